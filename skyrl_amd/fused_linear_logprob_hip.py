"""Autograd front ends of the HIP fused LM-head path, with the reference's call signatures.

* ``LinearCrossEntropy`` / ``linear_cross_entropy`` -- verl's interface, vendored in the reference at
  ``skyrl/backends/skyrl_train/distributed/megatron/fused_linear_logprob_triton.py:1763-1824``:
  ``(hidden, weight, labels, temperature: float, reduction: str, dist_process_group) -> (logprobs, entropy)`` and a backward
  that takes both upstream gradients.
* ``FusedLinearLogprobHip`` -- the SkyRL adapter contract of ``FusedLinearLogprobTriton`` (same file, :1839-1959) and
  ``FusedLinearChunkedDistributedLogprob`` (``.../megatron/model_utils.py:275-428``):
  ``apply(hidden[B,S,H], weight[V,H], target[B,S], vocab_start_index, vocab_end_index, chunk_size, tp_group, inference_only)``
  ``-> logprobs [B,S] fp32``; backward returns ``(grad_hidden, grad_weight, None x 6)``.

Both run the same two custom ops (``skyrl_amd::lmhead_fwd`` / ``lmhead_bwd``).  ``chunk_size`` is accepted and ignored: the
kernel tiles the problem itself and never holds more than one 256 x 256 logits tile per workgroup in registers.
"""

from __future__ import annotations

import typing
from typing import Any, Optional

import torch
import torch.distributed as dist

from . import ops

_OOV_LABEL_SENTINEL = torch.iinfo(torch.int64).max

_REDUCTIONS = ("none", "sum", "mean")


class EntropyReductionEnum:
    """Reduction of the log-probability output, as numbers (``fused_linear_logprob_triton.py:146-152``)."""

    _None = 0
    _Sum = 1
    _Mean = 2


_REDUCTION_NUMBER = {"none": EntropyReductionEnum._None, "sum": EntropyReductionEnum._Sum, "mean": EntropyReductionEnum._Mean}


def get_entropy_reduction_enum_number(reduction: str) -> int:
    """``"none" | "sum" | "mean"`` -> 0 | 1 | 2; anything else is a ``ValueError`` (``fused_linear_logprob_triton.py:155-166``)."""
    try:
        return _REDUCTION_NUMBER[reduction]
    except KeyError:
        raise ValueError(f"Invalid reduction: {reduction}") from None


def get_entropy_reduction_enum(ce_reduction: int) -> int:
    """The inverse check: 0, 1 or 2 is returned as it is, anything else is a ``ValueError`` (``...triton.py:169-180``)."""
    if ce_reduction not in _REDUCTION_NUMBER.values():
        raise ValueError(f"Invalid ce_reduction: {ce_reduction}")
    return int(ce_reduction)


class BackwardEnum:
    """The backward methods verl's kernels offer (``fused_linear_logprob_triton.py:185-195``).  One of them is built here:
    ``_Split_Dlogits_N`` -- d_logits formed one vocabulary chunk at a time and fed to two GEMMs -- which is also the
    reference's default and the only one SkyRL ever selects (:206, :213-216)."""

    _Total_Fuse_MN = 0
    _Total_Separate = 1
    _Split_Dlogits_N = 2
    _Split_Dlogits_M = 3


def set_backward_method(backward_method: int) -> None:
    """Counterpart of ``set_backward_method`` (``fused_linear_logprob_triton.py:213-216``).  Accepts the method that is built
    and refuses the others: ``_Total_Fuse_MN`` needs fp32 atomic adds of whole ``[256, H]`` tiles (280 GB of them at the 7B
    shape), ``_Total_Separate`` stores the full ``[T, V]`` d_logits, ``_Split_Dlogits_M`` re-reads the weight once per token
    split."""
    if backward_method != BackwardEnum._Split_Dlogits_N:
        raise NotImplementedError(
            f"backward method {backward_method!r}: the HIP path builds BackwardEnum._Split_Dlogits_N (value 2) only")


# Counterpart of the reference's module flag (``fused_linear_logprob_triton.py:603-611``), which switches fp32 operands from
# tf32 to IEEE products in its tests.  There is no reduced-precision route for fp32 operands here -- an fp32 weight always
# enters the matrix pipe as exact hi + lo bf16 terms -- so the flag is accepted and changes nothing.
FORCE_FP32_IEEE_PRECISION = False


def _group_size(group: Optional[dist.ProcessGroup]) -> int:
    if group is None or not (dist.is_available() and dist.is_initialized()):
        return 1
    return dist.get_world_size(group)


def _require_single_shard(group: Optional[dist.ProcessGroup], what: str) -> None:
    if _group_size(group) > 1:
        raise NotImplementedError(
            f"{what}: the HIP fused LM-head path is built for one vocab shard per GPU (tensor-parallel size 1); "
            f"got a process group of size {_group_size(group)}"
        )


class LinearCrossEntropy(torch.autograd.Function):
    """verl-style fused linear + log-prob + entropy.  See the module docstring for the reference lines."""

    @staticmethod
    def forward(  # type: ignore[override]
        ctx,
        hidden: torch.Tensor,
        weight: torch.Tensor,
        labels: torch.Tensor,
        temperature: typing.Optional[float] = 1.0,
        reduction: typing.Optional[str] = "none",
        dist_process_group: typing.Optional[dist.ProcessGroup] = None,
        want_entropy: bool = True,
    ):
        """``want_entropy`` (an extension; the reference always computes the entropy): with ``False`` the sum p*z accumulation is
        skipped, the second result is ``None`` and the backward runs the kernel variant without the entropy-gradient term."""
        assert isinstance(temperature, float), f"temperature must be a float, but got {type(temperature)}"
        assert isinstance(reduction, str), f"reduction must be a str, but got {type(reduction)}"
        reduction = reduction.lower()
        if reduction not in _REDUCTIONS:
            raise ValueError(f"Invalid reduction: {reduction}")
        _require_single_shard(dist_process_group, "linear_cross_entropy")
        assert hidden.shape[-1] == weight.shape[1] and weight.dim() == 2

        original_hidden_shape = hidden.shape
        hidden2 = hidden.reshape(-1, hidden.shape[-1])
        labels1 = labels.reshape(-1)
        assert hidden2.shape[0] == labels1.shape[0]
        labels1 = labels1.to(torch.int64).contiguous()  # what the kernel reads is what the backward gets back
        rcp_t = 1.0 / temperature
        with torch.no_grad():
            logprobs, entropy, row_lse, row_pz = ops.lmhead_fwd(hidden2, weight, labels1, rcp_t, bool(want_entropy))
        ctx.save_for_backward(hidden2, weight, labels1, row_lse, row_pz)
        # An output nobody uses arrives in backward as None, not as a tensor of zeros: an unused entropy then costs nothing.
        ctx.set_materialize_grads(False)
        ctx.want_entropy = bool(want_entropy)
        ctx.original_hidden_shape = original_hidden_shape
        ctx.reduction = reduction
        ctx.rcp_t = rcp_t
        # The reduction applies to the logprob output only; entropy stays per token (fused_linear_logprob_triton.py:468-475).
        if reduction == "sum":
            logprobs = logprobs.sum()
        elif reduction == "mean":
            logprobs = logprobs.mean()
        return logprobs, (entropy if want_entropy else None)

    @staticmethod
    def backward(ctx, dlogprobs: torch.Tensor, dentropy: torch.Tensor):  # type: ignore[override]
        hidden2, weight, labels1, row_lse, row_pz = ctx.saved_tensors
        T = hidden2.shape[0]
        dev = hidden2.device
        if dlogprobs is None:
            g = torch.zeros(T, dtype=torch.float32, device=dev)
        elif ctx.reduction == "none":
            g = dlogprobs.reshape(-1).to(torch.float32).contiguous()
        elif ctx.reduction == "sum":  # broadcast of the scalar gradient (fused_linear_logprob_triton.py:896-905)
            g = dlogprobs.to(torch.float32).expand(T).contiguous()
        else:
            g = (dlogprobs.to(torch.float32) / T).expand(T).contiguous()
        q = None if (dentropy is None or not ctx.want_entropy) else dentropy.reshape(-1).to(torch.float32).contiguous()
        d_hidden, d_weight = ops.lmhead_bwd_active_rows(hidden2, weight, labels1, row_lse, row_pz if q is not None else None,
                                                        g, q, ctx.rcp_t, 0, want_dweight=ctx.needs_input_grad[1],
                                                        dweight_dtype=weight.dtype)   # None for a frozen LM head
        return d_hidden.to(hidden2.dtype).view(ctx.original_hidden_shape), d_weight, None, None, None, None, None


linear_cross_entropy = LinearCrossEntropy.apply


class FusedLinearLogprobHip(torch.autograd.Function):
    """HIP fused LM-head + log-prob of the target token; drop-in for ``FusedLinearLogprobTriton`` at TP = 1."""

    @staticmethod
    def forward(  # type: ignore[override]
        ctx: Any,
        hidden: torch.Tensor,
        weight: torch.Tensor,
        target: torch.Tensor,
        vocab_start_index: int,
        vocab_end_index: int,
        chunk_size: int,
        tp_group: Optional[dist.ProcessGroup],
        inference_only: bool = False,
    ) -> torch.Tensor:
        _require_single_shard(tp_group, "FusedLinearLogprobHip")
        B, S, H = hidden.shape
        local_vocab = int(weight.shape[0])
        # Targets outside [vocab_start_index, vocab_end_index) get a label that matches no column: forward 0, backward keeps
        # -softmax * grad (fused_linear_logprob_triton.py:1876-1878, 1898-1905, 1929-1931).
        target_mask = (target < vocab_start_index) | (target >= vocab_end_index)
        target = target.to(torch.int64)  # int32 ids: the sentinel below does not fit their dtype
        labels = torch.where(target_mask, _OOV_LABEL_SENTINEL, target - vocab_start_index).reshape(-1).contiguous()
        # The kernel needs 2-D operands with matching dtypes: hidden follows the weight (model_utils.py:328-333).
        hidden_2d = ops.hidden_for_weight(hidden.reshape(B * S, H), weight).contiguous()
        weight_c = weight.contiguous()
        assert local_vocab == weight_c.shape[0]

        with torch.no_grad():
            logprobs, _, row_lse, _ = ops.lmhead_fwd(hidden_2d, weight_c, labels, 1.0, False)
        ctx.set_materialize_grads(False)
        if not inference_only:
            ctx.save_for_backward(hidden_2d, weight_c, labels, row_lse)
            ctx.shape = (B, S, H)
            ctx.hidden_dtype = hidden.dtype
        return logprobs.reshape(B, S)

    @staticmethod
    def backward(ctx: Any, *grad_outputs: torch.Tensor):  # type: ignore[override]
        grad_output = grad_outputs[0]
        hidden_2d, weight_c, labels, row_lse = ctx.saved_tensors
        B, S, H = ctx.shape
        if grad_output is None:
            g = torch.zeros(B * S, dtype=torch.float32, device=hidden_2d.device)
        else:
            g = grad_output.reshape(-1).to(torch.float32).contiguous()
        d_hidden, d_weight = ops.lmhead_bwd_active_rows(hidden_2d, weight_c, labels, row_lse, None, g, None, 1.0, 0,
                                                        want_dweight=ctx.needs_input_grad[1], dweight_dtype=weight_c.dtype)
        # grad_hidden in the hidden dtype, grad_weight in the weight dtype (model_utils.py:381, 428), rounded in the GEMM
        # epilogue; none for a frozen head.
        return d_hidden.reshape(B, S, H).to(ctx.hidden_dtype), d_weight, None, None, None, None, None, None
