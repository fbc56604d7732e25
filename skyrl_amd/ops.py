"""torch.library custom ops over the C ABI for the fused LM head: ``skyrl_amd::lmhead_fwd`` and the ``skyrl_amd::lmhead_bwd*``
family (fp32 / bf16 weight gradient, hidden gradient alone, all tokens or the tokens with an upstream gradient only).

Tensors stay torch-owned; the ops pass raw device pointers, sizes and the current HIP stream through ctypes.  Scratch is a torch ``uint8`` tensor sized by the library's
own ``*_workspace_bytes`` query, so ``torch.cuda.max_memory_allocated`` sees every byte the path uses.

Shapes: hidden ``[T, H]`` bf16 (row stride a multiple of 8), weight ``[V, H]`` bf16, labels ``[T]`` int64 (a value
outside ``[0, V)`` means "no target": logprob 0 and no one-hot term in the gradient, which is how the reference treats
targets outside the vocab shard, model_utils.py:314-337, 405-411).
"""

from __future__ import annotations

from typing import Optional, Tuple

import torch

from . import _lib

__all__ = ["hidden_for_weight", "lmhead_fwd", "lmhead_bwd", "lmhead_bwd_bf16", "lmhead_bwd_hidden", "lmhead_bwd_active_rows", "fwd_workspace_bytes",
           "bwd_workspace_bytes"]


def _require_device(*tensors: torch.Tensor) -> torch.device:
    dev = tensors[0].device
    if dev.type != "cuda":
        raise RuntimeError(
            "skyrl_amd fused LM-head ops run only on a ROCm GPU (device type 'cuda'); got a tensor on "
            f"'{dev}'. There is no CPU implementation of this path."
        )
    for t in tensors:
        if t.device != dev:
            raise RuntimeError(f"all tensors must be on {dev}, got one on {t.device}")
    return dev


def _check_operands(hidden: torch.Tensor, weight: torch.Tensor, labels: torch.Tensor) -> Tuple[int, int, int]:
    if hidden.dim() != 2 or weight.dim() != 2 or labels.dim() != 1:
        raise ValueError(f"expected hidden [T,H], weight [V,H], labels [T]; got {tuple(hidden.shape)}, "
                         f"{tuple(weight.shape)}, {tuple(labels.shape)}")
    if (hidden.dtype, weight.dtype) not in _DTYPE_TERMS:
        raise TypeError(f"hidden / weight must be (bf16, bf16), (bf16, fp32) or (fp32, fp32) -- the reference casts hidden to the "
                        f"weight's dtype (model_utils.py:328-333) -- got {hidden.dtype} and {weight.dtype}; an fp32 hidden with a "
                        "bf16 weight would be a down-cast: do it explicitly if it is intended")
    if labels.dtype != torch.int64:
        raise TypeError(f"labels must be int64, got {labels.dtype}")
    T, H = hidden.shape
    V, H2 = weight.shape
    if H != H2 or labels.shape[0] != T:
        raise ValueError(f"shape mismatch: hidden {tuple(hidden.shape)}, weight {tuple(weight.shape)}, labels {tuple(labels.shape)}")
    if hidden.stride(1) != 1 or weight.stride(1) != 1 or not labels.is_contiguous():
        raise ValueError("hidden and weight must have unit stride in the last dimension and labels must be contiguous")
    return int(T), int(H), int(V)


# Number of bf16 terms per product for each (hidden, weight) dtype pair: 1 = the native bf16 path; 2 = fp32 weight as
# [w_hi | w_lo] against [h | h]; 3 = both fp32, [w_hi | w_lo | w_hi] against [h_hi | h_hi | h_lo].
_DTYPE_TERMS = {(torch.bfloat16, torch.bfloat16): 1, (torch.bfloat16, torch.float32): 2, (torch.float32, torch.float32): 3}
_SPLIT_HI_LO, _SPLIT_HI_HI, _SPLIT_HI_LO_HI, _SPLIT_HI_HI_LO = 0, 1, 2, 3


def _bf16_terms(hidden: torch.Tensor, weight: torch.Tensor) -> Tuple[torch.Tensor, torch.Tensor, int]:
    """The operands as the kernels take them: bf16, stacked hi / lo terms along the contraction axis when the weight is fp32
    (``skyrl_lmhead_split_operand``).  Nothing is down-cast: the fp32 logits are reproduced to about 2^-16 of each product."""
    terms = _DTYPE_TERMS[(hidden.dtype, weight.dtype)]
    if terms == 1:
        return hidden, weight, 1
    lib = _lib.load()
    T, H = hidden.shape
    V = weight.shape[0]
    dev = hidden.device
    h2 = torch.empty((T, terms * H), dtype=torch.bfloat16, device=dev)
    w2 = torch.empty((V, terms * H), dtype=torch.bfloat16, device=dev)
    h_layout, w_layout = (_SPLIT_HI_HI, _SPLIT_HI_LO) if terms == 2 else (_SPLIT_HI_HI_LO, _SPLIT_HI_LO_HI)
    with torch.cuda.device(dev):
        stream = torch.cuda.current_stream(dev).cuda_stream
        if T > 0:
            _lib.check(lib.skyrl_lmhead_split_operand(hidden.data_ptr(), int(hidden.dtype == torch.float32), hidden.stride(0), T, H,
                                                      h_layout, h2.data_ptr(), terms * H, stream), "skyrl_lmhead_split_operand")
        _lib.check(lib.skyrl_lmhead_split_operand(weight.data_ptr(), 1, weight.stride(0), V, H, w_layout, w2.data_ptr(),
                                                  terms * H, stream), "skyrl_lmhead_split_operand")
    return h2, w2, terms


def hidden_for_weight(hidden: torch.Tensor, weight: torch.Tensor) -> torch.Tensor:
    """``hidden`` as the reference's ``hidden.to(weight.dtype)`` needs it (model_utils.py:328-333) without a cast that changes
    nothing: a bf16 hidden stays bf16 next to an fp32 weight (the up-cast is exact, and two bf16 terms per product are cheaper
    than three); an fp32 hidden next to a bf16 weight is cast down, as the reference does."""
    if hidden.dtype == torch.bfloat16 and weight.dtype == torch.float32:
        return hidden
    return hidden.to(weight.dtype)


def fwd_workspace_bytes(T: int, H: int, V: int) -> int:
    return int(_lib.load().skyrl_lmhead_fwd_workspace_bytes(T, H, V))


def bwd_workspace_bytes(T: int, H: int, V: int, vocab_chunk: int = 0) -> int:
    return int(_lib.load().skyrl_lmhead_bwd_workspace_bytes(T, H, V, vocab_chunk))


def _ptr(t: Optional[torch.Tensor]) -> Optional[int]:
    return None if t is None else t.data_ptr()


@torch.library.custom_op("skyrl_amd::lmhead_fwd", mutates_args=())
def lmhead_fwd(
    hidden: torch.Tensor,
    weight: torch.Tensor,
    labels: torch.Tensor,
    rcp_temperature: float,
    want_entropy: bool,
) -> Tuple[torch.Tensor, torch.Tensor, torch.Tensor, torch.Tensor]:
    """Returns ``(logprobs, entropy, row_lse, row_pz)``, each fp32 ``[T]``.

    With ``want_entropy=False`` the sum p*z accumulation is skipped and ``entropy`` / ``row_pz`` come back empty (0 elements).
    """
    T, H, V = _check_operands(hidden, weight, labels)
    dev = _require_device(hidden, weight, labels)
    lib = _lib.load()
    f32 = dict(dtype=torch.float32, device=dev)
    if T == 0:  # an empty micro-batch: nothing to launch
        return torch.empty(0, **f32), torch.empty(0, **f32), torch.empty(0, **f32), torch.empty(0, **f32)
    logprobs = torch.empty(T, **f32)
    row_lse = torch.empty(T, **f32)
    entropy = torch.empty(T if want_entropy else 0, **f32)
    row_pz = torch.empty(T if want_entropy else 0, **f32)
    ws_bytes = int(lib.skyrl_lmhead_fwd_workspace_bytes(T, H, V))
    ws = torch.empty(ws_bytes, dtype=torch.uint8, device=dev)
    hidden, weight, terms = _bf16_terms(hidden, weight)
    with torch.cuda.device(dev):
        stream = torch.cuda.current_stream(dev).cuda_stream
        st = lib.skyrl_lmhead_fwd(
            hidden.data_ptr(), hidden.stride(0), weight.data_ptr(), weight.stride(0), labels.data_ptr(), T, terms * H, V,
            float(rcp_temperature), logprobs.data_ptr(), _ptr(entropy if want_entropy else None), row_lse.data_ptr(),
            _ptr(row_pz if want_entropy else None), ws.data_ptr(), ws_bytes, stream,
        )
    _lib.check(st, "skyrl_lmhead_fwd")
    return logprobs, entropy, row_lse, row_pz


@lmhead_fwd.register_fake
def _(hidden, weight, labels, rcp_temperature, want_entropy):
    T = hidden.shape[0]
    f32 = dict(dtype=torch.float32, device=hidden.device)
    n = T if want_entropy else 0
    return torch.empty(T, **f32), torch.empty(n, **f32), torch.empty(T, **f32), torch.empty(n, **f32)


@torch.library.custom_op("skyrl_amd::lmhead_bwd", mutates_args=())
def lmhead_bwd(
    hidden: torch.Tensor,
    weight: torch.Tensor,
    labels: torch.Tensor,
    row_lse: torch.Tensor,
    row_pz: Optional[torch.Tensor],
    dlogprobs: torch.Tensor,
    dentropy: Optional[torch.Tensor],
    rcp_temperature: float,
    vocab_chunk: int,
    active_rows: bool = False,
) -> Tuple[torch.Tensor, torch.Tensor]:
    """Returns ``(d_hidden bf16 [T,H], d_weight fp32 [V,H])``.  ``active_rows``: run on the tokens that have an upstream gradient
    only (``skyrl_lmhead_bwd_active_rows``: compaction on the device, no host synchronisation)."""
    T, H, V = _check_operands(hidden, weight, labels)
    dev = _require_device(hidden, weight, labels, row_lse, dlogprobs)
    lib = _lib.load()
    d_hidden = torch.empty((T, H), dtype=torch.bfloat16, device=dev)
    if T == 0:  # an empty micro-batch contributes a zero weight gradient
        return d_hidden, torch.zeros((V, H), dtype=torch.float32, device=dev)
    d_weight = torch.empty((V, H), dtype=torch.float32, device=dev)
    _bwd_into(lib, hidden, weight, labels, row_lse, row_pz, dlogprobs, dentropy, rcp_temperature, vocab_chunk, d_hidden,
              d_weight, False, active_rows)
    return d_hidden, d_weight


@torch.library.custom_op("skyrl_amd::lmhead_bwd_bf16", mutates_args=())
def lmhead_bwd_bf16(
    hidden: torch.Tensor,
    weight: torch.Tensor,
    labels: torch.Tensor,
    row_lse: torch.Tensor,
    row_pz: Optional[torch.Tensor],
    dlogprobs: torch.Tensor,
    dentropy: Optional[torch.Tensor],
    rcp_temperature: float,
    vocab_chunk: int,
    active_rows: bool = False,
) -> Tuple[torch.Tensor, torch.Tensor]:
    """``(d_hidden bf16 [T,H], d_weight bf16 [V,H])``: the weight gradient leaves the GEMM epilogue already rounded to the
    weight's dtype (what the autograd adapters hand back), with no fp32 ``[V, H]`` buffer and no cast pass."""
    T, H, V = _check_operands(hidden, weight, labels)
    dev = _require_device(hidden, weight, labels, row_lse, dlogprobs)
    d_hidden = torch.empty((T, H), dtype=torch.bfloat16, device=dev)
    if T == 0:
        return d_hidden, torch.zeros((V, H), dtype=torch.bfloat16, device=dev)
    d_weight = torch.empty((V, H), dtype=torch.bfloat16, device=dev)
    _bwd_into(_lib.load(), hidden, weight, labels, row_lse, row_pz, dlogprobs, dentropy, rcp_temperature, vocab_chunk, d_hidden,
              d_weight, False, active_rows)
    return d_hidden, d_weight


@lmhead_bwd_bf16.register_fake
def _(hidden, weight, labels, row_lse, row_pz, dlogprobs, dentropy, rcp_temperature, vocab_chunk, active_rows=False):
    return (torch.empty(hidden.shape, dtype=torch.bfloat16, device=hidden.device),
            torch.empty(weight.shape, dtype=torch.bfloat16, device=weight.device))


@torch.library.custom_op("skyrl_amd::lmhead_bwd_hidden", mutates_args=())
def lmhead_bwd_hidden(
    hidden: torch.Tensor,
    weight: torch.Tensor,
    labels: torch.Tensor,
    row_lse: torch.Tensor,
    row_pz: Optional[torch.Tensor],
    dlogprobs: torch.Tensor,
    dentropy: Optional[torch.Tensor],
    rcp_temperature: float,
    vocab_chunk: int,
    active_rows: bool = False,
) -> torch.Tensor:
    """``d_hidden`` bf16 [T,H] alone, for a weight that takes no gradient (a frozen LM head): the dW product is skipped."""
    T, H, V = _check_operands(hidden, weight, labels)
    dev = _require_device(hidden, weight, labels, row_lse, dlogprobs)
    d_hidden = torch.empty((T, H), dtype=torch.bfloat16, device=dev)
    if T > 0:
        _bwd_into(_lib.load(), hidden, weight, labels, row_lse, row_pz, dlogprobs, dentropy, rcp_temperature, vocab_chunk,
                  d_hidden, None, False, active_rows)
    return d_hidden


@lmhead_bwd_hidden.register_fake
def _(hidden, weight, labels, row_lse, row_pz, dlogprobs, dentropy, rcp_temperature, vocab_chunk, active_rows=False):
    return torch.empty(hidden.shape, dtype=torch.bfloat16, device=hidden.device)


def lmhead_bwd_active_rows(
    hidden: torch.Tensor,
    weight: torch.Tensor,
    labels: torch.Tensor,
    row_lse: torch.Tensor,
    row_pz: Optional[torch.Tensor],
    dlogprobs: torch.Tensor,
    dentropy: Optional[torch.Tensor],
    rcp_temperature: float,
    vocab_chunk: int = 0,
    want_dweight: bool = True,
    dweight_dtype: torch.dtype = torch.float32,
) -> Tuple[torch.Tensor, Optional[torch.Tensor]]:
    """The backward on the tokens whose upstream gradients are not all zero -- what the autograd adapters call.

    A token with ``dlogprobs == 0`` (and ``dentropy == 0``) has a zero dz row: it adds nothing to dW and its dHidden row is
    zero.  In RL micro-batches those are the prompt and padding tokens the loss mask removes (``loss_mask`` in
    megatron_model_wrapper.py:607-985; half of the tokens in the Qwen2.5-1.5B benchmark configuration), so the three
    backward GEMMs run on the remaining rows only.  The rows are listed, counted, gathered and scattered back by kernels
    (``skyrl_lmhead_bwd_active_rows``): the host never reads the count, nothing synchronises, shapes are static, and the
    call can sit inside a captured HIP graph.  With ``want_dweight=False`` (the weight takes no gradient) the dW product is
    skipped and ``None`` is returned in its place; ``dweight_dtype`` is fp32 or bf16 (rounded in the GEMM epilogue).

    With every token active the compaction is pure overhead: one scan, one copy of the hidden rows, one scatter of d_hidden.
    Measured through ``linear_cross_entropy(...).backward()`` at T=16384, H=3584, V=152064 with all tokens active: 48.45 ms
    against 48.09 ms for the dense C-ABI step (``bench.py``, ``autograd``), custom-op dispatch and the bf16 dW included.
    ``d_hidden`` is bf16 also for an fp32 ``hidden`` (the adapters cast it back): one rounding of 2^-9 relative, inside the
    reference's 2e-3 tolerance for grad_hidden, where the reference returns an fp32-accurate tensor.
    """
    if dweight_dtype not in (torch.float32, torch.bfloat16):
        raise TypeError(f"d_weight is fp32 or bf16, not {dweight_dtype}")
    args = (hidden, weight, labels, row_lse, row_pz, dlogprobs, dentropy, rcp_temperature, vocab_chunk, True)
    if want_dweight:
        return lmhead_bwd(*args) if dweight_dtype == torch.float32 else lmhead_bwd_bf16(*args)
    return lmhead_bwd_hidden(*args), None


# SKYRL_BWD_FLUSH_TINY_DZ of include/skyrl_lmhead.h: an option of every backward call made through this module, off by default.
FLUSH_TINY_DZ_BIT = 0x100
_flush_tiny_dz = False


def set_flush_tiny_dz(enabled: bool) -> bool:
    """Switch on / off the backward option that takes softmax probabilities below 2^-24 as exactly zero when dz is formed
    (``SKYRL_BWD_FLUSH_TINY_DZ``; no counterpart in the reference).  Returns the previous setting.  Results stay inside the
    path's tolerances (the flushed mass of a row is below V * 2^-24); the gradient GEMMs run faster on a power-limited GPU
    because most of the dz panel becomes zeros.  A process-wide setting: set it once, before training starts."""
    global _flush_tiny_dz
    previous, _flush_tiny_dz = _flush_tiny_dz, bool(enabled)
    return previous


def _bwd_into(lib, hidden, weight, labels, row_lse, row_pz, dlogprobs, dentropy, rcp_temperature, vocab_chunk, d_hidden,
              d_weight, accumulate_dw: bool, active_rows: bool = False) -> None:
    T, H = hidden.shape
    V = weight.shape[0]
    dev = hidden.device
    if dentropy is not None and (row_pz is None or row_pz.numel() != T):
        raise ValueError("an entropy gradient needs row_pz from a forward call made with want_entropy=True")
    for name, t in (("row_lse", row_lse), ("dlogprobs", dlogprobs), ("row_pz", row_pz), ("dentropy", dentropy)):
        if t is None:
            continue
        if name == "row_pz" and dentropy is None:
            continue
        if t.dtype != torch.float32 or t.shape != (T,) or not t.is_contiguous():
            raise ValueError(f"{name} must be a contiguous fp32 tensor of shape [{T}], got {t.dtype} {tuple(t.shape)}")
    terms = _DTYPE_TERMS[(hidden.dtype, weight.dtype)]
    ws_bytes = int(lib.skyrl_lmhead_bwd_split_workspace_bytes(T, H, terms, V, int(vocab_chunk), int(bool(active_rows))))
    if ws_bytes == 0:
        if int(vocab_chunk) < 0 or int(vocab_chunk) % 256 != 0:
            raise ValueError(f"bad vocab_chunk {vocab_chunk}: must be 0 (library default) or a multiple of 256")
        raise ValueError(f"no backward workspace for T={T}, H={H}, V={V}: every extent must be at least 1")
    ws = torch.empty(ws_bytes, dtype=torch.uint8, device=dev)
    hidden, weight, terms = _bf16_terms(hidden, weight)  # recomputed rather than kept from the forward: a pass over W, no 2x copy held
    with torch.cuda.device(dev):
        stream = torch.cuda.current_stream(dev).cuda_stream
        st = lib.skyrl_lmhead_bwd_split(
            hidden.data_ptr(), hidden.stride(0), weight.data_ptr(), weight.stride(0), labels.data_ptr(),
            row_lse.data_ptr(), _ptr(row_pz if dentropy is not None else None), dlogprobs.data_ptr(), _ptr(dentropy),
            T, H, terms, V, float(rcp_temperature), d_hidden.data_ptr(), _ptr(d_weight),
            (2 if (d_weight is not None and d_weight.dtype == torch.bfloat16) else int(bool(accumulate_dw)))
            | (FLUSH_TINY_DZ_BIT if _flush_tiny_dz else 0),
            int(vocab_chunk), int(bool(active_rows)), ws.data_ptr(), ws_bytes, stream,
        )
    _lib.check(st, "skyrl_lmhead_bwd_split")


def lmhead_bwd_accumulate(hidden, weight, labels, row_lse, row_pz, dlogprobs, dentropy, rcp_temperature: float,
                          d_weight_accum: torch.Tensor, vocab_chunk: int = 0) -> torch.Tensor:
    """Backward that *adds* dW into an existing fp32 ``[V, H]`` buffer (Megatron's ``main_grad`` style accumulation
    across micro-batches, the role of ``grad_weight.add_`` at model_utils.py:425) and returns ``d_hidden``."""
    T, H, V = _check_operands(hidden, weight, labels)
    dev = _require_device(hidden, weight, labels, row_lse, dlogprobs, d_weight_accum)
    if d_weight_accum.dtype != torch.float32 or d_weight_accum.shape != (V, H) or not d_weight_accum.is_contiguous():
        raise ValueError(f"d_weight_accum must be contiguous fp32 [{V},{H}]")
    d_hidden = torch.empty((T, H), dtype=torch.bfloat16, device=dev)
    if T == 0:  # an empty micro-batch adds nothing
        return d_hidden
    _bwd_into(_lib.load(), hidden, weight, labels, row_lse, row_pz, dlogprobs, dentropy, rcp_temperature, vocab_chunk,
              d_hidden, d_weight_accum, True)
    return d_hidden


@lmhead_bwd.register_fake
def _(hidden, weight, labels, row_lse, row_pz, dlogprobs, dentropy, rcp_temperature, vocab_chunk, active_rows=False):
    return (torch.empty(hidden.shape, dtype=torch.bfloat16, device=hidden.device),
            torch.empty(weight.shape, dtype=torch.float32, device=weight.device))


def _setup_context(ctx, inputs, output):
    hidden, weight, labels, rcp_temperature, want_entropy = inputs
    _, _, row_lse, row_pz = output
    ctx.save_for_backward(hidden, weight, labels, row_lse, row_pz)
    ctx.rcp_temperature = rcp_temperature
    ctx.want_entropy = want_entropy
    ctx.set_materialize_grads(False)  # unused outputs arrive as None in _backward


def _backward(ctx, d_logprobs, d_entropy, d_row_lse, d_row_pz):
    if d_row_lse is not None or d_row_pz is not None:
        # row_lse and row_pz are what the backward kernel takes back, not differentiable results: a loss built on them
        # (a z-loss on the log-sum-exp, say) would silently get no gradient.
        raise NotImplementedError("skyrl_amd::lmhead_fwd: row_lse and row_pz carry no gradient; only logprobs and entropy do")
    hidden, weight, labels, row_lse, row_pz = ctx.saved_tensors
    T = hidden.shape[0]
    if d_logprobs is None:
        d_logprobs = torch.zeros(T, dtype=torch.float32, device=hidden.device)
    d_logprobs = d_logprobs.to(torch.float32).contiguous()
    dent = None
    if ctx.want_entropy and d_entropy is not None:
        dent = d_entropy.to(torch.float32).contiguous()
    d_hidden, d_weight = lmhead_bwd_active_rows(hidden, weight, labels, row_lse, row_pz if dent is not None else None,
                                                d_logprobs, dent, ctx.rcp_temperature, 0, want_dweight=ctx.needs_input_grad[1],
                                                dweight_dtype=weight.dtype)
    # grad_hidden in the hidden dtype, grad_weight in the weight's dtype, as the reference does (model_utils.py:381, 428).
    return d_hidden.to(hidden.dtype), d_weight, None, None, None


lmhead_fwd.register_autograd(_backward, setup_context=_setup_context)
