"""Draft-head soft cross-entropy of multi-token prediction, fused with the two output-layer products that feed it.

The reference (skyrl/backends/skyrl_train/mtp/soft_ce.py) projects the draft head's hidden states and the policy's hidden
states through the shared output layer, keeps both ``[B, S, V]`` logits tensors, rolls the teacher's, takes fp32 softmaxes
of both and reduces ``-sum_v softmax(teacher)_v log_softmax(student)_v`` (``draft_soft_ce``, :200-240;
``_VocabParallelSoftCrossEntropy``, :123-154) -- several full-vocabulary tensors per micro-batch, bounded only by sequence
chunking with recomputation (:162-197).  Here the loss and its gradient come straight from the hidden states:

* ``soft_ce_from_hidden(student_hidden, teacher_hidden, weight, shift=...)`` -> per-token loss ``[B, S]`` fp32, differentiable
  with respect to ``student_hidden`` only (teacher and weight are detached in the reference as well, soft_ce.py:16-19,
  mtp/adapter.py:51-56);
* ``draft_soft_ce_from_hidden(...)`` -> the masked-mean scalar, ``draft_soft_ce``'s contract with hidden states in place of
  logits and ``mtp_layer_number`` in place of a pre-rolled teacher;
* ``shift_mask_for_mtp`` (:37-79) -- the mask roll the caller applies, same signature and results;
* ``unpadded_vocab_shard_width`` (:79-95) -- how many rows of a vocabulary shard are real when Megatron padded the vocabulary;
  where the reference slices both logits tensors to that width (megatron_model_wrapper.py:738-748), the caller here passes
  ``weight[:width]``.

* ``topk_logits_from_hidden``, ``soft_ce_topk_from_hidden``, ``draft_soft_ce_topk_from_hidden`` -- the top-k variant
  (``draft_soft_ce_topk`` / ``_VocabParallelTopkSoftCE``, :243-341): the teacher's k largest logits per token straight from
  its hidden states, the student's logits at those columns as k gathered dot products, loss and gradient over the k columns.

No ``[T, V]`` tensor exists at any point.
"""

from __future__ import annotations

from typing import Optional, Tuple

import torch

from . import _lib
from .ops import _require_device

__all__ = ["soft_ce_from_hidden", "draft_soft_ce_from_hidden", "shift_mask_for_mtp", "softce_fwd", "softce_bwd",
           "topk_logits_from_hidden", "soft_ce_topk_from_hidden", "draft_soft_ce_topk_from_hidden", "topk_logits",
           "softce_topk_fwd", "softce_topk_bwd", "unpadded_vocab_shard_width"]


def _check(student: torch.Tensor, teacher: torch.Tensor, weight: torch.Tensor, seq_len: int) -> Tuple[int, int, int]:
    if student.dim() != 2 or teacher.dim() != 2 or weight.dim() != 2:
        raise ValueError(f"expected student [T,H], teacher [T,H], weight [V,H]; got {tuple(student.shape)}, "
                         f"{tuple(teacher.shape)}, {tuple(weight.shape)}")
    for name, t in (("student_hidden", student), ("teacher_hidden", teacher), ("weight", weight)):
        if t.dtype != torch.bfloat16:
            raise TypeError(f"the HIP path computes in bf16: {name} must be torch.bfloat16, got {t.dtype}")
        if t.stride(1) != 1:
            raise ValueError(f"{name} must have unit stride in the last dimension")
    T, H = student.shape
    if teacher.shape != student.shape or weight.shape[1] != H:
        raise ValueError(f"shape mismatch: student {tuple(student.shape)}, teacher {tuple(teacher.shape)}, weight "
                         f"{tuple(weight.shape)}")
    if seq_len < 1 or T % seq_len != 0:
        raise ValueError(f"seq_len {seq_len} does not divide the {T} tokens")
    return int(T), int(H), int(weight.shape[0])


@torch.library.custom_op("skyrl_amd::softce_fwd", mutates_args=())
def softce_fwd(student_hidden: torch.Tensor, teacher_hidden: torch.Tensor, weight: torch.Tensor, seq_len: int, shift: int,
               rcp_temperature: float) -> Tuple[torch.Tensor, torch.Tensor, torch.Tensor]:
    """``(loss, lse_student, lse_teacher)``, each fp32 ``[T]``, for bf16 ``[T, H]`` hidden states and a bf16 ``[V, H]`` weight;
    token ``b * seq_len + s`` is scored against teacher row ``b * seq_len + (s + shift) mod seq_len``."""
    T, H, V = _check(student_hidden, teacher_hidden, weight, seq_len)
    dev = _require_device(student_hidden, teacher_hidden, weight)
    lib = _lib.load()
    ws = torch.empty(int(lib.skyrl_softce_fwd_workspace_bytes(T, H, V)), dtype=torch.uint8, device=dev)
    loss, lse_s, lse_t = (torch.empty(T, dtype=torch.float32, device=dev) for _ in range(3))
    with torch.cuda.device(dev):
        st = lib.skyrl_softce_fwd(student_hidden.data_ptr(), student_hidden.stride(0), teacher_hidden.data_ptr(),
                                  teacher_hidden.stride(0), weight.data_ptr(), weight.stride(0), T, int(seq_len), int(shift), H, V,
                                  float(rcp_temperature), loss.data_ptr(), lse_s.data_ptr(), lse_t.data_ptr(), ws.data_ptr(),
                                  ws.numel(), torch.cuda.current_stream(dev).cuda_stream)
    _lib.check(st, "skyrl_softce_fwd")
    return loss, lse_s, lse_t


@softce_fwd.register_fake
def _(student_hidden, teacher_hidden, weight, seq_len, shift, rcp_temperature):
    T = student_hidden.shape[0]
    return tuple(student_hidden.new_empty(T, dtype=torch.float32) for _ in range(3))


@torch.library.custom_op("skyrl_amd::softce_bwd", mutates_args=())
def softce_bwd(student_hidden: torch.Tensor, teacher_hidden: torch.Tensor, weight: torch.Tensor, lse_student: torch.Tensor,
               lse_teacher: torch.Tensor, dloss: torch.Tensor, seq_len: int, shift: int, rcp_temperature: float,
               vocab_chunk: int) -> torch.Tensor:
    """d loss / d student_hidden, bf16 ``[T, H]``, for the upstream gradient ``dloss`` fp32 ``[T]``."""
    T, H, V = _check(student_hidden, teacher_hidden, weight, seq_len)
    dev = _require_device(student_hidden, teacher_hidden, weight, lse_student, lse_teacher, dloss)
    for name, t in (("lse_student", lse_student), ("lse_teacher", lse_teacher), ("dloss", dloss)):
        if t.dtype != torch.float32 or t.shape != (T,) or not t.is_contiguous():
            raise ValueError(f"{name} must be a contiguous fp32 tensor of shape [{T}], got {t.dtype} {tuple(t.shape)}")
    lib = _lib.load()
    ws_bytes = int(lib.skyrl_softce_bwd_workspace_bytes(T, H, V, int(vocab_chunk)))
    if ws_bytes == 0:
        raise ValueError(f"bad vocab_chunk {vocab_chunk}: must be 0 (library default) or a multiple of 256")
    ws = torch.empty(ws_bytes, dtype=torch.uint8, device=dev)
    d_student = torch.empty((T, H), dtype=torch.bfloat16, device=dev)
    with torch.cuda.device(dev):
        st = lib.skyrl_softce_bwd(student_hidden.data_ptr(), student_hidden.stride(0), teacher_hidden.data_ptr(),
                                  teacher_hidden.stride(0), weight.data_ptr(), weight.stride(0), lse_student.data_ptr(),
                                  lse_teacher.data_ptr(), dloss.data_ptr(), T, int(seq_len), int(shift), H, V,
                                  float(rcp_temperature), d_student.data_ptr(), int(vocab_chunk), ws.data_ptr(), ws.numel(),
                                  torch.cuda.current_stream(dev).cuda_stream)
    _lib.check(st, "skyrl_softce_bwd")
    return d_student


@softce_bwd.register_fake
def _(student_hidden, teacher_hidden, weight, lse_student, lse_teacher, dloss, seq_len, shift, rcp_temperature, vocab_chunk):
    return torch.empty_like(student_hidden, memory_format=torch.contiguous_format)


class _SoftCE(torch.autograd.Function):
    @staticmethod
    def forward(ctx, student_hidden, teacher_hidden, weight, seq_len, shift, rcp_temperature, vocab_chunk):
        loss, lse_s, lse_t = softce_fwd(student_hidden, teacher_hidden, weight, seq_len, shift, rcp_temperature)
        ctx.save_for_backward(student_hidden, teacher_hidden, weight, lse_s, lse_t)
        ctx.args = (seq_len, shift, rcp_temperature, vocab_chunk)
        return loss

    @staticmethod
    def backward(ctx, dloss):
        student_hidden, teacher_hidden, weight, lse_s, lse_t = ctx.saved_tensors
        seq_len, shift, rcp_temperature, vocab_chunk = ctx.args
        d_student = softce_bwd(student_hidden, teacher_hidden, weight, lse_s, lse_t, dloss.to(torch.float32).contiguous(), seq_len,
                               shift, rcp_temperature, vocab_chunk)
        return d_student, None, None, None, None, None, None


def soft_ce_from_hidden(student_hidden: torch.Tensor, teacher_hidden: torch.Tensor, weight: torch.Tensor, *, shift: int = 0,
                        temperature: float = 1.0, vocab_chunk: int = 0) -> torch.Tensor:
    """Per-token soft cross-entropy ``[B, S]`` (fp32) of ``softmax(student_hidden @ weight.T)`` against
    ``softmax(roll(teacher_hidden, -shift, dims=1) @ weight.T)``.

    ``student_hidden`` and ``teacher_hidden`` are ``[B, S, H]`` (or ``[T, H]`` = one row) and are cast to the weight's bf16
    as the output layer would; only ``student_hidden`` receives a gradient.  ``teacher_hidden`` and ``weight`` must not
    require grad (the reference asserts a detached teacher, soft_ce.py:16-19).
    """
    assert not teacher_hidden.requires_grad, "MTP draft loss: teacher_hidden must be detached"
    assert not weight.requires_grad, "MTP draft loss: the output weight must be detached"
    if student_hidden.shape != teacher_hidden.shape:
        raise ValueError(f"student {tuple(student_hidden.shape)} and teacher {tuple(teacher_hidden.shape)} differ in shape")
    if student_hidden.dim() not in (2, 3):
        raise ValueError("hidden states must be [B, S, H] or [T, H]")
    H = student_hidden.shape[-1]
    seq_len = student_hidden.shape[-2]
    out_shape = student_hidden.shape[:-1]
    if student_hidden.numel() == 0:
        return student_hidden.new_zeros(out_shape, dtype=torch.float32) + 0.0 * student_hidden.sum()
    flat = lambda t: t.reshape(-1, H).to(torch.bfloat16).contiguous()  # noqa: E731
    loss = _SoftCE.apply(flat(student_hidden), flat(teacher_hidden), weight.to(torch.bfloat16), int(seq_len), int(shift),
                         1.0 / float(temperature), int(vocab_chunk))
    return loss.reshape(out_shape)


def draft_soft_ce_from_hidden(
    student_hidden: torch.Tensor,
    teacher_hidden: torch.Tensor,
    weight: torch.Tensor,
    mask: torch.Tensor,
    mtp_layer_number: int = 0,
    global_normalization_factor: Optional[torch.Tensor] = None,
    *,
    vocab_parallel_group=None,
    vocab_chunk: int = 0,
) -> torch.Tensor:
    """Masked-mean soft cross-entropy between the draft head (student) and the policy (teacher), the scalar
    ``draft_soft_ce(student_logits, build_teacher_logits(main_logits, mtp_layer_number), mask, global_normalization_factor)``
    returns (soft_ce.py:22-34, 200-240), computed from the hidden states that feed the shared output layer.

    ``mask`` is the ``[B, S]`` supervision mask (already shifted with ``shift_mask_for_mtp``); with
    ``global_normalization_factor`` the masked sum is divided by ``clamp(factor, min=1)`` instead of the local mask count
    (soft_ce.py:154-159).  A vocabulary sharded over more than one rank is refused.
    """
    if vocab_parallel_group is not None and torch.distributed.is_initialized() \
            and torch.distributed.get_world_size(vocab_parallel_group) > 1:
        raise NotImplementedError("the fused soft cross-entropy covers one vocabulary shard")
    per_token = soft_ce_from_hidden(student_hidden, teacher_hidden, weight, shift=mtp_layer_number + 1, vocab_chunk=vocab_chunk)
    mask = mask.to(per_token.dtype)
    if global_normalization_factor is not None:
        return (per_token * mask).sum() / global_normalization_factor.clamp(min=1.0)
    return (per_token * mask).sum() / mask.sum().clamp(min=1.0)


@torch.library.custom_op("skyrl_amd::topk_logits", mutates_args=())
def topk_logits(hidden: torch.Tensor, weight: torch.Tensor, k: int, rcp_temperature: float) -> Tuple[torch.Tensor, torch.Tensor]:
    """``(values [T, k] fp32, columns [T, k] int32)``: the k largest entries of every row of ``hidden @ weight.T *
    rcp_temperature``, best first, the lower column first among equal values.  bf16 operands, ``1 <= k <= min(V, 1024)``."""
    T, H, V = _check(hidden, hidden, weight, 1)
    dev = _require_device(hidden, weight)
    lib = _lib.load()
    if not 1 <= int(k) <= min(V, 1024):
        raise ValueError(f"bad k {k}: must be between 1 and min(V, 1024) = {min(V, 1024)}")
    if T == 0:  # an empty batch: nothing to launch
        return torch.empty((0, k), dtype=torch.float32, device=dev), torch.empty((0, k), dtype=torch.int32, device=dev)
    ws_bytes = int(lib.skyrl_lmhead_topk_workspace_bytes(T, H, V, int(k)))
    if ws_bytes == 0:
        raise ValueError(f"no top-k workspace for T={T}, H={H}, V={V}, k={k}: an extent is out of range")
    ws = torch.empty(ws_bytes, dtype=torch.uint8, device=dev)
    values = torch.empty((T, k), dtype=torch.float32, device=dev)
    columns = torch.empty((T, k), dtype=torch.int32, device=dev)
    with torch.cuda.device(dev):
        st = lib.skyrl_lmhead_topk_logits(hidden.data_ptr(), hidden.stride(0), weight.data_ptr(), weight.stride(0), T, H, V, int(k),
                                          float(rcp_temperature), values.data_ptr(), columns.data_ptr(), ws.data_ptr(), ws.numel(),
                                          torch.cuda.current_stream(dev).cuda_stream)
    _lib.check(st, "skyrl_lmhead_topk_logits")
    return values, columns


@topk_logits.register_fake
def _(hidden, weight, k, rcp_temperature):
    T = hidden.shape[0]
    return hidden.new_empty((T, k), dtype=torch.float32), hidden.new_empty((T, k), dtype=torch.int32)


@torch.library.custom_op("skyrl_amd::softce_topk_fwd", mutates_args=())
def softce_topk_fwd(student_hidden: torch.Tensor, weight: torch.Tensor, teacher_values: torch.Tensor, teacher_columns: torch.Tensor,
                    seq_len: int, shift: int, rcp_temperature: float) -> Tuple[torch.Tensor, torch.Tensor, torch.Tensor]:
    """``(loss [T] fp32, coef [T, k] fp32, columns [T, k] int32)`` for bf16 ``student_hidden [T, H]``, ``weight [V, H]`` and the
    teacher's top-k lists; token ``b * seq_len + s`` is scored against the list of token ``b * seq_len + (s + shift) mod seq_len``."""
    T, H, V = _check(student_hidden, student_hidden, weight, seq_len)
    dev = _require_device(student_hidden, weight, teacher_values, teacher_columns)
    k = int(teacher_values.shape[1]) if teacher_values.dim() == 2 else 0
    if (teacher_values.shape != (T, k) or teacher_columns.shape != (T, k) or teacher_values.dtype != torch.float32
            or teacher_columns.dtype != torch.int32 or not teacher_values.is_contiguous() or not teacher_columns.is_contiguous()):
        raise ValueError(f"teacher_values must be contiguous fp32 [{T}, k] and teacher_columns contiguous int32 [{T}, k]")
    lib = _lib.load()
    loss = torch.empty(T, dtype=torch.float32, device=dev)
    coef = torch.empty((T, k), dtype=torch.float32, device=dev)
    columns = torch.empty((T, k), dtype=torch.int32, device=dev)
    with torch.cuda.device(dev):
        st = lib.skyrl_softce_topk_fwd(student_hidden.data_ptr(), student_hidden.stride(0), weight.data_ptr(), weight.stride(0),
                                       teacher_values.data_ptr(), teacher_columns.data_ptr(), T, int(seq_len), int(shift), H, V, k,
                                       float(rcp_temperature), loss.data_ptr(), coef.data_ptr(), columns.data_ptr(),
                                       torch.cuda.current_stream(dev).cuda_stream)
    _lib.check(st, "skyrl_softce_topk_fwd")
    return loss, coef, columns


@softce_topk_fwd.register_fake
def _(student_hidden, weight, teacher_values, teacher_columns, seq_len, shift, rcp_temperature):
    T = student_hidden.shape[0]
    return (student_hidden.new_empty(T, dtype=torch.float32), torch.empty_like(teacher_values), torch.empty_like(teacher_columns))


@torch.library.custom_op("skyrl_amd::softce_topk_bwd", mutates_args=())
def softce_topk_bwd(weight: torch.Tensor, coef: torch.Tensor, columns: torch.Tensor, dloss: torch.Tensor,
                    rcp_temperature: float) -> torch.Tensor:
    """d loss / d student_hidden, bf16 ``[T, H]``, from what ``softce_topk_fwd`` kept and the upstream gradient ``dloss [T]``."""
    T, k = int(coef.shape[0]), int(coef.shape[1])
    V, H = int(weight.shape[0]), int(weight.shape[1])
    dev = _require_device(weight, coef, columns, dloss)
    if weight.dtype != torch.bfloat16 or weight.stride(1) != 1:
        raise TypeError("weight must be bf16 with unit stride in the last dimension")
    if (coef.dtype != torch.float32 or columns.dtype != torch.int32 or columns.shape != coef.shape or not coef.is_contiguous()
            or not columns.is_contiguous() or dloss.dtype != torch.float32 or dloss.shape != (T,) or not dloss.is_contiguous()):
        raise ValueError("coef fp32 [T, k], columns int32 [T, k] and dloss fp32 [T] must be contiguous")
    lib = _lib.load()
    d_student = torch.empty((T, H), dtype=torch.bfloat16, device=dev)
    with torch.cuda.device(dev):
        st = lib.skyrl_softce_topk_bwd(weight.data_ptr(), weight.stride(0), coef.data_ptr(), columns.data_ptr(), dloss.data_ptr(), T, H,
                                       V, k, float(rcp_temperature), d_student.data_ptr(), H, torch.cuda.current_stream(dev).cuda_stream)
    _lib.check(st, "skyrl_softce_topk_bwd")
    return d_student


@softce_topk_bwd.register_fake
def _(weight, coef, columns, dloss, rcp_temperature):
    return weight.new_empty((coef.shape[0], weight.shape[1]))


class _SoftCETopk(torch.autograd.Function):
    @staticmethod
    def forward(ctx, student_hidden, teacher_hidden, weight, k, seq_len, shift, rcp_temperature):
        values, columns = topk_logits(teacher_hidden, weight, k, rcp_temperature)
        loss, coef, used = softce_topk_fwd(student_hidden, weight, values, columns, seq_len, shift, rcp_temperature)
        ctx.save_for_backward(weight, coef, used)
        ctx.rcp_temperature = rcp_temperature
        return loss

    @staticmethod
    def backward(ctx, dloss):
        weight, coef, used = ctx.saved_tensors
        return (softce_topk_bwd(weight, coef, used, dloss.to(torch.float32).contiguous(), ctx.rcp_temperature), None, None, None,
                None, None, None)


def topk_logits_from_hidden(hidden: torch.Tensor, weight: torch.Tensor, k: int, *, temperature: float = 1.0
                            ) -> Tuple[torch.Tensor, torch.Tensor]:
    """``(hidden @ weight.T / temperature).topk(min(k, V), dim=-1)`` without the logits: values fp32 and indices int64 of shape
    ``hidden.shape[:-1] + (k,)``.  Not differentiable (the reference takes the top-k of a detached teacher, soft_ce.py:273)."""
    H = hidden.shape[-1]
    k_eff = min(int(k), int(weight.shape[0]))
    with torch.no_grad():
        values, columns = topk_logits(hidden.detach().reshape(-1, H).to(torch.bfloat16).contiguous(), weight.detach().to(torch.bfloat16),
                                      k_eff, 1.0 / float(temperature))
    shape = tuple(hidden.shape[:-1]) + (k_eff,)
    return values.reshape(shape), columns.reshape(shape).to(torch.int64)


def soft_ce_topk_from_hidden(student_hidden: torch.Tensor, teacher_hidden: torch.Tensor, weight: torch.Tensor, k: int, *,
                             shift: int = 0, temperature: float = 1.0) -> torch.Tensor:
    """Per-token top-k soft cross-entropy ``[B, S]`` (fp32): the teacher's ``min(k, V)`` largest logits of position ``s + shift``
    (``roll(teacher, -shift, dims=1)``) and the student's logits at the same columns, both renormalised over those columns
    (``_VocabParallelTopkSoftCE.forward``, soft_ce.py:258-305, one vocabulary shard).  Differentiable with respect to
    ``student_hidden`` only; the gradient touches the k columns alone (:307-315)."""
    assert not teacher_hidden.requires_grad, "MTP draft loss: teacher_hidden must be detached"
    assert not weight.requires_grad, "MTP draft loss: the output weight must be detached"
    if student_hidden.shape != teacher_hidden.shape:
        raise ValueError(f"student {tuple(student_hidden.shape)} and teacher {tuple(teacher_hidden.shape)} differ in shape")
    if student_hidden.dim() not in (2, 3):
        raise ValueError("hidden states must be [B, S, H] or [T, H]")
    if int(k) < 1:
        raise ValueError(f"k must be positive, got {k}")
    H = student_hidden.shape[-1]
    seq_len = student_hidden.shape[-2]
    out_shape = student_hidden.shape[:-1]
    if student_hidden.numel() == 0:
        return student_hidden.new_zeros(out_shape, dtype=torch.float32) + 0.0 * student_hidden.sum()
    flat = lambda t: t.reshape(-1, H).to(torch.bfloat16).contiguous()  # noqa: E731
    loss = _SoftCETopk.apply(flat(student_hidden), flat(teacher_hidden), weight.to(torch.bfloat16), min(int(k), int(weight.shape[0])),
                             int(seq_len), int(shift), 1.0 / float(temperature))
    return loss.reshape(out_shape)


def draft_soft_ce_topk_from_hidden(
    student_hidden: torch.Tensor,
    teacher_hidden: torch.Tensor,
    weight: torch.Tensor,
    mask: torch.Tensor,
    k: int,
    global_normalization_factor: Optional[torch.Tensor] = None,
    vocab_parallel_group=None,
    roll_shift: int = 0,
) -> torch.Tensor:
    """Masked-mean top-k soft cross-entropy, the scalar ``draft_soft_ce_topk(student_logits, teacher_logits, mask, k,
    global_normalization_factor, vocab_parallel_group, roll_shift)`` returns (soft_ce.py:318-341), with the hidden states that
    feed the shared output layer in place of the two logits tensors.  ``teacher_hidden`` is the un-rolled policy hidden state
    and ``roll_shift`` the MTP depth roll, as there."""
    if vocab_parallel_group is not None and torch.distributed.is_initialized() \
            and torch.distributed.get_world_size(vocab_parallel_group) > 1:
        raise NotImplementedError("the fused top-k soft cross-entropy covers one vocabulary shard")
    per_token = soft_ce_topk_from_hidden(student_hidden, teacher_hidden, weight, k, shift=roll_shift)
    mask = mask.to(per_token.dtype)
    if global_normalization_factor is not None:
        return (per_token * mask).sum() / global_normalization_factor.clamp(min=1.0)
    return (per_token * mask).sum() / mask.sum().clamp(min=1.0)


def shift_mask_for_mtp(mask: torch.Tensor, mtp_layer_number: int = 0, cu_seqlens: Optional[torch.Tensor] = None) -> torch.Tensor:
    """Loss mask aligned with the teacher at MTP depth ``mtp_layer_number`` (reference ``shift_mask_for_mtp``,
    soft_ce.py:37-79): position ``t`` stays supervised only if both ``t`` and ``t + shift`` are real tokens of the same
    sequence; with ``cu_seqlens`` the ``[1, T]`` mask is one packed row and the roll stays inside each segment."""
    shift = mtp_layer_number + 1
    S = mask.shape[1]
    pos = torch.arange(S, device=mask.device)
    if cu_seqlens is None:
        end = torch.full((S,), S, device=mask.device, dtype=torch.long)
    else:
        cu = torch.as_tensor(cu_seqlens, device=mask.device, dtype=torch.long)
        if cu.numel() < 2:
            return torch.zeros_like(mask)
        seg = torch.searchsorted(cu[1:].contiguous(), pos, right=True).clamp(max=cu.numel() - 2)
        end = cu[1:][seg]
        end = torch.where(pos < cu[-1], end, torch.zeros_like(end))  # positions past the last segment are not supervised
    target = pos + shift
    ok = target < end
    rolled = torch.where(ok, mask[:, target.clamp(max=S - 1)], torch.zeros((), dtype=mask.dtype, device=mask.device))
    return mask * rolled


def unpadded_vocab_shard_width(true_vocab_size: Optional[int], vocab_shard_width: int, tp_rank: int) -> int:
    """Rows of rank ``tp_rank``'s vocabulary shard that belong to the true vocabulary (reference
    ``unpadded_vocab_shard_width``, soft_ce.py:79-95): the shard starts at ``tp_rank * vocab_shard_width`` and the padding sits
    at the end of the padded vocabulary, so the count is what is left of the true vocabulary from that start, between 0 and
    the shard's width; the whole width when the true size is unknown.  Padded rows are never trained and must not enter the
    teacher distribution: pass ``weight[:width]`` to the draft-loss functions of this module."""
    if true_vocab_size is None:
        return vocab_shard_width
    remaining = true_vocab_size - tp_rank * vocab_shard_width
    return min(vocab_shard_width, remaining) if remaining > 0 else 0
