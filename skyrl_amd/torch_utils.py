"""Log-probabilities and entropy from materialised logits, with the reference's call signatures.

For callers that already hold a ``[B, S, V]`` logits tensor (the FSDP worker's forward tail, models whose head is not a plain
linear layer):

* ``logprobs_from_logits(logits, labels, inplace_backward=True)``, ``logprobs_from_logits_v2(logits, labels)``,
  ``logprobs_from_logits_flash_attn`` -- ``skyrl/backends/skyrl_train/utils/torch_utils.py:115-177``;
* ``chunked_entropy_from_logits(logits, requires_grad=False, attention_mask=None, chunk_size=1024)`` -- ``:58-111``;
* ``logprobs_and_entropy_from_logits`` -- both from one pass over the logits (an extension);
* ``DistributedLogprob`` / ``ChunkedDistributedLogprob`` -- the apply signatures of the logits-input autograd functions of
  ``.../distributed/megatron/model_utils.py:66-272`` on one vocabulary shard, and ``from_parallel_logits_to_logprobs`` (:487-565).

Every forward is one HIP kernel that reads the logits once (the reference makes several passes and, in
``DistributedLogprob``, keeps an fp32 softmax of the whole tensor for the backward); the backward recomputes the softmax from the
logits and the saved ``[T]`` row statistics in one read + write pass, over the logits themselves when ``inplace_backward`` says so.
A sliced view such as ``logits[:, :-1]`` is walked where it lies (one launch per batch entry), not copied.
"""

from __future__ import annotations

from typing import Any, Optional, Tuple

import torch

from . import _lib
from .ops import _require_device as _require_device_all

__all__ = ["logprobs_from_logits", "logprobs_from_logits_v2", "logprobs_from_logits_flash_attn", "chunked_entropy_from_logits",
           "logprobs_and_entropy_from_logits", "DistributedLogprob", "ChunkedDistributedLogprob",
           "from_parallel_logits_to_logprobs", "from_parallel_logits_to_logprobs_packed_sequences", "vocab_parallel_entropy", "vocab_parallel_entropy_weighted_sum",
           "vocab_parallel_entropy_packed_sequences", "logits_fwd", "logits_bwd", "logits_bwd_"]

_DTYPES = {torch.bfloat16: 0, torch.float32: 1}


def _require_device(*tensors: Optional[torch.Tensor]) -> torch.device:
    return _require_device_all(*[t for t in tensors if t is not None])


def _rows(logits: torch.Tensor) -> Tuple[int, int, int]:
    """(T, V, leading dimension) of a 2-D logits matrix the kernels can walk."""
    if logits.dim() != 2:
        raise ValueError(f"expected logits [T, V], got {tuple(logits.shape)}")
    if logits.dtype not in _DTYPES:
        raise TypeError(f"logits must be torch.bfloat16 or torch.float32, got {logits.dtype}")
    if logits.stride(1) != 1 and logits.shape[1] > 1:
        raise ValueError("logits must have unit stride in the last dimension")
    T, V = int(logits.shape[0]), int(logits.shape[1])
    ld = int(logits.stride(0)) if T > 1 else V
    if ld < V:
        raise ValueError(f"logits rows overlap: row stride {ld} < {V}")
    return T, V, ld


def _pieces(logits: torch.Tensor) -> Tuple[int, int, list]:
    """``(T, V, pieces)`` of a ``[T, V]`` matrix or a ``[B, S, V]`` tensor: the runs of equally pitched rows the kernels walk,
    each ``(2-D view, index of its first row)``.  A 3-D tensor whose batch stride is ``S`` row pitches is one run; a view such
    as ``logits[:, :-1]`` (rows equally pitched inside a batch entry only) is one run per batch entry -- walked where it
    lies, never copied."""
    if logits.dim() == 2:
        T, V, _ = _rows(logits)
        return T, V, [(logits, 0)]
    if logits.dim() != 3:
        raise ValueError(f"expected logits [T, V] or [B, S, V], got {tuple(logits.shape)}")
    B, S, V = (int(x) for x in logits.shape)
    if B * S == 0:
        return 0, V, []
    flat = None
    if B == 1:
        flat = logits[0]
    elif S == 1:
        flat = logits[:, 0]
    elif logits.stride(0) == S * logits.stride(1):
        flat = logits.as_strided((B * S, V), (logits.stride(1), logits.stride(2)), logits.storage_offset())
    if flat is not None:
        _rows(flat)
        return B * S, V, [(flat, 0)]
    for b in range(B):
        _rows(logits[b])
    return B * S, V, [(logits[b], b * S) for b in range(B)]


def _check_rows(name: str, t: Optional[torch.Tensor], T: int, dtype: torch.dtype) -> None:
    if t is not None and (t.dtype != dtype or t.shape != (T,) or not t.is_contiguous()):
        raise ValueError(f"{name} must be a contiguous {dtype} tensor of shape [{T}], got {t.dtype} {tuple(t.shape)}")


@torch.library.custom_op("skyrl_amd::logits_fwd", mutates_args=())
def logits_fwd(logits: torch.Tensor, labels: Optional[torch.Tensor], rcp_temperature: float, want_entropy: bool
               ) -> Tuple[torch.Tensor, torch.Tensor, torch.Tensor, torch.Tensor]:
    """``(logprobs, entropy, row_lse, row_pz)``, fp32 ``[T]``, of ``logits [T, V] * rcp_temperature``.  Without ``labels`` the
    log-probabilities are zero; without ``want_entropy`` entropy and ``row_pz`` are zero (and cost nothing)."""
    T, V, pieces = _pieces(logits)
    dev = _require_device(logits, labels)
    _check_rows("labels", labels, T, torch.int64)
    f32 = dict(dtype=torch.float32, device=dev)
    lp, lse = (torch.zeros(T, **f32) if labels is None else torch.empty(T, **f32)), torch.empty(T, **f32)
    ent, pz = (torch.empty(T, **f32), torch.empty(T, **f32)) if want_entropy else (torch.zeros(T, **f32), torch.zeros(T, **f32))
    if T == 0:
        return lp, ent, lse, pz
    lib = _lib.load()
    with torch.cuda.device(dev):
        stream = torch.cuda.current_stream(dev).cuda_stream
        for view, r0 in pieces:
            rows, _, ld = _rows(view)
            st = lib.skyrl_logits_fwd(view.data_ptr(), _DTYPES[logits.dtype], ld, None if labels is None else labels.data_ptr() + 8 * r0,
                                      rows, V, float(rcp_temperature), None if labels is None else lp.data_ptr() + 4 * r0,
                                      ent.data_ptr() + 4 * r0 if want_entropy else None, lse.data_ptr() + 4 * r0,
                                      pz.data_ptr() + 4 * r0 if want_entropy else None, stream)
            _lib.check(st, "skyrl_logits_fwd")
    return lp, ent, lse, pz


@logits_fwd.register_fake
def _(logits, labels, rcp_temperature, want_entropy):
    T = logits.numel() // max(1, logits.shape[-1])
    return tuple(logits.new_empty(T, dtype=torch.float32) for _ in range(4))


def _row_run(pieces: list, r0: int, n: int) -> torch.Tensor:
    """Rows ``r0 .. r0 + n - 1`` of a tensor given by its pieces, as a 2-D view (the run lies inside one piece)."""
    for view, first in pieces:
        if first <= r0 and r0 + n <= first + view.shape[0]:
            return view[r0 - first:r0 - first + n]
    raise ValueError("the gradient's layout does not line up with the logits'")


def _bwd_into(out: torch.Tensor, logits, labels, row_lse, row_pz, dlogprobs, dentropy, rcp_temperature) -> None:
    T, V, pieces = _pieces(logits)
    To, Vo, out_pieces = _pieces(out)
    if (To, Vo) != (T, V):
        raise ValueError(f"the gradient has shape {tuple(out.shape)}, the logits {tuple(logits.shape)}")
    dev = _require_device(logits, labels, row_lse, row_pz, dlogprobs, dentropy, out)
    _check_rows("labels", labels, T, torch.int64)
    for name, t in (("row_lse", row_lse), ("row_pz", row_pz), ("dlogprobs", dlogprobs), ("dentropy", dentropy)):
        _check_rows(name, t, T, torch.float32)
    if dlogprobs is None and dentropy is None:
        raise ValueError("the backward needs an upstream gradient: dlogprobs, dentropy or both")
    if T == 0:
        return
    runs = pieces if len(pieces) >= len(out_pieces) else out_pieces        # the finer of the two partitions
    ptr = lambda t, r0, size: None if t is None else t.data_ptr() + size * r0  # noqa: E731
    lib = _lib.load()
    with torch.cuda.device(dev):
        stream = torch.cuda.current_stream(dev).cuda_stream
        for run, r0 in runs:
            n = int(run.shape[0])
            src, dst = _row_run(pieces, r0, n), _row_run(out_pieces, r0, n)
            _, _, ld = _rows(src)
            _, _, ldd = _rows(dst)
            st = lib.skyrl_logits_bwd(src.data_ptr(), _DTYPES[logits.dtype], ld, ptr(labels, r0, 8), ptr(row_lse, r0, 4), ptr(row_pz, r0, 4),
                                      ptr(dlogprobs, r0, 4), ptr(dentropy, r0, 4), n, V, float(rcp_temperature), dst.data_ptr(), ldd, stream)
            _lib.check(st, "skyrl_logits_bwd")


@torch.library.custom_op("skyrl_amd::logits_bwd", mutates_args=())
def logits_bwd(logits: torch.Tensor, labels: Optional[torch.Tensor], row_lse: torch.Tensor, row_pz: Optional[torch.Tensor],
               dlogprobs: Optional[torch.Tensor], dentropy: Optional[torch.Tensor], rcp_temperature: float) -> torch.Tensor:
    """d loss / d logits, a new ``[T, V]`` tensor in the logits' dtype."""
    out = torch.empty(logits.shape, dtype=logits.dtype, device=logits.device)
    _bwd_into(out, logits, labels, row_lse, row_pz, dlogprobs, dentropy, rcp_temperature)
    return out


@logits_bwd.register_fake
def _(logits, labels, row_lse, row_pz, dlogprobs, dentropy, rcp_temperature):
    return logits.new_empty(logits.shape)


@torch.library.custom_op("skyrl_amd::logits_bwd_", mutates_args=("logits",))
def logits_bwd_(logits: torch.Tensor, labels: Optional[torch.Tensor], row_lse: torch.Tensor, row_pz: Optional[torch.Tensor],
                dlogprobs: Optional[torch.Tensor], dentropy: Optional[torch.Tensor], rcp_temperature: float) -> None:
    """The same gradient written over the logits (what the flash-attn cross-entropy does with ``inplace_backward=True``)."""
    _bwd_into(logits, logits, labels, row_lse, row_pz, dlogprobs, dentropy, rcp_temperature)


class _FromLogits(torch.autograd.Function):
    """(logprobs, entropy) of a 2-D logits matrix; either output may go unused (its gradient then arrives as ``None``)."""

    @staticmethod
    def forward(ctx, logits, labels, rcp_temperature, want_entropy, inplace_backward):
        lp, ent, lse, pz = logits_fwd(logits, labels, rcp_temperature, want_entropy)
        ctx.save_for_backward(logits, labels, lse, pz if want_entropy else None)
        ctx.args = (rcp_temperature, want_entropy, inplace_backward)
        ctx.set_materialize_grads(False)
        return lp, ent

    @staticmethod
    def backward(ctx, dlp, dent):
        logits, labels, lse, pz = ctx.saved_tensors
        rcp_temperature, want_entropy, inplace = ctx.args
        if labels is None:
            dlp = None
        if not want_entropy:
            dent = None
        if dlp is None and dent is None:
            return None, None, None, None, None
        f = lambda t: None if t is None else t.to(torch.float32).contiguous()  # noqa: E731
        if inplace:
            logits_bwd_(logits, labels, lse, pz, f(dlp), f(dent), rcp_temperature)
            return logits, None, None, None, None
        return logits_bwd(logits, labels, lse, pz, f(dlp), f(dent), rcp_temperature), None, None, None, None


def _flat(logits: torch.Tensor) -> torch.Tensor:
    """``[..., V]`` in a form the kernels walk without a copy where the layout allows it: a 2-D matrix, or the ``[B, S, V]``
    tensor itself when its rows are equally pitched inside every batch entry (a slice such as ``logits[:, :-1]`` stays where
    it is; the kernels then run once per batch entry)."""
    V = logits.shape[-1]
    if logits.dtype not in _DTYPES:
        logits = logits.to(torch.float32)
    if logits.dim() == 3 and logits.shape[0] > 1 and logits.shape[1] > 1 and (logits.stride(2) == 1 or V == 1) \
            and logits.stride(1) >= V and logits.stride(0) != logits.shape[1] * logits.stride(1) and logits.stride(0) > 0:
        return logits          # reshape would copy: the rows of a batch entry are equally pitched, the entries are not adjacent
    flat = logits.reshape(-1, V)
    if flat.stride(1) != 1 and V > 1:
        flat = flat.contiguous()
    return flat


def logprobs_and_entropy_from_logits(logits: torch.Tensor, labels: torch.Tensor, *, temperature: float = 1.0,
                                     inplace_backward: bool = False) -> Tuple[torch.Tensor, torch.Tensor]:
    """``(logprobs, entropy)``, both fp32 of shape ``logits.shape[:-1]``, of ``logits / temperature`` from one pass over the
    logits.  Both carry gradients to ``logits``; with ``inplace_backward`` the gradient is written over the logits' storage."""
    shape = logits.shape[:-1]
    lp, ent = _FromLogits.apply(_flat(logits), labels.reshape(-1).to(torch.int64).contiguous(), 1.0 / float(temperature), True,
                                bool(inplace_backward))
    return lp.reshape(shape), ent.reshape(shape)


def logprobs_from_logits(logits: torch.Tensor, labels: torch.Tensor, inplace_backward: bool = True) -> torch.Tensor:
    """Reference ``logprobs_from_logits`` (torch_utils.py:115-152): the log-probability of ``labels`` under
    ``softmax(logits)``, fp32, shape ``logits.shape[:-1]``.  ``inplace_backward=True`` (the reference's default, honoured
    there when flash-attn is installed) lets the backward overwrite the logits with their gradient."""
    shape = logits.shape[:-1]
    lp, _ = _FromLogits.apply(_flat(logits), labels.reshape(-1).to(torch.int64).contiguous(), 1.0, False, bool(inplace_backward))
    return lp.reshape(shape)


def logprobs_from_logits_flash_attn(logits: torch.Tensor, labels: torch.Tensor, inplace_backward: bool = True) -> torch.Tensor:
    """Reference ``logprobs_from_logits_flash_attn`` (torch_utils.py:147-152), 2-D logits: same kernel."""
    return logprobs_from_logits(logits, labels, inplace_backward)


def logprobs_from_logits_v2(logits: torch.Tensor, labels: torch.Tensor) -> torch.Tensor:
    """Reference ``logprobs_from_logits_v2`` (torch_utils.py:156-177): same values, never in place, result in the logits'
    dtype as there (the reference takes the whole bf16 path in bf16; here only the result is rounded)."""
    return logprobs_from_logits(logits, labels, inplace_backward=False).to(logits.dtype)


def chunked_entropy_from_logits(logits: torch.Tensor, requires_grad: bool = False, attention_mask: Optional[torch.Tensor] = None,
                                chunk_size: int = 1024) -> torch.Tensor:
    """Reference ``chunked_entropy_from_logits`` (torch_utils.py:58-111): entropy of ``softmax(logits)`` per position, in the
    logits' dtype, zero where ``attention_mask`` is zero.  ``chunk_size`` is accepted and ignored: the kernel holds one row's
    running statistics, never a chunk of log-probabilities."""
    if attention_mask is not None and attention_mask.shape != (logits.shape[0], logits.shape[1]):
        raise ValueError(
            f"attention_mask shape {attention_mask.shape} does not match logits shape "
            f"(batch_size={logits.shape[0]}, seqlen={logits.shape[1]}). "
            f"Expected attention_mask shape: ({logits.shape[0]}, {logits.shape[1]})")
    if not isinstance(chunk_size, int) or chunk_size < 1:
        raise ValueError(f"chunk_size must be a positive integer, got {chunk_size!r}")
    shape = logits.shape[:-1]
    with (torch.enable_grad() if requires_grad else torch.no_grad()):
        _, ent = _FromLogits.apply(_flat(logits), None, 1.0, True, False)
        ent = ent.reshape(shape).to(logits.dtype)
        if attention_mask is not None:
            ent = ent * attention_mask
    return ent


def _require_single_shard(group: Any, what: str) -> None:
    if group is not None and torch.distributed.is_available() and torch.distributed.is_initialized() \
            and torch.distributed.get_world_size(group) > 1:
        raise NotImplementedError(f"{what}: built for one vocabulary shard per GPU (tensor-parallel size 1)")


class DistributedLogprob(torch.autograd.Function):
    """Apply signature of the reference's ``DistributedLogprob`` (model_utils.py:66-138) on one vocabulary shard:
    ``apply(vocab_parallel_logits[..., V], target[...], vocab_start_index, vocab_end_index, group, inference_only=False)``
    ``-> logprobs`` fp32; targets outside ``[vocab_start_index, vocab_end_index)`` give 0 and keep ``-softmax * grad`` in the
    backward.  Saves the logits and one fp32 per row instead of an fp32 softmax of the whole tensor."""

    @staticmethod
    def forward(ctx, vocab_parallel_logits, target, vocab_start_index, vocab_end_index, group, inference_only=False):
        _require_single_shard(group, "DistributedLogprob")
        shape = vocab_parallel_logits.shape[:-1]
        flat = _flat(vocab_parallel_logits.detach())
        t64 = target.reshape(-1).to(torch.int64)
        outside = (t64 < vocab_start_index) | (t64 >= vocab_end_index)
        labels = torch.where(outside, torch.full_like(t64, -1), t64 - vocab_start_index).contiguous()
        lp, _, lse, _ = logits_fwd(flat, labels, 1.0, False)
        if not inference_only:
            ctx.save_for_backward(flat, labels, lse)
        ctx.in_dtype, ctx.in_shape = vocab_parallel_logits.dtype, vocab_parallel_logits.shape
        return lp.reshape(shape)

    @staticmethod
    def backward(ctx, *grad_outputs):
        flat, labels, lse = ctx.saved_tensors
        g = grad_outputs[0].reshape(-1).to(torch.float32).contiguous()
        grad = logits_bwd(flat, labels, lse, None, g, None, 1.0)
        return grad.reshape(ctx.in_shape).to(ctx.in_dtype), None, None, None, None, None


class ChunkedDistributedLogprob(torch.autograd.Function):
    """Apply signature of ``ChunkedDistributedLogprob`` (model_utils.py:141-272): as above with a ``chunk_size`` that is
    accepted and ignored (nothing the size of a chunk of fp32 logits exists here)."""

    @staticmethod
    def forward(ctx, vocab_parallel_logits, target, vocab_start_index, vocab_end_index, chunk_size, tp_group, inference_only=False):
        return DistributedLogprob.forward(ctx, vocab_parallel_logits, target, vocab_start_index, vocab_end_index, tp_group,
                                          inference_only)

    @staticmethod
    def backward(ctx, *grad_outputs):
        return DistributedLogprob.backward(ctx, *grad_outputs) + (None,)


def from_parallel_logits_to_logprobs(vocab_parallel_logits: torch.Tensor, target: torch.Tensor, vocab_start_index: int,
                                     vocab_end_index: int, tp_group: Any, inference_only: bool = False, cp_group: Any = None,
                                     chunk_size: Optional[int] = None) -> torch.Tensor:
    """Reference ``from_parallel_logits_to_logprobs`` (model_utils.py:487-565) without context parallelism: the targets are
    rolled left by one, scored, and the last column is dropped -> ``[B, S - 1]`` fp32."""
    _require_single_shard(cp_group, "from_parallel_logits_to_logprobs (context parallelism)")
    rolled = target.roll(shifts=-1, dims=-1)
    logprobs = DistributedLogprob.apply(vocab_parallel_logits, rolled, vocab_start_index, vocab_end_index, tp_group, inference_only)
    return logprobs.contiguous()[:, :-1]


def from_parallel_logits_to_logprobs_packed_sequences(vocab_parallel_logits: torch.Tensor, target: torch.Tensor,
                                                      cu_seqlens_padded: torch.Tensor, unpacked_seqlen: int, vocab_start_index: int,
                                                      vocab_end_index: int, group: Any, inference_only: bool = False, cp_group: Any = None,
                                                      chunk_size: Optional[int] = None, attention_mask: Optional[torch.Tensor] = None,
                                                      sub_seq_lengths: Optional[list] = None) -> torch.Tensor:
    """Reference ``from_parallel_logits_to_logprobs_packed_sequences`` (model_utils.py:566-710) without context parallelism:
    packed logits ``[1, T, V]`` and packed targets ``[1, T]`` -> ``[batch, unpacked_seqlen - 1]`` fp32.  Every token is scored
    against its successor inside its own sequence (one index kernel), the log-probabilities come from the one-pass logits
    kernel, and the scatter back to rows is one kernel per direction instead of boolean-mask indexing."""
    from .model_utils import _packed_subseq_row_indices_offsets_and_lens
    from .packed import packed_next_token_labels, packed_scatter_logprobs

    _require_single_shard(cp_group, "from_parallel_logits_to_logprobs_packed_sequences (context parallelism)")
    target = target.squeeze(0)
    device = target.device
    batch_size = len(sub_seq_lengths) if sub_seq_lengths is not None else cu_seqlens_padded.shape[0] - 1
    cu = cu_seqlens_padded.to(device=device, dtype=torch.long)
    rolled = packed_next_token_labels(target.to(torch.long).contiguous(), cu).unsqueeze(0)
    if sub_seq_lengths is not None:
        rows, row_offs, seq_lens = _packed_subseq_row_indices_offsets_and_lens(cu, sub_seq_lengths, device)
        layout = dict(seg_row=rows, seg_col=row_offs, seg_len=seq_lens)
    elif attention_mask is not None:
        layout = dict(attention_mask=attention_mask.to(device=device, dtype=torch.bool))
    else:
        layout = {}
    probs = DistributedLogprob.apply(vocab_parallel_logits, rolled, vocab_start_index, vocab_end_index, group, inference_only)
    probs = probs.contiguous().squeeze(0)
    if probs.dim() != 1:
        raise ValueError(f"Expected probs to be 1D after squeezing, but got shape {probs.shape}.")
    return packed_scatter_logprobs(probs, cu, batch_size, unpacked_seqlen - 1, **layout)


def _check_entropy_chunking(chunk_size: Optional[int], chunk_memory_mb: int) -> None:
    """The argument errors of ``_resolve_vocab_entropy_chunk_size`` (model_utils.py:1352-1385).  The chunking itself bounds
    fp32 temporaries that do not exist here, so valid values change nothing."""
    if chunk_size is not None and chunk_size < 0:
        raise ValueError(f"chunk_size must be non-negative or None, got {chunk_size}")
    if chunk_size is not None and chunk_memory_mb <= 0:
        raise ValueError(f"chunk_memory_mb must be positive, got {chunk_memory_mb}")


def vocab_parallel_entropy(vocab_parallel_logits: torch.Tensor, chunk_size: Optional[int] = None, chunk_memory_mb: int = 512
                           ) -> torch.Tensor:
    """Reference ``vocab_parallel_entropy`` / ``_VocabParallelEntropy`` (model_utils.py:1316-1410) on one vocabulary shard:
    entropy of ``softmax(logits)`` per position, shape ``logits.shape[:-1]``, in the logits' dtype, with the gradient
    ``softmax * (sum softmax * logits - logits) * grad`` (:1337-1345) recomputed from the logits in the backward instead of
    kept as a second tensor of the logits' size."""
    _check_entropy_chunking(chunk_size, chunk_memory_mb)
    shape = vocab_parallel_logits.shape[:-1]
    _, ent = _FromLogits.apply(_flat(vocab_parallel_logits), None, 1.0, True, False)
    return ent.reshape(shape).to(vocab_parallel_logits.dtype)


def vocab_parallel_entropy_weighted_sum(vocab_parallel_logits: torch.Tensor, weights: torch.Tensor, chunk_size: Optional[int] = None,
                                        chunk_memory_mb: int = 512) -> torch.Tensor:
    """Reference ``vocab_parallel_entropy_weighted_sum`` (model_utils.py:1413-1440): ``sum(entropy * weights)``.  Rows whose
    weight is zero cost nothing in the backward (their gradient rows are written as zeros without reading the logits)."""
    return (vocab_parallel_entropy(vocab_parallel_logits, chunk_size, chunk_memory_mb) * weights).sum()


def vocab_parallel_entropy_packed_sequences(vocab_parallel_logits: torch.Tensor, cu_seqlens_padded: torch.Tensor, unpacked_seqlen: int,
                                            num_actions: int, attention_mask: torch.Tensor, loss_mask: Optional[torch.Tensor],
                                            cp_group: Any, sub_seq_lengths: Optional[list] = None, chunk_size: Optional[int] = None,
                                            chunk_memory_mb: int = 512) -> Tuple[torch.Tensor, torch.Tensor]:
    """Reference ``vocab_parallel_entropy_packed_sequences`` (model_utils.py:1001-1087) without context parallelism:
    ``(entropy, entropy_for_loss)``, the action-token mean of the per-token entropy of packed logits ``[1, T, V]``; the first
    is detached, the second carries the gradient.  The reference brings the ``[B, unpacked_seqlen - 1]`` action weights to
    the packed stream with boolean-mask indexing and one ``.item()``; here the per-token entropy goes the other way through
    the (differentiable) scatter-back kernel and the weighted mean is taken in the ``[B, unpacked_seqlen - 1]`` layout -- the
    same sums, no host synchronisation."""
    from .model_utils import _packed_subseq_row_indices_offsets_and_lens
    from .packed import packed_scatter_logprobs

    _require_single_shard(cp_group, "vocab_parallel_entropy_packed_sequences (context parallelism)")
    entropy_tokens = vocab_parallel_entropy(vocab_parallel_logits, chunk_size, chunk_memory_mb).reshape(-1).float()
    device = entropy_tokens.device
    batch_size, cols = attention_mask.shape[0], unpacked_seqlen - 1
    with torch.no_grad():
        action_weights = torch.zeros((batch_size, cols), dtype=torch.float32, device=device)
        action_weights[:, -num_actions:] = 1.0 if loss_mask is None else loss_mask.to(device=device, dtype=torch.float32)
        cu = cu_seqlens_padded.to(device=device, dtype=torch.long)
        if sub_seq_lengths is not None:
            rows, row_offs, seq_lens = _packed_subseq_row_indices_offsets_and_lens(cu, sub_seq_lengths, device)
            layout = dict(seg_row=rows, seg_col=row_offs, seg_len=seq_lens)
        else:
            layout = dict(attention_mask=attention_mask.to(device=device, dtype=torch.bool))
        landed = packed_scatter_logprobs(torch.ones_like(entropy_tokens), cu, batch_size, cols, **layout)
        count = (landed * action_weights).sum().clamp(min=1.0)
    entropy_bs = packed_scatter_logprobs(entropy_tokens.contiguous(), cu, batch_size, cols, **layout)
    entropy_for_loss = ((entropy_bs * action_weights).sum() / count).to(vocab_parallel_logits.dtype)
    return entropy_for_loss.detach().clone(), entropy_for_loss
