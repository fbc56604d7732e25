"""Packed-sequence label preparation and scatter-back as HIP kernels (one launch each, no host synchronisation).

What the reference computes with torch index arithmetic and boolean-mask indexing inside
``from_parallel_hidden_to_logprobs_packed_sequences``
(skyrl/backends/skyrl_train/distributed/megatron/model_utils.py:810-815 for the labels, :851-883 for the scatter-back):

* ``packed_next_token_labels(tokens, cu_seqlens)``: the successor of every token inside its own sequence;
* ``packed_scatter_logprobs(packed, cu_seqlens, rows, cols, ...)``: packed ``[T]`` values back to ``[rows, cols]``, for the
  plain, the sub-sequence and the attention-mask layout; differentiable, the gradient is the matching gather kernel.
"""

from __future__ import annotations

from typing import Optional

import torch

from . import _lib
from .ops import _require_device

__all__ = ["packed_next_token_labels", "packed_scatter_logprobs"]


def _i64_vector(name: str, t: torch.Tensor, dev: torch.device, numel: Optional[int] = None) -> torch.Tensor:
    if t.dim() != 1 or (numel is not None and t.numel() != numel):
        raise ValueError(f"{name} must be a vector" + (f" of {numel} elements" if numel is not None else "")
                         + f", got shape {tuple(t.shape)}")
    return t.to(device=dev, dtype=torch.int64).contiguous()


@torch.library.custom_op("skyrl_amd::packed_next_token_labels", mutates_args=())
def packed_next_token_labels(tokens: torch.Tensor, cu_seqlens: torch.Tensor) -> torch.Tensor:
    """``tokens`` int64 [T] (packed), ``cu_seqlens`` [n+1] -> labels int64 [T]: ``tokens[cu[s] + (off + 1) mod len_s]``."""
    dev = _require_device(tokens)
    if tokens.dim() != 1 or tokens.dtype != torch.int64:
        raise ValueError(f"tokens must be an int64 vector, got {tokens.dtype} {tuple(tokens.shape)}")
    tokens = tokens.contiguous()
    cu = _i64_vector("cu_seqlens", cu_seqlens, dev)
    if cu.numel() < 1:
        raise ValueError("cu_seqlens needs at least one element")
    labels = torch.empty_like(tokens)
    with torch.cuda.device(dev):
        st = _lib.load().skyrl_packed_next_token_labels(tokens.data_ptr(), cu.data_ptr(), cu.numel() - 1, tokens.numel(),
                                                        labels.data_ptr(), torch.cuda.current_stream(dev).cuda_stream)
    _lib.check(st, "skyrl_packed_next_token_labels")
    return labels


@packed_next_token_labels.register_fake
def _(tokens, cu_seqlens):
    return torch.empty_like(tokens)


def _scatter_call(fn_name: str, src: torch.Tensor, dst: torch.Tensor, cu, seg_row, seg_col, seg_len, attention_mask, T: int,
                  rows: int, cols: int, dev: torch.device) -> None:
    ptr = lambda t: None if t is None else t.data_ptr()  # noqa: E731
    with torch.cuda.device(dev):
        st = getattr(_lib.load(), fn_name)(src.data_ptr(), cu.data_ptr(), cu.numel() - 1, T, ptr(seg_row), ptr(seg_col),
                                           ptr(seg_len), ptr(attention_mask), rows, cols, dst.data_ptr(),
                                           torch.cuda.current_stream(dev).cuda_stream)
    _lib.check(st, fn_name)


def _scatter_operands(cu_seqlens, seg_row, seg_col, seg_len, attention_mask, rows: int, cols: int, dev: torch.device):
    cu = _i64_vector("cu_seqlens", cu_seqlens, dev)
    if cu.numel() < 1:
        raise ValueError("cu_seqlens needs at least one element")
    n = cu.numel() - 1
    segs = [seg_row, seg_col, seg_len]
    if any(s is not None for s in segs):
        if any(s is None for s in segs):
            raise ValueError("seg_row, seg_col and seg_len go together")
        if attention_mask is not None:
            raise ValueError("pass sub-sequence arrays or an attention mask, not both")
        segs = [_i64_vector(nm, s, dev, n) for nm, s in zip(("seg_row", "seg_col", "seg_len"), segs)]
    if attention_mask is not None:
        if tuple(attention_mask.shape) != (rows, cols + 1) or rows != n:
            raise ValueError(f"attention_mask must be [{n}, {cols + 1}] (one row per packed sequence, unpacked_seqlen "
                             f"columns), got {tuple(attention_mask.shape)} for rows={rows}")
        attention_mask = (attention_mask.to(device=dev) != 0).to(torch.uint8).contiguous()
    return cu, segs[0], segs[1], segs[2], attention_mask


@torch.library.custom_op("skyrl_amd::packed_scatter_logprobs", mutates_args=())
def _packed_scatter(packed: torch.Tensor, cu_seqlens: torch.Tensor, seg_row: Optional[torch.Tensor],
                    seg_col: Optional[torch.Tensor], seg_len: Optional[torch.Tensor],
                    attention_mask: Optional[torch.Tensor], rows: int, cols: int) -> torch.Tensor:
    dev = _require_device(packed)
    if packed.dim() != 1 or packed.dtype != torch.float32:
        raise ValueError(f"packed must be an fp32 vector, got {packed.dtype} {tuple(packed.shape)}")
    cu, seg_row, seg_col, seg_len, attention_mask = _scatter_operands(cu_seqlens, seg_row, seg_col, seg_len, attention_mask,
                                                                     rows, cols, dev)
    out = torch.empty((rows, cols), dtype=torch.float32, device=dev)
    _scatter_call("skyrl_packed_scatter_logprobs", packed.contiguous(), out, cu, seg_row, seg_col, seg_len, attention_mask,
                  packed.numel(), rows, cols, dev)
    return out


@_packed_scatter.register_fake
def _(packed, cu_seqlens, seg_row, seg_col, seg_len, attention_mask, rows, cols):
    return packed.new_empty((rows, cols))


@torch.library.custom_op("skyrl_amd::packed_gather_grad", mutates_args=())
def _packed_gather(d_out: torch.Tensor, cu_seqlens: torch.Tensor, seg_row: Optional[torch.Tensor],
                   seg_col: Optional[torch.Tensor], seg_len: Optional[torch.Tensor],
                   attention_mask: Optional[torch.Tensor], T: int) -> torch.Tensor:
    dev = _require_device(d_out)
    if d_out.dim() != 2 or d_out.dtype != torch.float32:
        raise ValueError(f"d_out must be an fp32 matrix, got {d_out.dtype} {tuple(d_out.shape)}")
    rows, cols = d_out.shape
    cu, seg_row, seg_col, seg_len, attention_mask = _scatter_operands(cu_seqlens, seg_row, seg_col, seg_len, attention_mask,
                                                                     rows, cols, dev)
    d_packed = torch.empty(T, dtype=torch.float32, device=dev)
    _scatter_call("skyrl_packed_gather_grad", d_out.contiguous(), d_packed, cu, seg_row, seg_col, seg_len, attention_mask, T,
                  rows, cols, dev)
    return d_packed


@_packed_gather.register_fake
def _(d_out, cu_seqlens, seg_row, seg_col, seg_len, attention_mask, T):
    return d_out.new_empty((T,))


def _scatter_setup(ctx, inputs, output):
    packed, cu, seg_row, seg_col, seg_len, mask, _, _ = inputs
    ctx.save_for_backward(cu, *(t for t in (seg_row, seg_col, seg_len, mask) if t is not None))
    ctx.has_segs, ctx.has_mask, ctx.T = seg_row is not None, mask is not None, packed.numel()


def _scatter_backward(ctx, d_out):
    saved = list(ctx.saved_tensors)
    cu = saved.pop(0)
    seg_row, seg_col, seg_len = (saved.pop(0), saved.pop(0), saved.pop(0)) if ctx.has_segs else (None, None, None)
    mask = saved.pop(0) if ctx.has_mask else None
    d_packed = _packed_gather(d_out.to(torch.float32).contiguous(), cu, seg_row, seg_col, seg_len, mask, ctx.T)
    return d_packed, None, None, None, None, None, None, None


_packed_scatter.register_autograd(_scatter_backward, setup_context=_scatter_setup)


def packed_scatter_logprobs(packed: torch.Tensor, cu_seqlens: torch.Tensor, rows: int, cols: int, *,
                            seg_row: Optional[torch.Tensor] = None, seg_col: Optional[torch.Tensor] = None,
                            seg_len: Optional[torch.Tensor] = None,
                            attention_mask: Optional[torch.Tensor] = None) -> torch.Tensor:
    """Packed fp32 ``[T]`` -> ``[rows, cols]`` (``cols = unpacked_seqlen - 1``), zeros where no token lands.

    Plain layout: token at offset ``o`` of sequence ``s`` goes to ``out[s, o]`` for ``o < len_s - 1``.  With ``seg_*``
    (row, first column and true length of every packed segment) it goes to ``out[seg_row[s], seg_col[s] + o]`` for
    ``o < seg_len[s] - 1``.  With ``attention_mask`` ``[rows, cols + 1]`` the j-th real token of row ``s`` takes packed
    token ``cu[s] + j`` (all real tokens but the last).  Differentiable with respect to ``packed``.
    """
    return _packed_scatter(packed, cu_seqlens, seg_row, seg_col, seg_len, attention_mask, int(rows), int(cols))
