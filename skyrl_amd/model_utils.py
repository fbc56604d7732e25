"""Host-side mirror of the reference's fused LM-head call sites, with ``"hip"`` as the backend.

Same names, argument order and return shapes as ``skyrl/backends/skyrl_train/distributed/megatron/model_utils.py`` so a
trainer can import these instead:

* ``_fused_lm_head_logprob_apply``                       (reference :431-484)
* ``from_parallel_hidden_to_logprobs``                   (:713-770)
* ``from_parallel_hidden_to_logprobs_packed_sequences``  (:773-883)
* ``_fused_vocab_parallel_entropy_from_hidden``          (:1090-1121)
* ``from_parallel_hidden_to_entropy_packed_sequences``   (:1124-1208)
* ``_packed_sequence_indices``, ``_packed_subseq_row_indices_offsets_and_lens``  (:920-928, :886-917)

The packed variant prepares its labels and scatters its result back with one HIP kernel each (``skyrl_amd/packed.py``)
instead of the reference's torch index arithmetic; ``_packed_sequence_indices`` is kept as the host-side statement of that
arithmetic.

Differences, all forced by the one-GPU scope: tensor/context-parallel groups must be ``None`` or of size 1, and the only
backend is ``"hip"`` -- there is no fallback to another implementation when the HIP library is missing.

Temperature: the reference divides the weight by the temperature in the weight's dtype and lets autograd chain the 1/T
factor (:734-740).  Here the kernel scales the fp32 logits (as the vendored verl kernel does,
fused_linear_logprob_triton.py:346, 957) and applies 1/T to both gradients itself, so no ``[V, H]`` temporary is made and
the gradients are with respect to the unscaled weight -- the same quantities autograd yields in the reference.
"""

from __future__ import annotations

from typing import Optional

import torch
import torch.distributed as dist

from . import ops
from .fused_linear_logprob_hip import FusedLinearLogprobHip, _group_size, _require_single_shard, linear_cross_entropy
from .packed import packed_next_token_labels, packed_scatter_logprobs

FUSED_LM_HEAD_LOGPROB_BACKENDS = ("hip",)


def validate_fused_backend(backend: str) -> str:
    """Mirror of the config check at skyrl/train/config/config.py:1539-1543, with this package's backend list."""
    if backend not in FUSED_LM_HEAD_LOGPROB_BACKENDS:
        raise ValueError(
            f"trainer.fused_lm_head_logprob_backend must be one of {FUSED_LM_HEAD_LOGPROB_BACKENDS}, got {backend!r} "
            "(the 'torch' and 'triton' backends live in the SkyRL tree, not in this package)"
        )
    return backend


def _fused_lm_head_logprob_apply(
    backend: str,
    hidden: torch.Tensor,
    weight: torch.Tensor,
    target: torch.Tensor,
    vocab_start_index: int,
    vocab_end_index: int,
    chunk_size: int,
    tp_group: Optional[dist.ProcessGroup],
    inference_only: bool,
    temperature: float = 1.0,
) -> torch.Tensor:
    """Dispatch the fused LM-head token-logprob to the HIP backend; returns ``[B, S]`` fp32.

    ``temperature`` is an extension over the reference signature (default 1.0 keeps it call-compatible): when it is not 1 the
    op scales the logits inside the kernel instead of the caller scaling the weight.
    """
    validate_fused_backend(backend)
    if temperature == 1.0:
        return FusedLinearLogprobHip.apply(hidden, weight, target, vocab_start_index, vocab_end_index, chunk_size, tp_group,
                                           inference_only)
    _require_single_shard(tp_group, "_fused_lm_head_logprob_apply")
    B, S, H = hidden.shape
    target_mask = (target < vocab_start_index) | (target >= vocab_end_index)
    target = target.to(torch.int64)
    labels = torch.where(target_mask, torch.iinfo(torch.int64).max, target - vocab_start_index)
    hidden_c = ops.hidden_for_weight(hidden, weight)
    # log-probabilities only: no entropy is accumulated in the forward, none differentiated in the backward
    if inference_only:
        with torch.no_grad():
            logprobs, _ = linear_cross_entropy(hidden_c, weight.contiguous(), labels, float(temperature), "none", None, False)
    else:
        logprobs, _ = linear_cross_entropy(hidden_c, weight.contiguous(), labels, float(temperature), "none", None, False)
    return logprobs.reshape(B, S)


def from_parallel_hidden_to_logprobs(
    hidden: torch.Tensor,
    lm_head_weight: torch.Tensor,
    target: torch.Tensor,
    vocab_start_index: int,
    vocab_end_index: int,
    tp_group: Optional[dist.ProcessGroup],
    inference_only: bool = False,
    cp_group: Optional[dist.ProcessGroup] = None,
    chunk_size: Optional[int] = None,
    temperature: float = 1.0,
    fused_backend: str = "hip",
    *,
    action_window: Optional[int] = None,
) -> torch.Tensor:
    """``hidden`` [B, S, H] + ``lm_head_weight`` [V, H] + token ids ``target`` [B, S] -> next-token logprobs [B, S-1].

    ``action_window = n`` (an extension) returns the last ``n`` columns only, ``[B, n]``, from an LM head run on positions
    ``S - 1 - n .. S - 2`` -- the slice the worker takes next -- instead of on all ``S`` positions."""
    if _group_size(cp_group) > 1:
        raise NotImplementedError("context parallelism is outside the one-GPU scope of the HIP fused LM-head path")
    target = target.roll(shifts=-1, dims=-1)
    if action_window is not None:
        n_act, S = int(action_window), hidden.shape[1]
        if not 0 < n_act <= S - 1:
            raise ValueError(f"action_window {action_window} does not fit sequences of length {S}")
        hidden, target = hidden[:, S - 1 - n_act:S - 1], target[:, S - 1 - n_act:S - 1].contiguous()
        return _fused_lm_head_logprob_apply(fused_backend, hidden, lm_head_weight, target, vocab_start_index, vocab_end_index,
                                            n_act, tp_group, inference_only, temperature).contiguous()
    seq_len_local = hidden.shape[1]
    eff_chunk = chunk_size if (chunk_size is not None and chunk_size < seq_len_local) else seq_len_local
    logprobs = _fused_lm_head_logprob_apply(
        fused_backend, hidden, lm_head_weight, target, vocab_start_index, vocab_end_index, eff_chunk, tp_group,
        inference_only, temperature,
    ).contiguous()
    return logprobs[:, :-1]


def _packed_sequence_indices(cu_seqlens_padded: torch.Tensor, total_tokens: int, device: torch.device):
    cu = cu_seqlens_padded.to(device=device, dtype=torch.long)
    token_indices = torch.arange(total_tokens, device=device)
    seq_indices = torch.searchsorted(cu[1:], token_indices, right=True)
    seq_offsets = token_indices - cu[seq_indices]
    seq_lens_padded = cu[1:] - cu[:-1]
    return cu, token_indices, seq_indices, seq_offsets, seq_lens_padded


def _packed_subseq_row_indices_offsets_and_lens(cu_seqlens_padded: torch.Tensor, sub_seq_lengths, device: torch.device):
    """Per-packed-segment (row, column offset, true length) for controller-side packing of several sequences per row."""
    bounds = cu_seqlens_padded.detach().cpu().tolist()
    padded = [bounds[i + 1] - bounds[i] for i in range(len(bounds) - 1)]
    rows, offs, lens = [], [], []
    seg = 0
    for row, row_lens in enumerate(sub_seq_lengths):
        col = 0
        for n in row_lens:
            if seg >= len(padded):
                raise ValueError("sub_seq_lengths contains more sub-sequences than cu_seqlens_padded")
            rows.append(row), offs.append(col), lens.append(int(n))
            col += padded[seg]
            seg += 1
    if seg != len(padded):
        raise ValueError(f"sub_seq_lengths describes {seg} sub-sequences, but cu_seqlens_padded describes {len(padded)}")
    mk = lambda x: torch.tensor(x, dtype=torch.long, device=device)  # noqa: E731
    return mk(rows), mk(offs), mk(lens)


def from_parallel_hidden_to_logprobs_packed_sequences(
    hidden: torch.Tensor,
    lm_head_weight: torch.Tensor,
    target: torch.Tensor,
    cu_seqlens_padded: torch.Tensor,
    unpacked_seqlen: int,
    vocab_start_index: int,
    vocab_end_index: int,
    group: Optional[dist.ProcessGroup],
    inference_only: bool = False,
    cp_group: Optional[dist.ProcessGroup] = None,
    chunk_size: Optional[int] = None,
    attention_mask: Optional[torch.Tensor] = None,
    sub_seq_lengths: Optional[list] = None,
    temperature: float = 1.0,
    fused_backend: str = "hip",
    *,
    action_window: Optional[int] = None,
) -> torch.Tensor:
    """Packed variant: ``hidden`` [1, T, H], ``target`` [1, T], ``cu_seqlens_padded`` [n+1] -> [batch, unpacked_seqlen-1].

    ``action_window = n`` (an extension) returns the last ``n`` columns only, ``[batch, n]`` -- what the Megatron worker
    slices next (``token_logprobs[:, -num_actions:]``, megatron_model_wrapper.py:707) -- and runs the LM head on just the
    packed tokens that land there: the scatter kernel, applied to the token numbers, is its own inverse map, so the rows are
    found without a host synchronisation and the shapes stay static (``batch * n`` rows, absent ones masked).
    """
    if _group_size(cp_group) > 1:
        raise NotImplementedError("context parallelism is outside the one-GPU scope of the HIP fused LM-head path")
    hidden = hidden.squeeze(0)
    target = target.squeeze(0)
    batch_size = len(sub_seq_lengths) if sub_seq_lengths is not None else cu_seqlens_padded.shape[0] - 1
    if attention_mask is not None:
        attention_mask = attention_mask.to(device=target.device, dtype=torch.bool)

    # Labels: every token's successor inside its own sequence, one kernel (reference: index arithmetic, :810-815).
    cu = cu_seqlens_padded.to(device=target.device, dtype=torch.long)
    rolled_targets = packed_next_token_labels(target.to(torch.long).contiguous(), cu).unsqueeze(0)
    hidden = hidden.unsqueeze(0)
    cols = unpacked_seqlen - 1
    if sub_seq_lengths is not None:
        rows, row_offs, seq_lens = _packed_subseq_row_indices_offsets_and_lens(cu, sub_seq_lengths, target.device)
        layout = dict(seg_row=rows, seg_col=row_offs, seg_len=seq_lens)
    elif attention_mask is not None:
        layout = dict(attention_mask=attention_mask)
    else:
        layout = {}

    if action_window is not None:
        n_act, T = int(action_window), hidden.shape[1]
        if not 0 < n_act <= cols:
            raise ValueError(f"action_window {action_window} does not fit {cols} columns")
        if T >= 1 << 24:
            raise ValueError("action_window numbers the packed tokens in fp32: at most 2^24 - 1 tokens")
        with torch.no_grad():  # token number + 1 where a token lands, 0 elsewhere
            number = torch.arange(1, T + 1, dtype=torch.float32, device=target.device)
            landed = packed_scatter_logprobs(number, cu, batch_size, cols, **layout)[:, cols - n_act:]
            src = landed.reshape(-1).to(torch.long) - 1
            present = (src >= 0).reshape(batch_size, n_act)
            src = src.clamp(min=0)
        rows_h = hidden.reshape(T, -1).index_select(0, src).unsqueeze(0)          # differentiable gather of the rows
        rows_y = rolled_targets.reshape(-1).index_select(0, src).unsqueeze(0).contiguous()
        window = _fused_lm_head_logprob_apply(fused_backend, rows_h, lm_head_weight, rows_y, vocab_start_index, vocab_end_index,
                                              rows_h.shape[1], group, inference_only, temperature)
        return window.reshape(batch_size, n_act) * present

    seq_len_local = hidden.shape[1]
    eff_chunk = chunk_size if (chunk_size is not None and chunk_size < seq_len_local) else seq_len_local
    probs = _fused_lm_head_logprob_apply(
        fused_backend, hidden, lm_head_weight, rolled_targets, vocab_start_index, vocab_end_index, eff_chunk, group,
        inference_only, temperature,
    ).contiguous().squeeze(0)
    if probs.dim() != 1:
        raise ValueError(f"Expected probs to be 1D after squeezing, but got shape {probs.shape}.")

    # Scatter-back to [batch, unpacked_seqlen - 1], one kernel per direction (reference: boolean-mask indexing, :851-883).
    return packed_scatter_logprobs(probs, cu, batch_size, cols, **layout)


def _fused_vocab_parallel_entropy_from_hidden(
    hidden: torch.Tensor,
    lm_head_weight: torch.Tensor,
    tp_group: Optional[dist.ProcessGroup],
    chunk_size: Optional[int] = None,
    temperature: float = 1.0,
) -> torch.Tensor:
    """Per-token entropy [B, S] fp32 from ``hidden`` [B, S, H] + LM-head weight, no gradient (the entropy *metric*)."""
    _require_single_shard(tp_group, "_fused_vocab_parallel_entropy_from_hidden")
    B, S, H = hidden.shape
    with torch.no_grad():
        labels = torch.full((B * S,), torch.iinfo(torch.int64).max, dtype=torch.int64, device=hidden.device)
        _, entropy, _, _ = ops.lmhead_fwd(ops.hidden_for_weight(hidden.reshape(B * S, H), lm_head_weight).contiguous(),
                                          lm_head_weight.contiguous(), labels, 1.0 / float(temperature), True)
    return entropy.reshape(B, S)


def from_parallel_hidden_to_entropy_packed_sequences(
    hidden: torch.Tensor,
    lm_head_weight: torch.Tensor,
    cu_seqlens_padded: torch.Tensor,
    unpacked_seqlen: int,
    num_actions: int,
    attention_mask: torch.Tensor,
    loss_mask: Optional[torch.Tensor],
    cp_group: Optional[dist.ProcessGroup],
    tp_group: Optional[dist.ProcessGroup],
    sub_seq_lengths: Optional[list] = None,
    chunk_size: Optional[int] = None,
    temperature: float = 1.0,
):
    """Action-token mean of the per-token entropy of a packed ``hidden`` [1, T, H]: ``(entropy, entropy_for_loss)``, both
    0-dim and without gradient (the metric the Megatron worker logs).

    The reference carries the ``[B, unpacked_seqlen - 1]`` action weights to the packed stream with boolean-mask indexing
    and one ``.item()`` (:1153-1179); here the per-token entropy goes the other way through the scatter-back kernel, together
    with a vector of ones that marks the positions a packed token lands on, and the weighted mean is taken in the
    ``[B, unpacked_seqlen - 1]`` layout -- the same sums, no host synchronisation.
    """
    if _group_size(cp_group) > 1:
        raise NotImplementedError("context parallelism is outside the one-GPU scope of the HIP fused LM-head path")
    entropy_tokens = _fused_vocab_parallel_entropy_from_hidden(hidden, lm_head_weight, tp_group, chunk_size=chunk_size,
                                                               temperature=temperature).squeeze(0)
    device = entropy_tokens.device
    batch_size = attention_mask.shape[0]
    cols = unpacked_seqlen - 1
    with torch.no_grad():
        action_weights = torch.zeros((batch_size, cols), dtype=entropy_tokens.dtype, device=device)
        action_weights[:, -num_actions:] = 1.0 if loss_mask is None else loss_mask.to(device=device, dtype=entropy_tokens.dtype)
        cu = cu_seqlens_padded.to(device=device, dtype=torch.long)
        if sub_seq_lengths is not None:
            rows, row_offs, seq_lens = _packed_subseq_row_indices_offsets_and_lens(cu, sub_seq_lengths, device)
            layout = dict(seg_row=rows, seg_col=row_offs, seg_len=seq_lens)
        else:
            layout = dict(attention_mask=attention_mask.to(device=device, dtype=torch.bool))
        entropy_bs = packed_scatter_logprobs(entropy_tokens.contiguous(), cu, batch_size, cols, **layout)
        landed = packed_scatter_logprobs(torch.ones_like(entropy_tokens), cu, batch_size, cols, **layout)
        total = (entropy_bs * action_weights).sum()
        count = (landed * action_weights).sum().clamp(min=1.0)
        entropy = total / count
    return entropy, entropy.clone()


def fused_logprobs_and_entropy_from_hidden(
    hidden: torch.Tensor,
    lm_head_weight: torch.Tensor,
    target: torch.Tensor,
    temperature: float = 1.0,
):
    """One pass for both outputs, both differentiable: ``(logprobs [B,S], entropy [B,S])`` for already-shifted ``target``.

    The reference needs two LM-head GEMMs for this (logprob op + entropy op, megatron_model_wrapper.py:648-679 and :852-878);
    the kernel produces both from one.  This is the entry the FSDP wrapper would use for ``compute_entropy=True`` with
    ``entropy_requires_grad`` (workers/worker.py:976-986, 1058-1065).
    """
    B, S, H = hidden.shape
    lp, ent = linear_cross_entropy(ops.hidden_for_weight(hidden, lm_head_weight), lm_head_weight.contiguous(), target.reshape(B, S),
                                   float(temperature), "none", None)
    return lp.reshape(B, S), ent.reshape(B, S)
