"""The tail of the FSDP worker's model forward on the fused LM head: hidden states in, action log-probabilities out.

The reference's ``HFModelWrapper.forward`` (skyrl/backends/skyrl_train/workers/model_wrapper.py:241-398) runs the HF model to
``logits_BSV`` -- a ``[B, S, V]`` tensor, 9-19 GiB in fp32 at the benchmark shapes -- and then divides by the temperature
(:334), takes the log-probability of the next token (:337-341), optionally the per-token entropy (:358-386), and slices the
action tokens (:393).  ``action_log_probs_from_hidden`` is that tail starting one step earlier, from the decoder's
``last_hidden_state`` and ``lm_head.weight``, so the logits are never materialised; the entropy comes from the same pass
and can carry its own gradient (``use_entropy_loss``, workers/worker.py:1058-1065).

Integration: in ``HFModelWrapper.forward`` call the decoder without its head (``self.model.model(...)`` for HF causal
LMs) and replace lines 333-393 by one call of this function with ``self.model.lm_head.weight``.
"""

from __future__ import annotations

from typing import List, Optional, Tuple, Union

import torch

from . import ops
from .fused_linear_logprob_hip import linear_cross_entropy
from .model_utils import _fused_lm_head_logprob_apply

__all__ = ["action_log_probs_from_hidden", "action_log_probs_from_logits"]


def _pad_back(values: torch.Tensor, nnz_indices: torch.Tensor, batch: int, seqlen: int) -> torch.Tensor:
    """``pad_input`` of the reference (:350-356): packed ``[nnz]`` values to ``[batch, seqlen]``, zeros at padding."""
    out = torch.zeros(batch * seqlen, dtype=values.dtype, device=values.device)
    return out.index_copy(0, nnz_indices.to(torch.long), values).view(batch, seqlen)


def action_log_probs_from_hidden(
    last_hidden_state: torch.Tensor,
    lm_head_weight: torch.Tensor,
    sequences: torch.Tensor,
    num_actions: Union[int, List[int]],
    attention_mask: Optional[torch.Tensor] = None,
    temperature: float = 1.0,
    return_output: bool = False,
    compute_entropy: bool = False,
    entropy_requires_grad: bool = True,
    nnz_indices: Optional[torch.Tensor] = None,
    action_only: bool = False,
) -> Union[torch.Tensor, Tuple[torch.Tensor, dict]]:
    """Action log-probabilities ``[B, num_actions]`` (and ``{"entropy": [B, S]}`` with ``return_output``).

    ``last_hidden_state`` is ``[B, S, H]``, or ``[1, nnz, H]`` when the worker removed the micro-batch padding, in which
    case ``nnz_indices`` are the flat positions of the real tokens (what ``unpad_input`` returned, :281-283) and
    ``sequences`` / ``attention_mask`` keep their ``[B, S]`` shape.  ``sequences`` are the token ids the model saw;
    targets are those ids rolled left by one over the stream the model ran on (:291), so with packing the last token of a
    sequence is scored against the first token of the next one, exactly as in the reference.

    Differences from the reference: the entropy is fp32 (the reference returns it in the logits' dtype, torch_utils.py:92),
    and both outputs come from one pass over the vocabulary.

    ``action_only=True`` (an extension) runs the LM head on the ``B * num_actions`` rows the result is read from -- positions
    ``S - num_actions - 1 .. S - 2`` of every sequence -- instead of on all tokens: the same action log-probabilities, and
    the same entropy inside that window, which is the only part the policy worker reads (workers/worker.py:1060-1062);
    outside it the entropy is 0.  Forward and backward then cost ``num_actions / S`` of the full pass.
    """
    if isinstance(num_actions, list):
        if len(num_actions) != 1:
            raise NotImplementedError("per-row num_actions is not supported (the reference slices with a numpy array here, "
                                      "which torch rejects as well)")
        num_actions = num_actions[0]
    batch, seqlen = sequences.shape
    packed = nnz_indices is not None
    if packed:
        tokens = sequences.reshape(-1)[nnz_indices.to(torch.long)].unsqueeze(0)
    else:
        tokens = sequences
    if last_hidden_state.shape[:2] != tokens.shape:
        raise ValueError(f"last_hidden_state {tuple(last_hidden_state.shape)} does not match the token stream "
                         f"{tuple(tokens.shape)}")
    rolled = torch.roll(tokens, shifts=-1, dims=1)
    V = lm_head_weight.shape[0]
    if action_only:
        return _action_rows_only(last_hidden_state, lm_head_weight, rolled, batch, seqlen, int(num_actions), attention_mask,
                                 float(temperature), return_output, compute_entropy, entropy_requires_grad, nnz_indices)

    output = {}
    if compute_entropy:
        hidden = ops.hidden_for_weight(last_hidden_state, lm_head_weight)
        log_probs, entropy = linear_cross_entropy(hidden, lm_head_weight.contiguous(), rolled.contiguous(), float(temperature),
                                                  "none", None)
        log_probs, entropy = log_probs.reshape(tokens.shape), entropy.reshape(tokens.shape)
        if not entropy_requires_grad:
            entropy = entropy.detach()
        if packed:
            entropy = _pad_back(entropy.reshape(-1), nnz_indices, batch, seqlen)
        elif attention_mask is not None:
            if attention_mask.shape != entropy.shape:
                raise ValueError(f"attention_mask shape {tuple(attention_mask.shape)} does not match {tuple(entropy.shape)}")
            entropy = entropy * attention_mask
        output["entropy"] = entropy
    else:
        log_probs = _fused_lm_head_logprob_apply("hip", last_hidden_state, lm_head_weight, rolled, 0, V, tokens.shape[1], None,
                                                 not torch.is_grad_enabled(), float(temperature))
    if packed:
        log_probs = _pad_back(log_probs.reshape(-1), nnz_indices, batch, seqlen)
    action_log_probs = log_probs[:, -num_actions - 1 : -1]
    return (action_log_probs, output) if return_output else action_log_probs


def action_log_probs_from_logits(
    logits_BSV: torch.Tensor,
    sequences: torch.Tensor,
    num_actions: Union[int, List[int]],
    attention_mask: Optional[torch.Tensor] = None,
    temperature: float = 1.0,
    return_output: bool = False,
    compute_entropy: bool = False,
    entropy_requires_grad: bool = True,
    nnz_indices: Optional[torch.Tensor] = None,
    inplace_backward: bool = True,
) -> Union[torch.Tensor, Tuple[torch.Tensor, dict]]:
    """The same tail for a worker that keeps its ``[B, S, V]`` logits (``[1, nnz, V]`` with the padding removed): lines
    333-393 of the reference's ``HFModelWrapper.forward`` as they stand, with the temperature division (:334), the
    log-probability (:337-341) and the entropy (:358-386) taken from ONE pass over the logits instead of an in-place division
    and six to eight elementwise passes, and the backward written over the logits' own storage (``inplace_backward``, what
    the reference gets from flash-attn's cross-entropy when it is installed, torch_utils.py:131-152).  The logits themselves
    are left undivided.  Entropy in the logits' dtype, as the reference returns it (torch_utils.py:92)."""
    from .torch_utils import _FromLogits, _flat

    if isinstance(num_actions, list):
        if len(num_actions) != 1:
            raise NotImplementedError("per-row num_actions is not supported (the reference slices with a numpy array here, "
                                      "which torch rejects as well)")
        num_actions = num_actions[0]
    batch, seqlen = sequences.shape
    packed = nnz_indices is not None
    tokens = sequences.reshape(-1)[nnz_indices.to(torch.long)].unsqueeze(0) if packed else sequences
    if logits_BSV.shape[:2] != tokens.shape:
        raise ValueError(f"logits {tuple(logits_BSV.shape)} do not match the token stream {tuple(tokens.shape)}")
    rolled = torch.roll(tokens, shifts=-1, dims=1)
    log_probs, entropy = _FromLogits.apply(_flat(logits_BSV), rolled.reshape(-1).to(torch.int64).contiguous(),
                                           1.0 / float(temperature), bool(compute_entropy), bool(inplace_backward))
    log_probs = log_probs.reshape(tokens.shape)
    output = {}
    if compute_entropy:
        entropy = entropy.reshape(tokens.shape).to(logits_BSV.dtype)
        if not entropy_requires_grad:
            entropy = entropy.detach()
        if packed:
            entropy = _pad_back(entropy.reshape(-1), nnz_indices, batch, seqlen)
        elif attention_mask is not None:
            if attention_mask.shape != entropy.shape:
                raise ValueError(f"attention_mask shape {tuple(attention_mask.shape)} does not match {tuple(entropy.shape)}")
            entropy = entropy * attention_mask
        output["entropy"] = entropy
    if packed:
        log_probs = _pad_back(log_probs.reshape(-1), nnz_indices, batch, seqlen)
    action_log_probs = log_probs[:, -num_actions - 1 : -1]
    return (action_log_probs, output) if return_output else action_log_probs


def _action_rows_only(last_hidden_state, lm_head_weight, rolled, batch, seqlen, num_actions, attention_mask, temperature,
                      return_output, compute_entropy, entropy_requires_grad, nnz_indices):
    """The LM head on the action window only: rows are gathered (differentiably) from the token stream, scored, and put back."""
    dev = last_hidden_state.device
    first = seqlen - num_actions - 1
    if num_actions < 1 or first < 0:
        raise ValueError(f"num_actions {num_actions} does not fit sequences of length {seqlen}")
    cols = torch.arange(first, seqlen - 1, device=dev)
    flat = (torch.arange(batch, device=dev).unsqueeze(1) * seqlen + cols.unsqueeze(0)).reshape(-1)   # positions in [B, S]
    if nnz_indices is not None:
        to_stream = torch.full((batch * seqlen,), -1, dtype=torch.long, device=dev)
        to_stream[nnz_indices.to(torch.long)] = torch.arange(nnz_indices.numel(), device=dev)
        src = to_stream[flat]
        present = src >= 0                                       # padding positions hold no token: 0, as pad_input leaves them
        src = src.clamp(min=0)
    else:
        src, present = flat, None
    H = last_hidden_state.shape[-1]
    rows = ops.hidden_for_weight(last_hidden_state.reshape(-1, H).index_select(0, src), lm_head_weight).unsqueeze(0)
    labels = rolled.reshape(-1).index_select(0, src).unsqueeze(0).contiguous()
    output = {}
    if compute_entropy:
        log_probs, entropy = linear_cross_entropy(rows, lm_head_weight.contiguous(), labels, temperature, "none", None)
        entropy = entropy.reshape(batch, num_actions)
        if not entropy_requires_grad:
            entropy = entropy.detach()
        if present is not None:
            entropy = entropy * present.reshape(batch, num_actions)
        elif attention_mask is not None:
            entropy = entropy * attention_mask[:, first:seqlen - 1]
        full = torch.zeros((batch, seqlen), dtype=entropy.dtype, device=dev)
        output["entropy"] = torch.cat([full[:, :first], entropy, full[:, seqlen - 1:]], dim=1)
    else:
        log_probs = _fused_lm_head_logprob_apply("hip", rows, lm_head_weight, labels, 0, lm_head_weight.shape[0], rows.shape[1],
                                                 None, not torch.is_grad_enabled(), temperature)
    action_log_probs = log_probs.reshape(batch, num_actions)
    if present is not None:
        action_log_probs = action_log_probs * present.reshape(batch, num_actions)
    return (action_log_probs, output) if return_output else action_log_probs
