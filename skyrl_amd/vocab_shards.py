"""Combining the fused LM head's per-shard statistics when the vocabulary is split over several weight shards.

The kernels already work on any ``[V_local, H]`` slice of the LM-head weight: ``lmhead_fwd`` returns, per token, the
log-sum-exp and the probability-weighted logit sum *of that slice* (``row_lse``, ``row_pz``) and the target's
log-probability relative to the slice (0 when the target lies in another slice); ``lmhead_bwd`` takes ``row_lse`` /
``row_pz`` back as inputs, so handing it the *global* values makes every slice produce its rows of ``d_weight`` and its
share of ``d_hidden`` of the global softmax.  What a tensor-parallel group has to exchange in between is therefore four
``[T]`` fp32 vectors -- the role of the MAX / SUM all-reduces of ``_compute_distributed_log_softmax``
(skyrl/backends/skyrl_train/distributed/megatron/model_utils.py:28-63) and of the tensor-parallel branch of the vendored
kernel's host code (fused_linear_logprob_triton.py:749-801).

``merge_shard_statistics`` is that exchange written for shards held by one process (stacked along dimension 0).  With one
shard per rank the same arithmetic is: ``m = all_reduce(row_lse, MAX)``; ``lse = m + log(all_reduce(exp(row_lse - m), SUM))``;
``pz = all_reduce(exp(row_lse - lse) * row_pz, SUM)``; ``z_y = all_reduce(owner ? logprob + row_lse : 0, SUM)``; and the
``d_hidden`` shares are summed by the all-reduce (or the sequence-parallel reduce-scatter) that follows the LM head.
The soft cross-entropy of the draft head shards the same way (``merge_soft_ce_shard_statistics``): per slice ``softce_fwd``
returns the two log-sum-exps of the slice and ``loss = lse_student - E_teacher[z_student]`` with the teacher normalised over
the slice; the group exchanges three ``[T]`` vectors (the MAX / SUM all-reduces of ``_vocab_parallel_softmax`` /
``_vocab_parallel_log_softmax`` and the SUM of the per-token dot product, skyrl/backends/skyrl_train/mtp/soft_ce.py:97-143), and
``softce_bwd`` with the global log-sum-exps gives every slice its share of the student's gradient.

This module runs no collective: process groups larger than one are refused by the autograd front ends.
"""

from __future__ import annotations

from typing import Tuple

import torch

__all__ = ["merge_shard_statistics", "merge_soft_ce_shard_statistics"]


def merge_shard_statistics(logprobs: torch.Tensor, row_lse: torch.Tensor, row_pz: torch.Tensor,
                           owner: torch.Tensor) -> Tuple[torch.Tensor, torch.Tensor, torch.Tensor, torch.Tensor]:
    """Per-shard outputs of ``lmhead_fwd`` (each ``[shards, T]`` fp32; ``owner`` bool, true where the token's target lies
    in that shard) -> global ``(logprobs, entropy, row_lse, row_pz)``, each ``[T]``.  A token whose target no shard owns
    gets log-probability 0, as in the single-shard case."""
    if not (logprobs.shape == row_lse.shape == row_pz.shape == owner.shape and logprobs.dim() == 2):
        raise ValueError("expected four [shards, T] tensors")
    m = row_lse.max(dim=0).values
    lse = m + torch.log(torch.exp(row_lse - m).sum(dim=0))
    pz = (torch.exp(row_lse - lse) * row_pz).sum(dim=0)
    owned = owner.any(dim=0)
    z_target = torch.where(owner, logprobs + row_lse, torch.zeros_like(logprobs)).sum(dim=0)
    merged_logprobs = torch.where(owned, z_target - lse, torch.zeros_like(lse))
    return merged_logprobs, lse - pz, lse, pz


def merge_soft_ce_shard_statistics(loss: torch.Tensor, lse_student: torch.Tensor,
                                   lse_teacher: torch.Tensor) -> Tuple[torch.Tensor, torch.Tensor, torch.Tensor]:
    """Per-shard outputs of ``softce_fwd`` (each ``[shards, T]`` fp32) -> global ``(loss, lse_student, lse_teacher)``.

    A shard's ``lse_student - loss`` is the teacher-weighted mean of the student's logits over that shard; weighting the
    shards by their share of the teacher's probability mass, ``exp(lse_teacher_shard - lse_teacher)``, gives the global mean."""
    if not (loss.shape == lse_student.shape == lse_teacher.shape and loss.dim() == 2):
        raise ValueError("expected three [shards, T] tensors")
    lse_s = torch.logsumexp(lse_student, dim=0)
    lse_t = torch.logsumexp(lse_teacher, dim=0)
    mean_z = (torch.exp(lse_teacher - lse_t) * (lse_student - loss)).sum(dim=0)
    return lse_s - mean_z, lse_s, lse_t
