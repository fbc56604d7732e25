"""CPU restatement of SkyRL's fused LM-head log-probability path.  TEST INFRASTRUCTURE ONLY.

This module is the checker for the HIP kernels, not a product path: only ``tests/``, ``__graft_entry__.smoke()`` and the
``cpu_baseline`` leg of ``bench.py`` may import it.  Nothing under ``skyrl_amd/`` does, and the product raises when the
HIP library is missing instead of routing here.

Every function restates one piece of the reference and cites it (paths relative to the SkyRL tree; ``MU`` =
``skyrl/backends/skyrl_train/distributed/megatron/model_utils.py``, ``TR`` = ``.../megatron/fused_linear_logprob_triton.py``).
Tensor-parallel all-reduces are identities here (one vocab shard holds the full vocabulary).

What pins each function (all in ``tests/test_oracle.py``; none of them re-types the formula under test):
  * log-softmax / logprob / entropy forward: ``torch.log_softmax`` + ``gather`` in fp64, the closed forms
    ``W = 0 -> logprob = -ln V, entropy = ln V`` (the reference's own known answer is ``ln 4``,
    tests/backends/skyrl_train/utils/test_torch_utils.py:31-35), ``sum_y exp(logprob(y)) = 1`` by brute force over every
    target, shift invariance, chunk-size invariance over the reference's cases {1, 7, 64, 512}
    (tests/backends/skyrl_train/gpu/gpu_ci/megatron/test_fused_linear_logprob.py:98).
  * split merge: any partition of the vocabulary merges to the one-shot result (hypothesis).
  * d_logits, dHidden, dW: torch autograd of the fp64 closed form, fp64 central finite differences, row sums of d_logits,
    linearity in (g, q), the reference's tolerances (test_fused_linear_logprob.py:89-95).
  * out-of-vocabulary targets: forward 0 / backward keeps -p*g, by construction of an autograd twin whose target logit is
    multiplied by the in-vocabulary mask.
  * packed-sequence roll and scatter-back (plain, sub-sequence and attention-mask layouts): per-sequence Python loops that
    place each token by hand, over ragged cases with length-1 and empty sequences, padded segments, left- and
    interior-padded masks and outputs narrower than a row's content.
  * packed action-token entropy: a per-row Python loop that walks each row's real tokens (or listed sub-sequences) and
    adds up entropy times weight by hand, with loss masks, left padding and a row without action weight.
  * PPO policy loss: hand-computed cases on both sides of every branch (unclipped, clipped high / low for either sign of
    the advantage, dual-clip active / inactive, the +-20 clamp of the log-ratio), fp64 central finite differences of the
    loss for the gradient autograd derives from it, and the masked-mean definition of clip_ratio counted by hand.
  * cross-entropy and importance-sampling losses, masked_mean: values worked out by hand on small inputs.
  * SAPO, GSPO, CISPO, rollout-IS and DPPO losses: per-token values worked out with ``math`` on either side of every branch
    (sign of the advantage, inside / on / outside the interval, both trust-region tests, the clamps at 20 and 10), the
    limits that tie them to pinned functions (GSPO on rows of one token is the clipped surrogate; DPPO with nothing masked
    and SAPO's gate near r = 1 are the importance-sampling surrogate; CISPO and rollout-IS agree inside the interval), and
    fp64 central finite differences of the surrogate with the stop-gradient factors held fixed.
  * clip-cov and kl-cov losses: the selection counted and listed by hand on a 2 x 4 batch (which tokens are candidates, how
    many are drawn, the top-k by sorting the hand-computed covariance terms), the limit in which every candidate is drawn
    (so that the random permutation cannot matter), loss values token by token with ``math``, and fp64 central finite
    differences with the selection held fixed.  CISPO's ratio diagnostics: hand values with and without a mask.
  * approximate KL: hand values at d = 0, ln 2, -1 and in both clamps; the identities the estimators are built on --
    under x ~ p the expectation of k1 and of k3 is KL(p || q) exactly, summed by brute force over a small alphabet and
    compared with ``torch.nn.functional.kl_div`` -- and k3 ~ k2 for small differences; the trainer's reduction against a
    per-row Python loop.
  * the assembled actor loss: a hand-computed two-row case (every term worked out on paper) on top of the pinned parts.
  * the FSDP forward tail: ``torch.distributions.Categorical`` for entropy and log-probability, and a Python loop that
    scores action token j of row b against position S - num_actions + j - 1, with and without padding removed.
  * MTP soft cross-entropy: the reference's own golden masks for ``shift_mask_for_mtp`` (tests/backends/skyrl_train/mtp/
    test_soft_ce.py:224-245) plus a per-position Python loop for the packed form; the decomposition soft CE = H(p) + KL(p || q)
    against ``torch.distributions`` / ``torch.nn.functional.kl_div``, the limits "teacher = student -> entropy" (the
    reference's known answer, test_soft_ce.py:248-284) and "one-hot teacher -> -log q(label)" (the pinned log-probability),
    and the gradient softmax(student) - softmax(teacher) (test_soft_ce.py:171-181) by fp64 finite differences.
  * MTP top-k soft cross-entropy: a per-token Python loop that picks the k largest teacher logits with ``sorted`` and sums
    the loss with ``math``; the limit k = V, where it is the full soft cross-entropy pinned above; the roll of the small
    [B, S, k] lists against a pre-rolled teacher (the reference's own check, test_soft_ce.py:122-144); the restated custom
    backward against autograd of the forward and fp64 finite differences, and its at most k non-zero columns per token
    (test_soft_ce.py:147-156).
  * logits-input functions (``logprobs_from_logits_v2``, ``DistributedLogprob`` forward / backward): ``torch.distributions.
    Categorical.log_prob``, the uniform-logits known answer ``-ln V``, autograd of ``log_softmax`` + ``gather`` in fp64 for the
    hand-written backward, its row sums (zero for a target inside the shard, ``-g`` outside), and the reference's own
    out-of-shard semantics (forward 0, backward keeps ``-softmax * g``).
  * off-policy correction: every step on a 3 x 4 batch whose ratios are powers of two, each mask, weight and metric
    written down by hand, and the order of the steps (a row removed as an outlier no longer counts in the token-mask and
    TIS statistics and has sequence ratio 1; the sequence mask sees the tokens the token mask left).
  * log-probability drift statistics: a six-token case worked out by hand, with a mask, with fractional weights and without.
  * the reference's own unit-test vectors for the off-policy correction, the policy losses and the approximate KL
    (tests/train/algorithms/test_off_policy_correction.py, tests/train/algorithms/test_losses.py,
    tests/backends/skyrl_train/utils/test_ppo_utils.py:38-98), transcribed into tests/golden/reference_unit_test_cases.json and run
    by tests/test_reference_unit_cases.py in fp32 and fp64 at the reference's tolerances.
No function is left "parity unpinned".
"""

from __future__ import annotations

from typing import List, Optional, Sequence, Tuple

import torch

OOV_LABEL_SENTINEL = torch.iinfo(torch.int64).max  # TR:1832


# ----------------------------------------------------------------------------------------------------------------------
# Torch backend of the reference: FusedLinearChunkedDistributedLogprob and helpers
# ----------------------------------------------------------------------------------------------------------------------
def distributed_log_softmax(logits: torch.Tensor) -> torch.Tensor:
    """MU:28-63 with the MAX / SUM all-reduces as identities: amax, subtract, exp, sum (as float), subtract log."""
    logits_max = torch.amax(logits, dim=-1, keepdim=True)
    shifted = logits - logits_max
    sum_exp = shifted.exp().sum(-1, keepdim=True).float()
    return shifted - sum_exp.log_().to(shifted.dtype)


def _mask_targets(target: torch.Tensor, vocab_start: int, vocab_end: int) -> Tuple[torch.Tensor, torch.Tensor]:
    """MU:314-316: mask of targets outside the shard; masked targets re-based to the shard and zeroed."""
    target_mask = (target < vocab_start) | (target >= vocab_end)
    masked_target = target - vocab_start
    masked_target[target_mask] = 0
    return target_mask, masked_target


def fused_chunked_logprob_forward(
    hidden: torch.Tensor, weight: torch.Tensor, target: torch.Tensor, vocab_start: int, vocab_end: int, chunk_size: int
) -> torch.Tensor:
    """MU:302-359.  hidden [B,S,H], weight [V,H], target [B,S] (already shifted) -> logprobs [B,S] fp32.

    Per sequence chunk: matmul in the weight dtype, cast to fp32, log-softmax, gather the target, force 0 where the target is
    outside [vocab_start, vocab_end).
    """
    target_mask, masked_target = _mask_targets(target.clone(), vocab_start, vocab_end)
    seq = int(hidden.shape[1])
    out: List[torch.Tensor] = []
    for c0 in range(0, seq, chunk_size):
        c1 = min(seq, c0 + chunk_size)
        logits = torch.matmul(hidden[:, c0:c1, :].to(weight.dtype), weight.t()).to(torch.float32)
        lp = distributed_log_softmax(logits)
        lp = torch.gather(lp, -1, masked_target[:, c0:c1].unsqueeze(-1)).squeeze(-1)
        lp[target_mask[:, c0:c1]] = 0.0
        out.append(lp)
    return torch.cat(out, dim=1)


def fused_chunked_logprob_backward(
    hidden: torch.Tensor,
    weight: torch.Tensor,
    target: torch.Tensor,
    vocab_start: int,
    vocab_end: int,
    chunk_size: int,
    grad_output: torch.Tensor,
) -> Tuple[torch.Tensor, torch.Tensor]:
    """MU:361-428.  Returns (grad_hidden in hidden dtype, grad_weight as the fp32 accumulator *before* the final cast to the
    weight dtype at MU:428 -- callers cast if they want the reference's returned dtype).

    Per chunk: recompute softmax, grad_logits = -softmax * g, scatter-add g at in-shard targets, cast to the weight dtype,
    grad_hidden[chunk] = grad_logits @ W, grad_weight += (grad_logits^T @ h).float().
    """
    target_mask, masked_target = _mask_targets(target.clone(), vocab_start, vocab_end)
    V, H = int(weight.shape[0]), int(weight.shape[1])
    B, seq = int(hidden.shape[0]), int(hidden.shape[1])
    grad_hidden = torch.empty_like(hidden)
    grad_weight = torch.zeros((V, H), dtype=torch.float32)
    for c0 in range(0, seq, chunk_size):
        c1 = min(seq, c0 + chunk_size)
        h_chunk = hidden[:, c0:c1, :]
        logits = torch.matmul(h_chunk.to(weight.dtype), weight.t()).to(torch.float32)
        grad_logits = distributed_log_softmax(logits).exp_().neg_()
        g = grad_output[:, c0:c1]
        grad_logits.mul_(g.unsqueeze(-1))
        valid = ~target_mask[:, c0:c1]
        # scatter-add of g at the chosen column (MU:396-411), written with 2-D indexing instead of flat offsets
        b_idx, s_idx = valid.nonzero(as_tuple=True)
        grad_logits[b_idx, s_idx, masked_target[:, c0:c1][b_idx, s_idx]] += g[b_idx, s_idx]
        grad_logits = grad_logits.to(weight.dtype)
        grad_hidden[:, c0:c1, :] = torch.matmul(grad_logits, weight)
        gl2 = grad_logits.reshape(-1, V)
        grad_weight.add_(torch.matmul(gl2.t(), h_chunk.reshape(-1, H).to(gl2.dtype)).to(torch.float32))
    return grad_hidden, grad_weight


def fused_entropy_from_hidden(
    hidden: torch.Tensor, weight: torch.Tensor, chunk_size: Optional[int] = None, temperature: float = 1.0
) -> torch.Tensor:
    """MU:1090-1121 (no-grad entropy metric): H = max + log(sum exp) - sum softmax*logits per token, weight divided by the
    temperature first (in the weight dtype)."""
    if temperature != 1.0:
        weight = weight / temperature
    B, S = int(hidden.shape[0]), int(hidden.shape[1])
    out = torch.empty((B, S), dtype=torch.float32)
    eff = chunk_size if (chunk_size is not None and chunk_size < S) else S
    for c0 in range(0, S, eff):
        c1 = min(S, c0 + eff)
        logits = torch.matmul(hidden[:, c0:c1, :].to(weight.dtype), weight.t()).to(torch.float32)
        logits_max = logits.max(dim=-1, keepdim=True).values
        e = (logits - logits_max).exp_()
        sum_exp = e.sum(dim=-1, keepdim=True)
        softmax = e / sum_exp
        spz = (softmax * logits).sum(dim=-1, keepdim=True)
        out[:, c0:c1] = (logits_max + sum_exp.log() - spz).squeeze(-1)
    return out


def vocab_parallel_entropy_backward(logits: torch.Tensor, grad_entropy: torch.Tensor) -> torch.Tensor:
    """MU:1339-1345: d entropy / d logits = softmax * (sum softmax*logits - logits) * grad."""
    p = torch.softmax(logits, dim=-1)
    spz = (p * logits).sum(dim=-1, keepdim=True)
    return p * (spz - logits) * grad_entropy.unsqueeze(-1)


# ----------------------------------------------------------------------------------------------------------------------
# Triton backend of the reference (vendored verl kernels): split statistics, merge, d_logits
# ----------------------------------------------------------------------------------------------------------------------
def split_statistics(logits: torch.Tensor) -> Tuple[torch.Tensor, torch.Tensor, torch.Tensor]:
    """TR:296-385 for one vocab split, logits already scaled by 1/temperature: (max, sum exp(z - max), sum z*exp(z - max))."""
    m = logits.max(dim=-1).values
    e = (logits - m.unsqueeze(-1)).exp()
    return m, e.sum(-1), (e * logits).sum(-1)


def merge_split_statistics(
    maxes: torch.Tensor, accus: torch.Tensor, entropy_bs: torch.Tensor
) -> Tuple[torch.Tensor, torch.Tensor, torch.Tensor]:
    """TR:417-446: merge per-split (max, accu, entropy_b) of shape [T, num_splits] into global (max, accu, entropy_b sum).

    The running maximum starts at -inf here; the reference kernel starts it at 0 (TR:421), which is the same number for any
    row with a non-negative logit and wrong (underflow) for rows whose logits are all very negative.  The HIP path follows
    this restatement, not that quirk.
    """
    gmax = maxes.max(dim=-1).values
    scale = (maxes - gmax.unsqueeze(-1)).exp()
    return gmax, (scale * accus).sum(-1), (scale * entropy_bs).sum(-1)


def linear_cross_entropy_forward(
    hidden: torch.Tensor, weight: torch.Tensor, labels: torch.Tensor, temperature: float = 1.0, vocab_per_split: int = 1024
) -> Tuple[torch.Tensor, torch.Tensor, torch.Tensor, torch.Tensor, torch.Tensor]:
    """efficient_entropy_forward, TR:614-803 (REDUCTION none, one rank): returns (logprobs, entropy, maximum, accumulate,
    entropy_b), each [T].  hidden [T,H], weight [V,H]; the dot products accumulate in fp32 from the stored dtype (TR:339),
    logits are scaled by 1/temperature (TR:346); labels matching no column contribute no label logit, and the adapter forces
    their logprob to 0 (TR:1898-1905)."""
    T, V = int(hidden.shape[0]), int(weight.shape[0])
    rcp_t = 1.0 / temperature
    acc_dtype = torch.float64 if hidden.dtype == torch.float64 else torch.float32
    ms, ss, es = [], [], []
    label_logit = torch.zeros(T, dtype=acc_dtype)
    for v0 in range(0, V, vocab_per_split):
        v1 = min(V, v0 + vocab_per_split)
        z = torch.matmul(hidden.to(acc_dtype), weight[v0:v1].to(acc_dtype).t()) * rcp_t
        m, s, e = split_statistics(z)
        ms.append(m), ss.append(s), es.append(e)
        own = (labels >= v0) & (labels < v1)
        idx = own.nonzero(as_tuple=True)[0]
        label_logit[idx] = z[idx, labels[idx] - v0]
    gmax, gacc, geb = merge_split_statistics(torch.stack(ms, 1), torch.stack(ss, 1), torch.stack(es, 1))
    entropy_b = geb / gacc  # TR:453
    entropy = gacc.log() + gmax - entropy_b  # TR:459
    logprobs = -(gmax + gacc.log() - label_logit)  # TR:463-467
    in_vocab = (labels >= 0) & (labels < V)
    logprobs = logprobs.masked_fill(~in_vocab, 0.0)  # TR:1898-1905
    return logprobs, entropy, gmax, gacc, entropy_b


def d_logits_formula(
    logits: torch.Tensor,
    maximum: torch.Tensor,
    accumulate: torch.Tensor,
    entropy_b: torch.Tensor,
    labels: torch.Tensor,
    dlogprobs: torch.Tensor,
    dentropy: torch.Tensor,
    rcp_temperature: float,
    vocab_offset: int = 0,
) -> torch.Tensor:
    """TR:947-957.  ``logits`` are already scaled by 1/temperature and cover columns [vocab_offset, vocab_offset + n).

    exp_logits = exp(z - max);  d = (-g) * (exp_logits/accu - onehot) + q * (-exp_logits/accu) * (z - entropy_b);  d *= 1/temperature.
    """
    p = (logits - maximum.unsqueeze(-1)).exp() / accumulate.unsqueeze(-1)
    cols = torch.arange(logits.shape[-1]) + vocab_offset
    onehot = (cols.unsqueeze(0) == labels.unsqueeze(-1)).to(logits.dtype)
    d = (-dlogprobs).unsqueeze(-1) * (p - onehot)
    d = d + dentropy.unsqueeze(-1) * (-p) * (logits - entropy_b.unsqueeze(-1))
    return d * rcp_temperature


def linear_cross_entropy_backward(
    dlogprobs: torch.Tensor,
    dentropy: torch.Tensor,
    hidden: torch.Tensor,
    weight: torch.Tensor,
    labels: torch.Tensor,
    maximum: torch.Tensor,
    accumulate: torch.Tensor,
    entropy_b: torch.Tensor,
    temperature: float = 1.0,
    vocab_per_split: int = 9504,
    round_d_logits_to: Optional[torch.dtype] = None,
) -> Tuple[torch.Tensor, torch.Tensor]:
    """efficient_entropy_backward with the default ``_Split_Dlogits_N`` method (TR:1689-1748): per vocab split, recompute the
    logits, form d_logits (rounded to the hidden dtype, TR:1402-1538 stores it in that dtype), then
    d_hidden += d_logits @ W_split and d_weight[split] = d_logits^T @ hidden.  Returns fp32 (or fp64) accumulators; the reference
    returns them in the hidden dtype."""
    T, H = int(hidden.shape[0]), int(hidden.shape[1])
    V = int(weight.shape[0])
    rcp_t = 1.0 / temperature
    acc_dtype = torch.float64 if hidden.dtype == torch.float64 else torch.float32
    round_to = hidden.dtype if round_d_logits_to is None else round_d_logits_to
    d_hidden = torch.zeros((T, H), dtype=acc_dtype)
    d_weight = torch.zeros((V, H), dtype=acc_dtype)
    h = hidden.to(acc_dtype)
    for v0 in range(0, V, vocab_per_split):
        v1 = min(V, v0 + vocab_per_split)
        w = weight[v0:v1].to(acc_dtype)
        z = torch.matmul(h, w.t()) * rcp_t
        d = d_logits_formula(z, maximum.to(acc_dtype), accumulate.to(acc_dtype), entropy_b.to(acc_dtype), labels,
                             dlogprobs.to(acc_dtype), dentropy.to(acc_dtype), rcp_t, vocab_offset=v0)
        d = d.to(round_to).to(acc_dtype)
        d_hidden += torch.matmul(d, w)
        d_weight[v0:v1] = torch.matmul(d.t(), h)
    return d_hidden, d_weight


# ----------------------------------------------------------------------------------------------------------------------
# Callers one level up: target roll, packed sequences
# ----------------------------------------------------------------------------------------------------------------------
def from_parallel_hidden_to_logprobs(
    hidden: torch.Tensor, weight: torch.Tensor, target: torch.Tensor, chunk_size: Optional[int] = None, temperature: float = 1.0
) -> torch.Tensor:
    """MU:713-770 at TP = CP = 1: weight / temperature (in the weight dtype, MU:739-740), targets rolled left by one
    (MU:741), fused op, last column dropped (MU:770).  -> [B, S-1]."""
    if temperature != 1.0:
        weight = weight / temperature
    target = target.roll(shifts=-1, dims=-1)
    S = int(hidden.shape[1])
    eff = chunk_size if (chunk_size is not None and chunk_size < S) else S
    lp = fused_chunked_logprob_forward(hidden, weight, target, 0, int(weight.shape[0]), eff)
    return lp[:, :-1]


def packed_sequence_indices(cu_seqlens: torch.Tensor, total_tokens: int) -> Tuple[torch.Tensor, torch.Tensor, torch.Tensor]:
    """MU:920-928: for every packed token its sequence index, offset inside the sequence, and the sequence lengths."""
    cu = cu_seqlens.to(torch.long)
    tok = torch.arange(total_tokens)
    seq_idx = torch.searchsorted(cu[1:], tok, right=True)
    seq_off = tok - cu[seq_idx]
    return seq_idx, seq_off, cu[1:] - cu[:-1]


def packed_rolled_targets(target: torch.Tensor, cu_seqlens: torch.Tensor) -> torch.Tensor:
    """MU:810-815: per-sequence roll(-1) inside a packed [T] stream: next = (offset + 1) mod len."""
    seq_idx, seq_off, seq_len = packed_sequence_indices(cu_seqlens, int(target.shape[0]))
    nxt = torch.remainder(seq_off + 1, seq_len[seq_idx])
    return target[cu_seqlens.to(torch.long)[seq_idx] + nxt]


def packed_subseq_rows_offsets_lens(cu_seqlens: torch.Tensor, sub_seq_lengths: Sequence[Sequence[int]]):
    """MU:886-917: with several sequences packed per output row, segment k (in stream order) belongs to the row that lists
    it, starts at the column where the *padded* lengths of the row's earlier segments end, and has the listed true length."""
    bounds = [int(x) for x in cu_seqlens.tolist()]
    padded = [bounds[i + 1] - bounds[i] for i in range(len(bounds) - 1)]
    rows, offs, lens = [], [], []
    k = 0
    for r, row_lens in enumerate(sub_seq_lengths):
        col = 0
        for n in row_lens:
            if k >= len(padded):
                raise ValueError("sub_seq_lengths contains more sub-sequences than cu_seqlens_padded")
            rows.append(r)
            offs.append(col)
            lens.append(int(n))
            col += padded[k]
            k += 1
    if k != len(padded):
        raise ValueError(f"sub_seq_lengths describes {k} sub-sequences, but cu_seqlens_padded describes {len(padded)}")
    return torch.tensor(rows, dtype=torch.long), torch.tensor(offs, dtype=torch.long), torch.tensor(lens, dtype=torch.long)


def packed_scatter_back(
    probs: torch.Tensor,
    cu_seqlens: torch.Tensor,
    batch_size: int,
    unpacked_seqlen: int,
    sub_seq_lengths: Optional[Sequence[Sequence[int]]] = None,
    attention_mask: Optional[torch.Tensor] = None,
) -> torch.Tensor:
    """MU:851-883, all three branches.  Plain: token at (seq i, offset o) goes to out[i, o] for o < len_i - 1 and
    o < unpacked_seqlen - 1.  Sub-sequences (MU:859-871): to out[row_i, col_i + o] for o < true_len_i - 1, column in bounds.
    Attention mask (MU:873-878): the positions of ``mask[:, :-1]`` that hold a real token other than the row's last one
    receive, in row-major order, the tokens with o < real_len_i - 1.  Everything else stays 0."""
    out = torch.zeros((batch_size, unpacked_seqlen - 1), dtype=probs.dtype)
    seq_idx, seq_off, seq_len = packed_sequence_indices(cu_seqlens, int(probs.shape[0]))
    if sub_seq_lengths is not None:
        rows, offs, lens = packed_subseq_rows_offsets_lens(cu_seqlens, sub_seq_lengths)
        valid = torch.clamp(lens - 1, min=0)
        mask = seq_off < valid[seq_idx]
        cols = offs[seq_idx[mask]] + seq_off[mask]
        rws = rows[seq_idx[mask]]
        inb = cols < unpacked_seqlen - 1
        out[rws[inb], cols[inb]] = probs[mask][inb]
        return out
    if attention_mask is not None:
        am = attention_mask.to(torch.bool)
        real = am.sum(dim=1, dtype=torch.long)
        ordinal = am.to(torch.long).cumsum(dim=1)
        out_mask = am[:, :-1] & (ordinal[:, :-1] < real.unsqueeze(1))
        valid = torch.clamp(real - 1, min=0)
        out[out_mask] = probs[seq_off < valid[seq_idx]]
        return out
    valid = torch.clamp(seq_len - 1, min=0)
    mask = (seq_off < valid[seq_idx]) & (seq_off < unpacked_seqlen - 1)
    out[seq_idx[mask], seq_off[mask]] = probs[mask]
    return out


# ----------------------------------------------------------------------------------------------------------------------
# Convenience used by the parity tests and the CPU baseline: one call = forward + backward of the whole path
# ----------------------------------------------------------------------------------------------------------------------
def packed_action_entropy(
    entropy_tokens: torch.Tensor,
    cu_seqlens: torch.Tensor,
    unpacked_seqlen: int,
    num_actions: int,
    attention_mask: torch.Tensor,
    loss_mask: Optional[torch.Tensor],
    sub_seq_lengths: Optional[Sequence[Sequence[int]]] = None,
) -> Tuple[torch.Tensor, torch.Tensor]:
    """MU:1124-1208 at CP = 1, after the per-token entropy: the action weights (ones, or the loss mask, in the last
    ``num_actions`` columns of [B, unpacked_seqlen - 1], MU:1153-1157) are carried to the packed stream by the inverse of the
    scatter-back mapping (sub-sequences MU:1160-1172, attention mask MU:1173-1179) and the entropy is their weighted mean
    with the weight sum clamped at 1 (MU:1196-1207).  Returns ``(entropy, entropy_for_loss)``, equal at CP = 1."""
    batch = int(attention_mask.shape[0])
    weights = torch.zeros((batch, unpacked_seqlen - 1), dtype=entropy_tokens.dtype)
    weights[:, -num_actions:] = 1.0 if loss_mask is None else loss_mask.to(entropy_tokens.dtype)
    packed = torch.zeros(int(cu_seqlens[-1]), dtype=entropy_tokens.dtype)
    if sub_seq_lengths is not None:
        seq_idx, seq_off, _ = packed_sequence_indices(cu_seqlens, int(packed.shape[0]))
        rows, offs, lens = packed_subseq_rows_offsets_lens(cu_seqlens, sub_seq_lengths)
        take = seq_off < torch.clamp(lens - 1, min=0)[seq_idx]
        cols = offs[seq_idx[take]] + seq_off[take]
        rws = rows[seq_idx[take]]
        inb = cols < weights.shape[1]
        packed[torch.arange(int(packed.shape[0]))[take][inb]] = weights[rws[inb], cols[inb]]
    else:
        am = attention_mask.to(torch.bool)
        real = am.sum(dim=1, dtype=torch.long)
        ordinal = am.to(torch.long).cumsum(dim=1)
        out_mask = am[:, :-1] & (ordinal[:, :-1] < real.unsqueeze(1))
        where = cu_seqlens.to(torch.long)[:-1].unsqueeze(1) + (ordinal - 1)
        packed[where[:, :-1][out_mask]] = weights[out_mask]
    total = (entropy_tokens * packed).sum()
    count = packed.sum().clamp(min=1.0)
    return total / count, total / count


def reference_faithful_fwd_bwd(
    hidden: torch.Tensor,
    weight: torch.Tensor,
    labels: torch.Tensor,
    temperature: float,
    dlogprobs: Optional[torch.Tensor],
    chunk_size: int = 1024,
    want_entropy: bool = True,
):
    """The reference's pure-torch path exactly as the trainer runs it on one rank (bf16 matmul, fp32 softmax, W / temperature
    in the weight dtype): logprobs via MU:302-359, entropy metric via MU:1090-1121, backward via MU:361-428.
    hidden [T,H], labels [T] already shifted.  Returns dict of tensors; gradients are w.r.t. the *scaled* weight W/temperature
    multiplied back by 1/temperature (the chain rule autograd applies for MU:739-740)."""
    w_scaled = weight / temperature if temperature != 1.0 else weight
    h3 = hidden.unsqueeze(0)
    y3 = labels.unsqueeze(0)
    V = int(weight.shape[0])
    out = {"logprobs": fused_chunked_logprob_forward(h3, w_scaled, y3, 0, V, chunk_size).squeeze(0)}
    if want_entropy:
        out["entropy"] = fused_entropy_from_hidden(h3, weight, chunk_size, temperature).squeeze(0)
    if dlogprobs is not None:
        gh, gw = fused_chunked_logprob_backward(h3, w_scaled, y3, 0, V, chunk_size, dlogprobs.unsqueeze(0))
        out["d_hidden"] = gh.squeeze(0)
        out["d_weight"] = gw / temperature
    return out


def exact_fwd_bwd(
    hidden: torch.Tensor,
    weight: torch.Tensor,
    labels: torch.Tensor,
    temperature: float,
    dlogprobs: Optional[torch.Tensor] = None,
    dentropy: Optional[torch.Tensor] = None,
    dtype: torch.dtype = torch.float64,
    vocab_per_split: int = 8192,
):
    """High-precision statement of the whole path (the verl formulas evaluated in ``dtype`` with no intermediate rounding).
    This is the "fp32 reference" side of the gradient-cosine criterion; fp64 by default."""
    h, w = hidden.to(dtype), weight.to(dtype)
    lp, ent, mx, acc, eb = linear_cross_entropy_forward(h, w, labels, temperature, vocab_per_split)
    out = {"logprobs": lp, "entropy": ent, "lse": mx + acc.log(), "pz": eb}
    if dlogprobs is not None:
        q = dentropy if dentropy is not None else torch.zeros_like(dlogprobs)
        dh, dw = linear_cross_entropy_backward(dlogprobs, q, h, w, labels, mx, acc, eb, temperature, vocab_per_split,
                                               round_d_logits_to=dtype)
        out["d_hidden"], out["d_weight"] = dh, dw
    return out


# ----------------------------------------------------------------------------------------------------------------------
# The consumer one step after the log-probabilities: PPO policy loss
# ----------------------------------------------------------------------------------------------------------------------
def ppo_policy_loss(
    log_probs: torch.Tensor,
    old_log_probs: torch.Tensor,
    advantages: torch.Tensor,
    eps_clip_low: float,
    eps_clip_high: float,
    clip_ratio_c: float = 3.0,
    dual_clip: bool = False,
    loss_mask: Optional[torch.Tensor] = None,
    loss_weight: Optional[torch.Tensor] = None,
) -> Tuple[torch.Tensor, torch.Tensor]:
    """skyrl/backends/skyrl_train/utils/ppo_utils.py:555-588 ("regular" and "dual_clip"), with safe_exp_delta and masked_mean of
    skyrl/backends/skyrl_train/utils/torch_utils.py:180-192 and reduce_loss of ppo_utils.py:1145-1149.  ``loss_weight`` stands
    for the importance ratio apply_off_policy_correction multiplies in (off_policy_correction_utils.py:383-384).  Returns
    ``(loss, clip_ratio)``; the gradient is whatever autograd derives from these torch ops, as in the reference."""
    ratio = torch.clamp(log_probs - old_log_probs, -20.0, 20.0).exp()                    # safe_exp_delta, clip=20
    surr1 = ratio * advantages
    surr2 = ratio.clamp(1 - eps_clip_low, 1 + eps_clip_high) * advantages
    loss = -torch.min(surr1, surr2)
    clipped = (-surr2 > -surr1).to(log_probs.dtype)
    if loss_mask is None:
        clip_ratio = clipped.mean()                                                      # masked_mean without a mask
    else:
        clip_ratio = (clipped * loss_mask).sum() / loss_mask.sum().clamp(min=1.0)
    if dual_clip:
        pg_losses3 = -advantages * clip_ratio_c
        loss = torch.where(advantages < 0, torch.min(pg_losses3, loss), loss)
    if loss_weight is not None:
        loss = loss * loss_weight
    loss = (loss * loss_mask).sum() if loss_mask is not None else loss.sum()            # reduce_loss
    return loss, clip_ratio.detach()


def _reduce(loss: torch.Tensor, loss_mask: Optional[torch.Tensor]) -> torch.Tensor:
    """reduce_loss, ppo_utils.py:1145-1149: the masked sum."""
    return (loss * loss_mask).sum() if loss_mask is not None else loss.sum()


def _safe_ratio(log_probs: torch.Tensor, behaviour: torch.Tensor) -> torch.Tensor:
    """safe_exp_delta with clip = 20, torch_utils.py:187-192."""
    return torch.clamp(log_probs - behaviour, -20.0, 20.0).exp()


def sapo_policy_loss(log_probs, old_log_probs, advantages, tau_pos: float, tau_neg: float, loss_mask=None):
    """ppo_utils.py:590-660: the sigmoid gate ``sigmoid(tau (r - 1)) 4 / tau`` in place of the clipped ratio, tau chosen by
    the sign of the advantage (:639-643: tau_pos where A > 0, tau_neg elsewhere).  Returns ``(loss, clip_ratio = 0)``."""
    ratio = _safe_ratio(log_probs, old_log_probs)
    taus = torch.where(advantages > 0, torch.as_tensor(tau_pos, dtype=advantages.dtype),
                       torch.as_tensor(tau_neg, dtype=advantages.dtype))
    gates = torch.sigmoid(taus * (ratio - 1.0)) * (4.0 / taus)
    return _reduce(-gates * advantages, loss_mask), torch.zeros(())


def gspo_policy_loss(log_probs, old_log_probs, advantages, eps_clip_low: float, eps_clip_high: float, loss_mask=None):
    """ppo_utils.py:663-729: every token of a sequence carries the sequence's importance weight, the masked row mean of the
    log-ratio (:701), re-attached to the token's own log-probability so that the gradient reaches it (:707), clamped from
    above at 10 (:709), then the clipped surrogate.  Returns ``(loss, clip_ratio)``."""
    row = masked_mean(log_probs - old_log_probs, loss_mask, dim=-1).unsqueeze(-1)
    log_w = torch.clamp(log_probs - log_probs.detach() + row.detach(), max=10)
    ratio = log_w.exp()
    surr1 = ratio * advantages
    surr2 = ratio.clamp(1 - eps_clip_low, 1 + eps_clip_high) * advantages
    clip_ratio = masked_mean((-surr2 > -surr1).to(log_probs.dtype), loss_mask)
    return _reduce(-torch.min(surr1, surr2), loss_mask), clip_ratio.detach()


def cispo_policy_loss(log_probs, behaviour_log_probs, advantages, eps_clip_low: float, eps_clip_high: float, loss_mask=None):
    """ppo_utils.py:732-821: ``-A stopgrad(clamp(r, 1 - lo, 1 + hi)) log_probs``; ``behaviour_log_probs`` is the anchor the
    config selects (:769-780).  Returns ``(loss, clip_ratio)``, the fraction of tokens whose ratio lies outside (:786-787)."""
    ratio = _safe_ratio(log_probs, behaviour_log_probs)
    clamped = torch.clamp(ratio, 1 - eps_clip_low, 1 + eps_clip_high)
    clipped = ((ratio < 1 - eps_clip_low) | (ratio > 1 + eps_clip_high)).to(log_probs.dtype)
    return _reduce(-advantages * clamped.detach() * log_probs, loss_mask), masked_mean(clipped, loss_mask).detach()


def rollout_is_policy_loss(log_probs, rollout_logprobs, advantages, eps_clip_low: float, eps_clip_high: float, loss_mask=None):
    """ppo_utils.py:824-863: as CISPO on the rollout log-probabilities, with the weight set to zero outside the open interval
    (1 - lo, 1 + hi) (:850-851).  Returns ``(loss, clip_ratio)``."""
    ratio = _safe_ratio(log_probs, rollout_logprobs)
    in_range = (ratio > 1 - eps_clip_low) & (ratio < 1 + eps_clip_high)
    weight = torch.where(in_range, ratio, torch.zeros_like(ratio))
    loss = -(weight.detach() * advantages * log_probs)
    return _reduce(loss, loss_mask), masked_mean((~in_range).to(log_probs.dtype), loss_mask).detach()


def dppo_policy_loss(log_probs, mu_log_probs, advantages, dppo_type: str, delta_low: float, delta_high: float, loss_mask=None):
    """ppo_utils.py:866-935: the unclipped surrogate times a 0/1 trust-region mask computed without gradient from the token's
    probability under the two policies -- "binary_tv" (:902-906) on the probability difference, "binary_kl" (:908-917) on the
    Bernoulli KL of the behaviour policy to the current one.  Returns ``(loss, clip_ratio)``, the fraction masked out."""
    ratio = _safe_ratio(log_probs, mu_log_probs)
    with torch.no_grad():
        p, mu = log_probs.exp(), mu_log_probs.exp()
        diff = p - mu
        keep = torch.ones_like(advantages)
        if dppo_type == "binary_tv":
            keep[(advantages > 0) & (diff > delta_high)] = 0.0
            keep[(advantages < 0) & (-diff > delta_low)] = 0.0
        elif dppo_type == "binary_kl":
            eps = 1e-8
            bkl = mu * (mu_log_probs - log_probs) + (1 - mu) * torch.log((1 - mu + eps) / (1 - p + eps))
            keep[(advantages > 0) & (diff > 0) & (bkl > delta_high)] = 0.0
            keep[(advantages < 0) & (diff < 0) & (bkl > delta_low)] = 0.0
        else:
            raise ValueError(f"Unknown DPPO type: {dppo_type}. Must be 'binary_tv' or 'binary_kl'.")
    return _reduce(-(ratio * advantages * keep), loss_mask), masked_mean((keep == 0).to(log_probs.dtype), loss_mask).detach()


def cispo_ratio_diagnostics(log_probs, behaviour_log_probs, eps_clip_low: float, eps_clip_high: float, loss_mask=None):
    """ppo_utils.py:790-815: the four ``cispo/ratio_*`` metrics -- masked means of the ratio and of the clamped ratio, and the
    largest / smallest ratio among the unmasked tokens (among all tokens when there is no mask or the mask is empty)."""
    ratio = _safe_ratio(log_probs, behaviour_log_probs).detach()
    clamped = torch.clamp(ratio, 1 - eps_clip_low, 1 + eps_clip_high)
    active = ratio[loss_mask.bool()] if (loss_mask is not None and bool(loss_mask.any())) else ratio
    return {"cispo/ratio_mean": float(masked_mean(ratio, loss_mask)), "cispo/ratio_clamped_mean": float(masked_mean(clamped, loss_mask)),
            "cispo/ratio_max": float(active.max()), "cispo/ratio_min": float(active.min())}


def clip_cov_policy_loss(log_probs, old_log_probs, advantages, eps_clip_low: float, eps_clip_high: float, clip_ratio: float,
                         clip_cov_lb: float, clip_cov_ub: float, loss_mask: torch.Tensor):
    """ppo_utils.py:938-999.  The clipped surrogate on the unclamped ratio (:962-967); among the unmasked tokens that the clip
    did not catch and whose covariance term (A - mean A)(logp - mean logp) lies strictly inside (lb, ub) (:970-978),
    ``max(int(clip_ratio * sum mask), 1)`` are drawn with ``torch.randperm`` -- the global CPU generator (:977-982) -- and their
    loss is removed (:987-996).  Returns ``(loss, fraction of unmasked tokens removed, the 0/1 factor)``."""
    ratio = torch.exp(log_probs - old_log_probs)
    pg1 = -advantages * ratio
    pg2 = -advantages * torch.clamp(ratio, 1 - eps_clip_low, 1 + eps_clip_high)
    clip_by_origin = (pg2 > pg1) & (loss_mask > 0)
    cov_all = ((advantages - masked_mean(advantages, loss_mask)) * (log_probs - masked_mean(log_probs.detach(), loss_mask))).detach().clone()
    cov_all[loss_mask == 0] = -torch.inf
    cov_all[clip_by_origin] = -torch.inf
    clip_num = max(int(clip_ratio * loss_mask.sum().item()), 1)
    candidates = torch.nonzero((cov_all < clip_cov_ub) & (cov_all > clip_cov_lb) & (loss_mask > 0))
    corr = torch.ones_like(advantages)
    if len(candidates) > 0:
        perm = torch.randperm(len(candidates))
        chosen = candidates[perm[: min(clip_num, len(candidates))]]
        corr[chosen[:, 0], chosen[:, 1]] = 0
    clip_frac = masked_mean((corr == 0).to(log_probs.dtype), loss_mask)
    return _reduce(torch.maximum(pg1, pg2) * corr, loss_mask), clip_frac.detach(), corr


def kl_cov_policy_loss(log_probs, old_log_probs, advantages, kl_cov_frac: float, ppo_kl_coef: float, loss_mask: torch.Tensor):
    """ppo_utils.py:1002-1053.  The importance-sampling surrogate -A r; the ``max(1, int(n * kl_cov_frac))`` unmasked tokens
    with the largest covariance term -- means over the unmasked tokens, computed on the CPU in the inputs' dtype (:1027-1036) --
    pay ``ppo_kl_coef * |logp - old|`` on top (:1038-1047).  Returns ``(loss, the 0/1 selector)``."""
    delta = log_probs - old_log_probs
    ratio = torch.exp(delta)
    pg = -advantages * ratio
    pg_kl = pg + ppo_kl_coef * delta.abs()
    valid = loss_mask > 0
    idx = torch.nonzero(valid.reshape(-1), as_tuple=True)[0]
    adv_v = advantages[valid].detach().reshape(-1).cpu()
    lp_v = log_probs[valid].detach().reshape(-1).cpu()
    selector = torch.zeros(advantages.numel(), dtype=log_probs.dtype)
    if len(adv_v) > 0:
        cov = (adv_v - adv_v.mean()) * (lp_v - lp_v.mean())
        k = max(1, int(len(cov) * kl_cov_frac))
        top = torch.topk(cov, min(k, len(cov)), largest=True).indices
        selector[idx[top]] = 1.0
    selector = selector.reshape(advantages.shape)
    return _reduce(torch.where(selector > 0, pg_kl, pg), loss_mask), selector


def cross_entropy_loss(log_probs: torch.Tensor, loss_mask: Optional[torch.Tensor] = None) -> torch.Tensor:
    """ppo_utils.py:1056-1092: the negative log-likelihood, reduced by reduce_loss (:1145-1149)."""
    loss = -log_probs
    return (loss * loss_mask).sum() if loss_mask is not None else loss.sum()


def importance_sampling_loss(
    log_probs: torch.Tensor, old_log_probs: torch.Tensor, advantages: torch.Tensor, loss_mask: Optional[torch.Tensor] = None
) -> Tuple[torch.Tensor, torch.Tensor]:
    """ppo_utils.py:1095-1142: ``(loss, mean importance ratio)``; neither the log-ratio nor the mask count is clamped."""
    ratio = torch.exp(log_probs - old_log_probs)
    elementwise = -(ratio * advantages)
    if loss_mask is not None:
        return (elementwise * loss_mask).sum(), ((ratio * loss_mask).sum() / loss_mask.sum()).detach()
    return elementwise.sum(), ratio.mean().detach()


def masked_mean(tensor: torch.Tensor, mask: Optional[torch.Tensor], dim: Optional[int] = None) -> torch.Tensor:
    """skyrl/backends/skyrl_train/utils/torch_utils.py:180-184."""
    if mask is None:
        return tensor.mean(dim=dim) if dim is not None else tensor.mean()
    if dim is None:
        return (tensor * mask).sum() / mask.sum().clamp(min=1.0)
    return (tensor * mask).sum(dim=dim) / mask.sum(dim=dim).clamp(min=1.0)


def compute_approx_kl(
    log_probs: torch.Tensor, log_probs_base: torch.Tensor, loss_mask: Optional[torch.Tensor] = None, kl_estimator_type: str = "k3"
) -> torch.Tensor:
    """ppo_utils.py:88-126: the k1 / abs / k2 / k3 estimators of KL(policy || base) per token; masked positions are set to 0
    by ``where`` rather than by the product alone."""
    if kl_estimator_type == "k1":
        kld = log_probs - log_probs_base
    elif kl_estimator_type == "abs":
        kld = (log_probs - log_probs_base).abs()
    elif kl_estimator_type == "k2":
        kld = 0.5 * (log_probs - log_probs_base).square()
    elif kl_estimator_type == "k3":
        kl = torch.clamp(log_probs_base - log_probs, min=-20, max=20)
        kld = torch.clamp(torch.exp(kl) - kl - 1, min=-10, max=10)
    else:
        raise ValueError(f"Invalid KL estimator type: {kl_estimator_type}")
    if loss_mask is not None:
        kld = torch.where(loss_mask.bool(), kld * loss_mask, torch.zeros((), dtype=kld.dtype))
    return kld


def approx_kl_loss(log_probs, log_probs_base, loss_mask=None, kl_estimator_type: str = "k3") -> torch.Tensor:
    """The KL loss term as the trainer reduces it (skyrl/backends/skyrl_train/workers/worker.py:1071-1077)."""
    return masked_mean(compute_approx_kl(log_probs, log_probs_base, loss_mask, kl_estimator_type), loss_mask, dim=-1).mean()


# ----------------------------------------------------------------------------------------------------------------------
# The FSDP worker's forward tail on materialised logits
# ----------------------------------------------------------------------------------------------------------------------
def chunked_entropy_from_logits(logits: torch.Tensor, attention_mask: Optional[torch.Tensor] = None, chunk_size: int = 1024):
    """skyrl/backends/skyrl_train/utils/torch_utils.py:58-111: per sequence chunk ``log_softmax``, ``-sum p log p``, times the
    attention mask; result in the logits' dtype."""
    out = torch.zeros(logits.shape[:2], dtype=logits.dtype)
    for start in range(0, logits.shape[1], chunk_size):
        chunk = torch.log_softmax(logits[:, start:start + chunk_size], dim=-1)
        ent = -(chunk.exp() * chunk).sum(-1)
        if attention_mask is not None:
            ent = ent * attention_mask[:, start:start + chunk_size]
        out[:, start:start + chunk_size] = ent
    return out


def hf_wrapper_tail(
    logits: torch.Tensor,
    sequences: torch.Tensor,
    num_actions: int,
    attention_mask: Optional[torch.Tensor],
    temperature: float,
    nnz_indices: Optional[torch.Tensor] = None,
):
    """skyrl/backends/skyrl_train/workers/model_wrapper.py:291, 333-393 on given logits ([B,S,V], or [1,nnz,V] with
    ``nnz_indices`` = flat positions of the real tokens): logits / temperature, log-prob of the stream rolled left by one
    (torch_utils.py:169-176: log_softmax + gather), entropy (masked by the attention mask only without packing), padding
    put back as zeros, action slice ``[:, -num_actions-1:-1]``.  Returns ``(action_log_probs, entropy [B,S])``."""
    batch, seqlen = sequences.shape
    tokens = sequences if nnz_indices is None else sequences.reshape(-1)[nnz_indices][None]
    rolled = torch.roll(tokens, shifts=-1, dims=1)
    z = logits / temperature
    log_probs = torch.log_softmax(z, dim=-1).gather(-1, rolled.unsqueeze(-1)).squeeze(-1)
    entropy = chunked_entropy_from_logits(z, None if nnz_indices is not None else attention_mask)
    if nnz_indices is not None:
        def pad(v):
            out = torch.zeros(batch * seqlen, dtype=v.dtype)
            out[nnz_indices] = v.reshape(-1)
            return out.view(batch, seqlen)
        log_probs, entropy = pad(log_probs), pad(entropy)
    return log_probs[:, -num_actions - 1:-1], entropy


def actor_loss(
    log_probs: torch.Tensor,
    old_log_probs: torch.Tensor,
    advantages: torch.Tensor,
    loss_mask: Optional[torch.Tensor],
    eps_clip_low: float,
    eps_clip_high: float,
    policy_scale: float = 1.0,
    term_scale: float = 1.0,
    base_log_probs: Optional[torch.Tensor] = None,
    kl_estimator_type: str = "k3",
    kl_coef: float = 0.0,
    entropy: Optional[torch.Tensor] = None,
    entropy_coef: float = 0.0,
):
    """The per-micro-batch loss the policy worker back-propagates (skyrl/backends/skyrl_train/workers/worker.py:989-1089):
    ``policy_loss * grad_sum_correction_factor + (kl_loss * kl_loss_coef - entropy * entropy_loss_coef) * microbatch_weight``
    with ``kl_loss = masked_mean(compute_approx_kl(...), loss_mask, dim=-1).mean()`` and ``entropy = masked_mean(entropy_BS,
    loss_mask)``.  Policy loss type "regular".  Returns ``(loss, policy_loss, kl, entropy_mean)``."""
    policy, _ = ppo_policy_loss(log_probs, old_log_probs, advantages, eps_clip_low, eps_clip_high, loss_mask=loss_mask)
    kl = approx_kl_loss(log_probs, base_log_probs, loss_mask, kl_estimator_type) if base_log_probs is not None else torch.zeros(())
    ent = masked_mean(entropy, loss_mask) if entropy is not None else torch.zeros(())
    return policy * policy_scale + (kl * kl_coef - ent * entropy_coef) * term_scale, policy, kl, ent


# ----------------------------------------------------------------------------------------------------------------------
# Multi-token-prediction draft loss: soft cross-entropy against the policy's own next-token distribution
# ----------------------------------------------------------------------------------------------------------------------
MTP = "skyrl/backends/skyrl_train/mtp/soft_ce.py"


def build_teacher_logits(main_logits: torch.Tensor, mtp_layer_number: int = 0) -> torch.Tensor:
    """mtp/soft_ce.py:22-34: the policy's logits rolled left by depth + 1 along the sequence, detached."""
    return torch.roll(main_logits.detach(), shifts=-(mtp_layer_number + 1), dims=1)


def shift_mask_for_mtp(mask: torch.Tensor, mtp_layer_number: int = 0, cu_seqlens=None) -> torch.Tensor:
    """mtp/soft_ce.py:37-79: the mask rolled like the teacher with the wrapped tail zeroed, AND-ed with the source mask;
    with ``cu_seqlens`` the roll is done segment by segment and each segment's tail is zeroed."""
    shift = mtp_layer_number + 1
    if cu_seqlens is None:
        rolled = torch.roll(mask, shifts=-shift, dims=1)
        rolled[:, -shift:] = 0
        return mask * rolled
    bounds = [int(b) for b in (cu_seqlens.tolist() if torch.is_tensor(cu_seqlens) else cu_seqlens)]
    rolled = torch.zeros_like(mask)
    for start, end in zip(bounds[:-1], bounds[1:]):
        if end - start <= 0:
            continue
        seg = torch.roll(mask[:, start:end], shifts=-shift, dims=1)
        if shift < end - start:
            seg[:, -shift:] = 0
        else:
            seg.zero_()
        rolled[:, start:end] = seg
    return mask * rolled


def soft_ce_per_token(student_logits: torch.Tensor, teacher_logits: torch.Tensor) -> torch.Tensor:
    """mtp/soft_ce.py:230-233 (and :137-143 for the vocabulary-parallel form on one shard):
    ``-sum_v softmax(teacher)_v log_softmax(student)_v`` in fp32 or wider."""
    up = torch.float64 if student_logits.dtype == torch.float64 else torch.float32
    return -(torch.softmax(teacher_logits.to(up), dim=-1) * torch.log_softmax(student_logits.to(up), dim=-1)).sum(dim=-1)


def draft_soft_ce(student_logits, teacher_logits, mask, global_normalization_factor=None) -> torch.Tensor:
    """mtp/soft_ce.py:200-240 with the reduction of :154-159: masked mean over the local mask count, or the masked sum over
    ``clamp(global_normalization_factor, min=1)``.  Sequence chunking (:162-197) does not change the value."""
    assert not teacher_logits.requires_grad, "MTP draft loss: teacher_logits must be detached"
    per_token = soft_ce_per_token(student_logits, teacher_logits)
    if global_normalization_factor is not None:
        return (per_token * mask).sum() / global_normalization_factor.clamp(min=1.0)
    return masked_mean(per_token, mask)


def draft_soft_ce_from_hidden(student_hidden, teacher_hidden, weight, mask, mtp_layer_number=0, global_normalization_factor=None):
    """The call chain around it: both hidden states through the shared, detached output layer (mtp/adapter.py:51-64), the
    teacher rolled to the draft depth, then ``draft_soft_ce`` (megatron_model_wrapper.py:766-775)."""
    w = weight.detach()
    student_logits = student_hidden @ w.t()
    teacher_logits = build_teacher_logits(teacher_hidden.detach() @ w.t(), mtp_layer_number)
    return draft_soft_ce(student_logits, teacher_logits, mask, global_normalization_factor)


def soft_ce_topk_per_token(student_logits: torch.Tensor, teacher_logits: torch.Tensor, k: int, roll_shift: int = 0):
    """mtp/soft_ce.py:258-305 (``_VocabParallelTopkSoftCE.forward`` with a group of one): the teacher's ``min(k, V)`` largest
    logits per position, the small ``[B, S, k]`` lists rolled left by ``roll_shift``, the student's logits gathered at those
    columns, both softmaxes over the k columns only.  Returns ``(per_token_loss, q_student, p_teacher, columns)``; autograd
    differentiates the loss through the gather."""
    up = torch.float64 if student_logits.dtype == torch.float64 else torch.float32
    k_eff = min(int(k), teacher_logits.shape[-1])
    t_vals, t_idx = teacher_logits.detach().topk(k_eff, dim=-1)
    if roll_shift:
        t_vals = torch.roll(t_vals, shifts=-int(roll_shift), dims=1)
        t_idx = torch.roll(t_idx, shifts=-int(roll_shift), dims=1)
    t_vals = t_vals.to(up)
    s_vals = student_logits.gather(-1, t_idx).to(up)
    t_exp = (t_vals - t_vals.max(dim=-1, keepdim=True).values).exp()
    t_p = t_exp / t_exp.sum(dim=-1, keepdim=True)
    s_shift = s_vals - s_vals.max(dim=-1, keepdim=True).values
    s_denom = s_shift.exp().sum(dim=-1, keepdim=True)
    q_s = s_shift.exp() / s_denom
    s_logp = s_shift - s_denom.log()
    return -(t_p * s_logp).sum(dim=-1), q_s, t_p, t_idx


def soft_ce_topk_backward(q_student, p_teacher, columns, grad_output, vocab_size: int) -> torch.Tensor:
    """mtp/soft_ce.py:307-315: ``(softmax(student) - softmax(teacher)) * grad`` scattered to the k columns, zero elsewhere."""
    grad_topk = (q_student - p_teacher) * grad_output.unsqueeze(-1)
    grad = torch.zeros(*columns.shape[:-1], vocab_size, dtype=grad_topk.dtype)
    grad.scatter_(-1, columns, grad_topk)
    return grad


def draft_soft_ce_topk(student_logits, teacher_logits, mask, k: int, global_normalization_factor=None, roll_shift: int = 0):
    """mtp/soft_ce.py:318-341 with the reduction of :154-159."""
    assert not teacher_logits.requires_grad, "MTP draft loss: teacher_logits must be detached"
    per_token = soft_ce_topk_per_token(student_logits, teacher_logits, k, roll_shift)[0]
    if global_normalization_factor is not None:
        return (per_token * mask).sum() / global_normalization_factor.clamp(min=1.0)
    return masked_mean(per_token, mask)


def draft_soft_ce_topk_from_hidden(student_hidden, teacher_hidden, weight, mask, k: int, global_normalization_factor=None,
                                   roll_shift: int = 0):
    """Both hidden states through the shared, detached output layer (mtp/adapter.py:51-64), the teacher un-rolled, then
    ``draft_soft_ce_topk`` with the MTP depth as ``roll_shift`` (megatron_model_wrapper.py passes ``mtp_layer_number + 1``)."""
    w = weight.detach()
    return draft_soft_ce_topk(student_hidden @ w.t(), teacher_hidden.detach() @ w.t(), mask, k, global_normalization_factor,
                              roll_shift)


# ----------------------------------------------------------------------------------------------------------------------
# Logits-input functions: the FSDP worker's log-probabilities and the Megatron path's materialised-logits autograd functions
# ----------------------------------------------------------------------------------------------------------------------
def logprobs_from_logits_v2(logits: torch.Tensor, labels: torch.Tensor) -> torch.Tensor:
    """skyrl/backends/skyrl_train/utils/torch_utils.py:156-177: fp32 / fp64 logits -> gathered logit minus ``logsumexp`` row by
    row; bf16 logits -> per-row ``log_softmax`` + ``gather`` (in bf16)."""
    if logits.dtype in (torch.float32, torch.float64):
        picked = torch.gather(logits, dim=-1, index=labels.unsqueeze(-1)).squeeze(-1)
        return picked - torch.stack([torch.logsumexp(row, dim=-1) for row in logits])
    rows = [torch.log_softmax(r, dim=-1).gather(dim=-1, index=y.unsqueeze(-1)).squeeze(-1) for r, y in zip(logits, labels)]
    return torch.stack(rows)


def distributed_logprob_forward(logits: torch.Tensor, target: torch.Tensor, vocab_start: int, vocab_end: int):
    """MU:73-106 (``DistributedLogprob.forward``) on one shard: fp32 (or wider) copy of the logits, a1's log-softmax, gather at
    the re-based target, 0 for targets outside the shard.  Returns ``(logprobs, softmax, target_mask, masked_target)``."""
    target_mask, masked_target = _mask_targets(target, vocab_start, vocab_end)
    wide = logits.to(torch.float64 if logits.dtype == torch.float64 else torch.float32)
    log_probs = distributed_log_softmax(wide)
    softmax = log_probs.exp()
    picked = torch.gather(log_probs, -1, masked_target.unsqueeze(-1)).squeeze(-1)
    picked[target_mask] = 0.0
    return picked, softmax, target_mask, masked_target


def distributed_logprob_backward(softmax: torch.Tensor, target_mask: torch.Tensor, masked_target: torch.Tensor,
                                 grad_output: torch.Tensor) -> torch.Tensor:
    """MU:108-137 (``DistributedLogprob.backward``): ``(onehot * in_shard - softmax) * grad``."""
    V = softmax.size(-1)
    is_chosen = (~target_mask).unsqueeze(-1) * torch.nn.functional.one_hot(masked_target, num_classes=V)
    return (is_chosen.to(softmax.dtype) - softmax) * grad_output.unsqueeze(-1)


# ----------------------------------------------------------------------------------------------------------------------
# Off-policy correction from the rollout engine's log-probabilities
# ----------------------------------------------------------------------------------------------------------------------
OPC = "skyrl/backends/skyrl_train/utils/off_policy_correction_utils.py"


def _cfg(cfg, name):
    return cfg.get(name) if isinstance(cfg, dict) else getattr(cfg, name, None)


def off_policy_correction(old_log_probs: torch.Tensor, rollout_logprobs: torch.Tensor, loss_mask: torch.Tensor, cfg):
    """OPC:257-348 with the helpers it calls (:24-254), in its order: is-ratio metrics on the incoming mask; outlier rows
    (any unmasked token's ratio beyond a threshold removes the row); the per-token hard mask (both bounds needed); the
    truncated importance weight, per token or per sequence, on the mask left so far; the sequence mask (geometric mean or
    product of the ratios outside its bounds removes the row).  Returns ``(tis_ratio | None, metrics, loss_mask)``."""
    tis_type, seq_metric = _cfg(cfg, "tis_ratio_type"), _cfg(cfg, "sequence_mask_metric")
    out_lo, out_hi = _cfg(cfg, "outlier_token_is_threshold_low"), _cfg(cfg, "outlier_token_is_threshold_high")
    tok_lo, tok_hi = _cfg(cfg, "token_mask_is_threshold_low"), _cfg(cfg, "token_mask_is_threshold_high")
    use_outlier, use_token = out_lo is not None or out_hi is not None, tok_lo is not None and tok_hi is not None
    if tis_type is None and seq_metric is None and not use_outlier and not use_token:
        return None, {}, loss_mask
    delta = old_log_probs - rollout_logprobs
    ratio = torch.clamp(delta, -20.0, 20.0).exp()
    rows = float(ratio.shape[0])
    m = {"is_ratio_mean": float(masked_mean(ratio, loss_mask)), "is_ratio_std": float((ratio * loss_mask).std()),
         "is_ratio_max": float((ratio * loss_mask).max()), "is_ratio_min": float((ratio * loss_mask).min())}
    mask = loss_mask
    if use_outlier:
        live = mask > 0
        over = (ratio > out_hi) & live if out_hi is not None else torch.zeros_like(live)
        under = (ratio < out_lo) & live if out_lo is not None else torch.zeros_like(live)
        ok = ((~over & ~under) | ~live).all(dim=-1, keepdim=True)
        m["outlier_seq_masked_ratio"] = float((~ok).sum() / rows)
        m["outlier_seq_over_high_ratio"] = float(over.any(dim=-1).sum() / rows)
        m["outlier_seq_under_low_ratio"] = float(under.any(dim=-1).sum() / rows)
        mask = mask * ok.to(mask.dtype)
    if use_token:
        inside = (ratio >= tok_lo) & (ratio <= tok_hi)
        m["token_mask_ratio"] = float(((~inside) & (mask > 0)).sum() / (mask > 0).sum().clamp(min=1))
        mask = mask * (inside | (mask == 0)).to(mask.dtype)
    tis = None
    if tis_type == "token":
        cap = _cfg(cfg, "token_tis_ratio_clip_high")
        m["tis_token_clip_high_ratio"] = float(((ratio > cap) & (mask > 0)).sum() / (mask > 0).sum().clamp(min=1))
        tis = torch.clamp(ratio, max=cap)
    elif tis_type == "sequence":
        cap = _cfg(cfg, "sequence_tis_ratio_clip_high")
        seq = torch.clamp((delta * mask).sum(dim=-1, keepdim=True), -20.0, 20.0).exp()
        m["tis_seq_clip_high_ratio"] = float((seq > cap).sum() / rows)
        tis = torch.clamp(seq, max=cap)
    elif tis_type is not None:
        raise ValueError(f"Unknown tis_ratio_type: {tis_type}")
    if seq_metric in ("geometric", "product"):
        total = (delta * mask).sum(dim=-1, keepdim=True)
        if seq_metric == "geometric":
            value = torch.clamp(total / mask.sum(dim=-1, keepdim=True).clamp(min=1.0), -20.0, 20.0).exp()
            lo, hi, name = _cfg(cfg, "geo_mask_low"), _cfg(cfg, "geo_mask_high"), "geo_sequence_mask"
        else:
            value = torch.clamp(total, -20.0, 20.0).exp()
            lo, hi, name = _cfg(cfg, "product_mask_low"), _cfg(cfg, "product_mask_high"), "product_sequence_mask"
        over, under = value > hi, value < lo
        m[f"{name}_masked_ratio"] = float((over | under).sum() / rows)
        m[f"{name}_over_high_ratio"] = float(over.sum() / rows)
        m[f"{name}_under_low_ratio"] = float(under.sum() / rows)
        mask = mask * (~over & ~under).to(mask.dtype)
    elif seq_metric is not None:
        raise ValueError(f"Unknown sequence_mask_metric: {seq_metric}")
    return tis, m, mask


def apply_off_policy_correction(loss, old_log_probs, rollout_logprobs, loss_mask, cfg):
    """OPC:351-391: the per-token loss times the weight (when there is one), the new mask, the metrics; nothing without
    rollout log-probabilities."""
    if rollout_logprobs is None:
        return loss, loss_mask, {}
    tis, metrics, mask = off_policy_correction(old_log_probs, rollout_logprobs, loss_mask, cfg)
    return (loss if tis is None else loss * tis), mask, metrics


def minibatch_rollout_logprob_diff_metrics(action_log_probs, rollout_logprobs, loss_mask):
    """workers/worker_utils.py:34-58: nothing without rollout log-probabilities; else the masked mean of the absolute
    difference and of its square, and the largest and smallest masked absolute difference."""
    if rollout_logprobs is None:
        return {}
    diff = (action_log_probs - rollout_logprobs).abs()
    weighted = diff if loss_mask is None else diff * loss_mask
    prefix = "minibatch_rollout_logprobs_abs_diff"
    return {f"{prefix}_mean": float(masked_mean(diff, loss_mask)), f"{prefix}_sq_mean": float(masked_mean(diff * diff, loss_mask)),
            f"{prefix}_max": float(weighted.max()), f"{prefix}_min": float(weighted.min())}
