"""Pins the CPU oracle (oracle/lmhead_oracle.py) without a GPU.

Each check compares an oracle function with something that does not share its code: a torch library routine in fp64,
autograd, central finite differences, a closed form, brute force, or the committed golden vectors (tests/golden/*.npz, made
by tests/golden/make_golden.py from library routines only).  The cases and tolerances follow the reference's own tests of this
path (tests/backends/skyrl_train/gpu/gpu_ci/megatron/test_fused_linear_logprob.py:89-141,
tests/backends/skyrl_train/distributed/test_vocab_entropy_chunking.py:34-51,
tests/backends/skyrl_train/utils/test_torch_utils.py:31-35).
"""

import glob
import math
import os

import numpy as np
import pytest
import torch
from hypothesis import given, settings
from hypothesis import strategies as st

from oracle import lmhead_oracle as O

GOLDEN = sorted(glob.glob(os.path.join(os.path.dirname(__file__), "golden", "*.npz")))


def load_golden(path):
    z = np.load(path, allow_pickle=False)
    d = {k: torch.from_numpy(z[k]) for k in z.files if k != "temperature"}
    d["hidden"] = d.pop("hidden_bits").view(torch.bfloat16)
    d["weight"] = d.pop("weight_bits").view(torch.bfloat16)
    d["temperature"] = float(z["temperature"])
    return d


def _inputs(B, S, H, V, seed=0, dtype=torch.float64):
    g = torch.Generator().manual_seed(seed)
    hidden = torch.randn(B, S, H, generator=g, dtype=torch.float64).to(dtype)
    weight = (torch.randn(V, H, generator=g, dtype=torch.float64) * 3 / H**0.5).to(dtype)
    target = torch.randint(0, V, (B, S), generator=g)
    return hidden, weight, target


def _materialised(hidden, weight, target, vs, ve, grad=None):
    """Library statement: log_softmax + gather on materialised fp64 logits; out-of-shard targets -> 0 / keep -p*g."""
    h = hidden.double().requires_grad_(True)
    w = weight.double().requires_grad_(True)
    z = h @ w.t()
    inside = (target >= vs) & (target < ve)
    safe = (target - vs).clamp(0, w.shape[0] - 1)
    lp = torch.log_softmax(z, -1).gather(-1, safe[..., None])[..., 0].masked_fill(~inside, 0.0)
    if grad is None:
        return lp.detach()
    lp_g = z.gather(-1, safe[..., None])[..., 0] * inside - torch.logsumexp(z, -1)
    (lp_g * grad.double()).sum().backward()
    return lp.detach(), h.grad, w.grad


# ---------------------------------------------------------------------------------------------------------------------
# forward
# ---------------------------------------------------------------------------------------------------------------------
@pytest.mark.parametrize("chunk", [1, 7, 64, 512])
@pytest.mark.parametrize("oov", [False, True])
def test_chunked_forward_matches_log_softmax(chunk, oov):
    B, S, H, V = 4, 32, 64, 512
    hidden, weight, target = _inputs(B, S, H, V, seed=1)
    vs, ve = (0, V)
    if oov:  # a shard that owns only the middle of the id range
        vs, ve = 100, 100 + V
        target = torch.randint(0, V + 200, (B, S), generator=torch.Generator().manual_seed(5))
    got = O.fused_chunked_logprob_forward(hidden, weight, target, vs, ve, chunk)
    want = _materialised(hidden, weight, target, vs, ve)
    assert got.dtype == torch.float32
    torch.testing.assert_close(got.double(), want, atol=1e-5, rtol=1e-5)


def test_zero_weight_known_answer():
    # uniform logits: logprob = -ln V, entropy = ln V
    T, H, V = 5, 64, 4
    hidden = torch.randn(1, T, H, dtype=torch.float64)
    weight = torch.zeros(V, H, dtype=torch.float64)
    target = torch.randint(0, V, (1, T))
    lp = O.fused_chunked_logprob_forward(hidden, weight, target, 0, V, 2)
    ent = O.fused_entropy_from_hidden(hidden, weight, 3)
    lp2, ent2, *_ = O.linear_cross_entropy_forward(hidden[0], weight, target[0], 1.0, vocab_per_split=3)
    for x in (lp, lp2):
        torch.testing.assert_close(x.double().flatten(), torch.full((T,), -math.log(V), dtype=torch.float64), atol=1e-6, rtol=0)
    for x in (ent, ent2):
        torch.testing.assert_close(x.double().flatten(), torch.full((T,), math.log(V), dtype=torch.float64), atol=1e-6, rtol=0)


def test_one_dominant_logit_limits():
    T, H, V = 3, 64, 50
    hidden = torch.zeros(T, H, dtype=torch.float64)
    hidden[:, 0] = 1.0
    weight = torch.zeros(V, H, dtype=torch.float64)
    weight[7, 0] = 200.0
    labels = torch.full((T,), 7)
    lp, ent, *_ = O.linear_cross_entropy_forward(hidden, weight, labels, 1.0, vocab_per_split=16)
    assert lp.abs().max() < 1e-12 and ent.abs().max() < 1e-12


def test_probabilities_sum_to_one_brute_force():
    T, H, V = 3, 64, 37
    hidden, weight, _ = _inputs(1, T, H, V, seed=3)
    total_a = torch.zeros(T, dtype=torch.float64)
    total_b = torch.zeros(T, dtype=torch.float64)
    for y in range(V):
        lab = torch.full((1, T), y)
        total_a += O.fused_chunked_logprob_forward(hidden, weight, lab, 0, V, 2)[0].double().exp()
        total_b += O.linear_cross_entropy_forward(hidden[0], weight, lab[0], 0.7, vocab_per_split=10)[0].exp()
    torch.testing.assert_close(total_a, torch.ones(T, dtype=torch.float64), atol=1e-5, rtol=0)
    torch.testing.assert_close(total_b, torch.ones(T, dtype=torch.float64), atol=1e-10, rtol=0)


def test_shift_invariance():
    # an extra hidden feature that adds the same constant to every logit changes neither output
    T, H, V = 6, 64, 90
    hidden, weight, target = _inputs(1, T, H, V, seed=4)
    h2 = torch.cat([hidden, torch.ones(1, T, 64, dtype=torch.float64)], -1)
    w2 = torch.cat([weight, torch.full((V, 64), 0.25, dtype=torch.float64)], -1)
    a = O.linear_cross_entropy_forward(hidden[0], weight, target[0], 0.8, 32)
    b = O.linear_cross_entropy_forward(h2[0], w2, target[0], 0.8, 32)
    torch.testing.assert_close(a[0], b[0], atol=1e-9, rtol=0)
    torch.testing.assert_close(a[1], b[1], atol=1e-9, rtol=0)


@pytest.mark.parametrize("temperature", [1.0, 0.6, 1.7])
def test_verl_forward_matches_library(temperature):
    T, H, V = 33, 64, 700
    hidden, weight, target = _inputs(1, T, H, V, seed=6)
    lp, ent, mx, acc, eb = O.linear_cross_entropy_forward(hidden[0], weight, target[0], temperature, vocab_per_split=128)
    z = (hidden[0] @ weight.t()) / temperature
    lsm = torch.log_softmax(z, -1)
    torch.testing.assert_close(lp, lsm.gather(-1, target[0][:, None])[:, 0], atol=1e-10, rtol=0)
    torch.testing.assert_close(ent, -(lsm.exp() * lsm).sum(-1), atol=1e-10, rtol=0)
    torch.testing.assert_close(mx + acc.log(), torch.logsumexp(z, -1), atol=1e-10, rtol=0)
    torch.testing.assert_close(eb, (lsm.exp() * z).sum(-1), atol=1e-10, rtol=0)
    assert (ent >= 0).all() and (ent <= math.log(V) + 1e-9).all() and (lp <= 0).all()


def test_entropy_metric_matches_closed_form_and_temperature():
    B, S, H, V = 2, 19, 64, 300
    hidden, weight, _ = _inputs(B, S, H, V, seed=7)
    for chunk in (None, 1, 5, 64):
        got = O.fused_entropy_from_hidden(hidden, weight, chunk, temperature=0.6)
        lsm = torch.log_softmax((hidden @ weight.t()) / 0.6, -1)
        torch.testing.assert_close(got.double(), -(lsm.exp() * lsm).sum(-1), atol=2e-5, rtol=1e-5)


@settings(max_examples=40, deadline=None)
@given(st.integers(2, 60), st.lists(st.integers(1, 59), min_size=0, max_size=6), st.integers(0, 10_000))
def test_split_merge_equals_one_shot(V, cuts, seed):
    g = torch.Generator().manual_seed(seed)
    z = torch.randn(4, V, generator=g, dtype=torch.float64) * 6 - 3
    z[1] -= 500.0  # a row of very negative logits: the merge must not lose it (the reference kernel's max starts at 0)
    bounds = sorted({0, V, *[c for c in cuts if c < V]})
    parts = [O.split_statistics(z[:, a:b]) for a, b in zip(bounds[:-1], bounds[1:])]
    m, s, e = O.merge_split_statistics(*[torch.stack(x, 1) for x in zip(*parts)])
    torch.testing.assert_close(m + s.log(), torch.logsumexp(z, -1), atol=1e-10, rtol=0)
    p = torch.softmax(z, -1)
    torch.testing.assert_close(e / s, (p * z).sum(-1), atol=1e-9, rtol=1e-12)


# ---------------------------------------------------------------------------------------------------------------------
# backward
# ---------------------------------------------------------------------------------------------------------------------
@pytest.mark.parametrize("chunk", [1, 7, 64, 512])
@pytest.mark.parametrize("oov", [False, True])
@pytest.mark.parametrize("dtypes", [("bf16", "bf16"), ("bf16", "fp32"), ("fp32", "fp32")])
def test_chunked_backward_matches_autograd(chunk, oov, dtypes):
    # the reference's own case and tolerances: test_fused_linear_logprob.py:57-59, 89-119
    B, S, H, V = 4, 32, 64, 512
    dt = {"bf16": torch.bfloat16, "fp32": torch.float32}
    hidden, weight, target = _inputs(B, S, H, V, seed=8)
    hidden, weight = hidden.to(dt[dtypes[0]]), weight.to(dt[dtypes[1]])
    vs, ve = 0, V
    if oov:
        vs, ve = 64, 64 + V
        target = torch.randint(0, V + 128, (B, S), generator=torch.Generator().manual_seed(9))
    grad = torch.linspace(0.5, 1.5, B * S).reshape(B, S)
    gh, gw = O.fused_chunked_logprob_backward(hidden, weight, target, vs, ve, chunk, grad)
    _, rh, rw = _materialised(hidden, weight, target, vs, ve, grad)
    assert gh.dtype == hidden.dtype and gw.dtype == torch.float32
    gw_tol = 4e-2 if weight.dtype == torch.bfloat16 else 2e-3
    gh_tol = 2e-2 if hidden.dtype == torch.bfloat16 else 2e-3  # grad_hidden is returned in bf16 when hidden is bf16
    torch.testing.assert_close(gh.double(), rh, atol=gh_tol, rtol=gh_tol)
    torch.testing.assert_close(gw.double(), rw, atol=gw_tol, rtol=gw_tol)


@pytest.mark.parametrize("case", ["S1", "all_in", "all_oov", "V8"])
def test_chunked_edge_cases(case):
    # test_fused_linear_logprob.py:122-141
    B, S, H, V = (2, 1, 64, 64) if case == "S1" else (2, 5, 64, 8) if case == "V8" else (2, 9, 64, 128)
    hidden, weight, target = _inputs(B, S, H, V, seed=10)
    vs, ve = (1000, 1000 + V) if case == "all_oov" else (0, V)
    grad = torch.ones(B, S)
    lp = O.fused_chunked_logprob_forward(hidden, weight, target, vs, ve, 4)
    gh, gw = O.fused_chunked_logprob_backward(hidden, weight, target, vs, ve, 4, grad)
    want, rh, rw = _materialised(hidden, weight, target, vs, ve, grad)
    torch.testing.assert_close(lp.double(), want, atol=1e-5, rtol=1e-5)
    torch.testing.assert_close(gh.double(), rh, atol=1e-5, rtol=1e-5)
    torch.testing.assert_close(gw.double(), rw, atol=1e-5, rtol=1e-5)
    if case == "all_oov":
        assert (lp == 0).all() and gw.abs().max() > 0  # forward forced to 0, backward keeps -softmax * g


def _scalar_loss(h, w, labels, temperature, g, q):
    z = (h @ w.t()) / temperature
    lsm = torch.log_softmax(z, -1)
    inside = (labels >= 0) & (labels < w.shape[0])
    safe = labels.clamp(0, w.shape[0] - 1)
    lp = z.gather(-1, safe[:, None])[:, 0] * inside - torch.logsumexp(z, -1)
    ent = -(lsm.exp() * lsm).sum(-1)
    return (lp * g).sum() + (ent * q).sum()


@pytest.mark.parametrize("temperature", [1.0, 0.6])
def test_verl_backward_matches_autograd_and_finite_differences(temperature):
    T, H, V = 9, 64, 150
    hidden, weight, target = _inputs(1, T, H, V, seed=11)
    h, w, y = hidden[0], weight, target[0].clone()
    y[2] = O.OOV_LABEL_SENTINEL
    gen = torch.Generator().manual_seed(12)
    g = torch.randn(T, generator=gen, dtype=torch.float64)
    q = torch.randn(T, generator=gen, dtype=torch.float64)
    _, _, mx, acc, eb = O.linear_cross_entropy_forward(h, w, y, temperature, 64)
    dh, dw = O.linear_cross_entropy_backward(g, q, h, w, y, mx, acc, eb, temperature, vocab_per_split=40)
    ha, wa = h.clone().requires_grad_(True), w.clone().requires_grad_(True)
    _scalar_loss(ha, wa, y, temperature, g, q).backward()
    torch.testing.assert_close(dh, ha.grad, atol=1e-10, rtol=1e-9)
    torch.testing.assert_close(dw, wa.grad, atol=1e-10, rtol=1e-9)
    # central finite differences on a few coordinates (independent of autograd as well)
    eps = 1e-6
    for (i, j) in [(0, 0), (3, 17), (8, 63)]:
        hp, hm = h.clone(), h.clone()
        hp[i, j] += eps
        hm[i, j] -= eps
        fd = (_scalar_loss(hp, w, y, temperature, g, q) - _scalar_loss(hm, w, y, temperature, g, q)) / (2 * eps)
        assert abs(fd - dh[i, j]) < 1e-6 * max(1.0, abs(fd))
    for (i, j) in [(int(y[0]), 5), (77, 0)]:
        wp, wm = w.clone(), w.clone()
        wp[i, j] += eps
        wm[i, j] -= eps
        fd = (_scalar_loss(h, wp, y, temperature, g, q) - _scalar_loss(h, wm, y, temperature, g, q)) / (2 * eps)
        assert abs(fd - dw[i, j]) < 1e-6 * max(1.0, abs(fd))


def test_d_logits_invariants():
    T, V = 7, 61
    gen = torch.Generator().manual_seed(13)
    z = torch.randn(T, V, generator=gen, dtype=torch.float64) * 3
    y = torch.randint(0, V, (T,), generator=gen)
    y[3] = O.OOV_LABEL_SENTINEL
    g, q = torch.randn(T, generator=gen, dtype=torch.float64), torch.randn(T, generator=gen, dtype=torch.float64)
    mx, s, e = O.split_statistics(z)
    eb = e / s
    zero = torch.zeros(T, dtype=torch.float64)
    d_lp = O.d_logits_formula(z, mx, s, eb, y, g, zero, 1.0)
    d_en = O.d_logits_formula(z, mx, s, eb, y, zero, q, 1.0)
    d_all = O.d_logits_formula(z, mx, s, eb, y, g, q, 1.0)
    # rows sum to 0 for in-vocab labels (softmax Jacobian annihilates constants); the out-of-vocab row sums to -g
    rs = d_lp.sum(-1)
    assert rs[[0, 1, 2, 4, 5, 6]].abs().max() < 1e-12 and abs(rs[3] + g[3]) < 1e-12
    assert d_en.sum(-1).abs().max() < 1e-12
    torch.testing.assert_close(d_all, d_lp + d_en, atol=1e-14, rtol=0)  # linear in (g, q)
    torch.testing.assert_close(d_en, O.vocab_parallel_entropy_backward(z, q), atol=1e-12, rtol=0)
    # column windows agree with the full formula
    torch.testing.assert_close(O.d_logits_formula(z[:, 20:45], mx, s, eb, y, g, q, 1.0, vocab_offset=20), d_all[:, 20:45])


def test_entropy_backward_matches_autograd():
    z = (torch.randn(5, 40, dtype=torch.float64) * 2).requires_grad_(True)
    q = torch.randn(5, dtype=torch.float64)
    lsm = torch.log_softmax(z, -1)
    (-(lsm.exp() * lsm).sum(-1) * q).sum().backward()
    torch.testing.assert_close(O.vocab_parallel_entropy_backward(z.detach(), q), z.grad, atol=1e-12, rtol=0)


# ---------------------------------------------------------------------------------------------------------------------
# golden vectors
# ---------------------------------------------------------------------------------------------------------------------
@pytest.mark.parametrize("path", GOLDEN, ids=[os.path.basename(p)[:-4] for p in GOLDEN])
def test_oracle_against_golden_vectors(path):
    d = load_golden(path)
    t = d["temperature"]
    ex = O.exact_fwd_bwd(d["hidden"], d["weight"], d["labels"], t, d["dlogprobs"], d["dentropy"], vocab_per_split=100)
    torch.testing.assert_close(ex["logprobs"], d["logprobs"], atol=1e-9, rtol=0)
    torch.testing.assert_close(ex["entropy"], d["entropy"], atol=1e-9, rtol=0)
    torch.testing.assert_close(ex["d_hidden"].float(), d["d_hidden"], atol=1e-5, rtol=1e-5)
    torch.testing.assert_close(ex["d_weight"].float(), d["d_weight"], atol=1e-5, rtol=1e-5)
    # The bf16 "reference-faithful" path rounds every logit to bf16 (matmul output dtype, model_utils.py:331-333): a target
    # logit in [8, 16) moves by up to 2^-5 = 0.031, so its distance to the exact value is bounded by that, not by 2e-2.
    # Run with fp32 operands the same code is exact; that is the comparator the GPU parity tests use for the 2e-2 bound.
    rf = O.reference_faithful_fwd_bwd(d["hidden"], d["weight"], d["labels"], t, d["dlogprobs"], chunk_size=16)
    assert (rf["logprobs"].double() - d["logprobs"]).abs().max() < 2 ** -4
    assert (rf["entropy"].double() - d["entropy"]).abs().max() < 5e-2  # entropies here are O(1): absolute bound
    rf32 = O.reference_faithful_fwd_bwd(d["hidden"].float(), d["weight"].float(), d["labels"], t, d["dlogprobs"], chunk_size=16)
    assert (rf32["logprobs"].double() - d["logprobs"]).abs().max() < 1e-4
    assert ((rf32["entropy"].double() - d["entropy"]).abs() / d["entropy"].abs().clamp_min(1e-3)).max() < 1e-4
    assert len(GOLDEN) >= 4


# ---------------------------------------------------------------------------------------------------------------------
# callers: roll, packing
# ---------------------------------------------------------------------------------------------------------------------
def test_roll_and_drop_last():
    B, S, H, V = 2, 11, 64, 97
    hidden, weight, tokens = _inputs(B, S, H, V, seed=14)
    got = O.from_parallel_hidden_to_logprobs(hidden, weight, tokens, chunk_size=4, temperature=0.9)
    lsm = torch.log_softmax((hidden @ weight.t()) / 0.9, -1)
    want = torch.stack([torch.stack([lsm[b, s, tokens[b, s + 1]] for s in range(S - 1)]) for b in range(B)])
    assert got.shape == (B, S - 1)
    torch.testing.assert_close(got.double(), want, atol=1e-5, rtol=1e-5)


def test_packed_roll_and_scatter_back_brute_force():
    lens = [5, 1, 9, 3]
    cu = torch.tensor([0, 5, 6, 15, 18])
    T = 18
    target = torch.arange(100, 100 + T)
    rolled = O.packed_rolled_targets(target, cu)
    want = []
    for i, n in enumerate(lens):
        seq = target[cu[i] : cu[i] + n]
        want.append(seq.roll(-1))
    assert torch.equal(rolled, torch.cat(want))
    probs = torch.arange(T, dtype=torch.float32) + 1
    L = 7
    out = O.packed_scatter_back(probs, cu, len(lens), L)
    ref = torch.zeros(len(lens), L - 1)
    for i, n in enumerate(lens):
        for o in range(n - 1):
            if o < L - 1:
                ref[i, o] = probs[cu[i] + o]
    assert torch.equal(out, ref)


def test_packed_roll_skips_empty_sequences():
    cu = torch.tensor([0, 0, 3, 3, 4, 9])
    target = torch.arange(50, 59)
    want = torch.cat([target[0:3].roll(-1), target[3:4], target[4:9].roll(-1)])
    assert torch.equal(O.packed_rolled_targets(target, cu), want)


def test_packed_scatter_back_sub_sequences_brute_force():
    # Two output rows; row 0 holds segments of true lengths 3 and 4 padded to 4 and 6, row 1 one segment of 5 padded to 8.
    sub = [[3, 4], [5]]
    cu = torch.tensor([0, 4, 10, 18])
    probs = torch.arange(18, dtype=torch.float32) + 1
    for L in (12, 8, 6):
        out = O.packed_scatter_back(probs, cu, 2, L, sub_seq_lengths=sub)
        ref = torch.zeros(2, L - 1)
        placements = [(0, 0, 0, 3), (0, 4, 4, 4), (1, 0, 10, 5)]  # (row, first column, first packed token, true length)
        for row, col0, tok0, n in placements:
            for o in range(n - 1):
                if col0 + o < L - 1:
                    ref[row, col0 + o] = probs[tok0 + o]
        assert torch.equal(out, ref), L
    with pytest.raises(ValueError):
        O.packed_scatter_back(probs, cu, 2, 12, sub_seq_lengths=[[3], [5]])
    with pytest.raises(ValueError):
        O.packed_scatter_back(probs, cu, 2, 12, sub_seq_lengths=[[3, 4], [5, 1]])


def test_packed_scatter_back_attention_mask_brute_force():
    # Rows with left padding, interior padding, a single real token, no real token, and a real token in the last column.
    am = torch.tensor([
        [0, 0, 1, 1, 1, 1, 0, 0],
        [1, 0, 1, 1, 0, 1, 1, 0],
        [0, 0, 0, 1, 0, 0, 0, 0],
        [0, 0, 0, 0, 0, 0, 0, 0],
        [1, 1, 1, 0, 0, 0, 0, 1],
    ])
    real = am.sum(1).tolist()
    padded = [6, 5, 2, 1, 4]  # packed segments may be longer than the real lengths
    cu = torch.tensor([0] + list(torch.tensor(padded).cumsum(0)))
    T = int(cu[-1])
    probs = torch.arange(T, dtype=torch.float32) + 1
    out = O.packed_scatter_back(probs, cu, 5, 8, attention_mask=am)
    ref = torch.zeros(5, 7)
    for b in range(5):
        positions = [c for c in range(8) if am[b, c]]
        for j, c in enumerate(positions[:-1]):  # every real token but the last of its row
            ref[b, c] = probs[cu[b] + j]
    assert torch.equal(out, ref)
    assert [int((ref[b] != 0).sum()) for b in range(5)] == [max(n - 1, 0) for n in real]


# ----------------------------------------------------------------------------------------------------------------------
# PPO policy loss
# ----------------------------------------------------------------------------------------------------------------------
def _ppo(lp, old, adv, **kw):
    lp = torch.tensor(lp, dtype=torch.float64, requires_grad=True)
    loss, clip = O.ppo_policy_loss(lp, torch.tensor(old, dtype=torch.float64), torch.tensor(adv, dtype=torch.float64), 0.2, 0.2, **kw)
    loss.backward()
    return loss.item(), clip.item(), lp.grad.tolist()


def test_ppo_loss_hand_computed_branches():
    ln2, ln4, lnhalf = math.log(2.0), math.log(4.0), math.log(0.5)
    # ratio 1: nothing clips; loss = -A, gradient -A (both branches of the min agree)
    loss, clip, g = _ppo([0.3], [0.3], [1.5])
    assert loss == pytest.approx(-1.5) and clip == 0.0 and g == pytest.approx([-1.5])
    # ratio 2, A > 0: the clipped branch 1.2*A is the smaller one -> loss -1.2*A, no gradient, counted as clipped
    loss, clip, g = _ppo([ln2], [0.0], [2.0])
    assert loss == pytest.approx(-2.4) and clip == 1.0 and g == pytest.approx([0.0])
    # ratio 2, A < 0: the unclipped branch 2*A is the smaller one -> loss -2*A = 4, gradient -ratio*A = 4, not clipped
    loss, clip, g = _ppo([ln2], [0.0], [-2.0])
    assert loss == pytest.approx(4.0) and clip == 0.0 and g == pytest.approx([4.0])
    # ratio 0.5, A < 0: clipped low, 0.8*A < 0.5*A -> loss 1.6, no gradient
    loss, clip, g = _ppo([lnhalf], [0.0], [-2.0])
    assert loss == pytest.approx(1.6) and clip == 1.0 and g == pytest.approx([0.0])
    # ratio 0.5, A > 0: unclipped branch is smaller -> loss -1, gradient -ratio*A = -1
    loss, clip, g = _ppo([lnhalf], [0.0], [2.0])
    assert loss == pytest.approx(-1.0) and clip == 0.0 and g == pytest.approx([-1.0])
    # dual clip, A < 0: ratio 2 stays below c = 3 (unchanged), ratio 4 is capped at -A*c = 6 with no gradient
    loss, clip, g = _ppo([ln2], [0.0], [-2.0], dual_clip=True, clip_ratio_c=3.0)
    assert loss == pytest.approx(4.0) and g == pytest.approx([4.0])
    loss, clip, g = _ppo([ln4], [0.0], [-2.0], dual_clip=True, clip_ratio_c=3.0)
    assert loss == pytest.approx(6.0) and g == pytest.approx([0.0])
    # dual clip leaves A > 0 alone
    loss, clip, g = _ppo([lnhalf], [0.0], [2.0], dual_clip=True, clip_ratio_c=3.0)
    assert loss == pytest.approx(-1.0) and g == pytest.approx([-1.0])
    # the log-ratio is clamped to +-20 before exp: ratio e^20, and no gradient passes the clamp
    loss, clip, g = _ppo([25.0], [0.0], [-1.0])
    assert loss == pytest.approx(math.exp(20.0)) and g == pytest.approx([0.0])


def test_ppo_loss_mask_weight_and_clip_ratio_by_hand():
    lp = [math.log(2.0), 0.0, math.log(2.0), math.log(0.5)]
    adv = [1.0, 1.0, 1.0, -1.0]
    mask = torch.tensor([1.0, 1.0, 0.0, 1.0], dtype=torch.float64)
    weight = torch.tensor([0.5, 2.0, 7.0, 1.0], dtype=torch.float64)
    loss, clip, g = _ppo(lp, [0.0] * 4, adv, loss_mask=mask, loss_weight=weight)
    # tokens: clipped (-1.2 * 0.5), unclipped (-1 * 2), masked out, clipped low (0.8 * 1)
    assert loss == pytest.approx(-0.6 - 2.0 + 0.8)
    assert clip == pytest.approx(2.0 / 3.0)  # two of the three unmasked tokens are clipped
    assert g == pytest.approx([0.0, -2.0, 0.0, 0.0])
    _, clip_all, _ = _ppo(lp, [0.0] * 4, adv)
    assert clip_all == pytest.approx(3.0 / 4.0)  # without a mask: plain mean


@pytest.mark.parametrize("dual", [False, True])
def test_ppo_loss_gradient_matches_finite_differences(dual):
    gen = torch.Generator().manual_seed(11)
    n = 64
    lp = torch.randn(n, generator=gen, dtype=torch.float64) * 0.4
    old = torch.randn(n, generator=gen, dtype=torch.float64) * 0.4
    adv = torch.randn(n, generator=gen, dtype=torch.float64)
    mask = (torch.rand(n, generator=gen) > 0.3).double()
    w = torch.rand(n, generator=gen, dtype=torch.float64) + 0.5
    f = lambda x: O.ppo_policy_loss(x, old, adv, 0.2, 0.28, 3.0, dual, mask, w)[0]  # noqa: E731
    x = lp.clone().requires_grad_(True)
    f(x).backward()
    eps = 1e-6
    for i in range(n):
        d = torch.zeros(n, dtype=torch.float64)
        d[i] = eps
        fd = (f(lp + d) - f(lp - d)).item() / (2 * eps)
        assert x.grad[i].item() == pytest.approx(fd, abs=1e-6), f"token {i}"


# ----------------------------------------------------------------------------------------------------------------------
# the other per-token losses: cross entropy, importance sampling, approximate KL, masked mean
# ----------------------------------------------------------------------------------------------------------------------
def test_cross_entropy_and_importance_sampling_by_hand():
    lp = torch.tensor([-1.0, -2.0, -0.5, -3.0], dtype=torch.float64)
    mask = torch.tensor([1.0, 0.0, 1.0, 1.0], dtype=torch.float64)
    assert O.cross_entropy_loss(lp).item() == pytest.approx(6.5)
    assert O.cross_entropy_loss(lp, mask).item() == pytest.approx(4.5)
    old = lp - torch.tensor([math.log(2.0), 0.0, math.log(0.5), math.log(3.0)], dtype=torch.float64)   # ratios 2, 1, 1/2, 3
    adv = torch.tensor([1.0, -1.0, 4.0, -2.0], dtype=torch.float64)
    loss, ratio = O.importance_sampling_loss(lp, old, adv)
    assert loss.item() == pytest.approx(-(2 - 1 + 2 - 6)) and ratio.item() == pytest.approx(6.5 / 4)
    loss, ratio = O.importance_sampling_loss(lp, old, adv, mask)
    assert loss.item() == pytest.approx(-(2 + 2 - 6)) and ratio.item() == pytest.approx(5.5 / 3)
    # no clamp of the log-ratio: a difference of 30 gives e^30, which safe_exp_delta would have cut at e^20
    big, _ = O.importance_sampling_loss(torch.tensor([0.0]), torch.tensor([-30.0]), torch.tensor([1.0]))
    assert big.item() == pytest.approx(-math.exp(30.0), rel=1e-6)


def _grad(fn, lp):
    x = torch.tensor(lp, dtype=torch.float64, requires_grad=True)
    loss, stat = fn(x)
    loss.backward()
    return loss.item(), stat.item(), x.grad.tolist()


def _t(v):
    return torch.tensor(v, dtype=torch.float64)


def test_sapo_by_hand():
    sig = lambda u: 1.0 / (1.0 + math.exp(-u))  # noqa: E731
    # ratio 1: the gate is sigmoid(0) * 4 / tau = 2 / tau, whatever the sign of A picks
    loss, stat, g = _grad(lambda x: O.sapo_policy_loss(x, _t([0.3, 0.3]), _t([1.5, -1.5]), 1.0, 1.25), [0.3, 0.3])
    assert loss == pytest.approx(-(2.0 / 1.0) * 1.5 + (2.0 / 1.25) * 1.5) and stat == 0.0
    # d gate / d lp at ratio 1 = 4 s (1 - s) ratio = 1 for every tau: there SAPO moves like the plain surrogate -ratio*A
    assert g == pytest.approx([-1.5, 1.5])
    # ratio 2, A = 3 > 0 -> tau_pos = 0.5; ratio 1/2, A = -2 (A <= 0 -> tau_neg = 2); A = 0 takes tau_neg and gives 0
    loss, _, g = _grad(lambda x: O.sapo_policy_loss(x, _t([0.0, 0.0, 0.0]), _t([3.0, -2.0, 0.0]), 0.5, 2.0),
                       [math.log(2.0), math.log(0.5), 0.7])
    s1, s2 = sig(0.5 * 1.0), sig(2.0 * -0.5)
    assert loss == pytest.approx(-s1 * 8.0 * 3.0 + s2 * 2.0 * 2.0)
    assert g == pytest.approx([-4 * 3.0 * s1 * (1 - s1) * 2.0, 4 * 2.0 * s2 * (1 - s2) * 0.5, 0.0])
    # the log-ratio is clamped at 20 and passes no gradient beyond
    loss, _, g = _grad(lambda x: O.sapo_policy_loss(x, _t([0.0]), _t([1.0]), 1.0, 1.0), [25.0])
    assert loss == pytest.approx(-4.0) and g == pytest.approx([0.0])
    # mask: the masked sum
    loss, _, _ = _grad(lambda x: O.sapo_policy_loss(x, _t([0.0, 0.0]), _t([1.0, 1.0]), 1.0, 1.0, _t([0.0, 1.0])), [0.0, 0.0])
    assert loss == pytest.approx(-2.0)


def test_gspo_by_hand_and_single_token_rows_are_ppo():
    ln2 = math.log(2.0)
    # one row, log-ratios (ln 2, 0, 3 ln 2) -> mean = 4/3 ln 2, masked (1, 1, 0) -> mean = ln 2 / 2: ratio sqrt 2 for all
    lp, old, adv = [[ln2, 0.0, 3 * ln2]], _t([[0.0, 0.0, 0.0]]), _t([[1.0, -1.0, 5.0]])
    mask = _t([[1.0, 1.0, 0.0]])
    r = math.sqrt(2.0)
    loss, clip, g = _grad(lambda x: O.gspo_policy_loss(x, old, adv, 0.2, 0.5, mask), lp)
    # token 0: A > 0, ratio 1.414 inside [0.8, 1.5] -> -r, gradient -r (to the token's own log-prob, weight 1);
    # token 1: A < 0 -> +r, gradient +r; token 2 masked
    assert loss == pytest.approx(-r + r) and clip == 0.0 and g[0] == pytest.approx([-r, r, 0.0])
    # tighter interval [0.8, 1.2]: token 0 clipped (-1.2, no gradient), token 1 takes the unclipped branch
    loss, clip, g = _grad(lambda x: O.gspo_policy_loss(x, old, adv, 0.2, 0.2, mask), lp)
    assert loss == pytest.approx(-1.2 + r) and clip == pytest.approx(0.5) and g[0] == pytest.approx([0.0, r, 0.0])
    # without a mask the row mean is the plain mean: ratio 2^(4/3)
    loss, _, _ = _grad(lambda x: O.gspo_policy_loss(x, old, adv, 0.2, 9.0), lp)
    assert loss == pytest.approx(-(2 ** (4 / 3)) * (1.0 - 1.0 + 5.0))
    # the clamp of the log weight at 10: ratio e^10, no gradient
    loss, _, g = _grad(lambda x: O.gspo_policy_loss(x, _t([[0.0]]), _t([[-1.0]]), 0.2, 0.2), [[12.0]])
    assert loss == pytest.approx(math.exp(10.0)) and g[0] == pytest.approx([0.0])
    # rows of one token: the sequence ratio is the token ratio, so GSPO is the clipped surrogate pinned above
    gen = torch.Generator().manual_seed(5)
    lp1 = torch.randn(40, 1, generator=gen, dtype=torch.float64) * 0.4
    old1 = torch.randn(40, 1, generator=gen, dtype=torch.float64) * 0.4
    adv1 = torch.randn(40, 1, generator=gen, dtype=torch.float64)
    x, y = lp1.clone().requires_grad_(True), lp1.clone().requires_grad_(True)
    a, ca = O.gspo_policy_loss(x, old1, adv1, 0.2, 0.28)
    b, cb = O.ppo_policy_loss(y, old1, adv1, 0.2, 0.28)
    a.backward(), b.backward()
    assert a.item() == pytest.approx(b.item()) and ca.item() == cb.item()
    assert torch.allclose(x.grad, y.grad, atol=1e-12)


def test_cispo_and_rollout_is_by_hand():
    ln2, ln3, lnh = math.log(2.0), math.log(3.0), math.log(0.5)
    lp = [ln2 - 1.0, ln3 - 1.0, lnh - 1.0, -1.0]                   # ratios 2, 3, 1/2, 1 against old = -1
    old, adv = _t([-1.0] * 4), _t([1.0, 2.0, -1.0, -3.0])
    # CISPO with [0.75, 2.5]: weights 2, 2.5 (capped), 0.75 (capped), 1
    loss, clip, g = _grad(lambda x: O.cispo_policy_loss(x, old, adv, 0.25, 1.5), lp)
    w = [2.0, 2.5, 0.75, 1.0]
    assert loss == pytest.approx(-sum(a * wi * l for a, wi, l in zip(adv.tolist(), w, lp)))
    assert clip == pytest.approx(0.5) and g == pytest.approx([-2.0, -5.0, 0.75, 3.0])
    # every token keeps a gradient; with a mask the clip fraction counts unmasked tokens only
    _, clip, g = _grad(lambda x: O.cispo_policy_loss(x, old, adv, 0.25, 1.5, _t([1.0, 0.0, 1.0, 1.0])), lp)
    assert clip == pytest.approx(1 / 3) and g == pytest.approx([-2.0, 0.0, 0.75, 3.0])
    # rollout-IS with the same interval: the two outside tokens drop to weight 0
    loss, clip, g = _grad(lambda x: O.rollout_is_policy_loss(x, old, adv, 0.25, 1.5), lp)
    assert loss == pytest.approx(-(1.0 * 2.0 * lp[0] + -3.0 * 1.0 * lp[3]))
    assert clip == pytest.approx(0.5) and g == pytest.approx([-2.0, 0.0, 0.0, 3.0])
    # the interval is open: a ratio exactly on the bound is out for rollout-IS, not clipped for CISPO
    loss, clip, g = _grad(lambda x: O.rollout_is_policy_loss(x, _t([0.0]), _t([1.0]), 0.5, 1.0), [ln2])
    assert loss == 0.0 and clip == 1.0 and g == [0.0]
    loss, clip, g = _grad(lambda x: O.cispo_policy_loss(x, _t([0.0]), _t([1.0]), 0.5, 1.0), [ln2])
    assert loss == pytest.approx(-2.0 * ln2) and clip == 0.0 and g == pytest.approx([-2.0])
    # inside the interval the two are the same function
    a = _grad(lambda x: O.cispo_policy_loss(x, old, adv, 0.9, 9.0), lp)
    b = _grad(lambda x: O.rollout_is_policy_loss(x, old, adv, 0.9, 9.0), lp)
    assert a[0] == pytest.approx(b[0]) and a[2] == pytest.approx(b[2]) and a[1] == b[1] == 0.0


def test_cov_losses_by_hand():
    """clip-cov and kl-cov (ppo_utils.py:938-1053) on a 2 x 4 batch whose selection can be listed by hand."""
    ln = math.log
    old = _t([[-1.0] * 4, [-1.0] * 4])
    # ratios 1, 2, 1/2, 1 | 1, 1, 3, 1
    lp = _t([[-1.0, ln(2) - 1, ln(0.5) - 1, -1.0], [-1.0, -1.0, ln(3) - 1, -1.0]])
    adv = _t([[1.0, 1.0, -2.0, 3.0], [-1.0, 2.0, 1.0, 0.5]])
    mask = _t([[1.0, 1.0, 1.0, 0.0], [1.0, 1.0, 1.0, 1.0]])
    # clipped by the surrogate with [0.8, 1.2]: (0,1) ratio 2 with A > 0, (0,2) ratio 1/2 with A < 0, (1,2) ratio 3 with A > 0
    m = mask.bool()
    mean_a, mean_l = float(adv[m].mean()), float(lp[m].mean())
    cov = {(i, j): (float(adv[i, j]) - mean_a) * (float(lp[i, j]) - mean_l) for i in range(2) for j in range(4)}
    candidates = [ij for ij in cov if ij not in [(0, 1), (0, 2), (1, 2), (0, 3)]]            # unmasked and not clipped
    inside = [ij for ij in candidates if -0.2 < cov[ij] < 0.3]
    assert sorted(candidates) == [(0, 0), (1, 0), (1, 1), (1, 3)] and len(inside) >= 2
    # a clip ratio large enough to draw every candidate inside the bounds: the permutation cannot matter
    x = lp.clone().requires_grad_(True)
    loss, frac, corr = O.clip_cov_policy_loss(x, old, adv, 0.2, 0.2, 1.0, -0.2, 0.3, mask)
    want_corr = torch.ones(2, 4, dtype=torch.float64)
    for ij in inside:
        want_corr[ij] = 0.0
    assert torch.equal(corr, want_corr) and float(frac) == pytest.approx(len(inside) / 7)
    tok = lambda i, j: max(-float(adv[i, j]) * math.exp(float(lp[i, j]) + 1), -float(adv[i, j]) * min(max(math.exp(float(lp[i, j]) + 1), 0.8), 1.2))  # noqa: E731
    want = sum(tok(i, j) * float(want_corr[i, j]) * float(mask[i, j]) for i in range(2) for j in range(4))
    assert loss.item() == pytest.approx(want)
    loss.backward()
    # gradient: -A r where the unclipped branch is active, the loss kept and the token unmasked; 0 elsewhere
    for (i, j), c in cov.items():
        live = (i, j) in candidates and want_corr[i, j] == 1.0
        assert float(x.grad[i, j]) == pytest.approx(-float(adv[i, j]) * math.exp(float(lp[i, j]) + 1) if live else 0.0)
    # clip_ratio = 0.3: int(0.3 * 7) = 2 tokens are drawn from the candidates inside the bounds, whichever the generator picks
    torch.manual_seed(3)
    _, frac, corr = O.clip_cov_policy_loss(lp, old, adv, 0.2, 0.2, 0.3, -10.0, 10.0, mask)
    removed = [(i, j) for i in range(2) for j in range(4) if corr[i, j] == 0]
    assert len(removed) == 2 and set(removed) <= set(candidates) and float(frac) == pytest.approx(2 / 7)
    torch.manual_seed(3)
    perm = torch.randperm(4)                                     # the draw the function makes: candidates in row-major order
    assert sorted(removed) == sorted(sorted(candidates)[k] for k in perm[:2].tolist())
    # a clip ratio that rounds to zero still draws one token; no candidate inside the bounds draws none
    assert int((O.clip_cov_policy_loss(lp, old, adv, 0.2, 0.2, 0.01, -10.0, 10.0, mask)[2] == 0).sum()) == 1
    assert int((O.clip_cov_policy_loss(lp, old, adv, 0.2, 0.2, 1.0, 50.0, 60.0, mask)[2] == 0).sum()) == 0

    # kl-cov: the top int(7 * 0.3) = 2 unmasked tokens by covariance pay coef * |log-ratio| on top of -A r
    order = sorted((ij for ij in cov if ij != (0, 3)), key=lambda ij: -cov[ij])
    x = lp.clone().requires_grad_(True)
    loss, sel = O.kl_cov_policy_loss(x, old, adv, 0.3, 0.5, mask)
    assert sorted((i, j) for i in range(2) for j in range(4) if sel[i, j] == 1) == sorted(order[:2])
    want = 0.0
    for i in range(2):
        for j in range(4):
            d = float(lp[i, j]) + 1.0
            want += float(mask[i, j]) * (-float(adv[i, j]) * math.exp(d) + (0.5 * abs(d) if (i, j) in order[:2] else 0.0))
    assert loss.item() == pytest.approx(want)
    loss.backward()
    for i in range(2):
        for j in range(4):
            d = float(lp[i, j]) + 1.0
            sign = (d > 0) - (d < 0)
            gw = float(mask[i, j]) * (-float(adv[i, j]) * math.exp(d) + (0.5 * sign if (i, j) in order[:2] else 0.0))
            assert float(x.grad[i, j]) == pytest.approx(gw)
    # a fraction that rounds to zero still selects one token; finite differences with the selection held fixed
    assert int(O.kl_cov_policy_loss(lp, old, adv, 0.01, 0.5, mask)[1].sum()) == 1
    eps = 1e-6
    for (i, j) in [(0, 1), (1, 2), (1, 3)]:
        up, dn = lp.clone(), lp.clone()
        up[i, j] += eps
        dn[i, j] -= eps
        fd = (float(O.kl_cov_policy_loss(up, old, adv, 0.3, 0.5, mask)[0]) - float(O.kl_cov_policy_loss(dn, old, adv, 0.3, 0.5, mask)[0])) / (2 * eps)
        assert fd == pytest.approx(float(x.grad[i, j]), rel=1e-5, abs=1e-6)
    # with nothing selected to pay (coef 0) it is the importance-sampling surrogate pinned above
    assert float(O.kl_cov_policy_loss(lp, old, adv, 0.3, 0.0, mask)[0]) == pytest.approx(float(O.importance_sampling_loss(lp, old, adv, mask)[0]))


def test_cispo_ratio_diagnostics_by_hand():
    ln = math.log
    lp, old = _t([ln(2) - 1, ln(3) - 1, ln(0.5) - 1, -1.0]), _t([-1.0] * 4)     # ratios 2, 3, 1/2, 1
    d = O.cispo_ratio_diagnostics(lp, old, 0.25, 1.5)                           # clamp to [0.75, 2.5]
    assert d["cispo/ratio_mean"] == pytest.approx(6.5 / 4) and d["cispo/ratio_clamped_mean"] == pytest.approx((2 + 2.5 + 0.75 + 1) / 4)
    assert d["cispo/ratio_max"] == pytest.approx(3.0) and d["cispo/ratio_min"] == pytest.approx(0.5)
    d = O.cispo_ratio_diagnostics(lp, old, 0.25, 1.5, _t([1.0, 0.0, 0.0, 1.0]))  # the masked extremes do not count
    assert d["cispo/ratio_mean"] == pytest.approx(1.5) and d["cispo/ratio_max"] == pytest.approx(2.0) and d["cispo/ratio_min"] == pytest.approx(1.0)
    d = O.cispo_ratio_diagnostics(lp, old, 0.25, 1.5, _t([0.0] * 4))             # an empty mask: extremes over all tokens, means 0
    assert d["cispo/ratio_mean"] == 0.0 and d["cispo/ratio_max"] == pytest.approx(3.0) and d["cispo/ratio_min"] == pytest.approx(0.5)


def test_dppo_by_hand():
    ln = math.log
    # probabilities now / behaviour: (0.5, 0.2), (0.2, 0.5), (0.5, 0.2), (0.2, 0.5), (0.3, 0.2)
    lp = [ln(0.5), ln(0.2), ln(0.5), ln(0.2), ln(0.3)]
    mu = _t([ln(0.2), ln(0.5), ln(0.2), ln(0.5), ln(0.2)])
    adv = _t([1.0, 1.0, -1.0, -1.0, 2.0])
    # TV, delta_low 0.25, delta_high 0.2: token 0 (A > 0, rose by 0.3 > 0.2) out; token 3 (A < 0, fell by 0.3 > 0.25) out;
    # tokens 1 and 2 moved against their advantage's direction and stay; token 4 rose by 0.1 only
    loss, clip, g = _grad(lambda x: O.dppo_policy_loss(x, mu, adv, "binary_tv", 0.25, 0.2), lp)
    assert loss == pytest.approx(-(0.4 * 1.0) + 2.5 * 1.0 - 1.5 * 2.0) and clip == pytest.approx(0.4)
    assert g == pytest.approx([0.0, -0.4, 2.5, 0.0, -3.0])
    # the thresholds are per direction: delta_low 0.35 lets token 3 back in
    loss, clip, _ = _grad(lambda x: O.dppo_policy_loss(x, mu, adv, "binary_tv", 0.35, 0.2), lp)
    assert loss == pytest.approx(-0.4 + 2.5 + 0.4 - 3.0) and clip == pytest.approx(0.2)
    # KL: Bernoulli KL(mu || p) = mu ln(mu/p) + (1-mu) ln((1-mu)/(1-p))
    bkl = lambda m, p: m * ln(m / p) + (1 - m) * ln((1 - m) / (1 - p))  # noqa: E731
    k0, k3, k4 = bkl(0.2, 0.5), bkl(0.5, 0.2), bkl(0.2, 0.3)
    assert k4 < 0.05 < k0 < 0.21 < k3                                  # 0.0257, 0.1927, 0.2231
    loss, clip, g = _grad(lambda x: O.dppo_policy_loss(x, mu, adv, "binary_kl", 0.21, 0.05), lp)
    assert clip == pytest.approx(0.4) and g == pytest.approx([0.0, -0.4, 2.5, 0.0, -3.0])
    loss, clip, g = _grad(lambda x: O.dppo_policy_loss(x, mu, adv, "binary_kl", 0.23, 0.2), lp)
    assert clip == 0.0 and g == pytest.approx([-2.5, -0.4, 2.5, 0.4, -3.0])
    # nothing masked: the importance-sampling surrogate pinned above
    ref, _ = O.importance_sampling_loss(_t(lp), mu, adv)
    assert loss == pytest.approx(ref.item())
    with pytest.raises(ValueError):
        O.dppo_policy_loss(_t(lp), mu, adv, "topk_tv", 0.2, 0.2)


@pytest.mark.parametrize("kind", ["sapo", "gspo", "cispo", "rollout_is", "dppo_tv", "dppo_kl"])
def test_further_losses_gradient_matches_finite_differences(kind):
    """Autograd of the restatement against fp64 central differences of the same surrogate with its stop-gradient factors
    (the CISPO / rollout-IS weight, the DPPO mask, GSPO's sequence weight) evaluated once at the base point."""
    gen = torch.Generator().manual_seed(23)
    rows, cols = 6, 9
    old = -torch.rand(rows, cols, generator=gen, dtype=torch.float64) * 2 - 0.1
    lp = (old + torch.randn(rows, cols, generator=gen, dtype=torch.float64) * 0.3).clamp(max=-0.01)
    adv = torch.randn(rows, cols, generator=gen, dtype=torch.float64)
    mask = (torch.rand(rows, cols, generator=gen) > 0.3).double()
    ratio0 = (lp - old).exp()
    if kind == "sapo":
        f = lambda x: O.sapo_policy_loss(x, old, adv, 1.0, 1.05, mask)[0]  # noqa: E731
        frozen = f
    elif kind == "gspo":
        f = lambda x: O.gspo_policy_loss(x, old, adv, 0.1, 0.15, mask)[0]  # noqa: E731
        row0 = O.masked_mean(lp - old, mask, dim=-1).unsqueeze(-1)

        def frozen(x):  # s_i fixed at the base point, times pi(x) / pi(base)
            r = (x - lp + row0).exp()
            return -(torch.min(r * adv, r.clamp(0.9, 1.15) * adv) * mask).sum()
    elif kind == "cispo":
        f = lambda x: O.cispo_policy_loss(x, old, adv, 0.2, 0.3, mask)[0]  # noqa: E731
        frozen = lambda x: -(adv * ratio0.clamp(0.8, 1.3) * x * mask).sum()  # noqa: E731
    elif kind == "rollout_is":
        f = lambda x: O.rollout_is_policy_loss(x, old, adv, 0.2, 0.3, mask)[0]  # noqa: E731
        w0 = torch.where((ratio0 > 0.8) & (ratio0 < 1.3), ratio0, torch.zeros_like(ratio0))
        frozen = lambda x: -(adv * w0 * x * mask).sum()  # noqa: E731
    else:
        name = "binary_tv" if kind == "dppo_tv" else "binary_kl"
        lo, hi = (0.05, 0.04) if kind == "dppo_tv" else (0.02, 0.015)
        f = lambda x: O.dppo_policy_loss(x, old, adv, name, lo, hi, mask)[0]  # noqa: E731
        x0 = lp.clone().requires_grad_(True)
        keep0 = (torch.autograd.grad(f(x0), x0)[0] != 0) | (mask == 0) | (adv == 0)
        assert 0 < (~keep0).sum() < keep0.numel() / 2                   # the mask does cut some tokens, not most
        frozen = lambda x: -((x - old).exp() * adv * keep0 * mask).sum()  # noqa: E731
    x = lp.clone().requires_grad_(True)
    f(x).backward()
    assert frozen(lp).item() == pytest.approx(f(lp).item(), rel=1e-12)
    eps = 1e-6
    for i in range(rows):
        for j in range(cols):
            d = torch.zeros(rows, cols, dtype=torch.float64)
            d[i, j] = eps
            fd = (frozen(lp + d) - frozen(lp - d)).item() / (2 * eps)
            assert x.grad[i, j].item() == pytest.approx(fd, abs=1e-6), f"token {i},{j}"


def test_masked_mean_by_hand():
    t = torch.tensor([[1.0, 2.0, 3.0], [4.0, 5.0, 6.0]])
    m = torch.tensor([[1.0, 0.0, 1.0], [0.0, 0.0, 0.0]])
    assert O.masked_mean(t, None).item() == pytest.approx(3.5)
    assert O.masked_mean(t, m).item() == pytest.approx(2.0)
    assert O.masked_mean(t, None, dim=-1).tolist() == pytest.approx([2.0, 5.0])
    assert O.masked_mean(t, m, dim=-1).tolist() == pytest.approx([2.0, 0.0])       # an all-masked row: 0 / clamp(0, 1)
    half = torch.tensor([[0.5, 0.5, 0.0], [0.25, 0.0, 0.0]])                        # fractional weights, count below 1
    assert O.masked_mean(t, half, dim=-1).tolist() == pytest.approx([1.5, 1.0])


def test_approx_kl_hand_values_and_clamps():
    base = torch.zeros(6, dtype=torch.float64)
    # base - lp = k:            0      ln 2             -1      25 (clamped to 20)  -25 (clamped)   2
    lp = torch.tensor([0.0, -math.log(2.0), 1.0, -25.0, 25.0, -2.0], dtype=torch.float64)
    k3 = O.compute_approx_kl(lp, base, None, "k3").tolist()
    assert k3[0] == 0.0
    assert k3[1] == pytest.approx(1.0 - math.log(2.0))
    assert k3[2] == pytest.approx(math.exp(-1.0))
    assert k3[3] == 10.0                                                      # e^20 - 21 cut by the outer clamp
    assert k3[4] == 10.0                                                      # e^-20 + 19 cut by the outer clamp
    assert k3[5] == pytest.approx(math.exp(2.0) - 3.0)
    assert O.compute_approx_kl(torch.tensor([-3.0]), torch.tensor([0.0]), None, "k3").item() == 10.0   # e^3 - 4 = 16.1
    assert O.compute_approx_kl(lp, base, None, "k1").tolist() == lp.tolist()
    assert O.compute_approx_kl(lp, base, None, "abs").tolist() == lp.abs().tolist()
    assert O.compute_approx_kl(lp, base, None, "k2").tolist() == pytest.approx((0.5 * lp * lp).tolist())
    with pytest.raises(ValueError):
        O.compute_approx_kl(lp, base, None, "k4")
    # masked positions are exactly zero even where the value is not finite
    m = torch.tensor([1.0, 0.0, 2.0, 0.0, 1.0, 0.0], dtype=torch.float64)
    lp_nan = lp.clone()
    lp_nan[1] = float("nan")
    out = O.compute_approx_kl(lp_nan, base, m, "k1")
    assert out.tolist() == [0.0, 0.0, 2.0, 0.0, 25.0, 0.0]


def test_approx_kl_estimators_are_unbiased_for_the_true_kl():
    gen = torch.Generator().manual_seed(3)
    # spreads small enough that no term reaches the clamps (|log ratio| < 20, value < 10)
    logp = torch.log_softmax(0.5 * torch.randn(50, dtype=torch.float64, generator=gen), 0)
    logq = torch.log_softmax(0.5 * torch.randn(50, dtype=torch.float64, generator=gen), 0)
    assert float((logq - logp).abs().max()) < 3.0
    true_kl = torch.nn.functional.kl_div(logq, logp, reduction="sum", log_target=True)   # KL(p || q)
    p = logp.exp()
    assert float((p * O.compute_approx_kl(logp, logq, None, "k1")).sum()) == pytest.approx(float(true_kl), rel=1e-12)
    assert float((p * O.compute_approx_kl(logp, logq, None, "k3")).sum()) == pytest.approx(float(true_kl), rel=1e-12)
    # second order: k3 and k2 agree for nearby distributions
    near = logp + 1e-4 * torch.randn(50, dtype=torch.float64, generator=gen)
    k2, k3 = O.compute_approx_kl(logp, near, None, "k2"), O.compute_approx_kl(logp, near, None, "k3")
    torch.testing.assert_close(k3, k2, rtol=1e-3, atol=1e-14)


def test_approx_kl_loss_reduction_brute_force():
    gen = torch.Generator().manual_seed(4)
    lp = torch.randn(3, 7, dtype=torch.float64, generator=gen)
    base = torch.randn(3, 7, dtype=torch.float64, generator=gen)
    mask = (torch.rand(3, 7, generator=gen) < 0.6).double()
    mask[2] = 0
    got = O.approx_kl_loss(lp, base, mask, "k2").item()
    rows = []
    for b in range(3):
        vals = [0.5 * (lp[b, s] - base[b, s]).item() ** 2 for s in range(7) if mask[b, s] > 0]
        rows.append(sum(vals) / max(len(vals), 1))
    assert got == pytest.approx(sum(rows) / 3)
    got = O.approx_kl_loss(lp, base, None, "abs").item()
    assert got == pytest.approx(float((lp - base).abs().mean()))


def test_actor_loss_combination_by_hand():
    # two rows of two tokens; ratios 1 (unclipped), so the policy loss is -sum A * mask
    lp = torch.tensor([[-1.0, -2.0], [-0.5, -3.0]], dtype=torch.float64)
    adv = torch.tensor([[1.0, -2.0], [0.5, 4.0]], dtype=torch.float64)
    mask = torch.tensor([[1.0, 1.0], [1.0, 0.0]], dtype=torch.float64)
    base = lp - torch.tensor([[0.2, -0.4], [0.6, 9.0]], dtype=torch.float64)        # k1 = lp - base
    ent = torch.tensor([[2.0, 4.0], [6.0, 100.0]], dtype=torch.float64)
    loss, policy, kl, e = O.actor_loss(lp, lp.clone(), adv, mask, 0.2, 0.2, policy_scale=8.0, term_scale=0.25,
                                       base_log_probs=base, kl_estimator_type="k1", kl_coef=0.1, entropy=ent, entropy_coef=0.01)
    assert policy.item() == pytest.approx(-(1.0 - 2.0 + 0.5))
    assert kl.item() == pytest.approx(((0.2 - 0.4) / 2 + 0.6 / 1) / 2)            # row means over masked tokens, then over rows
    assert e.item() == pytest.approx((2.0 + 4.0 + 6.0) / 3)
    assert loss.item() == pytest.approx(8.0 * 0.5 + 0.25 * (0.1 * 0.25 - 0.01 * 4.0))
    bare, _, kl0, e0 = O.actor_loss(lp, lp.clone(), adv, mask, 0.2, 0.2)
    assert bare.item() == pytest.approx(0.5) and kl0.item() == 0.0 and e0.item() == 0.0


# ----------------------------------------------------------------------------------------------------------------------
# the FSDP worker's forward tail
# ----------------------------------------------------------------------------------------------------------------------
def test_hf_wrapper_tail_brute_force():
    gen = torch.Generator().manual_seed(21)
    B, S, V, A, t = 3, 9, 13, 4, 0.7
    logits = torch.randn(B, S, V, dtype=torch.float64, generator=gen)
    seqs = torch.randint(0, V, (B, S), generator=gen)
    am = torch.ones(B, S, dtype=torch.long)
    am[0, :3] = 0                                          # left padding
    am[2, :1] = 0
    alp, ent = O.hf_wrapper_tail(logits, seqs, A, am, t)
    dist = torch.distributions.Categorical(logits=logits / t)
    assert alp.shape == (B, A) and ent.shape == (B, S)
    for b in range(B):
        for j in range(A):
            pos = S - A + j                                 # the j-th action token; predicted from position pos - 1
            one = torch.distributions.Categorical(logits=logits[b, pos - 1] / t)
            assert alp[b, j].item() == pytest.approx(one.log_prob(seqs[b, pos]).item(), rel=1e-12)
    torch.testing.assert_close(ent, dist.entropy() * am, rtol=1e-12, atol=1e-12)

    # padding removed: the model ran on the real tokens only, as one stream
    nnz = am.flatten().nonzero().flatten()
    packed_logits = logits.reshape(B * S, V)[nnz][None]
    alp_p, ent_p = O.hf_wrapper_tail(packed_logits, seqs, A, am, t, nnz_indices=nnz)
    assert alp_p.shape == (B, A) and ent_p.shape == (B, S)
    # inside a row the successor in the stream is the successor in the row, so all but each row's last action agree
    torch.testing.assert_close(alp_p[:, :], alp[:, :], rtol=1e-12, atol=0)
    torch.testing.assert_close(ent_p, dist.entropy() * am, rtol=1e-12, atol=1e-12)   # zeros come from the padding here
    # the stream's roll wraps a row's last token onto the next row's first real token (the slice drops that position)
    tokens = seqs.flatten()[nnz]
    full, _ = O.hf_wrapper_tail(packed_logits, seqs, S - 1, am, t, nnz_indices=nnz)
    row0_last = int(am[0].sum()) - 1                                      # stream position of row 0's last token
    want = torch.log_softmax(packed_logits[0, row0_last] / t, -1)[tokens[row0_last + 1]]
    lp_all = torch.log_softmax(packed_logits[0] / t, -1).gather(-1, torch.roll(tokens, -1)[:, None])[:, 0]
    assert lp_all[row0_last].item() == pytest.approx(want.item(), rel=1e-12)
    assert full.shape == (B, S - 1)


def test_packed_action_entropy_brute_force():
    gen = torch.Generator().manual_seed(21)
    # attention-mask layout: rows with left, right and interior padding; row b owns packed tokens cu[b] .. cu[b]+real_b-1
    L, num_actions = 9, 4
    am = torch.tensor([[1, 1, 1, 1, 1, 1, 1, 1, 1],
                       [0, 0, 1, 1, 1, 1, 1, 0, 0],
                       [1, 1, 0, 1, 1, 0, 1, 1, 1],
                       [0, 0, 0, 0, 0, 0, 0, 1, 1]])
    real = am.sum(1).tolist()
    padded = [r + (-r) % 4 for r in real]                       # segments padded to a multiple of 4
    cu = torch.tensor([0] + list(np.cumsum(padded)))
    ent = torch.rand(int(cu[-1]), generator=gen, dtype=torch.float64) * 3
    for loss_mask in (None, (torch.rand(4, num_actions, generator=gen) > 0.4).double()):
        total = count = 0.0
        for b in range(4):
            j = 0                                               # index of the real token inside row b
            for c in range(L - 1):
                if am[b, c]:
                    if j + 1 < real[b] and c >= L - 1 - num_actions:
                        wgt = 1.0 if loss_mask is None else loss_mask[b, c - (L - 1 - num_actions)].item()
                        total += ent[cu[b] + j].item() * wgt
                        count += wgt
                    j += 1
        got, for_loss = O.packed_action_entropy(ent, cu, L, num_actions, am, loss_mask)
        assert got.item() == pytest.approx(total / max(count, 1.0)) and for_loss.item() == got.item()
    # no action weight at all: 0 / clamp(0, 1)
    got, _ = O.packed_action_entropy(ent, cu, L, num_actions, am, torch.zeros(4, num_actions, dtype=torch.float64))
    assert got.item() == 0.0

    # sub-sequence layout: two output rows, three and two packed segments; true lengths shorter than the padded ones
    sub = [[3, 1, 4], [5, 2]]
    pad = [4, 4, 4, 8, 4]
    cu = torch.tensor([0] + list(np.cumsum(pad)))
    ent = torch.rand(int(cu[-1]), generator=gen, dtype=torch.float64)
    L, num_actions = 12, 6
    loss_mask = (torch.rand(2, num_actions, generator=gen) > 0.3).double()
    total = count = 0.0
    k = 0
    for r, row in enumerate(sub):
        col0 = 0
        for n in row:
            for o in range(max(n - 1, 0)):
                c = col0 + o
                if c < L - 1 and c >= L - 1 - num_actions:
                    wgt = loss_mask[r, c - (L - 1 - num_actions)].item()
                    total += ent[cu[k] + o].item() * wgt
                    count += wgt
            col0 += pad[k]
            k += 1
    got, _ = O.packed_action_entropy(ent, cu, L, num_actions, torch.ones(2, L), loss_mask, sub)
    assert count > 0 and got.item() == pytest.approx(total / count)


# ----------------------------------------------------------------------------------------------------------------------
# MTP draft loss: soft cross-entropy
# ----------------------------------------------------------------------------------------------------------------------
def test_shift_mask_for_mtp_reference_golden_masks():
    """The masks the reference's tests spell out (tests/backends/skyrl_train/mtp/test_soft_ce.py:224-245)."""
    m = torch.ones(1, 4)
    assert O.shift_mask_for_mtp(m, 0).tolist() == [[1.0, 1.0, 1.0, 0.0]]
    assert O.shift_mask_for_mtp(m, 1).tolist() == [[1.0, 1.0, 0.0, 0.0]]
    left = torch.tensor([[0.0, 0.0, 1.0, 1.0, 1.0]])
    assert O.shift_mask_for_mtp(left, 0).tolist() == [[0.0, 0.0, 1.0, 1.0, 0.0]]
    assert O.shift_mask_for_mtp(left, 1).tolist() == [[0.0, 0.0, 1.0, 0.0, 0.0]]
    right = torch.tensor([[1.0, 1.0, 1.0, 0.0, 0.0]])
    assert O.shift_mask_for_mtp(right, 0).tolist() == [[1.0, 1.0, 0.0, 0.0, 0.0]]


def _shift_mask_loop(mask, shift, bounds):
    out = torch.zeros_like(mask)
    for b in range(mask.shape[0]):
        for start, end in zip(bounds[:-1], bounds[1:]):
            for t in range(start, end):
                if t + shift < end and mask[b, t] != 0 and mask[b, t + shift] != 0:
                    out[b, t] = mask[b, t] * mask[b, t + shift]
    return out


def test_shift_mask_for_mtp_packed_brute_force_and_product_mirror():
    from skyrl_amd.mtp_soft_ce import shift_mask_for_mtp as product

    gen = torch.Generator().manual_seed(3)
    for bounds in ([0, 5, 5, 6, 14, 20], [0, 1, 3, 20], [0, 20], [0, 7, 12]):   # empty / one-token segments, a tail outside
        mask = (torch.rand(2, 20, generator=gen) > 0.25).float()
        for depth in (0, 1, 2, 6):
            want = _shift_mask_loop(mask, depth + 1, bounds)
            assert torch.equal(O.shift_mask_for_mtp(mask.clone(), depth, torch.tensor(bounds)), want), (bounds, depth)
            assert torch.equal(product(mask.clone(), depth, torch.tensor(bounds)), want), (bounds, depth)
            assert torch.equal(product(mask.clone(), depth, bounds), want)
    mask = (torch.rand(3, 9, generator=gen) > 0.3).float()
    for depth in (0, 1, 3, 8, 11):
        want = _shift_mask_loop(mask, depth + 1, [0, 9])
        assert torch.equal(O.shift_mask_for_mtp(mask.clone(), depth), want)
        assert torch.equal(product(mask.clone(), depth), want)


def test_soft_ce_is_entropy_plus_kl_and_its_limits():
    gen = torch.Generator().manual_seed(12)
    student = torch.randn(3, 5, 11, generator=gen, dtype=torch.float64) * 2
    teacher = torch.randn(3, 5, 11, generator=gen, dtype=torch.float64) * 2
    got = O.soft_ce_per_token(student, teacher)
    p = torch.distributions.Categorical(logits=teacher)
    kl = torch.nn.functional.kl_div(torch.log_softmax(student, -1), torch.softmax(teacher, -1), reduction="none").sum(-1)
    torch.testing.assert_close(got, p.entropy() + kl, rtol=1e-12, atol=1e-12)
    torch.testing.assert_close(got, p.entropy() + torch.distributions.kl_divergence(p, torch.distributions.Categorical(logits=student)))
    # teacher = student: the entropy; a shift of either logits row changes nothing
    torch.testing.assert_close(O.soft_ce_per_token(teacher + 3.0, teacher - 1.0), p.entropy())
    # a one-hot teacher: minus the student's log-probability of that token, i.e. the pinned forward with these labels
    labels = torch.randint(0, 11, (3, 5), generator=gen)
    hot = torch.full((3, 5, 11), -1e4, dtype=torch.float64).scatter_(-1, labels[..., None], 0.0)
    want = -O.distributed_log_softmax(student).gather(-1, labels[..., None])[..., 0]
    torch.testing.assert_close(O.soft_ce_per_token(student, hot), want)
    # uniform teacher over V: ln V + mean of (lse - z)
    uni = torch.zeros(3, 5, 11, dtype=torch.float64)
    torch.testing.assert_close(O.soft_ce_per_token(student, uni), torch.logsumexp(student, -1) - student.mean(-1))


def test_draft_soft_ce_reduction_gradient_and_teacher_checks():
    gen = torch.Generator().manual_seed(13)
    student = torch.randn(2, 4, 6, generator=gen, dtype=torch.float64)
    teacher = torch.randn(2, 4, 6, generator=gen, dtype=torch.float64)
    mask = torch.tensor([[1.0, 1.0, 0.0, 1.0], [0.0, 1.0, 1.0, 0.0]], dtype=torch.float64)
    per = O.soft_ce_per_token(student, teacher)
    by_hand = sum(per[b, t].item() for b in range(2) for t in range(4) if mask[b, t]) / 5
    assert O.draft_soft_ce(student, teacher, mask).item() == pytest.approx(by_hand)
    assert O.draft_soft_ce(student, teacher, mask, torch.tensor(20.0)).item() == pytest.approx(by_hand * 5 / 20)
    assert O.draft_soft_ce(student, teacher, mask, torch.tensor(0.25)).item() == pytest.approx(by_hand * 5)   # clamp(min=1)
    # masked-out positions do not enter (test_soft_ce.py:184-194)
    other = teacher.clone()
    other[0, 2] = torch.randn(6, generator=gen, dtype=torch.float64)
    assert O.draft_soft_ce(student, other, mask).item() == pytest.approx(by_hand)
    # gradient: (softmax(student) - softmax(teacher)) * mask / n (test_soft_ce.py:171-181), against central differences
    x = student.clone().requires_grad_(True)
    O.draft_soft_ce(x, teacher, mask).backward()
    want = (torch.softmax(student, -1) - torch.softmax(teacher, -1)) * mask[..., None] / 5
    torch.testing.assert_close(x.grad, want, rtol=1e-10, atol=1e-12)
    eps = 1e-6
    for idx in [(0, 0, 1), (0, 2, 3), (1, 1, 5), (1, 2, 0)]:
        d = torch.zeros_like(student)
        d[idx] = eps
        fd = (O.draft_soft_ce(student + d, teacher, mask) - O.draft_soft_ce(student - d, teacher, mask)).item() / (2 * eps)
        assert x.grad[idx].item() == pytest.approx(fd, abs=1e-8)
    assert x.grad.sum(-1).abs().max().item() < 1e-14                  # rows of the gradient sum to zero
    with pytest.raises(AssertionError, match="must be detached"):
        O.draft_soft_ce(student, teacher.clone().requires_grad_(True), mask)


def test_build_teacher_logits_and_hidden_chain():
    ml = torch.arange(2 * 4 * 3, dtype=torch.float64, requires_grad=True).reshape(2, 4, 3)
    assert torch.equal(O.build_teacher_logits(ml, 0), torch.roll(ml.detach(), -1, dims=1))
    assert torch.equal(O.build_teacher_logits(ml, 1), torch.roll(ml.detach(), -2, dims=1))
    assert not O.build_teacher_logits(ml, 0).requires_grad
    # the hidden-state chain: position t of the student against position t + depth + 1 of the policy, by a per-position loop
    gen = torch.Generator().manual_seed(14)
    B, S, H, V, depth = 2, 6, 8, 13, 1
    hs = torch.randn(B, S, H, generator=gen, dtype=torch.float64, requires_grad=True)
    ht = torch.randn(B, S, H, generator=gen, dtype=torch.float64)
    w = torch.randn(V, H, generator=gen, dtype=torch.float64, requires_grad=True)
    mask = O.shift_mask_for_mtp(torch.ones(B, S, dtype=torch.float64), depth)
    got = O.draft_soft_ce_from_hidden(hs, ht, w, mask, depth)
    total, n = 0.0, 0
    for b in range(B):
        for t in range(S - depth - 1):
            p = torch.softmax(w.detach() @ ht[b, t + depth + 1], -1)
            total += -(p * torch.log_softmax(w.detach() @ hs[b, t].detach(), -1)).sum().item()
            n += 1
    assert got.item() == pytest.approx(total / n)
    got.backward()
    assert w.grad is None and hs.grad is not None                      # the output weight is detached


def test_soft_ce_topk_by_brute_force_and_its_limits():
    """The top-k draft loss (mtp/soft_ce.py:243-341): selection by ``sorted``, sums with ``math``; k = V is the full soft
    cross-entropy; rolling the small lists equals pre-rolling the teacher; custom backward = autograd = finite differences."""
    gen = torch.Generator().manual_seed(5)
    B, S, V, k = 2, 6, 11, 4
    student = torch.randn(B, S, V, generator=gen, dtype=torch.float64)
    teacher = torch.randn(B, S, V, generator=gen, dtype=torch.float64)
    x = student.clone().requires_grad_(True)
    per_token, q_s, t_p, cols = O.soft_ce_topk_per_token(x, teacher, k)
    for b in range(B):
        for s in range(S):
            best = sorted(range(V), key=lambda v: -float(teacher[b, s, v]))[:k]
            assert sorted(cols[b, s].tolist()) == sorted(best)
            zt = [float(teacher[b, s, v]) for v in best]
            zs = [float(student[b, s, v]) for v in best]
            pt = [math.exp(z) / sum(math.exp(u) for u in zt) for z in zt]
            logq = [z - math.log(sum(math.exp(u) for u in zs)) for z in zs]
            assert float(per_token[b, s].detach()) == pytest.approx(-sum(p * lq for p, lq in zip(pt, logq)), rel=1e-12)
    # k >= V: every column is kept and the loss is the full soft cross-entropy
    full = O.soft_ce_topk_per_token(student, teacher, V + 3)[0]
    assert torch.allclose(full, O.soft_ce_per_token(student, teacher), rtol=1e-12, atol=1e-12)
    # roll_shift on the un-rolled teacher = top-k of the pre-rolled teacher (the reference's own check, test_soft_ce.py:122-144)
    for shift in (1, 2, 5):
        a = O.soft_ce_topk_per_token(student, teacher, k, roll_shift=shift)[0]
        b_ = O.soft_ce_topk_per_token(student, torch.roll(teacher, shifts=-shift, dims=1), k)[0]
        assert torch.equal(a, b_)
    # gradient: the restated custom backward, autograd through the gather, and central finite differences
    g = torch.randn(B, S, generator=gen, dtype=torch.float64)
    (per_token * g).sum().backward()
    custom = O.soft_ce_topk_backward(q_s.detach(), t_p, cols, g, V)
    assert torch.allclose(x.grad, custom, rtol=1e-12, atol=1e-14)
    assert int((custom != 0).sum(-1).max()) <= k and int((custom != 0).sum(-1).min()) == k
    eps = 1e-6
    for (b, s, v) in [(0, 0, int(cols[0, 0, 0])), (1, 3, int(cols[1, 3, 2])), (1, 5, int(cols[1, 5, 3]))]:
        up, dn = student.clone(), student.clone()
        up[b, s, v] += eps
        dn[b, s, v] -= eps
        fd = ((O.soft_ce_topk_per_token(up, teacher, k)[0] - O.soft_ce_topk_per_token(dn, teacher, k)[0]) * g).sum() / (2 * eps)
        assert float(fd) == pytest.approx(float(custom[b, s, v]), rel=1e-6, abs=1e-9)
    # the reductions, and the call chain from hidden states
    mask = torch.ones(B, S, dtype=torch.float64)
    mask[0, 4:] = 0
    pt = O.soft_ce_topk_per_token(student, teacher, k, roll_shift=1)[0]
    assert float(O.draft_soft_ce_topk(student, teacher, mask, k, roll_shift=1)) == pytest.approx(float((pt * mask).sum() / 10))
    assert float(O.draft_soft_ce_topk(student, teacher, mask, k, torch.tensor(40.0), roll_shift=1)) == pytest.approx(float((pt * mask).sum() / 40))
    H = 5
    hs, ht = torch.randn(B, S, H, generator=gen, dtype=torch.float64), torch.randn(B, S, H, generator=gen, dtype=torch.float64)
    w = torch.randn(V, H, generator=gen, dtype=torch.float64)
    assert float(O.draft_soft_ce_topk_from_hidden(hs, ht, w, mask, k, roll_shift=2)) == pytest.approx(
        float(O.draft_soft_ce_topk(hs @ w.t(), ht @ w.t(), mask, k, roll_shift=2)))
    with pytest.raises(AssertionError):
        O.draft_soft_ce_topk(student, teacher.clone().requires_grad_(True), mask, k)


def test_logits_input_functions_against_library_distributions():
    """logprobs_from_logits_v2 (torch_utils.py:156-177) and DistributedLogprob (model_utils.py:66-138) on one shard."""
    gen = torch.Generator().manual_seed(9)
    B, S, V = 2, 5, 13
    logits = torch.randn(B, S, V, generator=gen, dtype=torch.float64) * 2
    labels = torch.randint(0, V, (B, S), generator=gen)
    want = torch.distributions.Categorical(logits=logits).log_prob(labels)
    assert torch.allclose(O.logprobs_from_logits_v2(logits, labels), want, rtol=1e-12, atol=1e-12)
    assert torch.allclose(O.logprobs_from_logits_v2(logits.float(), labels).double(), want, atol=1e-5)
    bf = O.logprobs_from_logits_v2(logits.bfloat16(), labels)
    assert bf.dtype == torch.bfloat16 and torch.allclose(bf.double(), want, atol=0.1)
    flat = O.logprobs_from_logits_v2(torch.zeros(3, 2, V, dtype=torch.float64), labels[:, :2].repeat(2, 1)[:3])
    assert torch.allclose(flat, torch.full((3, 2), -math.log(V), dtype=torch.float64))
    # DistributedLogprob on a shard [3, 3 + V): targets re-based, outside -> 0 forward and -softmax * g backward
    target = labels + 3
    target[0, 1], target[1, 4] = 1, 3 + V
    lp, softmax, mask, masked = O.distributed_logprob_forward(logits, target, 3, 3 + V)
    inside = ~mask
    assert mask.sum() == 2 and bool((lp[mask] == 0).all())
    # the reference's log-softmax takes the row sum through fp32 (model_utils.py:52-60): fp32 accuracy even on fp64 logits
    assert torch.allclose(lp[inside], want[inside], atol=1e-6)
    assert torch.allclose(softmax, torch.softmax(logits, -1), atol=1e-6)
    g = torch.randn(B, S, generator=gen, dtype=torch.float64)
    grad = O.distributed_logprob_backward(softmax, mask, masked, g)
    x = logits.clone().requires_grad_(True)
    picked = torch.log_softmax(x, -1).gather(-1, masked.unsqueeze(-1)).squeeze(-1) * inside
    (picked * g).sum().backward()
    # autograd of the masked closed form gives the in-shard rows; out-of-shard rows keep -softmax * g in the reference
    assert torch.allclose(grad[inside], x.grad[inside], atol=1e-6)
    assert torch.allclose(grad[mask], -(torch.softmax(logits, -1) * g.unsqueeze(-1))[mask], atol=1e-6)
    assert torch.allclose(grad.sum(-1)[inside], torch.zeros(int(inside.sum()), dtype=torch.float64), atol=1e-6)
    assert torch.allclose(grad.sum(-1)[mask], -g[mask], atol=1e-6)


def _opc_cfg(**kw):
    from types import SimpleNamespace

    base = dict(tis_ratio_type=None, token_tis_ratio_clip_high=2.0, sequence_tis_ratio_clip_high=5.0, sequence_mask_metric=None,
                geo_mask_high=1.01, geo_mask_low=0.99, product_mask_high=2.0, product_mask_low=0.5,
                outlier_token_is_threshold_low=None, outlier_token_is_threshold_high=None,
                token_mask_is_threshold_low=None, token_mask_is_threshold_high=None)
    base.update(kw)
    return SimpleNamespace(**base)


def _opc_batch():
    """Ratios old / rollout that are powers of two, so that every product and threshold decision can be read off."""
    ratio = _t([[1.0, 2.0, 0.5, 4.0], [1.0, 8.0, 1.0, 1.0], [0.25, 1.0, 2.0, 1.0]])
    mask = _t([[1.0, 1.0, 1.0, 0.0], [1.0, 1.0, 1.0, 1.0], [1.0, 0.0, 1.0, 1.0]])
    rollout = _t([[-1.0, -2.0, -0.5, -3.0]] * 3)
    return rollout + ratio.log(), rollout, mask, ratio


def test_off_policy_correction_by_hand():
    """off_policy_correction_utils.py:24-391 on a 3 x 4 batch: masks, weights and metrics of every step written down by hand,
    and the order of the steps."""
    import statistics

    old, rollout, mask, ratio = _opc_batch()
    assert O.off_policy_correction(old, rollout, mask, _opc_cfg()) == (None, {}, mask)
    # outlier rows: row 1 holds an 8 (> 6); the 4 of row 0 is masked and does not count
    tis, m, out = O.off_policy_correction(old, rollout, mask, _opc_cfg(outlier_token_is_threshold_high=6.0))
    assert tis is None and torch.equal(out, _t([[1, 1, 1, 0], [0, 0, 0, 0], [1, 0, 1, 1]]))
    assert m["outlier_seq_masked_ratio"] == pytest.approx(1 / 3) and m["outlier_seq_over_high_ratio"] == pytest.approx(1 / 3)
    assert m["outlier_seq_under_low_ratio"] == 0.0
    x = [1, 2, .5, 0, 1, 8, 1, 1, .25, 0, 2, 1]                      # ratio * mask, all twelve entries
    assert m["is_ratio_mean"] == pytest.approx(17.75 / 10) and m["is_ratio_std"] == pytest.approx(statistics.stdev(x))
    assert m["is_ratio_max"] == pytest.approx(8.0) and m["is_ratio_min"] == 0.0
    _, m, out = O.off_policy_correction(old, rollout, mask, _opc_cfg(outlier_token_is_threshold_low=0.3))
    assert torch.equal(out, _t([[1, 1, 1, 0], [1, 1, 1, 1], [0, 0, 0, 0]])) and m["outlier_seq_under_low_ratio"] == pytest.approx(1 / 3)
    # + the per-token hard mask [0.4, 3]: of the six tokens the outlier step left, the 0.25 of row 2 goes
    both = dict(outlier_token_is_threshold_high=6.0, token_mask_is_threshold_low=0.4, token_mask_is_threshold_high=3.0)
    _, m, out = O.off_policy_correction(old, rollout, mask, _opc_cfg(**both))
    assert torch.equal(out, _t([[1, 1, 1, 0], [0, 0, 0, 0], [0, 0, 1, 1]])) and m["token_mask_ratio"] == pytest.approx(1 / 6)
    # one bound alone does not switch the token mask on
    assert O.off_policy_correction(old, rollout, mask, _opc_cfg(token_mask_is_threshold_low=0.4))[0:2] == (None, {})
    # + token-level TIS capped at 1.5: two of the five tokens still alive exceed it
    tis, m, _ = O.off_policy_correction(old, rollout, mask, _opc_cfg(tis_ratio_type="token", token_tis_ratio_clip_high=1.5, **both))
    assert torch.allclose(tis, _t([[1, 1.5, .5, 1.5], [1, 1.5, 1, 1], [.25, 1, 1.5, 1]])) and m["tis_token_clip_high_ratio"] == pytest.approx(0.4)
    # sequence-level TIS on the same masks: products 1, 1 (the removed row) and 2; without the other steps row 1 has 8
    tis, m, _ = O.off_policy_correction(old, rollout, mask, _opc_cfg(tis_ratio_type="sequence", sequence_tis_ratio_clip_high=1.5, **both))
    assert torch.allclose(tis, _t([[1.0], [1.0], [1.5]])) and m["tis_seq_clip_high_ratio"] == pytest.approx(1 / 3)
    tis, m, out = O.off_policy_correction(old, rollout, mask, _opc_cfg(tis_ratio_type="sequence"))
    assert torch.allclose(tis, _t([[1.0], [5.0], [0.5]])) and m["tis_seq_clip_high_ratio"] == pytest.approx(1 / 3) and torch.equal(out, mask)
    half = mask.clone()
    half[0, 1] = 0.5                                                # a fractional mask weighs the log-ratio: 2 ** 0.5 * 0.5
    tis, _, _ = O.off_policy_correction(old, rollout, half, _opc_cfg(tis_ratio_type="sequence"))
    assert float(tis[0]) == pytest.approx(2 ** -0.5)
    # sequence masks on the masks the first two steps left: geometric means 1, 1, sqrt 2; products 1, 1, 2
    _, m, out = O.off_policy_correction(old, rollout, mask, _opc_cfg(sequence_mask_metric="geometric", geo_mask_low=0.9, geo_mask_high=1.3, **both))
    assert torch.equal(out, _t([[1, 1, 1, 0], [0, 0, 0, 0], [0, 0, 0, 0]]))
    assert (m["geo_sequence_mask_masked_ratio"], m["geo_sequence_mask_over_high_ratio"], m["geo_sequence_mask_under_low_ratio"]) == \
        (pytest.approx(1 / 3), pytest.approx(1 / 3), 0.0)
    _, m, out = O.off_policy_correction(old, rollout, mask, _opc_cfg(sequence_mask_metric="geometric", geo_mask_low=1.05, geo_mask_high=1.3, **both))
    assert float(out.sum()) == 0.0 and m["geo_sequence_mask_masked_ratio"] == 1.0 and m["geo_sequence_mask_under_low_ratio"] == pytest.approx(2 / 3)
    _, m, out = O.off_policy_correction(old, rollout, mask, _opc_cfg(sequence_mask_metric="product", product_mask_low=0.5, product_mask_high=1.5, **both))
    assert torch.equal(out, _t([[1, 1, 1, 0], [0, 0, 0, 0], [0, 0, 0, 0]])) and m["product_sequence_mask_over_high_ratio"] == pytest.approx(1 / 3)
    _, m, out = O.off_policy_correction(old, rollout, mask, _opc_cfg(sequence_mask_metric="product", product_mask_low=0.6, product_mask_high=6.0))
    assert torch.equal(out, _t([[1, 1, 1, 0], [0, 0, 0, 0], [0, 0, 0, 0]]))          # products 1, 8, 0.5 without the other steps
    assert m["product_sequence_mask_under_low_ratio"] == pytest.approx(1 / 3) and m["product_sequence_mask_masked_ratio"] == pytest.approx(2 / 3)
    # the clamp of the log-ratio at +-20, unknown names, and the wrapper on a per-token loss
    far = old.clone()
    far[0, 0] += 50.0
    tis, _, _ = O.off_policy_correction(far, rollout, mask, _opc_cfg(tis_ratio_type="token", token_tis_ratio_clip_high=1e30))
    assert float(tis[0, 0]) == pytest.approx(math.exp(20.0))
    with pytest.raises(ValueError):
        O.off_policy_correction(old, rollout, mask, _opc_cfg(tis_ratio_type="rows"))
    with pytest.raises(ValueError):
        O.off_policy_correction(old, rollout, mask, _opc_cfg(sequence_mask_metric="median"))
    loss = _t([[1.0, 2.0, 3.0, 4.0]] * 3)
    got, got_mask, m = O.apply_off_policy_correction(loss, old, rollout, mask, _opc_cfg(tis_ratio_type="token", token_tis_ratio_clip_high=1.5, **both))
    assert torch.allclose(got, loss * _t([[1, 1.5, .5, 1.5], [1, 1.5, 1, 1], [.25, 1, 1.5, 1]])) and "token_mask_ratio" in m
    assert torch.equal(got_mask, _t([[1, 1, 1, 0], [0, 0, 0, 0], [0, 0, 1, 1]]))
    assert O.apply_off_policy_correction(loss, old, None, mask, _opc_cfg(tis_ratio_type="token")) == (loss, mask, {})


def test_minibatch_rollout_logprob_diff_metrics_by_hand():
    """workers/worker_utils.py:34-58 on six tokens whose differences are 0.5, -1, 2, 0, -0.25, 4."""
    lp = _t([[-1.0, -2.0, -0.5], [-3.0, -1.25, -0.5]])
    rollout = _t([[-1.5, -1.0, -2.5], [-3.0, -1.0, -4.5]])
    assert O.minibatch_rollout_logprob_diff_metrics(lp, None, None) == {}
    pre = "minibatch_rollout_logprobs_abs_diff"
    m = O.minibatch_rollout_logprob_diff_metrics(lp, rollout, None)
    assert sorted(m) == [f"{pre}_max", f"{pre}_mean", f"{pre}_min", f"{pre}_sq_mean"]
    assert m[f"{pre}_mean"] == pytest.approx(7.75 / 6) and m[f"{pre}_sq_mean"] == pytest.approx((0.25 + 1 + 4 + 0 + 0.0625 + 16) / 6)
    assert m[f"{pre}_max"] == 4.0 and m[f"{pre}_min"] == 0.0
    mask = _t([[1, 1, 0], [0, 1, 0]])                              # the tokens with 0.5, 1 and 0.25
    m = O.minibatch_rollout_logprob_diff_metrics(lp, rollout, mask)
    assert m[f"{pre}_mean"] == pytest.approx(1.75 / 3) and m[f"{pre}_sq_mean"] == pytest.approx(1.3125 / 3)
    assert m[f"{pre}_max"] == 1.0 and m[f"{pre}_min"] == 0.0       # masked tokens count as 0 in the extremes
    half = _t([[0.5, 1, 0], [0, 0, 2]])                           # weights: 0.5 * 0.5, 1 * 1, 2 * 4 over a weight sum of 3.5
    m = O.minibatch_rollout_logprob_diff_metrics(lp, rollout, half)
    assert m[f"{pre}_mean"] == pytest.approx(9.25 / 3.5) and m[f"{pre}_sq_mean"] == pytest.approx((0.125 + 1 + 32) / 3.5)
    assert m[f"{pre}_max"] == 8.0
    none = torch.zeros(2, 3, dtype=torch.float64)                  # nothing counts: the denominators are clamped at 1
    m = O.minibatch_rollout_logprob_diff_metrics(lp, rollout, none)
    assert (m[f"{pre}_mean"], m[f"{pre}_sq_mean"], m[f"{pre}_max"], m[f"{pre}_min"]) == (0.0, 0.0, 0.0, 0.0)
