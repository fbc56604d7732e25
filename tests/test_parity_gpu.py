"""GPU parity tests: the HIP path (through the C ABI) against the CPU oracle, the golden vectors and size-independent properties.

Tolerances are the ones the task states for this path: log-probabilities within 2e-2 absolute, entropy within 1e-2 relative,
gradient cosine similarity >= 0.999, all against an fp32 (here fp64) statement of the reference on the same seeded inputs.
Where a comparison is tighter than that, the tighter bound documents what the kernel actually achieves.
"""

import glob
import math
import os

import numpy as np
import pytest
import torch

from oracle import lmhead_oracle as O
from skyrl_amd import _lib, model_utils, ops
from skyrl_amd.bench_inputs import CONFIGS, SMALL_TWINS, make_inputs
from skyrl_amd.fused_linear_logprob_hip import FusedLinearLogprobHip, linear_cross_entropy

pytestmark = pytest.mark.gpu

LOGPROB_ATOL = 2e-2
ENTROPY_RTOL = 1e-2
GRAD_COS = 0.999
GOLDEN = sorted(glob.glob(os.path.join(os.path.dirname(__file__), "golden", "*.npz")))
SENTINEL = torch.iinfo(torch.int64).max


def cos(a, b):
    a, b = a.detach().double().flatten().cpu(), b.detach().double().flatten().cpu()
    return float(torch.dot(a, b) / (a.norm() * b.norm()).clamp_min(1e-300))


def rel_l2(a, b):
    a, b = a.detach().double().cpu(), b.detach().double().cpu()
    return float((a - b).norm() / b.norm().clamp_min(1e-300))


def worst_row(a, b):
    """Largest row-wise relative L2 distance of ``a`` from ``b`` ([rows, cols]).  A row is measured against its own norm, with a
    floor of 1e-3 of the largest row norm so that rows that are (nearly) zero in ``b`` are held to an absolute bound instead.
    One wrong row -- a ragged tile edge, one vocabulary row -- stands out here however many good rows surround it."""
    a, b = a.detach().double().cpu(), b.detach().double().cpu()
    a, b = a.reshape(-1, a.shape[-1]), b.reshape(-1, b.shape[-1])
    norms = b.norm(dim=1)
    floor = 1e-3 * float(norms.max().clamp_min(1e-300))
    return float(((a - b).norm(dim=1) / norms.clamp_min(floor)).max())


GRAD_REL_L2 = 1e-2    # whole gradient; dz is rounded to bf16 once (2^-9 per element), d_hidden is stored in bf16
GRAD_ROW_REL_L2 = 5e-2  # every single row of it


def check_grads(d_hidden, d_weight, ref, tag=""):
    c1, c2 = cos(d_hidden, ref["d_hidden"]), cos(d_weight, ref["d_weight"])
    assert c1 >= GRAD_COS and c2 >= GRAD_COS, f"{tag} grad cosine dH {c1} dW {c2}"
    r1, r2 = rel_l2(d_hidden, ref["d_hidden"]), rel_l2(d_weight, ref["d_weight"])
    assert r1 < GRAD_REL_L2 and r2 < GRAD_REL_L2, f"{tag} grad rel L2 dH {r1} dW {r2}"
    w1, w2 = worst_row(d_hidden, ref["d_hidden"]), worst_row(d_weight, ref["d_weight"])
    assert w1 < GRAD_ROW_REL_L2 and w2 < GRAD_ROW_REL_L2, f"{tag} worst row rel L2 dH {w1} dW {w2}"


def run_hip(dev, hidden, weight, labels, temperature, g=None, q=None, want_entropy=True, vocab_chunk=0):
    h, w, y = hidden.to(dev), weight.to(dev), labels.to(dev)
    lp, ent, lse, pz = ops.lmhead_fwd(h, w, y, 1.0 / temperature, want_entropy)
    out = {"logprobs": lp.cpu(), "lse": lse.cpu()}
    if want_entropy:
        out["entropy"], out["pz"] = ent.cpu(), pz.cpu()
    if g is not None:
        dh, dw = ops.lmhead_bwd(h, w, y, lse, pz if q is not None else None, g.to(dev), None if q is None else q.to(dev),
                                1.0 / temperature, vocab_chunk)
        out["d_hidden"], out["d_weight"] = dh.cpu(), dw.cpu()
    torch.cuda.synchronize()
    return out


def check_against(out, ref, want_entropy, backward, tag=""):
    assert out["logprobs"].dtype == torch.float32
    err = (out["logprobs"].double() - ref["logprobs"].double()).abs().max().item()
    assert err <= LOGPROB_ATOL, f"{tag} logprob max abs err {err}"
    if want_entropy:
        rel = ((out["entropy"].double() - ref["entropy"].double()).abs() / ref["entropy"].double().abs().clamp_min(1e-3)).max().item()
        assert rel <= ENTROPY_RTOL, f"{tag} entropy max rel err {rel}"
    if backward:
        assert out["d_hidden"].dtype == torch.bfloat16 and out["d_weight"].dtype == torch.float32
        check_grads(out["d_hidden"], out["d_weight"], ref, tag)
    return err


# ---------------------------------------------------------------------------------------------------------------------
# the five benchmark configurations at CPU-checkable size
# ---------------------------------------------------------------------------------------------------------------------
@pytest.mark.parametrize("name", list(SMALL_TWINS))
def test_small_twin_of_each_config(name, cuda_device):
    cfg = SMALL_TWINS[name]
    d = make_inputs(cfg)
    g = d.get("dlogprobs")
    q = d.get("dentropy")
    out = run_hip(cuda_device, d["hidden"], d["weight"], d["labels"], cfg.temperature, g, q, cfg.entropy)
    # (1) exact statement (fp64): the "fp32 reference" of the acceptance criterion
    ex = O.exact_fwd_bwd(d["hidden"], d["weight"], d["labels"], cfg.temperature, g, q)
    err = check_against(out, ex, cfg.entropy, cfg.backward, f"{name} vs exact")
    assert err < 1e-3  # fp32 accumulation of exact bf16 products: far inside the stated tolerance
    if cfg.backward:
        # dz is rounded to bf16 once (as the reference does): ~2^-9 relative noise per element
        assert rel_l2(out["d_hidden"], ex["d_hidden"]) < 1e-2 and rel_l2(out["d_weight"], ex["d_weight"]) < 1e-2
    # (2) the reference's torch implementation run on fp32 copies of the same operands
    rf = O.reference_faithful_fwd_bwd(d["hidden"].float(), d["weight"].float(), d["labels"], cfg.temperature,
                                      g if q is None else None, chunk_size=128, want_entropy=cfg.entropy)
    check_against(out, rf, cfg.entropy, cfg.backward and q is None, f"{name} vs reference(fp32 operands)")
    # (3) ... and on the bf16 operands as the trainer runs it.  That path rounds W/temperature and every logit to bf16
    #     (model_utils.py:739-740, 331-333), so it sits up to ~2^-4 away from the exact value itself; the HIP result must
    #     lie inside that path's own error ball: |hip - ref_bf16| <= |ref_bf16 - exact| + 2e-3 for every token.
    rb = O.reference_faithful_fwd_bwd(d["hidden"], d["weight"], d["labels"], cfg.temperature, g if q is None else None,
                                      chunk_size=128, want_entropy=cfg.entropy)
    diff = (out["logprobs"].double() - rb["logprobs"].double()).abs()
    ref_err = (rb["logprobs"].double() - ex["logprobs"].double()).abs()
    excess = (diff - ref_err).max().item()
    assert excess <= 2e-3, f"{name} vs reference(bf16 operands): exceeds the reference's own rounding error by {excess}"
    assert diff.max().item() < 0.25, f"{name}: {diff.max().item()}"
    if cfg.backward and q is None:
        assert cos(out["d_hidden"], rb["d_hidden"]) >= GRAD_COS and cos(out["d_weight"], rb["d_weight"]) >= GRAD_COS
    # masked tokens (g = 0 and no entropy gradient) get exactly zero dHidden rows
    if cfg.backward and q is None:
        masked = d["mask"] == 0
        if masked.any():
            assert out["d_hidden"][masked].abs().max().item() == 0.0


@pytest.mark.parametrize("path", GOLDEN, ids=[os.path.basename(p)[:-4] for p in GOLDEN])
def test_golden_vectors(path, cuda_device):
    z = np.load(path, allow_pickle=False)
    hidden = torch.from_numpy(z["hidden_bits"]).view(torch.bfloat16)
    weight = torch.from_numpy(z["weight_bits"]).view(torch.bfloat16)
    labels = torch.from_numpy(z["labels"])
    t = float(z["temperature"])
    g, q = torch.from_numpy(z["dlogprobs"]), torch.from_numpy(z["dentropy"])
    out = run_hip(cuda_device, hidden, weight, labels, t, g, q, True)
    ref = {k: torch.from_numpy(z[k]) for k in ("logprobs", "entropy", "d_hidden", "d_weight")}
    err = check_against(out, ref, True, True, os.path.basename(path))
    assert err < 1e-3


# ---------------------------------------------------------------------------------------------------------------------
# edge cases (the reference's: S=1, all in / all out of vocabulary, V=8 -- test_fused_linear_logprob.py:122-141 -- plus
# ragged tile edges, strided rows, several vocab chunks, accumulation)
# ---------------------------------------------------------------------------------------------------------------------
def _rand(T, H, V, seed, oov=None):
    gen = torch.Generator().manual_seed(seed)
    hidden = torch.randn(T, H, generator=gen).to(torch.bfloat16)
    weight = (torch.randn(V, H, generator=gen) * 3 / H**0.5).to(torch.bfloat16)
    labels = torch.randint(0, V, (T,), generator=gen)
    if oov == "all":
        labels[:] = SENTINEL
    elif oov == "some":
        labels[::3] = SENTINEL
        labels[1::7] = -5
    g = torch.randn(T, generator=gen)
    q = torch.randn(T, generator=gen) * 0.2
    return hidden, weight, labels, g, q


@pytest.mark.parametrize(
    "T,H,V,temperature,oov,vc",
    [
        (1, 64, 8, 1.0, None, 0),
        (1, 128, 300, 0.7, "all", 0),
        (5, 64, 8, 1.0, "some", 0),
        (255, 64, 257, 1.0, None, 0),
        (257, 192, 255, 1.3, "some", 0),
        (300, 128, 1001, 0.6, None, 256),
        (513, 256, 3000, 1.0, "some", 1024),
        (64, 64, 5000, 2.0, "all", 2048),
        # vocabularies that are multiples of 64: the dHidden GEMM reads the weight in place (K-major), also with a hidden size
        # that is not a multiple of the tile (overhanging columns) and ragged token counts
        (300, 192, 1024, 0.8, None, 0),
        (257, 128, 64, 1.0, "some", 0),
        (100, 320, 4096, 1.0, None, 1024),
        (513, 448, 1984, 0.6, "some", 512),
    ],
)
def test_edge_shapes(T, H, V, temperature, oov, vc, cuda_device):
    hidden, weight, labels, g, q = _rand(T, H, V, seed=T * 7 + V, oov=oov)
    out = run_hip(cuda_device, hidden, weight, labels, temperature, g, q, True, vc)
    ex = O.exact_fwd_bwd(hidden, weight, labels, temperature, g, q)
    err = check_against(out, ex, True, True, f"T={T} H={H} V={V}")
    assert err < 1e-3
    inside = (labels >= 0) & (labels < V)
    assert (out["logprobs"][~inside] == 0).all()
    assert (out["logprobs"] <= 1e-6).all()
    assert (out["entropy"] >= -1e-4).all() and (out["entropy"] <= math.log(V) + 1e-4).all()


def test_random_shapes_against_the_oracle(cuda_device):
    """Seeded sweep over ragged shapes: token counts and vocabulary sizes that are not multiples of any tile edge, every
    hidden size class, chunk widths that split the vocabulary unevenly, temperatures, with and without an entropy gradient."""
    gen = torch.Generator().manual_seed(2024)
    ri = lambda lo, hi: int(torch.randint(lo, hi + 1, (1,), generator=gen))  # noqa: E731
    for case in range(24):
        T, H, V = ri(1, 700), 64 * ri(1, 8), ri(2, 3500)
        temperature = [1.0, 0.6, 1.7][ri(0, 2)]
        oov = [None, "some", "all"][ri(0, 2)] if case % 3 == 0 else None
        vc = [0, 256, 512, 1024][ri(0, 3)]
        use_q = case % 2 == 0
        hidden, weight, labels, g, q = _rand(T, H, V, seed=1000 + case, oov=oov)
        tag = f"case {case}: T={T} H={H} V={V} t={temperature} oov={oov} vc={vc} q={use_q}"
        print(tag, flush=True)
        out = run_hip(cuda_device, hidden, weight, labels, temperature, g, q if use_q else None, True, vc)
        ex = O.exact_fwd_bwd(hidden, weight, labels, temperature, g, q if use_q else None)
        check_against(out, ex, True, True, tag)
        assert torch.isfinite(out["d_hidden"].float()).all() and torch.isfinite(out["d_weight"]).all(), tag


def test_zero_weight_known_answer(cuda_device):
    T, H, V = 70, 64, 1000
    hidden = torch.randn(T, H).to(torch.bfloat16)
    weight = torch.zeros(V, H, dtype=torch.bfloat16)
    labels = torch.randint(0, V, (T,))
    out = run_hip(cuda_device, hidden, weight, labels, 1.0)
    torch.testing.assert_close(out["logprobs"], torch.full((T,), -math.log(V)), atol=1e-5, rtol=0)
    torch.testing.assert_close(out["entropy"], torch.full((T,), math.log(V)), atol=1e-5, rtol=0)


def test_empty_micro_batch(cuda_device):
    """Zero tokens: empty outputs, a zero weight gradient, no launch (the C ABI itself rejects T < 1)."""
    from types import SimpleNamespace

    from skyrl_amd.policy_loss import ppo_policy_loss

    H, V = 128, 512
    hidden = torch.zeros(1, 0, H, dtype=torch.bfloat16, device=cuda_device, requires_grad=True)
    weight = torch.randn(V, H, device=cuda_device).bfloat16().requires_grad_(True)
    target = torch.zeros(1, 0, dtype=torch.int64, device=cuda_device)
    lp = FusedLinearLogprobHip.apply(hidden, weight, target, 0, V, 1024, None, False)
    assert lp.shape == (1, 0) and lp.dtype == torch.float32
    cfg = SimpleNamespace(policy_loss_type="regular", eps_clip_low=0.2, eps_clip_high=0.2)
    loss, metrics = ppo_policy_loss(lp, torch.zeros_like(lp), torch.zeros_like(lp), cfg, torch.zeros_like(lp))
    assert loss.item() == 0.0 and metrics["clip_ratio"] == 0.0
    loss.backward()
    assert hidden.grad.shape == hidden.shape and float(weight.grad.abs().max()) == 0.0
    lp2, ent2 = linear_cross_entropy(hidden.detach()[0], weight.detach(), target[0], 1.0, "none")
    assert lp2.numel() == 0 and ent2.numel() == 0


def test_adapter_corner_cases(cuda_device):
    """Strided and int32 target ids through both adapters, the log-probability-only temperature path, an empty micro-batch into
    an accumulating weight gradient, and a loss built on an output that carries no gradient."""
    dev = cuda_device
    B, S, H, V = 2, 150, 128, 2000
    gen = torch.Generator().manual_seed(21)
    hidden = torch.randn(B, S, H, generator=gen).bfloat16()
    weight = (torch.randn(V, H, generator=gen) * 3 / H**0.5).bfloat16()
    wide = torch.randint(0, V, (B, 2 * S), generator=gen)
    g = torch.randn(B, S, generator=gen)
    target = wide[:, ::2]                                   # non-contiguous view
    ex = O.exact_fwd_bwd(hidden.reshape(-1, H), weight, target.reshape(-1), 0.7, g.reshape(-1), None)
    for ids in (target.to(dev), target.to(torch.int32).to(dev)):
        h = hidden.to(dev).requires_grad_(True)
        w = weight.to(dev).requires_grad_(True)
        lp = model_utils._fused_lm_head_logprob_apply("hip", h, w, ids, 0, V, 64, None, False, temperature=0.7)
        lp.backward(g.to(dev))
        assert (lp.cpu().double().reshape(-1) - ex["logprobs"]).abs().max() <= 1e-3
        check_grads(h.grad.reshape(-1, H), w.grad.float(), ex, "temperature path")
        h1 = hidden.to(dev).requires_grad_(True)
        lp1 = FusedLinearLogprobHip.apply(h1, weight.to(dev), ids, 0, V, 64, None, False)
        lp1.sum().backward()
        assert h1.grad.shape == h1.shape
        # verl interface with a strided 1-D label tensor, entropy output unused: the backward gets no entropy gradient
        h2 = hidden.to(dev).reshape(-1, H).requires_grad_(True)
        lp2, ent2 = linear_cross_entropy(h2, weight.to(dev), wide.to(dev).reshape(-1)[::2].to(ids.dtype), 0.7, "none")
        assert ent2 is not None and torch.equal(lp2.reshape(B, S), lp.detach())
        lp2.backward(g.to(dev).reshape(-1))
        assert torch.equal(h2.grad, h.grad.reshape(-1, H))
    # an empty micro-batch adds nothing to an accumulating weight gradient
    acc = torch.ones(V, H, dtype=torch.float32, device=dev)
    e = torch.empty(0, device=dev)
    dh = ops.lmhead_bwd_accumulate(torch.empty(0, H, dtype=torch.bfloat16, device=dev), weight.to(dev),
                                   torch.empty(0, dtype=torch.int64, device=dev), e, None, e, None, 1.0, acc)
    assert dh.shape == (0, H) and float((acc - 1).abs().max()) == 0.0
    with pytest.raises(ValueError, match="vocab_chunk"):
        ops.lmhead_bwd(hidden.to(dev).reshape(-1, H), weight.to(dev), target.reshape(-1).contiguous().to(dev),
                       torch.zeros(B * S, device=dev), None, torch.zeros(B * S, device=dev), None, 1.0, 100)
    # row_lse / row_pz of the custom op are inputs of its backward, not differentiable results
    h3 = hidden.to(dev).reshape(-1, H).requires_grad_(True)
    _, _, lse3, _ = ops.lmhead_fwd(h3, weight.to(dev), target.reshape(-1).contiguous().to(dev), 1.0, True)
    with pytest.raises(NotImplementedError, match="row_lse"):
        lse3.square().sum().backward()


@pytest.mark.parametrize("with_oov_targets", [False, True])
@pytest.mark.parametrize("hidden_dtype", [torch.bfloat16, torch.float32])
def test_fp32_weight_matches_the_fp32_product(hidden_dtype, with_oov_targets, cuda_device):
    """The reference's dtype matrix (tests/backends/skyrl_train/gpu/gpu_ci/megatron/test_fused_linear_logprob.py:89-118): an fp32
    output weight with a bf16 or an fp32 hidden, same shapes, same upstream gradient, same tolerances -- log-probabilities
    1e-5, grad_hidden 2e-3, grad_weight 2e-3 against logits materialised in fp32 -- and results in the reference's dtypes.
    Here the fp32 operands reach the bf16 matrix pipe as stacked hi / lo terms."""
    dev = cuda_device
    B, S, V, H = 4, 32, 4096, 256
    gen = torch.Generator().manual_seed(0)
    hidden = torch.randn(B, S, H, generator=gen).to(hidden_dtype)
    weight = torch.randn(V, H, generator=gen) * H ** -0.5
    target = torch.randint(0, V + 1024 if with_oov_targets else V, (B, S), generator=gen)
    g = torch.linspace(0.5, 1.5, steps=B * S).reshape(B, S)          # the reference's non-uniform upstream gradient
    h = hidden.to(dev).requires_grad_(True)
    w = weight.to(dev).requires_grad_(True)
    out = FusedLinearLogprobHip.apply(h, w, target.to(dev), 0, V, 64, None, False)
    out.backward(g.to(dev))
    assert out.dtype == torch.float32 and h.grad.dtype == hidden_dtype and w.grad.dtype == torch.float32
    # materialised fp32 logits + autograd, as the reference's own check does (hidden cast to the weight's dtype)
    hr = hidden.float().clone().requires_grad_(True)
    wr = weight.clone().requires_grad_(True)
    logits = hr @ wr.t()
    in_vocab = target < V
    ref = torch.log_softmax(logits, -1).gather(-1, target.clamp(max=V - 1)[..., None])[..., 0] * in_vocab
    # targets outside the shard: forward 0, backward keeps -softmax * g (model_utils.py:337, 405-411), the gradient of -lse * g
    lse = torch.logsumexp(logits, -1)
    ((ref - (~in_vocab) * lse) * g).sum().backward()
    torch.testing.assert_close(out.cpu(), ref.detach(), atol=1e-5, rtol=1e-5)
    torch.testing.assert_close(h.grad.cpu().float(), hr.grad, atol=2e-3, rtol=2e-3)
    torch.testing.assert_close(w.grad.cpu(), wr.grad, atol=2e-3, rtol=2e-3)
    # the verl interface with temperature and a grad-carrying entropy, against the fp64 statement
    q = torch.randn(B * S, generator=gen) * 0.1
    h2 = hidden.reshape(-1, H).to(dev).requires_grad_(True)
    w2 = weight.to(dev).requires_grad_(True)
    labels = torch.where(in_vocab, target, SENTINEL).reshape(-1)
    lp, ent = linear_cross_entropy(h2, w2, labels.to(dev), 0.7, "none")
    (lp * g.reshape(-1).to(dev) + ent * q.to(dev)).sum().backward()
    ex = O.exact_fwd_bwd(hidden.reshape(-1, H), weight, labels, 0.7, g.reshape(-1), q)
    lp_err = float((lp.detach().cpu().double() - ex["logprobs"]).abs().max())
    ent_err = float(((ent.detach().cpu().double() - ex["entropy"]).abs() / ex["entropy"].abs()).max())
    assert lp_err <= 5e-5 and ent_err <= 2e-5, (lp_err, ent_err)
    check_grads(h2.grad, w2.grad, ex, "fp32 weight, entropy gradient")
    # rows without upstream gradient are dropped on this path too
    gm = g.reshape(-1).clone()
    gm[::2] = 0
    _, _, lse_d, _ = ops.lmhead_fwd(h2.detach(), w2.detach(), labels.to(dev), 1.0, False)
    dense = ops.lmhead_bwd(h2.detach(), w2.detach(), labels.to(dev), lse_d, None, gm.to(dev), None, 1.0, 0)
    compact = ops.lmhead_bwd(h2.detach(), w2.detach(), labels.to(dev), lse_d, None, gm.to(dev), None, 1.0, 0, True)
    assert float(compact[0][::2].abs().max()) == 0.0 and torch.equal(compact[0][1::2], dense[0][1::2])
    assert rel_l2(compact[1], dense[1]) < 1e-5


@pytest.mark.parametrize("weight_dtype,V,H", [(torch.float32, 152064, 8192), (torch.bfloat16, 139264, 16384)])
def test_operands_beyond_four_gib(weight_dtype, V, H, cuda_device):
    """A weight whose bf16 form exceeds 4 GiB -- the fp32 output layer of a 70B-class model as stacked bf16 terms
    ([152064, 2 * 8192], 4.98 GB), and a plain bf16 [139264, 16384] (4.56 GB): the copy plan addresses every tile from its own
    first row, so rows beyond the 4 GiB mark are read and written like any other.  Half of the labels lie beyond it.  Checked
    on the GPU against the library's fp32 product, log-softmax and autograd (test_fused_linear_logprob.py:71-95)."""
    dev = cuda_device
    T = 192
    gen = torch.Generator(device=dev).manual_seed(11)
    hidden = torch.randn(T, H, generator=gen, device=dev).to(torch.bfloat16)
    weight = (torch.randn(V, H, generator=gen, device=dev) * (2.0 / H ** 0.5)).to(weight_dtype)
    first_high = (1 << 32) // (2 * (2 * H if weight_dtype == torch.float32 else H)) + 1   # first row wholly beyond 4 GiB
    assert first_high < V - 1000
    labels = torch.cat([torch.randint(0, V, (T // 2,), generator=gen, device=dev),
                        torch.randint(first_high, V, (T - T // 2,), generator=gen, device=dev)])
    g = torch.randn(T, generator=gen, device=dev)
    h = hidden.clone().requires_grad_(True)
    w = weight.clone().requires_grad_(True)
    out = FusedLinearLogprobHip.apply(h.view(1, T, H), w, labels.view(1, T), 0, V, 1024, None, False).view(T)
    out.backward(g)
    hr = hidden.float().requires_grad_(True)
    wr = weight.float().requires_grad_(True)
    ref = torch.log_softmax(hr @ wr.t(), -1).gather(-1, labels[:, None])[:, 0]
    (ref * g).sum().backward()
    assert float((out.detach() - ref.detach()).abs().max()) <= (1e-4 if weight_dtype == torch.float32 else 2e-3)
    assert w.grad.dtype == weight_dtype and h.grad.dtype == torch.bfloat16
    for got, want, what in ((h.grad.float(), hr.grad, "grad_hidden"), (w.grad.float(), wr.grad, "grad_weight"),
                            (w.grad[first_high:].float(), wr.grad[first_high:], "grad_weight beyond 4 GiB")):
        c = float(torch.nn.functional.cosine_similarity(got.flatten().double(), want.flatten().double(), dim=0))
        r = float((got.double() - want.double()).norm() / want.double().norm())
        assert c >= 0.9999 and r < GRAD_REL_L2, (what, c, r)   # dz and grad_hidden are rounded to bf16 once each
    hot = labels[T // 2:]                                  # label rows beyond the mark carry the one-hot term
    assert float((w.grad[hot].float() - wr.grad[hot]).abs().max()) <= 2e-2 * float(wr.grad[hot].abs().max())


@pytest.mark.parametrize("entgrad", [False, True])
def test_tiny_dz_flush_option(entgrad, cuda_device):
    """SKYRL_BWD_FLUSH_TINY_DZ (off by default; no counterpart in the reference): softmax probabilities below 2^-24 are taken
    as zero when dz is formed.  The gradients stay inside the path's tolerances against the fp64 statement and close to the
    exact path's; a vocabulary row that no token gives a probability of 2^-24 gets an exactly zero weight gradient, and one
    that some token does keeps that token's term; switched off again, the backward is bit-identical to before."""
    dev = cuda_device
    T, H, V, temperature = 300, 128, 5000, 0.5
    hidden, weight, labels, g, q = _rand(T, H, V, seed=31)
    if not entgrad:
        q = None
    # 200 vocabulary rows that every token finds hopeless: a feature all tokens share, against a large negative weight
    low = torch.arange(100, 300)
    hidden[:, 0] = 4.0
    weight[:, 0] = 0.0
    weight[low, 0] = -8.0
    labels[(labels >= 100) & (labels < 300)] = 7
    ex = O.exact_fwd_bwd(hidden, weight, labels, temperature, g, q)
    h, w, y = hidden.to(dev), weight.to(dev), labels.to(dev)
    _, _, lse, pz = ops.lmhead_fwd(h, w, y, 1.0 / temperature, True)
    args = (h, w, y, lse, pz if entgrad else None, g.to(dev), None if q is None else q.to(dev), 1.0 / temperature, 1024)
    exact = ops.lmhead_bwd(*args)
    assert ops.set_flush_tiny_dz(True) is False
    try:
        flushed = ops.lmhead_bwd(*args)
    finally:
        assert ops.set_flush_tiny_dz(False) is True
    again = ops.lmhead_bwd(*args)
    assert torch.equal(again[0], exact[0]) and torch.equal(again[1], exact[1])
    check_grads(flushed[0].cpu(), flushed[1].cpu(), ex, "tiny dz flushed")
    assert rel_l2(flushed[0].float(), exact[0].float()) < 1e-3 and rel_l2(flushed[1], exact[1]) < 1e-3
    # probabilities in fp64: which vocabulary rows are below / above the threshold for every / some token
    z = (hidden.double() @ weight.double().t()) / temperature
    p = torch.softmax(z, -1)
    is_label = torch.zeros(V, dtype=torch.bool)
    is_label[labels] = True
    never = (p.max(0).values < 2.0 ** -25) & ~is_label
    some = (p.max(0).values > 2.0 ** -20) & ~is_label
    assert int(never.sum()) > 50 and int(some.sum()) > 50, (int(never.sum()), int(some.sum()))
    assert float(flushed[1][never.to(dev)].abs().max()) == 0.0
    assert float(exact[1][never.to(dev)].abs().max()) > 0.0
    kept = flushed[1][some.to(dev)].cpu().double()
    assert rel_l2(kept, ex["d_weight"][some]) < GRAD_REL_L2
    share = float((p < 2.0 ** -24).double().mean())
    assert share > 0.5                                       # most of the panel is zeros on a peaked distribution


def test_fp32_weight_gradient_spread_run_to_run(cuda_device):
    """The one place with atomics: on the fp32-weight path the label term of dW is added with fp32 atomic adds (tokens may
    share a label), so the last bits of those rows depend on the order of the adds.  Many tokens on few labels, several runs:
    d_hidden is bit-identical, d_weight rows without a label are bit-identical, label rows agree to fp32 rounding."""
    dev = cuda_device
    T, H, V = 2048, 128, 1024
    gen = torch.Generator().manual_seed(3)
    hidden = torch.randn(T, H, generator=gen).to(torch.bfloat16).to(dev)
    weight = (torch.randn(V, H, generator=gen) * 3 / H ** 0.5).to(dev)          # fp32
    labels = torch.randint(0, 16, (T,), generator=gen).to(dev)                   # 128 tokens per label
    g = torch.randn(T, generator=gen).to(dev)
    _, _, lse, _ = ops.lmhead_fwd(hidden, weight, labels, 1.0, False)
    runs = [ops.lmhead_bwd(hidden, weight, labels, lse, None, g, None, 1.0, 0) for _ in range(4)]
    for dh, dw in runs[1:]:
        assert torch.equal(dh, runs[0][0])
        assert torch.equal(dw[16:], runs[0][1][16:])
        spread = float((dw[:16] - runs[0][1][:16]).abs().max())
        assert spread <= 1e-5 * float(runs[0][1][:16].abs().max()), spread


def test_extreme_logits(cuda_device):
    # one dominant logit -> logprob, entropy -> 0; all logits very negative -> the split merge must not underflow
    T, H, V = 40, 64, 700
    hidden = torch.zeros(T, H)
    hidden[:, 0] = 1.0
    weight = torch.zeros(V, H)
    weight[13, 0] = 200.0
    out = run_hip(cuda_device, hidden.bfloat16(), weight.bfloat16(), torch.full((T,), 13), 1.0)
    assert out["logprobs"].abs().max().item() < 1e-4 and out["entropy"].abs().max().item() < 1e-4  # fp32 ulp at lse = 200 is 1.5e-5
    weight = torch.full((V, H), 0.0)
    weight[:, 0] = -300.0 - torch.arange(V) * 0.25
    hb, wb = hidden.bfloat16(), weight.bfloat16()
    labels = torch.randint(0, V, (T,))
    out = run_hip(cuda_device, hb, wb, labels, 1.0)
    ex = O.exact_fwd_bwd(hb, wb, labels, 1.0)
    assert torch.isfinite(out["logprobs"]).all() and torch.isfinite(out["entropy"]).all()
    torch.testing.assert_close(out["logprobs"].double(), ex["logprobs"], atol=1e-3, rtol=1e-5)
    torch.testing.assert_close(out["lse"].double(), ex["lse"], atol=1e-3, rtol=1e-6)


def test_strided_rows_and_no_entropy_path(cuda_device):
    T, H, V = 200, 128, 900
    hidden, weight, labels, g, _ = _rand(T, H, V, seed=5)
    big_h = torch.zeros(T, H + 64, dtype=torch.bfloat16, device=cuda_device)
    big_w = torch.zeros(V, H + 8, dtype=torch.bfloat16, device=cuda_device)
    big_h[:, :H] = hidden.to(cuda_device)
    big_w[:, :H] = weight.to(cuda_device)
    hv, wv = big_h[:, :H], big_w[:, :H]
    assert hv.stride(0) == H + 64 and not hv.is_contiguous()
    y = labels.to(cuda_device)
    lp, ent, lse, pz = ops.lmhead_fwd(hv, wv, y, 1.0, False)
    assert ent.numel() == 0 and pz.numel() == 0
    dh, dw = ops.lmhead_bwd(hv, wv, y, lse, None, g.to(cuda_device), None, 1.0, 0)
    ex = O.exact_fwd_bwd(hidden, weight, labels, 1.0, g, None)
    check_against({"logprobs": lp.cpu(), "d_hidden": dh.cpu(), "d_weight": dw.cpu()}, ex, False, True)


def test_vocab_chunk_invariance_and_accumulate(cuda_device):
    T, H, V = 400, 128, 3000
    hidden, weight, labels, g, q = _rand(T, H, V, seed=9, oov="some")
    dev = cuda_device
    h, w, y, gd, qd = (x.to(dev) for x in (hidden, weight, labels, g, q))
    lp, ent, lse, pz = ops.lmhead_fwd(h, w, y, 1.0, True)
    ref_dh, ref_dw = ops.lmhead_bwd(h, w, y, lse, pz, gd, qd, 1.0, 0)
    for vc in (256, 768, 4096):
        dh, dw = ops.lmhead_bwd(h, w, y, lse, pz, gd, qd, 1.0, vc)
        # dW rows are complete within one chunk: bit-identical.  dHidden sums chunk partials in a different order.
        assert torch.equal(dw, ref_dw)
        assert rel_l2(dh.float(), ref_dh.float()) < 1e-2
    acc = torch.full((V, H), 0.5, dtype=torch.float32, device=dev)
    dh2 = ops.lmhead_bwd_accumulate(h, w, y, lse, pz, gd, qd, 1.0, acc, 768)
    torch.testing.assert_close(acc, ref_dw + 0.5, atol=1e-6, rtol=1e-6)
    with pytest.raises(ValueError):
        ops.lmhead_bwd(h, w, y, lse, pz, gd, qd, 1.0, 100)


def test_backward_is_linear_in_upstream_grads_and_deterministic(cuda_device):
    T, H, V = 300, 128, 2000
    hidden, weight, labels, g, q = _rand(T, H, V, seed=21)
    dev = cuda_device
    h, w, y, gd, qd = (x.to(dev) for x in (hidden, weight, labels, g, q))
    lp, ent, lse, pz = ops.lmhead_fwd(h, w, y, 1.0 / 0.8, True)
    z = torch.zeros_like(gd)
    a = ops.lmhead_bwd(h, w, y, lse, pz, gd, z, 1.0 / 0.8, 0)
    b = ops.lmhead_bwd(h, w, y, lse, pz, z, qd, 1.0 / 0.8, 0)
    c = ops.lmhead_bwd(h, w, y, lse, pz, gd, qd, 1.0 / 0.8, 0)
    c2 = ops.lmhead_bwd(h, w, y, lse, pz, gd, qd, 1.0 / 0.8, 0)
    assert torch.equal(c[0], c2[0]) and torch.equal(c[1], c2[1])  # no atomics anywhere: bit-reproducible
    assert rel_l2(a[1] + b[1], c[1]) < 1e-2 and rel_l2(a[0].float() + b[0].float(), c[0].float()) < 2e-2
    lp2, *_ = ops.lmhead_fwd(h, w, y, 1.0 / 0.8, True)
    assert torch.equal(lp, lp2)


def test_backward_skips_rows_without_upstream_gradient(cuda_device):
    # the masked configurations (prompt tokens carry no gradient): compacted and dense backward agree, masked rows are exactly 0
    cfg = SMALL_TWINS["qwen2.5-1.5b-fwdbwd"]
    d = make_inputs(cfg)
    dev = cuda_device
    h, w, y, g = (d[k].to(dev) for k in ("hidden", "weight", "labels", "dlogprobs"))
    lp, _, lse, _ = ops.lmhead_fwd(h, w, y, 1.0, False)
    dense = ops.lmhead_bwd(h, w, y, lse, None, g, None, 1.0, 0)
    compact = ops.lmhead_bwd_active_rows(h, w, y, lse, None, g, None, 1.0, 0)
    masked = (d["mask"] == 0).to(dev)
    assert masked.float().mean().item() == pytest.approx(0.5)
    assert compact[0][masked].abs().max().item() == 0.0
    assert rel_l2(compact[0].float(), dense[0].float()) < 2e-2 and rel_l2(compact[1], dense[1]) < 1e-3
    ex = O.exact_fwd_bwd(d["hidden"], d["weight"], d["labels"], 1.0, d["dlogprobs"], None)
    check_grads(compact[0], compact[1], ex, "compacted")
    # all-zero upstream gradient: zeros
    z = ops.lmhead_bwd_active_rows(h, w, y, lse, None, torch.zeros_like(g), None, 1.0, 0)
    assert z[0].abs().max().item() == 0.0 and z[1].abs().max().item() == 0.0
    # through autograd (FusedLinearLogprobHip uses the compacting path)
    B, S = cfg.n_seqs, cfg.T // cfg.n_seqs
    hd = d["hidden"].reshape(B, S, cfg.H).to(dev).requires_grad_(True)
    wd = w.clone().requires_grad_(True)
    out = FusedLinearLogprobHip.apply(hd, wd, d["labels"].reshape(B, S).to(dev), 0, cfg.V, S, None, False)
    (out * g.reshape(B, S)).sum().backward()
    assert cos(hd.grad.reshape(-1, cfg.H), ex["d_hidden"]) >= GRAD_COS and cos(wd.grad, ex["d_weight"]) >= GRAD_COS


@pytest.mark.parametrize("T,H,V,vc,keep,entgrad", [
    (700, 128, 2048, 512, 0.4, True),     # four vocab chunks: the dHidden partial sums cross chunks under a device-side count
    (700, 128, 2001, 0, 0.4, False),      # V not a multiple of 64: the dHidden GEMM on the transposed weight copy
    (515, 64, 900, 256, 0.999, True),     # (nearly) everything active
    (1000, 192, 1500, 0, 0.003, False),   # a handful of active rows: far less than one tile
    (300, 64, 777, 0, 0.5, True),
])
def test_active_rows_backward_equals_the_backward_on_gathered_rows(T, H, V, vc, keep, entgrad, cuda_device):
    """skyrl_lmhead_bwd_active_rows compacts on the device; the same compaction done here with torch indexing, followed by the
    dense backward, must give the same bits: d_weight of the compacted problem, d_hidden rows scattered back, zeros elsewhere."""
    dev = cuda_device
    hidden, weight, labels, g, q = _rand(T, H, V, seed=int(1000 * keep) + T)
    gen = torch.Generator().manual_seed(T + V)
    active = torch.rand(T, generator=gen) < keep
    if keep > 0.9:
        active[:] = True
        active[T // 2] = False
    g = g * active
    q = q * active if entgrad else None
    h, w, y = hidden.to(dev), weight.to(dev), labels.to(dev)
    gd, qd = g.to(dev), None if q is None else q.to(dev)
    _, _, lse, pz = ops.lmhead_fwd(h, w, y, 1.0 / 0.9, True)
    pzq = pz if entgrad else None
    idx = active.nonzero()[:, 0].to(dev)
    take = lambda t: None if t is None else t.index_select(0, idx)  # noqa: E731
    for op, kw in ((ops.lmhead_bwd, {}), (ops.lmhead_bwd_bf16, {}), (ops.lmhead_bwd_hidden, {})):
        got = op(h, w, y, lse, pzq, gd, qd, 1.0 / 0.9, vc, True)
        want = op(take(h), w, take(y), take(lse), take(pzq), take(gd), take(qd), 1.0 / 0.9, vc)
        got, want = (got, want) if isinstance(got, tuple) else ((got,), (want,))
        full = torch.zeros(T, H, dtype=torch.bfloat16, device=dev)
        full.index_copy_(0, idx, want[0])
        assert torch.equal(got[0], full), op.__name__
        if len(got) > 1:
            assert torch.equal(got[1], want[1]), op.__name__
    # and against the oracle
    dh, dw = ops.lmhead_bwd(h, w, y, lse, pzq, gd, qd, 1.0 / 0.9, vc, True)
    ex = O.exact_fwd_bwd(hidden, weight, labels, 0.9, g, q)
    check_grads(dh, dw, ex, "active rows")
    # accumulation into an existing dW goes through the same entry point
    lib = _lib.load()
    acc = torch.full((V, H), 0.5, dtype=torch.float32, device=dev)
    n = lib.skyrl_lmhead_bwd_active_rows_workspace_bytes(T, H, V, vc)
    ws = torch.empty(n, dtype=torch.uint8, device=dev)
    dh2 = torch.empty(T, H, dtype=torch.bfloat16, device=dev)
    st = lib.skyrl_lmhead_bwd_active_rows(h.data_ptr(), H, w.data_ptr(), H, y.data_ptr(), lse.data_ptr(),
                                          None if pzq is None else pzq.data_ptr(), gd.data_ptr(),
                                          None if qd is None else qd.data_ptr(), T, H, V, 1.0 / 0.9, dh2.data_ptr(),
                                          acc.data_ptr(), 1, vc, ws.data_ptr(), n, torch.cuda.current_stream().cuda_stream)
    assert st == 0
    torch.cuda.synchronize()
    assert torch.equal(dh2, dh) and torch.equal(acc, dw + 0.5)
    assert lib.skyrl_lmhead_bwd_active_rows(h.data_ptr(), H, w.data_ptr(), H, y.data_ptr(), lse.data_ptr(), None, gd.data_ptr(),
                                            None, T, H, V, 1.0, dh2.data_ptr(), acc.data_ptr(), 1, vc, ws.data_ptr(), n - 1,
                                            None) == -4


def test_forward_and_backward_in_token_blocks(cuda_device):
    """More than 32768 tokens: both passes walk the tokens in blocks.  Tokens are independent, so each block must reproduce a
    call on that block alone bit for bit, and dW must be the blocks' dW added up -- in every dw_mode, with and without
    row compaction."""
    dev = cuda_device
    T, H, V, cut = 40000, 64, 1000, 32768
    hidden, weight, labels, g, q = _rand(T, H, V, seed=77)
    g[torch.rand(T, generator=torch.Generator().manual_seed(5)) < 0.3] = 0.0
    q = q * (g != 0)
    h, w, y, gd, qd = hidden.to(dev), weight.to(dev), labels.to(dev), g.to(dev), q.to(dev)
    out = ops.lmhead_fwd(h, w, y, 1.0, True)
    parts = [ops.lmhead_fwd(h[a:b], w, y[a:b], 1.0, True) for a, b in ((0, cut), (cut, T))]
    for k in range(4):
        assert torch.equal(out[k], torch.cat([p[k] for p in parts]))
    assert ops.fwd_workspace_bytes(T, H, V) == ops.fwd_workspace_bytes(cut, H, V)
    lse, pz = out[2], out[3]
    halves = [ops.lmhead_bwd(h[a:b], w, y[a:b], lse[a:b], pz[a:b], gd[a:b], qd[a:b], 1.0, 512) for a, b in ((0, cut), (cut, T))]
    want_dh = torch.cat([p[0] for p in halves])
    want_dw = halves[0][1] + halves[1][1]
    for active_rows in (False, True):
        dh, dw = ops.lmhead_bwd(h, w, y, lse, pz, gd, qd, 1.0, 512, active_rows)
        if not active_rows:
            assert torch.equal(dh, want_dh) and torch.equal(dw, want_dw)
        ex_rows = torch.arange(cut - 300, cut + 300)
        assert rel_l2(dh[ex_rows.to(dev)].float(), want_dh[ex_rows.to(dev)].float()) < 1e-2
        assert rel_l2(dw, want_dw) < 1e-3 and worst_row(dw, want_dw) < 2e-2
        _, dwb = ops.lmhead_bwd_bf16(h, w, y, lse, pz, gd, qd, 1.0, 512, active_rows)
        assert torch.equal(dwb, dw.bfloat16())          # summed over the blocks in fp32, rounded once
        acc = torch.full((V, H), -2.0, dtype=torch.float32, device=dev)
        ops._bwd_into(_lib.load(), h, w, y, lse, pz, gd, qd, 1.0, 512, torch.empty_like(h), acc, True, active_rows)
        assert rel_l2(acc + 2.0, dw) < 1e-5           # the same sums, added to what was there in a different order
    ex = O.exact_fwd_bwd(hidden, weight, labels, 1.0, g, q)
    dh, dw = ops.lmhead_bwd(h, w, y, lse, pz, gd, qd, 1.0, 0, True)
    check_grads(dh, dw, ex, "token blocks, active rows")
    assert (out[0].cpu().double() - ex["logprobs"]).abs().max() <= 1e-3


def test_c_abi_called_directly(cuda_device):
    """No torch op wrapper in between: raw pointers into the exported symbols."""
    lib = _lib.load()
    T, H, V = 100, 64, 500
    hidden, weight, labels, g, _ = _rand(T, H, V, seed=3)
    dev = cuda_device
    h, w, y, gd = (x.to(dev) for x in (hidden, weight, labels, g))
    lp = torch.empty(T, device=dev)
    lse = torch.empty(T, device=dev)
    n = lib.skyrl_lmhead_fwd_workspace_bytes(T, H, V)
    ws = torch.empty(n, dtype=torch.uint8, device=dev)
    st = lib.skyrl_lmhead_fwd(h.data_ptr(), H, w.data_ptr(), H, y.data_ptr(), T, H, V, 1.0, lp.data_ptr(), None,
                              lse.data_ptr(), None, ws.data_ptr(), n, torch.cuda.current_stream().cuda_stream)
    assert st == 0
    nb = lib.skyrl_lmhead_bwd_workspace_bytes(T, H, V, 0)
    wsb = torch.empty(nb, dtype=torch.uint8, device=dev)
    dh = torch.empty(T, H, dtype=torch.bfloat16, device=dev)
    dw = torch.empty(V, H, dtype=torch.float32, device=dev)
    st = lib.skyrl_lmhead_bwd(h.data_ptr(), H, w.data_ptr(), H, y.data_ptr(), lse.data_ptr(), None, gd.data_ptr(), None, T, H,
                              V, 1.0, dh.data_ptr(), dw.data_ptr(), 0, 0, wsb.data_ptr(), nb,
                              torch.cuda.current_stream().cuda_stream)
    assert st == 0
    torch.cuda.synchronize()
    ex = O.exact_fwd_bwd(hidden, weight, labels, 1.0, g, None)
    check_against({"logprobs": lp.cpu(), "d_hidden": dh.cpu(), "d_weight": dw.cpu()}, ex, False, True)
    # too-small workspace is refused, nothing is launched
    assert lib.skyrl_lmhead_fwd(h.data_ptr(), H, w.data_ptr(), H, y.data_ptr(), T, H, V, 1.0, lp.data_ptr(), None,
                                lse.data_ptr(), None, ws.data_ptr(), n - 1, None) == -4


# ---------------------------------------------------------------------------------------------------------------------
# the reference's call signatures
# ---------------------------------------------------------------------------------------------------------------------
@pytest.mark.parametrize("loss_type", ["regular", "dual_clip"])
@pytest.mark.parametrize("masked", [False, True])
@pytest.mark.parametrize("B", [6, 67])   # 3102 tokens: one workgroup; 34639 tokens: five slices and their partial sums
def test_ppo_policy_loss_matches_oracle(loss_type, masked, B, cuda_device):
    from types import SimpleNamespace

    from skyrl_amd.policy_loss import ppo_policy_loss

    gen = torch.Generator().manual_seed(5)
    S = 517
    lp = (torch.randn(B, S, generator=gen) * 0.5 - 2.0)
    old = lp + torch.randn(B, S, generator=gen) * 0.3
    old[0, :4] = lp[0, :4]                       # exact ties of the two surrogates
    old[1, 0], old[1, 1] = lp[1, 0] - 30.0, lp[1, 1] + 30.0  # beyond the +-20 clamp
    adv = torch.randn(B, S, generator=gen)
    mask = (torch.rand(B, S, generator=gen) > 0.4).float() if masked else None
    weight = (torch.rand(B, S, generator=gen) + 0.5) if masked else None
    cfg = SimpleNamespace(policy_loss_type=loss_type, eps_clip_low=0.2, eps_clip_high=0.28, clip_ratio_c=3.0)

    ref_lp = lp.double().requires_grad_(True)
    ref_loss, ref_clip = O.ppo_policy_loss(ref_lp, old.double(), adv.double(), 0.2, 0.28, 3.0, loss_type == "dual_clip",
                                           None if mask is None else mask.double(), None if weight is None else weight.double())
    ref_loss.backward()

    dlp = lp.to(cuda_device).requires_grad_(True)
    to = lambda t: None if t is None else t.to(cuda_device)  # noqa: E731
    loss, metrics = ppo_policy_loss(dlp, to(old), to(adv), cfg, to(mask), loss_weight=to(weight))
    loss.backward()
    assert loss.dtype == torch.float32 and isinstance(metrics["clip_ratio"], float)
    # fp32 sum of ~3000 terms, one of them about e^20 (the clamped log-ratio): a relative bound
    assert abs(loss.item() - ref_loss.item()) <= 5e-6 * max(abs(ref_loss.item()), 1e3)
    assert metrics["clip_ratio"] == pytest.approx(ref_clip.item(), abs=1e-6)
    err = (dlp.grad.double().cpu() - ref_lp.grad).abs().max().item()
    assert err <= 1e-5 * max(1.0, ref_lp.grad.abs().max().item()), f"gradient max abs err {err}"
    # scaling the loss scales the gradient; metrics without a host synchronisation come back as tensors
    dlp2 = lp.to(cuda_device).requires_grad_(True)
    loss2, m2 = ppo_policy_loss(dlp2, to(old), to(adv), cfg, to(mask), loss_weight=to(weight), sync_metrics=False)
    (loss2 * 3.0).backward()
    assert torch.equal(dlp2.grad, dlp.grad * 3.0) and torch.is_tensor(m2["clip_ratio"])
    assert loss2.item() == loss.item()                           # fixed summation order: reproducible bit for bit


def test_policy_loss_feeds_the_fused_backward(cuda_device):
    """log-probabilities from the fused forward -> PPO loss -> backward through the fused LM head, against the oracle chain."""
    from types import SimpleNamespace

    from skyrl_amd.policy_loss import ppo_policy_loss

    gen = torch.Generator().manual_seed(9)
    T, H, V = 384, 128, 1000
    hidden = torch.randn(T, H, generator=gen).bfloat16()
    weight = (torch.randn(V, H, generator=gen) * 3 / H ** 0.5).bfloat16()
    labels = torch.randint(0, V, (T,), generator=gen)
    adv = torch.randn(T, generator=gen)
    mask = (torch.rand(T, generator=gen) > 0.5).float()
    cfg = SimpleNamespace(policy_loss_type="regular", eps_clip_low=0.2, eps_clip_high=0.2)

    h64, w64 = hidden.double().requires_grad_(True), weight.double().requires_grad_(True)
    ref_lp = torch.log_softmax(h64 @ w64.t(), -1).gather(-1, labels[:, None])[:, 0]
    old = (ref_lp.detach() + torch.randn(T, generator=gen).double() * 0.3).float()
    O.ppo_policy_loss(ref_lp, old.double(), adv.double(), 0.2, 0.2, loss_mask=mask.double())[0].backward()

    dh = hidden.to(cuda_device).requires_grad_(True)
    dw = weight.to(cuda_device).requires_grad_(True)
    lp = FusedLinearLogprobHip.apply(dh[None], dw, labels.to(cuda_device)[None], 0, V, 1024, None, False)[0]
    loss, _ = ppo_policy_loss(lp, old.to(cuda_device), adv.to(cuda_device), cfg, mask.to(cuda_device))
    loss.backward()
    assert cos(dh.grad.float(), h64.grad) >= GRAD_COS and cos(dw.grad.float(), w64.grad) >= GRAD_COS


@pytest.mark.parametrize("masked", [False, True])
def test_cross_entropy_and_importance_sampling_losses_match_oracle(masked, cuda_device):
    from skyrl_amd.policy_loss import cross_entropy_loss, importance_sampling_loss

    gen = torch.Generator().manual_seed(15)
    B, S = 5, 333
    lp = torch.randn(B, S, generator=gen) * 0.5 - 2.0
    old = lp + torch.randn(B, S, generator=gen) * 0.3
    old[0, 0] = lp[0, 0] - 23.0                    # no clamp in this loss: a ratio of e^23
    adv = torch.randn(B, S, generator=gen)
    mask = (torch.rand(B, S, generator=gen) > 0.4).float() if masked else None
    to = lambda t: None if t is None else t.to(cuda_device)  # noqa: E731
    m64 = None if mask is None else mask.double()

    ref_lp = lp.double().requires_grad_(True)
    ref = O.cross_entropy_loss(ref_lp, m64)
    ref.backward()
    dlp = lp.to(cuda_device).requires_grad_(True)
    loss, metrics = cross_entropy_loss(dlp, None, None, None, to(mask))
    loss.backward()
    assert metrics == {"clip_ratio": 0.0} and loss.item() == pytest.approx(ref.item(), rel=2e-6)
    assert torch.equal(dlp.grad.cpu().double(), ref_lp.grad)

    ref_lp = lp.double().requires_grad_(True)
    ref, ref_ratio = O.importance_sampling_loss(ref_lp, old.double(), adv.double(), m64)
    ref.backward()
    dlp = lp.to(cuda_device).requires_grad_(True)
    loss, metrics = importance_sampling_loss(dlp, to(old), to(adv), None, to(mask))
    loss.backward()
    assert abs(loss.item() - ref.item()) <= 5e-6 * max(abs(ref.item()), float((lp - old).exp().abs().max()))
    assert metrics["importance_ratio"] == pytest.approx(ref_ratio.item(), rel=1e-5)
    err = (dlp.grad.double().cpu() - ref_lp.grad).abs()
    assert bool((err <= 1e-5 * ref_lp.grad.abs().clamp(min=1.0)).all())


def _further_loss_case(kind, masked):
    """Inputs for one of the further loss types, its config, and the oracle's loss / clip ratio / gradient in fp64.  Tokens
    whose branch decision sits within 1e-4 of a threshold in fp64 are moved to ratio 1 so that fp32 takes the same branch."""
    from types import SimpleNamespace

    gen = torch.Generator().manual_seed(31)
    B, S = 7, 411
    lp = (torch.randn(B, S, generator=gen) * 0.7 - 1.5).clamp(max=-0.02)
    old = lp + torch.randn(B, S, generator=gen) * 0.35
    adv = torch.randn(B, S, generator=gen)
    adv[3, :5] = 0.0                                            # A = 0: tau_neg side of SAPO, neither DPPO direction
    mask = None
    if masked:
        mask = (torch.rand(B, S, generator=gen) > 0.4).float()
        mask[2] = 0                                             # a row without loss tokens
        mask[4, :7] = 0.5                                       # fractional weights
    weight = (torch.rand(B, S, generator=gen) + 0.5) if masked else None
    lo, hi = {"sapo": (1.0, 1.05), "gspo": (0.02, 0.03), "cispo": (0.3, 0.5), "rollout_is": (0.3, 0.5),
              "dppo_tv": (0.06, 0.05), "dppo_kl": (0.02, 0.015)}[kind]
    ratio = (lp.double() - old.double()).exp()
    fragile = torch.zeros(B, S, dtype=torch.bool)
    if kind in ("cispo", "rollout_is"):
        fragile = ((ratio - (1 - lo)).abs() < 1e-4) | ((ratio - (1 + hi)).abs() < 1e-4)
    elif kind == "dppo_tv":
        diff = lp.double().exp() - old.double().exp()
        fragile = ((diff - hi).abs() < 1e-4) | ((-diff - lo).abs() < 1e-4)
    elif kind == "dppo_kl":
        p, mu = lp.double().exp(), old.double().exp()
        bkl = mu * (old.double() - lp.double()) + (1 - mu) * torch.log((1 - mu) / (1 - p))
        fragile = ((bkl - hi).abs() < 1e-4) | ((bkl - lo).abs() < 1e-4) | ((p - mu).abs() < 1e-6)
    old = torch.where(fragile, lp, old)
    old[1, 0], old[1, 1] = lp[1, 0] - 30.0, lp[1, 1] + 30.0     # beyond the +-20 clamp of the log-ratio
    if kind == "gspo":
        old[5] = lp[5] - 11.0                                   # a row beyond the clamp of the sequence weight at 10
        row = O.masked_mean(lp.double() - old.double(), None if mask is None else mask.double(), dim=-1).exp()
        assert bool((((row - (1 - lo)).abs() > 1e-3) & ((row - (1 + hi)).abs() > 1e-3)).all())
        assert bool((row < 1 - lo).any()) and bool((row > 1 + hi).any())

    cfg = SimpleNamespace(policy_loss_type={"dppo_tv": "dppo", "dppo_kl": "dppo"}.get(kind, kind), eps_clip_low=lo,
                          eps_clip_high=hi, loss_reduction="sequence_mean",
                          sapo=SimpleNamespace(tau_pos=lo, tau_neg=hi),
                          cispo=SimpleNamespace(cispo_eps_clip_low=lo, cispo_eps_clip_high=hi, cispo_anchor="old"),
                          dppo=SimpleNamespace(dppo_type="binary_kl" if kind == "dppo_kl" else "binary_tv", delta_low=lo,
                                               delta_high=hi),
                          off_policy_correction=SimpleNamespace(tis_ratio_type=None, sequence_mask_metric=None))
    m64 = None if mask is None else mask.double()
    x = lp.double().requires_grad_(True)
    if kind == "dppo_tv" or kind == "dppo_kl":
        per_token = lambda msk: O.dppo_policy_loss(x, old.double(), adv.double(), cfg.dppo.dppo_type, lo, hi, msk)  # noqa: E731
    else:
        fn = {"sapo": O.sapo_policy_loss, "gspo": O.gspo_policy_loss, "cispo": O.cispo_policy_loss,
              "rollout_is": O.rollout_is_policy_loss}[kind]
        per_token = lambda msk: fn(x, old.double(), adv.double(), lo, hi, msk)  # noqa: E731
    # the importance weight of off-policy correction multiplies the per-token loss before the masked sum: fold it into the mask
    # for the loss, keep the plain mask for the statistic (and, for GSPO, for the row mean)
    if weight is None:
        ref_loss, ref_clip = per_token(m64)
    elif kind == "gspo":
        row = O.masked_mean(x - old.double(), m64, dim=-1).unsqueeze(-1)
        r = torch.clamp(x - x.detach() + row.detach(), max=10).exp()
        a64 = adv.double()
        ref_loss = (-torch.min(r * a64, r.clamp(1 - lo, 1 + hi) * a64) * weight.double() * m64).sum()
        ref_clip = per_token(m64)[1]
    else:
        ref_loss, ref_clip = per_token(m64 * weight.double())[0], per_token(m64)[1]
    ref_loss.backward()
    return lp, old, adv, mask, weight, cfg, ref_loss.item(), ref_clip.item(), x.grad


@pytest.mark.parametrize("kind", ["sapo", "gspo", "cispo", "rollout_is", "dppo_tv", "dppo_kl"])
@pytest.mark.parametrize("masked", [False, True])
def test_further_policy_losses_match_oracle(kind, masked, cuda_device):
    from skyrl_amd import policy_loss as PL

    lp, old, adv, mask, weight, cfg, ref_loss, ref_clip, ref_grad = _further_loss_case(kind, masked)
    fn = {"sapo": PL.sapo_policy_loss, "gspo": PL.gspo_policy_loss, "cispo": PL.compute_policy_loss_cispo,
          "rollout_is": PL.rollout_is_policy_loss, "dppo_tv": PL.dppo_policy_loss, "dppo_kl": PL.dppo_policy_loss}[kind]
    to = lambda t: None if t is None else t.to(cuda_device)  # noqa: E731
    dlp = lp.to(cuda_device).requires_grad_(True)
    if kind == "rollout_is":     # anchored on the rollout log-probabilities; the old ones are not read
        loss, metrics = fn(dlp, to(old) + 5.0, to(adv), cfg, to(mask), to(old), loss_weight=to(weight))
    else:
        loss, metrics = fn(dlp, to(old), to(adv), cfg, to(mask), loss_weight=to(weight))
    loss.backward()
    scale = max(abs(ref_loss), float(ref_grad.abs().max()), 1e3)
    assert abs(loss.item() - ref_loss) <= 5e-6 * scale, (loss.item(), ref_loss)
    assert metrics["clip_ratio"] == pytest.approx(ref_clip, abs=1e-6)
    if kind not in ("sapo",):
        assert 0.0 < ref_clip < 1.0                             # both sides of the branch are exercised
    err = (dlp.grad.double().cpu() - ref_grad).abs().max().item()
    assert err <= 1e-5 * max(1.0, ref_grad.abs().max().item()), f"gradient max abs err {err}"
    if mask is not None:
        assert bool((dlp.grad.cpu()[mask == 0] == 0).all())

    # the same type inside the assembled actor loss, with a KL term on top
    cfg.use_kl_loss, cfg.kl_loss_coef, cfg.kl_estimator_type, cfg.use_entropy_loss = True, 0.05, "k2", False
    base = lp + 0.25
    d2 = lp.to(cuda_device).requires_grad_(True)
    rollout = to(old) if kind == "rollout_is" else None
    loss2, m2 = PL.actor_loss(d2, to(old), to(adv), cfg, to(mask), base_log_probs=to(base), loss_weight=to(weight),
                              rollout_logprobs=rollout, policy_scale=2.0, term_scale=0.5)
    loss2.backward()
    kl_ref_lp = lp.double().requires_grad_(True)
    kl_ref = O.approx_kl_loss(kl_ref_lp, base.double(), None if mask is None else mask.double(), "k2")
    kl_ref.backward()
    want = 2.0 * ref_loss + 0.5 * 0.05 * kl_ref.item()
    assert abs(loss2.item() - want) <= 5e-6 * scale
    assert m2["clip_ratio"].item() == pytest.approx(ref_clip, abs=1e-6)
    want_grad = 2.0 * ref_grad + 0.5 * 0.05 * kl_ref_lp.grad
    err = (d2.grad.double().cpu() - want_grad).abs().max().item()
    assert err <= 2e-5 * max(1.0, want_grad.abs().max().item()), f"actor-loss gradient max abs err {err}"


def _cov_case(seed=47, B=6, S=203):
    from types import SimpleNamespace

    gen = torch.Generator().manual_seed(seed)
    lp = (torch.randn(B, S, generator=gen) * 0.7 - 1.5).clamp(max=-0.02)
    old = lp + torch.randn(B, S, generator=gen) * 0.3
    adv = torch.randn(B, S, generator=gen)
    mask = (torch.rand(B, S, generator=gen) > 0.3).float()
    mask[1] = 0
    cfg = SimpleNamespace(policy_loss_type="clip_cov", eps_clip_low=0.2, eps_clip_high=0.25, loss_reduction="sequence_mean",
                          clip_cov=SimpleNamespace(clip_ratio=0.05, clip_cov_lb=0.05, clip_cov_ub=2.0),
                          kl_cov=SimpleNamespace(kl_cov_frac=0.1, ppo_kl_coef=0.7))
    return lp, old, adv, mask, cfg


def test_clip_cov_policy_loss_matches_oracle(cuda_device):
    """The clip-cov loss (ppo_utils.py:938-999): same tokens drawn as the oracle draws from the same generator state, same
    loss, removed fraction and gradient.  Tokens whose candidate decision is within 1e-4 of a bound in fp64 are masked out."""
    from skyrl_amd import policy_loss as PL

    lp, old, adv, mask, cfg = _cov_case()
    cc = cfg.clip_cov
    m64 = mask.double()
    cov = (adv.double() - O.masked_mean(adv.double(), m64)) * (lp.double() - O.masked_mean(lp.double(), m64))
    ratio = (lp.double() - old.double()).exp()
    fragile = ((cov - cc.clip_cov_lb).abs() < 1e-4) | ((cov - cc.clip_cov_ub).abs() < 1e-4) | \
              ((ratio - 0.8).abs() < 1e-4) | ((ratio - 1.25).abs() < 1e-4)
    mask = torch.where(fragile, torch.zeros(()), mask)
    m64 = mask.double()
    cov = (adv.double() - O.masked_mean(adv.double(), m64)) * (lp.double() - O.masked_mean(lp.double(), m64))
    assert not bool((((cov - cc.clip_cov_lb).abs() < 5e-5) | ((cov - cc.clip_cov_ub).abs() < 5e-5))[mask > 0].any())
    x = lp.double().requires_grad_(True)
    torch.manual_seed(11)
    ref, ref_frac, corr = O.clip_cov_policy_loss(x, old.double(), adv.double(), cfg.eps_clip_low, cfg.eps_clip_high, cc.clip_ratio,
                                                 cc.clip_cov_lb, cc.clip_cov_ub, m64)
    ref.backward()
    removed = int((corr == 0).sum())
    assert removed == max(int(cc.clip_ratio * float(mask.sum())), 1)      # enough candidates: the draw is a strict subset
    to = lambda t: t.to(cuda_device)  # noqa: E731
    d = to(lp).requires_grad_(True)
    torch.manual_seed(11)
    loss, metrics = PL.compute_policy_loss_clip_cov(d, to(old), to(adv), cfg, to(mask))
    loss.backward()
    scale = max(abs(ref.item()), 1e3)
    assert abs(loss.item() - ref.item()) <= 5e-6 * scale, (loss.item(), ref.item())
    assert metrics["clip_ratio"] == pytest.approx(ref_frac.item(), abs=1e-6)
    err = (d.grad.double().cpu() - x.grad).abs().max().item()
    assert err <= 1e-5 * max(1.0, x.grad.abs().max().item()), f"gradient max abs err {err}"
    # exactly the drawn tokens, the masked ones and the ones the clip catches carry no gradient
    assert bool((d.grad.cpu()[(corr == 0) | (mask == 0)] == 0).all())
    # another generator state draws other tokens
    torch.manual_seed(12)
    d2 = to(lp).requires_grad_(True)
    PL.compute_policy_loss_clip_cov(d2, to(old), to(adv), cfg, to(mask))[0].backward()
    assert not torch.equal(d2.grad == 0, d.grad == 0)
    # no candidate inside the bounds: the clipped surrogate on the unclamped ratio
    cfg.clip_cov.clip_cov_lb, cfg.clip_cov.clip_cov_ub = 500.0, 600.0
    x = lp.double().requires_grad_(True)
    ref, ref_frac, _ = O.clip_cov_policy_loss(x, old.double(), adv.double(), 0.2, 0.25, cc.clip_ratio, 500.0, 600.0, m64)
    loss, metrics = PL.compute_policy_loss_clip_cov(to(lp), to(old), to(adv), cfg, to(mask))
    assert abs(loss.item() - ref.item()) <= 5e-6 * scale and metrics["clip_ratio"] == 0.0 == ref_frac.item()


def test_kl_cov_policy_loss_matches_oracle(cuda_device):
    """The kl-cov loss (ppo_utils.py:1002-1053): the same top-k tokens as the oracle, loss and gradient."""
    from skyrl_amd import policy_loss as PL

    lp, old, adv, mask, cfg = _cov_case(seed=53)
    kc = cfg.kl_cov
    old[0, 0] = lp[0, 0]                                          # a log-ratio of exactly zero: |.| has subgradient 0 there
    x = lp.double().requires_grad_(True)
    ref, sel = O.kl_cov_policy_loss(x, old.double(), adv.double(), kc.kl_cov_frac, kc.ppo_kl_coef, mask.double())
    ref.backward()
    k = max(1, int(float((mask > 0).sum()) * kc.kl_cov_frac))
    assert int(sel.sum()) == k
    # the k-th and (k+1)-th covariance terms are far enough apart for fp32 to order them alike
    valid = mask > 0
    c = ((adv.double()[valid] - adv.double()[valid].mean()) * (lp.double()[valid] - lp.double()[valid].mean())).sort(descending=True).values
    assert float(c[k - 1] - c[k]) > 1e-5
    to = lambda t: t.to(cuda_device)  # noqa: E731
    d = to(lp).requires_grad_(True)
    loss, metrics = PL.compute_policy_loss_kl_cov(d, to(old), to(adv), cfg, to(mask))
    loss.backward()
    assert metrics == {"clip_ratio": 0.0}
    assert abs(loss.item() - ref.item()) <= 5e-6 * max(abs(ref.item()), 1e3)
    err = (d.grad.double().cpu() - x.grad).abs().max().item()
    assert err <= 1e-5 * max(1.0, x.grad.abs().max().item()), f"gradient max abs err {err}"
    # with a zero coefficient it is the importance-sampling loss of the same kernel, bit for bit
    cfg.kl_cov.ppo_kl_coef = 0.0
    a, _ = PL.compute_policy_loss_kl_cov(to(lp), to(old), to(adv), cfg, to(mask))
    b, _ = PL.importance_sampling_loss(to(lp), to(old), to(adv), None, to(mask))
    assert a.item() == pytest.approx(b.item(), rel=1e-6)


@pytest.mark.parametrize("masked", ["none", "some", "empty"])
def test_cispo_ratio_diagnostics_match_oracle(masked, cuda_device):
    from skyrl_amd import policy_loss as PL

    lp, old, adv, mask, _weight, cfg, *_ = _further_loss_case("cispo", masked == "some")
    if masked == "empty":
        mask = torch.zeros_like(lp)
    m64 = None if mask is None else mask.double()
    want = O.cispo_ratio_diagnostics(lp.double(), old.double(), cfg.cispo.cispo_eps_clip_low, cfg.cispo.cispo_eps_clip_high, m64)
    to = lambda t: None if t is None else t.to(cuda_device)  # noqa: E731
    _, metrics = PL.compute_policy_loss_cispo(to(lp), to(old), to(adv), cfg, to(mask))
    _, lazy = PL.compute_policy_loss_cispo(to(lp), to(old), to(adv), cfg, to(mask), sync_metrics=False)
    for key, value in want.items():
        assert metrics[key] == pytest.approx(value, rel=1e-5, abs=1e-9), key
        assert isinstance(lazy[key], torch.Tensor) and lazy[key].item() == metrics[key]
    assert want["cispo/ratio_max"] == pytest.approx(math.exp(20.0)) or masked == "some"   # the clamp of the log-ratio at +-20


def test_further_policy_losses_argument_handling(cuda_device):
    from types import SimpleNamespace

    from skyrl_amd import policy_loss as PL

    x = torch.full((2, 8), -1.0, device=cuda_device)
    cfg = SimpleNamespace(policy_loss_type="cispo", eps_clip_low=0.2, eps_clip_high=0.2,
                          cispo=SimpleNamespace(cispo_eps_clip_low=1.0, cispo_eps_clip_high=4.0, cispo_anchor="rollout"),
                          dppo=SimpleNamespace(dppo_type="topk", delta_low=0.2, delta_high=0.2),
                          off_policy_correction=SimpleNamespace(tis_ratio_type="token", sequence_mask_metric=None))
    with pytest.raises(AssertionError):                          # the rollout anchor needs rollout log-probabilities
        PL.compute_policy_loss_cispo(x, x, x, cfg)
    # a correction switched on is applied, not skipped: old / rollout = e^0.5 on every token, capped at 1.5
    tis_cfg = SimpleNamespace(policy_loss_type="regular", eps_clip_low=0.2, eps_clip_high=0.2,
                              off_policy_correction=SimpleNamespace(tis_ratio_type="token", token_tis_ratio_clip_high=1.5,
                                                                    sequence_mask_metric=None))
    loss, m = PL.ppo_policy_loss(x, x, x, tis_cfg, None, x - 0.5)
    assert loss.item() == pytest.approx(16.0 * 1.5) and m["tis_token_clip_high_ratio"] == 1.0
    with pytest.raises(ValueError):                              # the rollout anchor already is the correction: TIS would double-count
        PL.compute_policy_loss_cispo(x, x, x, cfg, None, x)
    cfg.off_policy_correction.tis_ratio_type = None
    loss, m = PL.compute_policy_loss_cispo(x, x + 9.0, x, cfg, None, x)   # ratio 1 against the rollout anchor
    assert loss.item() == pytest.approx(-16.0) and m["clip_ratio"] == 0.0
    with pytest.raises(AssertionError):
        PL.rollout_is_policy_loss(x, x, x, cfg)
    with pytest.raises(ValueError):
        PL.dppo_policy_loss(x, x, x, cfg)
    with pytest.raises(ValueError):
        PL.gspo_policy_loss(x[0], x[0], x[0], cfg)
    cfg.policy_loss_type = "clip_cov"
    with pytest.raises(NotImplementedError):
        PL.actor_loss(x, x, x, cfg)


@pytest.mark.parametrize("estimator", ["k1", "abs", "k2", "k3"])
@pytest.mark.parametrize("masked", [False, True])
def test_approx_kl_matches_oracle(estimator, masked, cuda_device):
    from skyrl_amd.policy_loss import approx_kl_loss, compute_approx_kl

    gen = torch.Generator().manual_seed(16)
    B, S = 7, 600
    lp = torch.randn(B, S, generator=gen) * 0.5 - 2.0
    base = lp + torch.randn(B, S, generator=gen) * 0.4
    base[0, 0], base[0, 1] = lp[0, 0] + 25.0, lp[0, 1] - 25.0   # inner clamp on both sides
    base[0, 2] = lp[0, 2] + 3.0                                 # outer clamp: e^3 - 4 > 10
    base[0, 3] = lp[0, 3]                                       # zero difference (|.| has derivative 0 there)
    mask = None
    if masked:
        mask = (torch.rand(B, S, generator=gen) > 0.4).float()
        mask[1] = 0                                             # a row without loss tokens
        mask[2, :10] = 0.5                                      # fractional weights
        mask[0, :4] = 1
    to = lambda t: None if t is None else t.to(cuda_device)  # noqa: E731
    m64 = None if mask is None else mask.double()

    # per-token values and their elementwise gradient
    ref_lp = lp.double().requires_grad_(True)
    ref = O.compute_approx_kl(ref_lp, base.double(), m64, estimator)
    G = torch.randn(B, S, generator=gen)
    (ref * G.double()).sum().backward()
    dlp = lp.to(cuda_device).requires_grad_(True)
    got = compute_approx_kl(dlp, to(base), to(mask), estimator)
    (got * G.to(cuda_device)).sum().backward()
    assert got.dtype == torch.float32 and got.shape == (B, S)
    torch.testing.assert_close(got.detach().cpu().double(), ref.detach(), rtol=2e-5, atol=2e-6)
    if masked:
        assert bool((got.detach().cpu()[mask == 0] == 0).all())
    torch.testing.assert_close(dlp.grad.cpu().double(), ref_lp.grad, rtol=2e-5, atol=2e-6)

    # the trainer's reduction and its gradient
    ref_lp = lp.double().requires_grad_(True)
    ref = O.approx_kl_loss(ref_lp, base.double(), m64, estimator)
    ref.backward()
    dlp = lp.to(cuda_device).requires_grad_(True)
    got = approx_kl_loss(dlp, to(base), to(mask), estimator)
    (got * 1.0).backward()
    assert got.dim() == 0 and got.item() == pytest.approx(ref.item(), rel=1e-5, abs=1e-7)
    torch.testing.assert_close(dlp.grad.cpu().double(), ref_lp.grad, rtol=2e-5, atol=1e-9)


def test_masked_mean_matches_oracle(cuda_device):
    from skyrl_amd.policy_loss import masked_mean

    gen = torch.Generator().manual_seed(17)
    B, S = 9, 1031
    v = torch.randn(B, S, generator=gen)
    mask = (torch.rand(B, S, generator=gen) > 0.5).float()
    mask[3] = 0
    mask[4, :] = 0
    mask[4, 5] = 0.25
    for m in (None, mask):
        for dim in (None, -1):
            ref_v = v.double().requires_grad_(True)
            ref = O.masked_mean(ref_v, None if m is None else m.double(), dim)
            w = torch.randn(ref.shape, generator=gen).double()
            (ref * w).sum().backward()
            dv = v.to(cuda_device).requires_grad_(True)
            got = masked_mean(dv, None if m is None else m.to(cuda_device), dim)
            (got * w.float().to(cuda_device)).sum().backward()
            assert got.shape == ref.shape
            torch.testing.assert_close(got.detach().cpu().double(), ref.detach(), rtol=1e-5, atol=1e-6)
            torch.testing.assert_close(dv.grad.cpu().double(), ref_v.grad, rtol=1e-5, atol=1e-9)
    with pytest.raises(NotImplementedError):
        masked_mean(v.to(cuda_device), None, 0)


def test_loss_argument_errors(cuda_device):
    lib = _lib.load()
    x = torch.zeros(16, dtype=torch.float32, device=cuda_device)
    p = x.data_ptr()
    assert lib.skyrl_ppo_policy_loss(p, None, None, None, None, 16, 0.2, 0.2, 3.0, 2, p, None, None, None) == 0   # cross entropy
    assert lib.skyrl_ppo_policy_loss(p, None, None, None, None, 16, 0.2, 0.2, 3.0, 3, p, None, None, None) == -1
    assert lib.skyrl_ppo_policy_loss(p, p, p, None, None, 16, 0.2, 0.2, 3.0, 4, p, None, None, None) == -5
    assert lib.skyrl_approx_kl(p, p, None, 4, 4, 3, None, None, p, 0, None, None) == -1
    assert lib.skyrl_approx_kl(p, p, None, 4, 4, 4, None, p, p, 0, None, None) == -5
    assert lib.skyrl_approx_kl(p, p, None, 4, 4, 3, None, p, p, 2, None, None) == -1
    assert lib.skyrl_approx_kl(p, p, None, 0, 4, 3, None, p, p, 0, None, None) == -2
    assert lib.skyrl_masked_mean(p, None, 4, 4, None, None, None) == -1
    assert lib.skyrl_masked_mean(p, None, 4, 0, p, None, None) == -2
    args = lambda **kw: [kw.get("lp", p), p, p, None, None, None, kw.get("ent"), 4, 4, kw.get("type", 0), 0.2, 0.2, 3.0,  # noqa: E731
                         3, 1.0, 1.0, 0.0, 0.0, kw.get("rows", p), p, None, kw.get("dent"), None]
    assert lib.skyrl_actor_loss(*args()) == 0
    assert lib.skyrl_actor_loss(*args(rows=None)) == -1
    assert lib.skyrl_actor_loss(*args(dent=p)) == -1          # an entropy gradient without the entropy
    assert lib.skyrl_actor_loss(*args(type=4)) == 0           # the sequence-level type is part of this entry point only
    assert lib.skyrl_actor_loss(*args(type=10)) == -5
    # SAPO's temperatures divide: zero is refused
    assert lib.skyrl_ppo_policy_loss(p, p, p, None, None, 16, 0.0, 1.0, 0.0, 5, p, None, None, None) == -5
    # more than one workgroup's worth of tokens needs the scratch for the partial sums
    big = torch.zeros(20000, dtype=torch.float32, device=cuda_device)
    assert lib.skyrl_ppo_policy_loss(big.data_ptr(), None, None, None, None, 20000, 0.2, 0.2, 3.0, 2, p, None, None, None) == -4
    torch.cuda.synchronize()


@pytest.mark.parametrize("use_kl,use_ent,masked", [(False, False, True), (True, False, False), (True, True, True)])
def test_actor_loss_matches_oracle(use_kl, use_ent, masked, cuda_device):
    """The assembled loss (policy + KL - entropy) and both upstream gradients from the row / finish / entropy-gradient kernels."""
    from types import SimpleNamespace

    from skyrl_amd.policy_loss import actor_loss

    gen = torch.Generator().manual_seed(23)
    B, S = 6, 700
    lp = torch.randn(B, S, generator=gen) * 0.5 - 2.0
    old = lp + torch.randn(B, S, generator=gen) * 0.3
    base = lp + torch.randn(B, S, generator=gen) * 0.4
    adv = torch.randn(B, S, generator=gen)
    ent = torch.rand(B, S, generator=gen) * 3
    mask = None
    if masked:
        mask = (torch.rand(B, S, generator=gen) > 0.4).float()
        mask[2] = 0
    cfg = SimpleNamespace(policy_loss_type="regular", eps_clip_low=0.2, eps_clip_high=0.28, use_kl_loss=use_kl, kl_loss_coef=0.05,
                          kl_estimator_type="k3", use_entropy_loss=use_ent, entropy_loss_coef=0.01)
    m64 = None if mask is None else mask.double()
    r_lp, r_ent = lp.double().requires_grad_(True), ent.double().requires_grad_(True)
    ref, ref_pol, ref_kl, ref_e = O.actor_loss(r_lp, old.double(), adv.double(), m64, 0.2, 0.28, policy_scale=4.0, term_scale=0.125,
                                               base_log_probs=base.double() if use_kl else None, kl_estimator_type="k3",
                                               kl_coef=0.05 if use_kl else 0.0, entropy=r_ent, entropy_coef=0.01 if use_ent else 0.0)
    ref.backward()
    to = lambda t: None if t is None else t.to(cuda_device)  # noqa: E731
    d_lp, d_ent = lp.to(cuda_device).requires_grad_(True), ent.to(cuda_device).requires_grad_(True)
    loss, metrics = actor_loss(d_lp, to(old), to(adv), cfg, to(mask), base_log_probs=to(base), entropy=d_ent, policy_scale=4.0,
                               term_scale=0.125)
    loss.backward()
    assert loss.item() == pytest.approx(ref.item(), rel=2e-5, abs=1e-4)
    assert metrics["policy_loss"].item() == pytest.approx(ref_pol.item(), rel=2e-5, abs=1e-4)
    assert metrics["policy_kl"].item() == pytest.approx(ref_kl.item() if use_kl else 0.0, rel=2e-5, abs=1e-7)
    assert metrics["policy_entropy"].item() == pytest.approx(ref_e.item(), rel=2e-5)
    torch.testing.assert_close(d_lp.grad.cpu().double(), r_lp.grad, rtol=2e-5, atol=1e-7)
    want_dent = r_ent.grad if r_ent.grad is not None else torch.zeros(B, S, dtype=torch.float64)
    torch.testing.assert_close(d_ent.grad.cpu().double(), want_dent, rtol=2e-5, atol=1e-12)
    # the same loss from the separate kernels
    from skyrl_amd.policy_loss import approx_kl_loss, masked_mean, ppo_policy_loss
    pol, _ = ppo_policy_loss(to(lp), to(old), to(adv), cfg, to(mask))
    parts = pol * 4.0
    if use_kl:
        parts = parts + 0.125 * 0.05 * approx_kl_loss(to(lp), to(base), to(mask), "k3")
    if use_ent:
        parts = parts - 0.125 * 0.01 * masked_mean(to(ent), to(mask))
    assert loss.item() == pytest.approx(parts.item(), rel=1e-5, abs=1e-4)


def test_whole_path_hidden_to_actor_loss_gradients(cuda_device):
    """Decoder output -> fused LM head (log-probabilities and grad-carrying entropy, padding removed) -> assembled actor loss
    -> gradients in hidden and weight, against the same chain on materialised fp64 logits."""
    from types import SimpleNamespace

    from skyrl_amd.model_wrapper import action_log_probs_from_hidden
    from skyrl_amd.policy_loss import actor_loss

    dev = cuda_device
    gen = torch.Generator().manual_seed(77)
    B, S, H, V, A, t = 4, 48, 128, 900, 20, 0.9
    seqs = torch.randint(0, V, (B, S), generator=gen)
    am = torch.ones(B, S, dtype=torch.long)
    am[0, :9] = 0
    am[3, :17] = 0
    nnz = am.flatten().nonzero().flatten()
    hidden = torch.randn(1, len(nnz), H, generator=gen).to(torch.bfloat16)
    weight = (torch.randn(V, H, generator=gen) * 3 / H ** 0.5).to(torch.bfloat16)
    adv = torch.randn(B, A, generator=gen)
    loss_mask = (torch.rand(B, A, generator=gen) > 0.3).float()
    cfg = SimpleNamespace(policy_loss_type="regular", eps_clip_low=0.2, eps_clip_high=0.2, use_kl_loss=True, kl_loss_coef=0.02,
                          kl_estimator_type="k2", use_entropy_loss=True, entropy_loss_coef=0.005)

    h64, w64 = hidden.double().requires_grad_(True), weight.double().requires_grad_(True)
    alp, ent = O.hf_wrapper_tail(h64 @ w64.t(), seqs, A, am.double(), t, nnz_indices=nnz)
    old = (alp.detach() + 0.2 * torch.randn(B, A, generator=gen).double()).float()
    base = (alp.detach() + 0.3 * torch.randn(B, A, generator=gen).double()).float()
    ent_act = ent[:, -A - 1:-1]
    ref, _, _, _ = O.actor_loss(alp, old.double(), adv.double(), loss_mask.double(), 0.2, 0.2, policy_scale=2.0, term_scale=0.5,
                                base_log_probs=base.double(), kl_estimator_type="k2", kl_coef=0.02, entropy=ent_act,
                                entropy_coef=0.005)
    ref.backward()

    hd, wd = hidden.to(dev).requires_grad_(True), weight.to(dev).requires_grad_(True)
    got_alp, out = action_log_probs_from_hidden(hd, wd, seqs.to(dev), A, am.to(dev), t, return_output=True,
                                                compute_entropy=True, entropy_requires_grad=True, nnz_indices=nnz.to(dev))
    loss, metrics = actor_loss(got_alp, old.to(dev), adv.to(dev), cfg, loss_mask.to(dev), base_log_probs=base.to(dev),
                               entropy=out["entropy"][:, -A - 1:-1], policy_scale=2.0, term_scale=0.5)
    loss.backward()
    assert loss.item() == pytest.approx(ref.item(), rel=1e-3, abs=1e-3)
    assert all(v.dim() == 0 and v.is_cuda for v in metrics.values())
    assert cos(hd.grad, h64.grad) >= GRAD_COS and cos(wd.grad, w64.grad) >= GRAD_COS


def test_mfma_probe_sums_exactly(cuda_device):
    """The measurement kernel runs the mainloop's MFMA sequence on caller-given operands: with small integers the sum of
    every wavefront's accumulators has a closed form, sum_k (sum_m A[m,k]) (sum_n B[n,k]) per pair of fragments."""
    lib = _lib.load()
    gen = torch.Generator().manual_seed(3)
    ops_cpu = torch.randint(-3, 4, (2, 8, 2, 256, 8), generator=gen).to(torch.float32)  # [k-step, fragment, A/B, thread, 8 k]
    dev_ops = ops_cpu.to(torch.bfloat16).to(cuda_device).contiguous()
    wgs, iters = 3, 5
    sink = torch.empty(256 * wgs, dtype=torch.float32, device=cuda_device)
    st = lib.skyrl_lmhead_mfma_probe(dev_ops.data_ptr(), wgs, iters, sink.data_ptr(), torch.cuda.current_stream().cuda_stream)
    _lib.check(st, "skyrl_lmhead_mfma_probe")
    torch.cuda.synchronize()
    got = sink.view(wgs, 4, 64).sum(-1).double().cpu()  # per workgroup and wavefront
    want = torch.zeros(4, dtype=torch.float64)
    for w in range(4):
        frag = ops_cpu[:, :, :, 64 * w:64 * (w + 1), :].double()             # [2, 8, 2, 64 lanes, 8]
        # lane l holds row l & 15 and the k values (l >> 4) * 8 .. + 7: sum over the 16 rows -> [2, 8, 2, 32 k]
        colsum = frag.view(2, 8, 2, 4, 16, 8).sum(4).reshape(2, 8, 2, 32)
        a, b = colsum[:, :, 0].sum(1), colsum[:, :, 1].sum(1)                 # sums over the 8 A / 8 B fragments: [2, 32]
        want[w] = iters * (a * b).sum()
    for g in range(wgs):
        assert torch.equal(got[g], want), f"workgroup {g}: {got[g].tolist()} vs {want.tolist()}"


@pytest.mark.parametrize("oov", [False, True])
@pytest.mark.parametrize("chunk", [1, 7, 64, 512])
def test_fused_linear_logprob_apply_matches_reference_statement(oov, chunk, cuda_device):
    # shapes of the reference's test (test_fused_linear_logprob.py:98-119) with H raised to the kernel's multiple of 64
    B, S, H, V = 4, 32, 256, 4096
    gen = torch.Generator().manual_seed(0)
    hidden = torch.randn(B, S, H, generator=gen).to(torch.bfloat16)
    weight = (torch.randn(V, H, generator=gen) * H**-0.5).to(torch.bfloat16)
    vs, ve = (0, V)
    target = torch.randint(0, V, (B, S), generator=gen)
    if oov:
        vs, ve = 1024, 1024 + V
        target = torch.randint(0, V + 2048, (B, S), generator=gen)
    grad = torch.linspace(0.5, 1.5, B * S).reshape(B, S)
    hd = hidden.to(cuda_device).requires_grad_(True)
    wd = weight.to(cuda_device).requires_grad_(True)
    lp = FusedLinearLogprobHip.apply(hd, wd, target.to(cuda_device), vs, ve, chunk, None, False)
    assert lp.shape == (B, S) and lp.dtype == torch.float32
    (lp * grad.to(cuda_device)).sum().backward()
    assert hd.grad.dtype == torch.bfloat16 and wd.grad.dtype == torch.bfloat16
    ref_lp = O.fused_chunked_logprob_forward(hidden.float(), weight.float(), target, vs, ve, chunk)
    ref_gh, ref_gw = O.fused_chunked_logprob_backward(hidden.float(), weight.float(), target, vs, ve, chunk, grad)
    torch.testing.assert_close(lp.cpu(), ref_lp, atol=1e-3, rtol=1e-4)
    assert cos(hd.grad, ref_gh) >= GRAD_COS and cos(wd.grad, ref_gw) >= GRAD_COS
    # the reference's tolerances for bf16 operands: grad_hidden 2e-3 (+ bf16 output rounding), grad_weight 4e-2
    torch.testing.assert_close(hd.grad.float().cpu(), ref_gh, atol=2e-2, rtol=2e-2)
    torch.testing.assert_close(wd.grad.float().cpu(), ref_gw, atol=4e-2, rtol=4e-2)
    # inference_only saves nothing and returns the same numbers
    with torch.no_grad():
        lp2 = FusedLinearLogprobHip.apply(hd, wd, target.to(cuda_device), vs, ve, chunk, None, True)
    assert torch.equal(lp2, lp.detach())


@pytest.mark.parametrize("reduction", ["none", "sum", "mean"])
def test_linear_cross_entropy_interface(reduction, cuda_device):
    T, H, V, t = 150, 128, 1500, 0.6
    hidden, weight, labels, g, q = _rand(T, H, V, seed=33)
    hd = hidden.to(cuda_device).requires_grad_(True)
    wd = weight.to(cuda_device).requires_grad_(True)
    lp, ent = linear_cross_entropy(hd, wd, labels.to(cuda_device), t, reduction, None)
    ex = O.exact_fwd_bwd(hidden, weight, labels, t)
    want = {"none": ex["logprobs"], "sum": ex["logprobs"].sum(), "mean": ex["logprobs"].mean()}[reduction]
    torch.testing.assert_close(lp.double().cpu(), want, atol=2e-3 * (T if reduction == "sum" else 1), rtol=1e-4)
    torch.testing.assert_close(ent.double().cpu(), ex["entropy"], atol=1e-3, rtol=1e-3)
    if reduction == "none":
        loss = (lp * g.to(cuda_device)).sum() + (ent * q.to(cuda_device)).sum()
        gg = g
    else:
        loss = lp * 1.7 + (ent * q.to(cuda_device)).sum()
        gg = torch.full((T,), 1.7 if reduction == "sum" else 1.7 / T)
    loss.backward()
    exb = O.exact_fwd_bwd(hidden, weight, labels, t, gg.double(), q.double())
    assert cos(hd.grad, exb["d_hidden"]) >= GRAD_COS and cos(wd.grad, exb["d_weight"]) >= GRAD_COS


def test_wrappers_roll_packing_entropy(cuda_device):
    dev = cuda_device
    B, S, H, V, t = 3, 40, 128, 777, 0.9
    gen = torch.Generator().manual_seed(44)
    hidden = torch.randn(B, S, H, generator=gen).to(torch.bfloat16)
    weight = (torch.randn(V, H, generator=gen) * 3 / H**0.5).to(torch.bfloat16)
    tokens = torch.randint(0, V, (B, S), generator=gen)
    got = model_utils.from_parallel_hidden_to_logprobs(hidden.to(dev), weight.to(dev), tokens.to(dev), 0, V, None,
                                                       inference_only=True, chunk_size=16, temperature=t)
    want = O.from_parallel_hidden_to_logprobs(hidden.float(), weight.float(), tokens, chunk_size=16, temperature=t)
    assert got.shape == (B, S - 1)
    torch.testing.assert_close(got.cpu(), want, atol=2e-3, rtol=1e-4)

    ent = model_utils._fused_vocab_parallel_entropy_from_hidden(hidden.to(dev), weight.to(dev), None, chunk_size=8, temperature=t)
    want_e = O.fused_entropy_from_hidden(hidden.float(), weight.float(), 8, t)
    torch.testing.assert_close(ent.cpu(), want_e, atol=1e-3, rtol=1e-3)

    # packed: 4 sequences in one stream
    lens = [9, 1, 17, 13]
    cu = torch.tensor([0, 9, 10, 27, 40])
    T = 40
    ph = hidden[0:1, :T]
    ptok = tokens[0:1, :T]
    L = 15
    got_p = model_utils.from_parallel_hidden_to_logprobs_packed_sequences(
        ph.to(dev), weight.to(dev), ptok.to(dev), cu.to(dev), L, 0, V, None, inference_only=True, temperature=t)
    rolled = O.packed_rolled_targets(ptok[0], cu)
    probs = O.fused_chunked_logprob_forward(ph.float(), weight.float() / t, rolled[None], 0, V, 8)[0]
    want_p = O.packed_scatter_back(probs, cu, len(lens), L)
    assert got_p.shape == (len(lens), L - 1)
    torch.testing.assert_close(got_p.cpu(), want_p, atol=2e-3, rtol=1e-4)

    # both outputs with gradients from one pass
    hd = hidden.to(dev).requires_grad_(True)
    wd = weight.to(dev).requires_grad_(True)
    lp, en = model_utils.fused_logprobs_and_entropy_from_hidden(hd, wd, tokens.to(dev), t)
    (lp.sum() * 0.3 - en.sum() * 0.01).backward()
    ex = O.exact_fwd_bwd(hidden.reshape(-1, H), weight, tokens.reshape(-1), t, torch.full((B * S,), 0.3, dtype=torch.float64),
                         torch.full((B * S,), -0.01, dtype=torch.float64))
    assert cos(hd.grad.reshape(-1, H), ex["d_hidden"]) >= GRAD_COS and cos(wd.grad, ex["d_weight"]) >= GRAD_COS


# ---------------------------------------------------------------------------------------------------------------------
# packed-sequence label preparation and scatter-back: integer / index work, bit-exact against the oracle
# ---------------------------------------------------------------------------------------------------------------------
def _ragged_cu(n, max_len, seed, empties=True):
    gen = torch.Generator().manual_seed(seed)
    lens = torch.randint(0 if empties else 1, max_len + 1, (n,), generator=gen)
    lens[torch.randint(0, n, (1,), generator=gen)] = 1
    if int(lens.sum()) == 0:
        lens[0] = 3
    return torch.cat([torch.zeros(1, dtype=torch.long), lens.cumsum(0)]), lens


@pytest.mark.parametrize("n,max_len,seed", [(1, 1, 0), (4, 17, 1), (37, 300, 2), (700, 50, 3), (3, 40000, 4)])
def test_packed_next_token_labels_bit_exact(cuda_device, n, max_len, seed):
    from skyrl_amd.packed import packed_next_token_labels
    cu, _ = _ragged_cu(n, max_len, seed)
    T = int(cu[-1])
    tokens = torch.randint(0, 1 << 40, (T,), generator=torch.Generator().manual_seed(seed))
    got = packed_next_token_labels(tokens.to(cuda_device), cu.to(cuda_device))
    assert got.dtype == torch.int64 and torch.equal(got.cpu(), O.packed_rolled_targets(tokens, cu))
    # a stream longer than cu_seqlens describes: the excess tokens have no sequence and get the "no target" label
    longer = torch.cat([tokens, tokens[:5]])
    got = packed_next_token_labels(longer.to(cuda_device), cu.to(cuda_device)).cpu()
    assert torch.equal(got[:T], O.packed_rolled_targets(tokens, cu)) and bool((got[T:] == SENTINEL).all())


@pytest.mark.parametrize("n,max_len,L,seed", [(1, 1, 2, 0), (4, 17, 9, 1), (37, 300, 301, 2), (700, 50, 33, 3), (5, 3000, 2500, 4)])
def test_packed_scatter_plain_and_adjoint_bit_exact(cuda_device, n, max_len, L, seed):
    from skyrl_amd.packed import packed_scatter_logprobs
    cu, _ = _ragged_cu(n, max_len, seed)
    T = int(cu[-1])
    gen = torch.Generator().manual_seed(seed)
    probs = torch.randn(T, generator=gen)
    pd = probs.to(cuda_device).requires_grad_(True)
    out = packed_scatter_logprobs(pd, cu.to(cuda_device), n, L - 1)
    want = O.packed_scatter_back(probs, cu, n, L)
    assert torch.equal(out.detach().cpu(), want)
    # adjoint: <scatter(p), G> = <p, gather(G)> with both sides exact sums of selected products
    G = torch.randn(n, L - 1, generator=gen)
    out.backward(G.to(cuda_device))
    idx, off, lens = O.packed_sequence_indices(cu, T)
    keep = (off < (lens - 1).clamp(min=0)[idx]) & (off < L - 1)
    want_grad = torch.where(keep, G[idx.clamp(max=n - 1), off.clamp(max=L - 2)], torch.zeros(()))
    assert torch.equal(pd.grad.cpu(), want_grad)


def test_packed_scatter_sub_sequences_bit_exact(cuda_device):
    from skyrl_amd.packed import packed_scatter_logprobs
    gen = torch.Generator().manual_seed(9)
    sub, padded = [], []
    for r in range(23):
        k = int(torch.randint(1, 5, (1,), generator=gen))
        row = [int(x) for x in torch.randint(1, 40, (k,), generator=gen)]
        sub.append(row)
        padded += [n + int(torch.randint(0, 4, (1,), generator=gen)) for n in row]
    cu = torch.cat([torch.zeros(1, dtype=torch.long), torch.tensor(padded).cumsum(0)])
    T = int(cu[-1])
    probs = torch.randn(T, generator=gen)
    rows, offs, lens = model_utils._packed_subseq_row_indices_offsets_and_lens(cu, sub, torch.device("cpu"))
    r2, o2, l2 = O.packed_subseq_rows_offsets_lens(cu, sub)
    assert torch.equal(rows, r2) and torch.equal(offs, o2) and torch.equal(lens, l2)
    for L in (200, 61, 17):
        pd = probs.to(cuda_device).requires_grad_(True)
        out = packed_scatter_logprobs(pd, cu.to(cuda_device), len(sub), L - 1, seg_row=rows, seg_col=offs, seg_len=lens)
        want = O.packed_scatter_back(probs, cu, len(sub), L, sub_seq_lengths=sub)
        assert torch.equal(out.detach().cpu(), want), L
        G = torch.randn(len(sub), L - 1, generator=gen)
        out.backward(G.to(cuda_device))
        pr = probs.clone().requires_grad_(True)  # the oracle's scatter is differentiable torch indexing: autograd is its adjoint
        O.packed_scatter_back(pr, cu, len(sub), L, sub_seq_lengths=sub).backward(G)
        assert torch.equal(pd.grad.cpu(), pr.grad), L


@pytest.mark.parametrize("rows,L,seed", [(1, 2, 0), (5, 8, 1), (19, 257, 2), (7, 1500, 3)])
def test_packed_scatter_attention_mask_bit_exact(cuda_device, rows, L, seed):
    from skyrl_amd.packed import packed_scatter_logprobs
    gen = torch.Generator().manual_seed(seed)
    am = torch.rand(rows, L, generator=gen) < 0.7
    am[0] = False          # a row without tokens
    if rows > 1:
        am[1] = True       # a full row: its last real token sits in the last column
    if rows > 2:
        am[2] = False
        am[2, L // 2] = True  # a single real token
    real = am.sum(1)
    padded = real + torch.randint(0, 3, (rows,), generator=gen)
    cu = torch.cat([torch.zeros(1, dtype=torch.long), padded.cumsum(0)])
    T = int(cu[-1])
    probs = torch.randn(max(T, 1), generator=gen)[:T]
    pd = probs.to(cuda_device).requires_grad_(True)
    out = packed_scatter_logprobs(pd, cu.to(cuda_device), rows, L - 1, attention_mask=am.to(cuda_device))
    want = O.packed_scatter_back(probs, cu, rows, L, attention_mask=am)
    assert torch.equal(out.detach().cpu(), want)
    G = torch.randn(rows, L - 1, generator=gen)
    out.backward(G.to(cuda_device))
    pr = probs.clone().requires_grad_(True)
    O.packed_scatter_back(pr, cu, rows, L, attention_mask=am).backward(G)
    assert torch.equal(pd.grad.cpu(), pr.grad)


def test_packed_wrapper_all_layouts_with_gradient(cuda_device):
    """from_parallel_hidden_to_logprobs_packed_sequences end to end (labels kernel -> LM head -> scatter kernel), the three
    layouts against the oracle's statement of the same pipeline, and the gradient through scatter + LM head."""
    dev = cuda_device
    H, V, t = 128, 515, 0.8
    gen = torch.Generator().manual_seed(52)
    true_lens = [9, 1, 17, 13, 6]
    padded = [10, 2, 17, 16, 6]
    cu = torch.cat([torch.zeros(1, dtype=torch.long), torch.tensor(padded).cumsum(0)])
    T = int(cu[-1])
    hidden = torch.randn(1, T, H, generator=gen).to(torch.bfloat16)
    weight = (torch.randn(V, H, generator=gen) * 3 / H**0.5).to(torch.bfloat16)
    tokens = torch.randint(0, V, (1, T), generator=gen)
    rolled = O.packed_rolled_targets(tokens[0], cu)
    probs = O.fused_chunked_logprob_forward(hidden.float(), weight.float() / t, rolled[None], 0, V, 8)[0]
    L = 20
    am = torch.zeros(len(true_lens), L, dtype=torch.bool)
    for b, n in enumerate(true_lens):
        am[b, L - n:] = True  # left padded rows
    sub = [[9, 1], [17], [13, 6]]
    cases = {
        "plain": (dict(), O.packed_scatter_back(probs, cu, len(padded), L)),
        "mask": (dict(attention_mask=am.to(dev)), O.packed_scatter_back(probs, cu, len(padded), L, attention_mask=am)),
        "sub": (dict(sub_seq_lengths=sub), O.packed_scatter_back(probs, cu, len(sub), 30, sub_seq_lengths=sub)),
    }
    for name, (kw, want) in cases.items():
        hd = hidden.to(dev).requires_grad_(True)
        wd = weight.to(dev).requires_grad_(True)
        got = model_utils.from_parallel_hidden_to_logprobs_packed_sequences(
            hd, wd, tokens.to(dev), cu.to(dev), want.shape[1] + 1, 0, V, None, temperature=t, **kw)
        assert got.shape == want.shape, name
        torch.testing.assert_close(got.detach().cpu(), want, atol=2e-3, rtol=1e-4, msg=name)
        assert torch.equal(got.detach().cpu() == 0, want == 0), name
        G = torch.randn(want.shape, generator=gen)
        (got * G.to(dev)).sum().backward()
        # upstream gradient per packed token = the oracle scatter's adjoint applied to G
        pr = probs.clone().requires_grad_(True)
        O.packed_scatter_back(pr, cu, want.shape[0], want.shape[1] + 1, **{k: (v.cpu() if torch.is_tensor(v) else v)
                                                                          for k, v in kw.items()}).backward(G)
        ex = O.exact_fwd_bwd(hidden[0], weight, rolled, t, pr.grad.double(), None)
        assert cos(hd.grad[0], ex["d_hidden"]) >= GRAD_COS and cos(wd.grad, ex["d_weight"]) >= GRAD_COS, name


def test_packed_wrapper_action_window(cuda_device):
    """action_window = n: the last n columns of the full result, from an LM head that ran on the landing rows only -- equal
    values (a token's row is computed independently of the others) and the same gradients as the full pass with an
    upstream gradient that is zero outside the window."""
    dev = cuda_device
    H, V, t = 128, 515, 0.8
    gen = torch.Generator().manual_seed(53)
    true_lens = [9, 1, 17, 13, 6]
    padded = [10, 2, 17, 16, 6]
    cu = torch.cat([torch.zeros(1, dtype=torch.long), torch.tensor(padded).cumsum(0)]).to(dev)
    T = int(cu[-1])
    hidden = torch.randn(1, T, H, generator=gen).to(torch.bfloat16).to(dev)
    weight = (torch.randn(V, H, generator=gen) * 3 / H**0.5).to(torch.bfloat16).to(dev)
    tokens = torch.randint(0, V, (1, T), generator=gen).to(dev)
    L = 20
    am = torch.zeros(len(true_lens), L, dtype=torch.bool)
    for b, n in enumerate(true_lens):
        am[b, L - n:] = True
    cases = {"plain": (dict(), L), "mask": (dict(attention_mask=am.to(dev)), L), "sub": (dict(sub_seq_lengths=[[9, 1], [17], [13, 6]]), 31)}
    for name, (kw, seqlen) in cases.items():
        for window in (4, 11, seqlen - 1):
            hd, wd = hidden.clone().requires_grad_(True), weight.clone().requires_grad_(True)
            full = model_utils.from_parallel_hidden_to_logprobs_packed_sequences(hd, wd, tokens, cu, seqlen, 0, V, None,
                                                                                 temperature=t, **kw)
            G = torch.randn(full.shape[0], window, generator=gen).to(dev)
            (full[:, -window:] * G).sum().backward()
            h2, w2 = hidden.clone().requires_grad_(True), weight.clone().requires_grad_(True)
            got = model_utils.from_parallel_hidden_to_logprobs_packed_sequences(h2, w2, tokens, cu, seqlen, 0, V, None,
                                                                                temperature=t, action_window=window, **kw)
            assert got.shape == (full.shape[0], window), name
            torch.testing.assert_close(got.detach(), full.detach()[:, -window:], rtol=0, atol=1e-6, msg=f"{name} {window}")
            (got * G).sum().backward()
            if full.detach()[:, -window:].abs().sum() > 0:
                assert cos(h2.grad, hd.grad) >= 0.9999 and cos(w2.grad, wd.grad) >= 0.9999, (name, window)
    with pytest.raises(ValueError):
        model_utils.from_parallel_hidden_to_logprobs_packed_sequences(hidden, weight, tokens, cu, L, 0, V, None, action_window=L)


def test_dense_wrapper_action_window(cuda_device):
    dev = cuda_device
    gen = torch.Generator().manual_seed(54)
    B, S, H, V, t = 3, 37, 128, 700, 0.7
    hidden = torch.randn(B, S, H, generator=gen).to(torch.bfloat16).to(dev)
    weight = (torch.randn(V, H, generator=gen) * 3 / H**0.5).to(torch.bfloat16).to(dev)
    tokens = torch.randint(0, V, (B, S), generator=gen).to(dev)
    for window in (1, 9, S - 1):
        hd, wd = hidden.clone().requires_grad_(True), weight.clone().requires_grad_(True)
        full = model_utils.from_parallel_hidden_to_logprobs(hd, wd, tokens, 0, V, None, temperature=t)
        G = torch.randn(B, window, generator=gen).to(dev)
        (full[:, -window:] * G).sum().backward()
        h2, w2 = hidden.clone().requires_grad_(True), weight.clone().requires_grad_(True)
        got = model_utils.from_parallel_hidden_to_logprobs(h2, w2, tokens, 0, V, None, temperature=t, action_window=window)
        assert got.shape == (B, window)
        torch.testing.assert_close(got.detach(), full.detach()[:, -window:], rtol=0, atol=1e-6)
        (got * G).sum().backward()
        assert cos(h2.grad, hd.grad) >= 0.9999 and cos(w2.grad, wd.grad) >= 0.9999
    with pytest.raises(ValueError):
        model_utils.from_parallel_hidden_to_logprobs(hidden, weight, tokens, 0, V, None, action_window=S)


def test_packed_argument_errors(cuda_device):
    lib = _lib.load()
    x = torch.zeros(8, dtype=torch.float32, device=cuda_device)
    i = torch.zeros(8, dtype=torch.int64, device=cuda_device)
    m = torch.zeros(8, dtype=torch.uint8, device=cuda_device)
    p = lambda t: t.data_ptr()  # noqa: E731
    assert lib.skyrl_packed_next_token_labels(None, p(i), 1, 4, p(i), None) == -1
    assert lib.skyrl_packed_next_token_labels(p(i), p(i), -1, 4, p(i), None) == -2
    assert lib.skyrl_packed_scatter_logprobs(p(x), p(i), 1, 4, p(i), None, None, None, 1, 4, p(x), None) == -1
    assert lib.skyrl_packed_scatter_logprobs(p(x), p(i), 1, 4, p(i), p(i), p(i), p(m), 1, 4, p(x), None) == -5
    assert lib.skyrl_packed_scatter_logprobs(p(x), p(i), 2, 4, None, None, None, p(m), 1, 4, p(x), None) == -2
    assert lib.skyrl_packed_gather_grad(p(x), p(i), 1, 4, None, None, None, None, 1, -1, p(x), None) == -2
    torch.cuda.synchronize()


@pytest.mark.parametrize("packed", [False, True])
@pytest.mark.parametrize("compute_entropy,entropy_grad", [(False, False), (True, False), (True, True)])
def test_fsdp_forward_tail_from_hidden(cuda_device, packed, compute_entropy, entropy_grad):
    """action_log_probs_from_hidden against the reference tail evaluated on materialised fp64 logits: values, shapes, the
    zero padding, and the gradients into hidden and weight (log-probability loss, plus an entropy term when it has a grad)."""
    from skyrl_amd.model_wrapper import action_log_probs_from_hidden
    dev = cuda_device
    gen = torch.Generator().manual_seed(61)
    B, S, H, V, A, t = 3, 24, 128, 700, 7, 0.8
    seqs = torch.randint(0, V, (B, S), generator=gen)
    am = torch.ones(B, S, dtype=torch.long)
    am[0, :5] = 0
    am[1, :2] = 0
    weight = (torch.randn(V, H, generator=gen) * 3 / H ** 0.5).to(torch.bfloat16)
    nnz = am.flatten().nonzero().flatten() if packed else None
    n_tok = int(am.sum()) if packed else B * S
    hidden = torch.randn(1 if packed else B, n_tok if packed else S, H, generator=gen).to(torch.bfloat16)

    h64, w64 = hidden.double().requires_grad_(True), weight.double().requires_grad_(True)
    want_alp, want_ent = O.hf_wrapper_tail(h64 @ w64.t(), seqs, A, am.double(), t, nnz_indices=nnz)
    G = torch.randn(B, A, generator=gen).double()
    Q = torch.randn(B, S, generator=gen).double() * 0.1
    loss = (want_alp * G).sum() + ((want_ent * Q).sum() if entropy_grad else 0.0)
    loss.backward()

    hd, wd = hidden.to(dev).requires_grad_(True), weight.to(dev).requires_grad_(True)
    got = action_log_probs_from_hidden(hd, wd, seqs.to(dev), A, am.to(dev), t, return_output=True,
                                       compute_entropy=compute_entropy, entropy_requires_grad=entropy_grad,
                                       nnz_indices=None if nnz is None else nnz.to(dev))
    alp, out = got
    assert alp.shape == (B, A) and alp.dtype == torch.float32
    torch.testing.assert_close(alp.detach().cpu().double(), want_alp.detach(), atol=LOGPROB_ATOL, rtol=0)
    loss = (alp * G.float().to(dev)).sum()
    if compute_entropy:
        ent = out["entropy"]
        assert ent.shape == (B, S) and ent.requires_grad == entropy_grad
        torch.testing.assert_close(ent.detach().cpu().double(), want_ent.detach(), rtol=ENTROPY_RTOL, atol=1e-6)
        assert bool((ent.detach().cpu()[am == 0] == 0).all())
        if entropy_grad:
            loss = loss + (ent * Q.float().to(dev)).sum()
    else:
        assert out == {}
    loss.backward()
    assert cos(hd.grad, h64.grad) >= GRAD_COS and cos(wd.grad, w64.grad) >= GRAD_COS


def test_masked_training_step_replays_from_a_hip_graph(cuda_device):
    """Forward -> actor loss (its gradient is the backward's upstream gradient, zero on masked tokens) -> backward on the active
    rows, captured as one HIP graph: nothing on that path reads a value back on the host.  Every replay, on new inputs and a new
    mask (so a new number of active rows), must equal the eager step bit for bit."""
    from types import SimpleNamespace

    from skyrl_amd.policy_loss import actor_loss

    dev = cuda_device
    B, S, H, V = 3, 120, 128, 1500
    gen = torch.Generator().manual_seed(17)
    weight = (torch.randn(V, H, generator=gen) * 3 / H ** 0.5).bfloat16().to(dev)
    hidden = torch.zeros(B * S, H, dtype=torch.bfloat16, device=dev)
    labels = torch.zeros(B * S, dtype=torch.int64, device=dev)
    old = torch.zeros(B, S, device=dev)
    adv = torch.zeros(B, S, device=dev)
    mask = torch.zeros(B, S, device=dev)
    cfg = SimpleNamespace(policy_loss_type="regular", eps_clip_low=0.2, eps_clip_high=0.2, use_kl_loss=False,
                          use_entropy_loss=False)

    def step():
        h = hidden.detach().requires_grad_(True)
        w = weight.detach().requires_grad_(True)
        lp, _ = linear_cross_entropy(h, w, labels, 1.0, "none", None, False)
        loss, _ = actor_loss(lp.reshape(B, S), old, adv, cfg, mask)
        gh, gw = torch.autograd.grad(loss, (h, w))
        return loss.detach(), gh, gw

    def refill(seed):
        gen_ = torch.Generator().manual_seed(seed)
        hidden.copy_(torch.randn(B * S, H, generator=gen_).bfloat16())
        labels.copy_(torch.randint(0, V, (B * S,), generator=gen_))
        old.copy_(torch.randn(B, S, generator=gen_) * 0.1 - 7.0)
        adv.copy_(torch.randn(B, S, generator=gen_))
        mask.copy_((torch.rand(B, S, generator=gen_) < 0.2 * seed).float())

    refill(1)
    side = torch.cuda.Stream(device=dev)
    side.wait_stream(torch.cuda.current_stream(dev))
    with torch.cuda.stream(side):
        step()
    torch.cuda.current_stream(dev).wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        captured = step()
    for seed in (2, 4, 0, 3):               # 40 %, 80 %, none and 60 % of the tokens active
        refill(seed)
        graph.replay()
        torch.cuda.synchronize()
        got = [t.clone() for t in captured]
        want = step()
        torch.cuda.synchronize()
        for a, b in zip(got, want):
            assert torch.equal(a, b)
        assert float(got[1][(mask.reshape(-1) == 0)].abs().max() if (mask == 0).any() else 0.0) == 0.0


def test_vocab_shards_reproduce_the_full_vocabulary(cuda_device):
    """How the path shards over a vocabulary-parallel group, on one GPU: forward per weight slice, the four [T] vectors
    merged (what the group's all-reduces would do), backward per slice with the global statistics.  The slices' d_weight
    rows concatenate to the full d_weight and their d_hidden shares add up to the full d_hidden."""
    from skyrl_amd.vocab_shards import merge_shard_statistics
    dev = cuda_device
    T, H, V, t = 300, 128, 1000, 0.7
    hidden, weight, labels, g, q = _rand(T, H, V, seed=31)
    labels[:7] = SENTINEL                                  # targets no shard owns
    h, w, y = hidden.to(dev), weight.to(dev), labels.to(dev)
    gd, qd = g.to(dev), q.to(dev)
    full_lp, full_ent, full_lse, full_pz = ops.lmhead_fwd(h, w, y, 1.0 / t, True)
    full_dh, full_dw = ops.lmhead_bwd(h, w, y, full_lse, full_pz, gd, qd, 1.0 / t, 0)

    bounds = [0, 256, 333, 1000]                           # uneven slices, one narrower than a tile
    outs, owners, local_labels = [], [], []
    for lo, hi in zip(bounds[:-1], bounds[1:]):
        own = (y >= lo) & (y < hi)
        yl = torch.where(own, y - lo, torch.full_like(y, SENTINEL))
        outs.append(ops.lmhead_fwd(h, w[lo:hi].contiguous(), yl, 1.0 / t, True))
        owners.append(own)
        local_labels.append(yl)
    lp, ent, lse, pz = merge_shard_statistics(torch.stack([o[0] for o in outs]), torch.stack([o[2] for o in outs]),
                                              torch.stack([o[3] for o in outs]), torch.stack(owners))
    torch.testing.assert_close(lp, full_lp, atol=2e-5, rtol=0)
    torch.testing.assert_close(ent, full_ent, atol=2e-5, rtol=1e-5)
    torch.testing.assert_close(lse, full_lse, atol=2e-5, rtol=0)
    assert bool((lp[:7] == 0).all())

    dh_sum = torch.zeros(T, H, dtype=torch.float32, device=dev)
    for (lo, hi), yl in zip(zip(bounds[:-1], bounds[1:]), local_labels):
        dh, dw = ops.lmhead_bwd(h, w[lo:hi].contiguous(), yl, lse, pz, gd, qd, 1.0 / t, 0)
        # same dz values up to the rounding of the merged lse and sum p z: now and then one bf16 dz value lands on the other
        # side of a rounding boundary (2^-8 of one term of the sum)
        torch.testing.assert_close(dw, full_dw[lo:hi], atol=1e-3, rtol=5e-3)
        dh_sum += dh.float()
    assert cos(dh_sum, full_dh) >= 0.9999 and rel_l2(dh_sum, full_dh.float()) < 1e-2   # three bf16 roundings instead of one


def test_opcheck_registration(cuda_device):
    T, H, V = 64, 64, 300
    hidden, weight, labels, _, _ = _rand(T, H, V, seed=2)
    args = (hidden.to(cuda_device), weight.to(cuda_device), labels.to(cuda_device), 1.0, True)
    torch.library.opcheck(torch.ops.skyrl_amd.lmhead_fwd.default, args, test_utils=("test_schema", "test_faketensor"))


# ---------------------------------------------------------------------------------------------------------------------
# full benchmark sizes: row / column sub-sampling against the oracle and size-independent invariants
# ---------------------------------------------------------------------------------------------------------------------
def _full_size_check(cfg, dev, n_rows=24, n_vocab=12):
    d = make_inputs(cfg)
    T, H, V = cfg.T, cfg.H, cfg.V
    h, w, y = d["hidden"].to(dev), d["weight"].to(dev), d["labels"].to(dev)
    torch.cuda.synchronize()
    torch.cuda.reset_peak_memory_stats()
    base = torch.cuda.memory_allocated()
    lp, ent, lse, pz = ops.lmhead_fwd(h, w, y, 1.0 / cfg.temperature, cfg.entropy or cfg.entropy_grad)
    torch.cuda.synchronize()
    peak_fwd = torch.cuda.max_memory_allocated() - base
    assert peak_fwd < ops.fwd_workspace_bytes(T, H, V) + 16 * 4 * T + (64 << 20)  # allocator rounding
    assert peak_fwd < 2 * T * V / 8  # far below one bf16 T x V buffer

    gen = torch.Generator().manual_seed(7)
    rows = torch.randperm(T, generator=gen)[:n_rows].sort().values
    w64 = d["weight"].double()
    z = (d["hidden"][rows].double() @ w64.t()) / cfg.temperature
    lsm = torch.log_softmax(z, -1)
    want_lp = lsm.gather(-1, d["labels"][rows][:, None])[:, 0]
    assert (lp.cpu()[rows].double() - want_lp).abs().max() <= 1e-3
    if cfg.entropy or cfg.entropy_grad:
        want_ent = -(lsm.exp() * lsm).sum(-1)
        assert ((ent.cpu()[rows].double() - want_ent).abs() / want_ent).max() <= 1e-3
        assert (ent >= 0).all() and (ent <= math.log(V) + 1e-3).all()
    assert (lp <= 0).all() and torch.isfinite(lp).all()
    want_lse = torch.logsumexp(z, -1)
    assert (lse.cpu()[rows].double() - want_lse).abs().max() <= 1e-3
    _check_every_token_against_the_library(cfg, h, w, y, lp, ent if (cfg.entropy or cfg.entropy_grad) else None, lse)
    if not cfg.backward:
        return

    g = d["dlogprobs"].to(dev)
    q = d["dentropy"].to(dev) if cfg.entropy_grad else None
    torch.cuda.reset_peak_memory_stats()
    base = torch.cuda.memory_allocated()
    dh, dw = ops.lmhead_bwd(h, w, y, lse, pz if q is not None else None, g, q, 1.0 / cfg.temperature, 0)
    torch.cuda.synchronize()
    peak_bwd = torch.cuda.max_memory_allocated() - base
    assert peak_bwd < ops.bwd_workspace_bytes(T, H, V) + 2 * T * H + 4 * V * H + (64 << 20)  # allocator rounding
    assert ops.bwd_workspace_bytes(T, H, V) < 2 * T * V  # no buffer the size of bf16 logits

    # dHidden rows: exact dz for the sampled rows, times W
    rt = 1.0 / cfg.temperature
    p = lsm.exp()
    gg = d["dlogprobs"][rows].double()
    dz = -p * gg[:, None]
    dz[torch.arange(n_rows), d["labels"][rows]] += gg
    if cfg.entropy_grad:
        qq = d["dentropy"][rows].double()
        pzr = (p * z).sum(-1)
        dz = dz - qq[:, None] * p * (z - pzr[:, None])
    dz = dz * rt
    want_dh = dz @ w64
    got_dh = dh.cpu()[rows].double()
    assert cos(got_dh, want_dh) >= GRAD_COS
    assert rel_l2(got_dh, want_dh) < GRAD_REL_L2 and worst_row(got_dh, want_dh) < GRAD_ROW_REL_L2
    masked = d["mask"] == 0
    if masked.any() and not cfg.entropy_grad:  # tokens without an upstream gradient get exactly zero rows
        assert float(dh[masked.to(dev)].abs().max()) == 0.0
    del z, lsm, p, dz

    # dW rows for a few vocab ids (incl. some that are labels): needs every token, uses the verified lse / pz from the GPU
    vs = torch.cat([d["labels"][rows[: n_vocab // 2]], torch.randperm(V, generator=gen)[: n_vocab - n_vocab // 2]])
    hd64 = d["hidden"].double()
    zc = (hd64 @ w64[vs].t()) * rt  # [T, n_vocab]
    pc = (zc - lse.cpu().double()[:, None]).exp()
    gall = d["dlogprobs"].double()
    dzc = -pc * gall[:, None]
    dzc += (d["labels"][:, None] == vs[None, :]).double() * gall[:, None]
    if cfg.entropy_grad:
        dzc = dzc - d["dentropy"].double()[:, None] * pc * (zc - pz.cpu().double()[:, None])
    want_dw = (dzc * rt).t() @ hd64
    got_dw = dw[vs.to(dev)].cpu().double()
    assert cos(got_dw, want_dw) >= GRAD_COS
    assert rel_l2(got_dw, want_dw) < GRAD_REL_L2 and worst_row(got_dw, want_dw) < GRAD_ROW_REL_L2
    # checksum over the whole gradient: every row of dz sums to 0 (labels all in vocabulary), so the columns of dW sum to ~0
    col = dw.sum(0).abs().max().item()
    scale = dw.abs().sum(0).max().item()
    assert col < 2e-3 * scale
    assert torch.isfinite(dh).all() and torch.isfinite(dw).all()


def _check_every_token_against_the_library(cfg, h, w, y, lp, ent, lse, slab=512):
    """Log-sum-exp, log-probability and entropy of ALL tokens against an independent computation on the GPU with library
    routines only: fp32 ``torch.matmul`` of 512-token slabs with the weight (a [512, V] fp32 slab, never T x V), then
    ``torch.logsumexp`` / ``gather`` / ``softmax``.  The sampled fp64 rows above pin the library's result; this pins every
    row of the kernel's -- the expected dW rows below are built from the kernel's own lse of all tokens."""
    T, V = cfg.T, cfg.V
    w32 = w.float()
    rt = 1.0 / cfg.temperature
    worst_lse = worst_lp = worst_ent = 0.0
    for t0 in range(0, T, slab):
        t1 = min(T, t0 + slab)
        z = torch.matmul(h[t0:t1].float(), w32.t()) * rt
        ref_lse = torch.logsumexp(z, -1)
        worst_lse = max(worst_lse, float((lse[t0:t1] - ref_lse).abs().max()))
        ref_lp = z.gather(-1, y[t0:t1, None])[:, 0] - ref_lse
        worst_lp = max(worst_lp, float((lp[t0:t1] - ref_lp).abs().max()))
        if ent is not None:
            ref_ent = ref_lse - (torch.softmax(z, -1) * z).sum(-1)
            worst_ent = max(worst_ent, float(((ent[t0:t1] - ref_ent).abs() / ref_ent.abs().clamp(min=1e-3)).max()))
        del z
    assert worst_lse <= 1e-3 and worst_lp <= 1e-3 and worst_ent <= 2e-3, (worst_lse, worst_lp, worst_ent)


def test_full_size_packed_wrapper_qwen7b(cuda_device):
    """The 7B configuration as the Megatron worker feeds it: one packed stream of 16384 tokens with the configuration's own
    ``cu_seqlens`` through ``from_parallel_hidden_to_logprobs_packed_sequences`` and autograd (model_utils.py:773-883).
    Checked: every landed log-probability against the flat op on the rolled labels (bit-exact: same kernels), padding exactly
    zero, sampled rows against fp64, and the gradients against the flat backward on the scattered-back upstream gradient."""
    from skyrl_amd.model_utils import from_parallel_hidden_to_logprobs_packed_sequences

    dev = cuda_device
    cfg = CONFIGS["qwen2.5-7b-fwdbwd"]
    d = make_inputs(cfg)
    T, H, V = cfg.T, cfg.H, cfg.V
    cu = d["cu_seqlens"]
    lens = (cu[1:] - cu[:-1]).tolist()
    n, L = len(lens), max(lens)
    hidden = d["hidden"].to(dev).requires_grad_(True)
    weight = d["weight"].to(dev).requires_grad_(True)
    tokens = d["labels"].to(dev)                     # the packed input ids; the wrapper rolls them per sequence
    out = from_parallel_hidden_to_logprobs_packed_sequences(hidden.unsqueeze(0), weight, tokens.unsqueeze(0), cu.to(dev), L, 0, V,
                                                            None, temperature=cfg.temperature, fused_backend="hip")
    assert out.shape == (n, L - 1) and out.dtype == torch.float32
    gen = torch.Generator().manual_seed(5)
    up = torch.randn(n, L - 1, generator=gen)
    out.backward(up.to(dev))

    # expectation by a per-sequence loop on the host: successor labels, landing positions, upstream gradient per token
    rolled = torch.empty(T, dtype=torch.int64)
    g_tok = torch.zeros(T)
    landed = torch.zeros(n, L - 1, dtype=torch.bool)
    for i, ln in enumerate(lens):
        a = int(cu[i])
        rolled[a:a + ln] = torch.roll(d["labels"][a:a + ln], -1)
        g_tok[a:a + ln - 1] = up[i, :ln - 1]
        landed[i, :ln - 1] = True
    lp_flat, _, lse, _ = ops.lmhead_fwd(hidden.detach(), weight.detach(), rolled.to(dev), 1.0 / cfg.temperature, False)
    got = out.detach().cpu()
    assert float(got[~landed].abs().max()) == 0.0
    for i, ln in enumerate(lens):
        a = int(cu[i])
        assert torch.equal(got[i, :ln - 1], lp_flat[a:a + ln - 1].cpu())
    rows = torch.randperm(T, generator=gen)[:16]
    z = (d["hidden"][rows].double() @ d["weight"].double().t()) / cfg.temperature
    want = torch.log_softmax(z, -1).gather(-1, rolled[rows][:, None])[:, 0]
    assert float((lp_flat.cpu()[rows].double() - want).abs().max()) <= 1e-3
    dh, dw = ops.lmhead_bwd(hidden.detach(), weight.detach(), rolled.to(dev), lse, None, g_tok.to(dev), None, 1.0 / cfg.temperature, 0)
    assert hidden.grad.dtype == torch.bfloat16 and weight.grad.dtype == torch.bfloat16
    last = torch.tensor([int(cu[i + 1]) - 1 for i in range(n)])
    assert float(hidden.grad[last.to(dev)].abs().max()) == 0.0          # the last token of a sequence predicts nothing
    assert torch.equal(hidden.grad, dh)                                    # rows dropped or not, same products
    assert rel_l2(weight.grad.float(), dw) < 5e-3                          # bf16 rounding of the fp32 sums
    p = torch.softmax(z, -1)
    gg = g_tok[rows].double()
    dz = -p * gg[:, None]
    dz[torch.arange(len(rows)), rolled[rows]] += gg
    want_dh = (dz / cfg.temperature) @ d["weight"].double()
    assert cos(hidden.grad.cpu()[rows].double(), want_dh) >= GRAD_COS


def test_full_size_forward_qwen05b(cuda_device):
    _full_size_check(CONFIGS["qwen2.5-0.5b-fwd"], cuda_device)


def test_full_size_forward_backward_qwen7b(cuda_device):
    _full_size_check(CONFIGS["qwen2.5-7b-fwdbwd"], cuda_device)


def test_full_size_forward_backward_qwen15b(cuda_device):
    _full_size_check(CONFIGS["qwen2.5-1.5b-fwdbwd"], cuda_device)


def test_full_size_forward_backward_llama8b(cuda_device):
    # T = 32768, H = 4096: the panel cap decides the chunk width, the largest scratch offsets of the five configurations
    _full_size_check(CONFIGS["llama3.1-8b-fwdbwd"], cuda_device)


def test_full_size_forward_qwen32b(cuda_device):
    _full_size_check(CONFIGS["qwen3-32b-fwd"], cuda_device)


def test_full_size_long_context_262k(cuda_device):
    """One sequence of 262144 tokens at H = 2048 against one TP=4 vocabulary shard (62080 columns), the long-context point of
    the reference's harness (skyrl/benchmarks/bench_fused_linear_logprob.py:39-47): eight token blocks in both passes, dW
    summed over them, scratch sized by the block."""
    cfg = CONFIGS["longctx-s262144-v62080"]
    T, H, V = cfg.T, cfg.H, cfg.V
    assert ops.fwd_workspace_bytes(T, H, V) == ops.fwd_workspace_bytes(32768, H, V)
    assert ops.bwd_workspace_bytes(T, H, V) < 2 * 32768 * V // 2 + 4 * V * H + (1 << 30)  # nothing of the size of T x V (32 GB in bf16)
    _full_size_check(cfg, cuda_device, n_rows=16, n_vocab=8)


# ---------------------------------------------------------------------------------------------------------------------
# MTP draft loss: soft cross-entropy from hidden states
# ---------------------------------------------------------------------------------------------------------------------
SOFTCE_ATOL = 5e-3   # per-token loss, absolute (values are of the order of ln V)


def _softce_case(B, S, H, V, seed, spread=3.0):
    gen = torch.Generator().manual_seed(seed)
    hs = torch.randn(B, S, H, generator=gen).bfloat16()
    ht = torch.randn(B, S, H, generator=gen).bfloat16()
    w = (torch.randn(V, H, generator=gen) * spread / H ** 0.5).bfloat16()
    return hs, ht, w


@pytest.mark.parametrize("B,S,H,V,depth,temperature,vocab_chunk", [
    (3, 50, 128, 1000, 0, 1.0, 0),        # ragged tokens and vocabulary, transposed-weight fallback (V % 64 != 0)
    (2, 200, 192, 1088, 1, 0.7, 0),       # weight read in place, depth 1, a temperature
    (1, 333, 128, 1000, 2, 1.0, 256),     # one packed row, four vocabulary chunks
    (4, 128, 256, 8192, 0, 1.0, 2048),    # whole tiles, four chunks in place
])
def test_soft_ce_from_hidden_matches_oracle(B, S, H, V, depth, temperature, vocab_chunk, cuda_device):
    from skyrl_amd.mtp_soft_ce import soft_ce_from_hidden

    hs, ht, w = _softce_case(B, S, H, V, 40 + depth)
    gen = torch.Generator().manual_seed(77)
    g = torch.randn(B, S, generator=gen) * (torch.rand(B, S, generator=gen) > 0.3)

    hs64 = hs.double().requires_grad_(True)
    student_logits = hs64 @ w.double().t() / temperature
    teacher_logits = O.build_teacher_logits(ht.double() @ w.double().t() / temperature, depth)
    ref = O.soft_ce_per_token(student_logits, teacher_logits)
    (ref * g.double()).sum().backward()

    d_hs = hs.to(cuda_device).requires_grad_(True)
    got = soft_ce_from_hidden(d_hs, ht.to(cuda_device), w.to(cuda_device), shift=depth + 1, temperature=temperature,
                              vocab_chunk=vocab_chunk)
    assert got.shape == (B, S) and got.dtype == torch.float32
    (got * g.to(cuda_device)).sum().backward()
    err = (got.detach().cpu().double() - ref.detach()).abs().max().item()
    assert err <= SOFTCE_ATOL, f"per-token loss max abs err {err}"
    assert d_hs.grad.dtype == torch.bfloat16 and d_hs.grad.shape == hs.shape
    assert cos(d_hs.grad.float(), hs64.grad) >= GRAD_COS
    rel = (d_hs.grad.cpu().double() - hs64.grad).norm() / hs64.grad.norm()
    assert rel.item() <= 2e-2, f"gradient relative error {rel.item()}"
    assert bool((d_hs.grad.cpu()[g == 0] == 0).all())           # tokens without an upstream gradient get exact zeros


def test_soft_ce_limits_against_the_logprob_kernels(cuda_device):
    """Teacher = student, no roll: the loss is the entropy the log-probability forward reports, and the gradient is exactly
    zero (both softmaxes come from the same accumulator values)."""
    from skyrl_amd.mtp_soft_ce import soft_ce_from_hidden

    hs, _, w = _softce_case(2, 300, 128, 2000, 51)
    d_hs = hs.to(cuda_device).requires_grad_(True)
    dw = w.to(cuda_device)
    loss = soft_ce_from_hidden(d_hs, d_hs.detach(), dw, shift=0)
    loss.sum().backward()
    labels = torch.zeros(600, dtype=torch.int64, device=cuda_device)
    _, entropy, _, _ = ops.lmhead_fwd(d_hs.detach().reshape(600, 128), dw, labels, 1.0, True)
    torch.testing.assert_close(loss.detach().reshape(-1), entropy, rtol=1e-5, atol=1e-5)
    assert bool((d_hs.grad == 0).all())


def test_draft_soft_ce_from_hidden_matches_oracle(cuda_device):
    from skyrl_amd.mtp_soft_ce import draft_soft_ce_from_hidden, shift_mask_for_mtp

    B, S, H, V, depth = 3, 70, 128, 1500, 1
    hs, ht, w = _softce_case(B, S, H, V, 60)
    gen = torch.Generator().manual_seed(61)
    attn = (torch.rand(B, S, generator=gen) > 0.2).float()
    attn[1, :9] = 0                                              # left padding
    mask = O.shift_mask_for_mtp(attn.clone(), depth)
    for factor in (None, torch.tensor(57.0), torch.tensor(0.5)):
        hs64 = hs.double().requires_grad_(True)
        ref = O.draft_soft_ce_from_hidden(hs64, ht.double(), w.double(), mask.double(), depth, factor)
        ref.backward()
        d_hs = hs.to(cuda_device).requires_grad_(True)
        d_mask = shift_mask_for_mtp(attn.to(cuda_device), depth)
        assert torch.equal(d_mask.cpu(), mask)
        got = draft_soft_ce_from_hidden(d_hs, ht.to(cuda_device), w.to(cuda_device), d_mask, depth,
                                        None if factor is None else factor.to(cuda_device))
        got.backward()
        assert got.dim() == 0 and got.item() == pytest.approx(ref.item(), abs=SOFTCE_ATOL * max(1.0, ref.item() / 10))
        assert cos(d_hs.grad.float(), hs64.grad) >= GRAD_COS
    with pytest.raises(AssertionError, match="must be detached"):
        draft_soft_ce_from_hidden(d_hs, ht.to(cuda_device).requires_grad_(True), w.to(cuda_device), d_mask, depth)


def test_soft_ce_argument_errors(cuda_device):
    lib = _lib.load()
    x = torch.zeros(256, 128, dtype=torch.bfloat16, device=cuda_device)
    f = torch.zeros(256, dtype=torch.float32, device=cuda_device)
    ws = torch.zeros(lib.skyrl_softce_fwd_workspace_bytes(256, 128, 256), dtype=torch.uint8, device=cuda_device)
    p, fp = x.data_ptr(), f.data_ptr()

    def fwd(**kw):
        a = dict(s=p, lds=128, t=p, ldt=128, w=p, ldw=128, T=256, seq=64, shift=1, H=128, V=256, rt=1.0, loss=fp, ls=fp, lt=fp,
                 ws=ws.data_ptr(), wsb=ws.numel())
        a.update(kw)
        return lib.skyrl_softce_fwd(a["s"], a["lds"], a["t"], a["ldt"], a["w"], a["ldw"], a["T"], a["seq"], a["shift"], a["H"],
                                    a["V"], a["rt"], a["loss"], a["ls"], a["lt"], a["ws"], a["wsb"], None)

    assert fwd() == 0
    assert fwd(t=None) == -1 and fwd(loss=None) == -1
    assert fwd(seq=100) == -2 and fwd(seq=0) == -2 and fwd(shift=-1) == -2 and fwd(ldt=64) == -2
    assert fwd(t=p + 8) == -3
    assert fwd(wsb=1024) == -4 and fwd(ws=None) == -4
    assert fwd(rt=0.0) == -5
    assert lib.skyrl_softce_bwd_workspace_bytes(256, 128, 256, 100) == 0
    assert lib.skyrl_softce_bwd(p, 128, p, 128, p, 128, fp, fp, None, 256, 64, 1, 128, 256, 1.0, p, 0, ws.data_ptr(), ws.numel(),
                                None) == -1
    assert lib.skyrl_softce_bwd(p, 128, p, 128, p, 128, fp, fp, fp, 256, 64, 1, 128, 256, 1.0, p, 0, ws.data_ptr(), 1024,
                                None) == -4
    torch.cuda.synchronize()


def test_soft_ce_full_size_properties(cuda_device):
    """The benchmark shape (T=16384, H=3584, V=152064), through size-independent properties: teacher = student gives the
    entropy of the log-probability forward and an exactly zero gradient; the per-token loss is at least the teacher's
    entropy (Gibbs); the gradient is linear in the upstream gradient for power-of-two factors, bit for bit."""
    from skyrl_amd.mtp_soft_ce import softce_bwd, softce_fwd

    T, H, V = 16384, 3584, 152064
    gen = torch.Generator(device=cuda_device).manual_seed(9)
    hs = torch.randn(T, H, generator=gen, device=cuda_device).bfloat16()
    ht = torch.randn(T, H, generator=gen, device=cuda_device).bfloat16()
    w = (torch.randn(V, H, generator=gen, device=cuda_device) * 3 / H ** 0.5).bfloat16()
    g = torch.randn(T, generator=gen, device=cuda_device)
    labels = torch.zeros(T, dtype=torch.int64, device=cuda_device)

    loss_self, lse_s, lse_t = softce_fwd(ht, ht, w, T, 0, 1.0)
    _, entropy, lse, _ = ops.lmhead_fwd(ht, w, labels, 1.0, True)
    torch.testing.assert_close(loss_self, entropy, rtol=1e-5, atol=1e-5)
    torch.testing.assert_close(lse_t, lse, rtol=1e-6, atol=1e-6)
    assert bool((softce_bwd(ht, ht, w, lse_s, lse_t, g, T, 0, 1.0, 0) == 0).all())

    lib = _lib.load()
    torch.cuda.synchronize()
    torch.cuda.reset_peak_memory_stats()
    base = torch.cuda.memory_allocated()
    loss, lse_s, lse_t = softce_fwd(hs, ht, w, T, 1, 1.0)
    torch.cuda.synchronize()
    peak = torch.cuda.max_memory_allocated() - base
    assert peak < lib.skyrl_softce_fwd_workspace_bytes(T, H, V) + 16 * 4 * T + (64 << 20)
    assert peak < 2 * T * V / 4                                   # far below one bf16 T x V buffer, let alone two in fp32
    # sampled tokens against fp64 logits of just those rows
    rows = torch.randperm(T - 1, generator=torch.Generator().manual_seed(3))[:12].sort().values
    w64 = w.cpu().double()
    zs = hs.cpu()[rows].double() @ w64.t()
    zt = ht.cpu()[rows + 1].double() @ w64.t()
    want = O.soft_ce_per_token(zs, zt)
    assert (loss.cpu()[rows].double() - want).abs().max().item() <= SOFTCE_ATOL
    rolled_entropy = torch.roll(entropy, -1)                      # the teacher of token t is row t + 1
    assert bool((loss >= rolled_entropy - 1e-3).all()) and bool(torch.isfinite(loss).all())
    torch.cuda.reset_peak_memory_stats()
    base = torch.cuda.memory_allocated()
    d1 = softce_bwd(hs, ht, w, lse_s, lse_t, g, T, 1, 1.0, 0)
    torch.cuda.synchronize()
    peak = torch.cuda.max_memory_allocated() - base
    assert peak < lib.skyrl_softce_bwd_workspace_bytes(T, H, V, 0) + 2 * T * H + (64 << 20)
    assert lib.skyrl_softce_bwd_workspace_bytes(T, H, V, 0) < 2 * T * V
    want_rows = ((torch.softmax(zs, -1) - torch.softmax(zt, -1)) * g.cpu()[rows].double()[:, None]) @ w64
    assert cos(d1.cpu()[rows].float(), want_rows) >= GRAD_COS
    d4 = softce_bwd(hs, ht, w, lse_s, lse_t, g * 4.0, T, 1, 1.0, 0)
    assert torch.equal(d4.float(), d1.float() * 4.0) and bool(torch.isfinite(d1.float()).all())
    # a different vocabulary chunking changes the order of the fp32 partial sums only
    d_chunked = softce_bwd(hs, ht, w, lse_s, lse_t, g, T, 1, 1.0, 16384)
    assert cos(d_chunked.float(), d1.float()) >= 0.99999


@pytest.mark.parametrize("layout", ["attention_mask", "sub_sequences"])
@pytest.mark.parametrize("with_loss_mask", [False, True])
def test_packed_action_entropy_matches_oracle(layout, with_loss_mask, cuda_device):
    """The Megatron worker's entropy metric on a packed micro-batch: per-token entropy from the forward kernel, action-token
    weighted mean through the scatter kernels, against the oracle's restatement of the reference's packed-weight route."""
    gen = torch.Generator().manual_seed(33)
    H, V, temperature = 128, 1500, 0.8
    if layout == "attention_mask":
        L, num_actions = 40, 17
        real = [40, 23, 31, 5, 1]
        am = torch.zeros(len(real), L, dtype=torch.long)
        am[0] = 1
        am[1, L - 23:] = 1                                       # left padding
        am[2, :31] = 1                                           # right padding
        am[3, 10:15] = 1
        am[4, L - 1] = 1                                         # a single real token: nothing to score
        padded = [r + (-r) % 8 for r in real]
        sub = None
    else:
        L, num_actions = 48, 30
        sub = [[9, 1, 14], [20, 6], [33]]
        padded = [16, 8, 16, 24, 8, 40]
        am = torch.ones(len(sub), L, dtype=torch.long)
    B = am.shape[0]
    cu = torch.tensor([0] + list(np.cumsum(padded)))
    T = int(cu[-1])
    hidden = torch.randn(1, T, H, generator=gen).bfloat16()
    weight = (torch.randn(V, H, generator=gen) * 3 / H ** 0.5).bfloat16()
    loss_mask = (torch.rand(B, num_actions, generator=gen) > 0.35).float() if with_loss_mask else None

    ent64 = O.fused_entropy_from_hidden(hidden.double(), weight.double(), None, temperature).double().squeeze(0)
    want, want_loss = O.packed_action_entropy(ent64, cu, L, num_actions, am, None if loss_mask is None else loss_mask.double(), sub)

    to = lambda t: None if t is None else t.to(cuda_device)  # noqa: E731
    got, got_loss = model_utils.from_parallel_hidden_to_entropy_packed_sequences(
        to(hidden), to(weight), to(cu), L, num_actions, to(am), to(loss_mask), None, None, sub_seq_lengths=sub,
        temperature=temperature)
    assert got.dim() == 0 and not got.requires_grad
    assert want.item() > 0.5                                     # the case does put weight on real tokens
    assert got.item() == pytest.approx(want.item(), rel=ENTROPY_RTOL) and got_loss.item() == pytest.approx(want_loss.item(), rel=ENTROPY_RTOL)


@pytest.mark.parametrize("B,S,H,V,shift,vocab_chunk", [
    (1, 1, 64, 5, 1, 0),             # one token, a vocabulary smaller than a tile; the roll of a one-token row is itself
    (1, 63, 64, 255, 2, 0),          # one token short of the 64-token pairing unit, one row short of a vocabulary tile
    (3, 43, 320, 257, 1, 256),       # 129 tokens: one more than a 128-token tile; second chunk holds a single vocab row
    (5, 128, 128, 4104, 3, 1024),    # whole token tiles, V a multiple of 8 but not of 64, five chunks
    (7, 19, 192, 777, 20, 0),        # a shift larger than the row: wraps modulo the row length
    (1, 100, 128, 20032, 1, 4096),   # V a multiple of 64 (weight read in place), five chunks with a short last one
])
def test_soft_ce_edge_shapes_match_oracle(B, S, H, V, shift, vocab_chunk, cuda_device):
    from skyrl_amd.mtp_soft_ce import soft_ce_from_hidden

    hs, ht, w = _softce_case(B, S, H, V, 500 + V)
    gen = torch.Generator().manual_seed(V)
    g = torch.randn(B, S, generator=gen)
    hs64 = hs.double().requires_grad_(True)
    teacher_logits = torch.roll(ht.double() @ w.double().t(), -shift, dims=1)
    ref = O.soft_ce_per_token(hs64 @ w.double().t(), teacher_logits)
    (ref * g.double()).sum().backward()
    d_hs = hs.to(cuda_device).requires_grad_(True)
    got = soft_ce_from_hidden(d_hs, ht.to(cuda_device), w.to(cuda_device), shift=shift, vocab_chunk=vocab_chunk)
    (got * g.to(cuda_device)).sum().backward()
    err = (got.detach().cpu().double() - ref.detach()).abs().max().item()
    assert err <= SOFTCE_ATOL, f"per-token loss max abs err {err}"
    assert bool(torch.isfinite(d_hs.grad.float()).all())
    if hs64.grad.norm() > 0:
        assert cos(d_hs.grad.float(), hs64.grad) >= GRAD_COS
        rel = (d_hs.grad.cpu().double() - hs64.grad).norm() / hs64.grad.norm()
        assert rel.item() <= 2e-2, f"gradient relative error {rel.item()}"


@pytest.mark.parametrize("B,S,chunk", [(2, 4, 3), (2, 4, 8), (2, 4, 16), (1, 8, 3), (4, 1, 2), (1, 1, 1)])
def test_identity_lm_head_known_answer(B, S, chunk, cuda_device):
    """The reference's chunk-boundary cases (tests/tx/utils/test_logits_processor.py:39-58) on its deterministic input: an
    identity LM head and hidden = arange / n, so the logits are the hidden states themselves and the answer is
    log_softmax(hidden)[target] whatever the sequence chunk is.  H = V = 64 here (the kernel's k-tile) instead of 16."""
    V = 64
    hidden = (torch.arange(B * S * V, dtype=torch.float32).reshape(B, S, V) / (B * S * V)).bfloat16()
    target = (torch.arange(B * S).reshape(B, S) % V)
    weight = torch.eye(V).bfloat16()
    want = torch.log_softmax(hidden.double(), -1).gather(-1, target[..., None])[..., 0]
    got = FusedLinearLogprobHip.apply(hidden.to(cuda_device), weight.to(cuda_device), target.to(cuda_device), 0, V, chunk, None,
                                      True)
    assert got.shape == (B, S)
    torch.testing.assert_close(got.cpu().double(), want, rtol=1e-5, atol=1e-5)   # the reference's own tolerance


def test_entry_points_replay_from_a_hip_graph(cuda_device):
    """The C-ABI entry points neither allocate nor synchronise, so a forward + backward step can be captured into a HIP graph
    (workspaces and outputs come from the capturing allocator's pool).  Three replays, with eager work and synchronisations
    of the program's own between them and new values in the static inputs each time, must each reproduce the eager result
    bit for bit."""
    gen = torch.Generator().manual_seed(91)
    T, H, V = 300, 128, 1500
    weight = (torch.randn(V, H, generator=gen) * 3 / H ** 0.5).bfloat16().to(cuda_device)
    hidden = torch.zeros(T, H, dtype=torch.bfloat16, device=cuda_device)
    labels = torch.zeros(T, dtype=torch.int64, device=cuda_device)
    g = torch.zeros(T, device=cuda_device)
    q = torch.zeros(T, device=cuda_device)

    def step():
        lp, ent, lse, pz = ops.lmhead_fwd(hidden, weight, labels, 0.8, True)
        dh, dw = ops.lmhead_bwd(hidden, weight, labels, lse, pz, g, q, 0.8, 512)
        return lp, ent, dh, dw

    def refill(seed):
        gen_ = torch.Generator().manual_seed(seed)
        hidden.copy_(torch.randn(T, H, generator=gen_).bfloat16())
        labels.copy_(torch.randint(0, V, (T,), generator=gen_))
        g.copy_(torch.randn(T, generator=gen_))
        q.copy_(torch.randn(T, generator=gen_) * 0.01)

    refill(0)
    side = torch.cuda.Stream(device=cuda_device)
    side.wait_stream(torch.cuda.current_stream(cuda_device))
    with torch.cuda.stream(side):
        step()                                                   # warm-up outside the capture (library load, first launches)
    torch.cuda.current_stream(cuda_device).wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        captured = step()
    for seed in (1, 2, 3):
        refill(seed)
        graph.replay()
        torch.cuda.synchronize()
        got = [t.clone() for t in captured]
        want = step()                                            # eager, on the same inputs
        torch.cuda.synchronize()
        for a, b in zip(got, want):
            assert torch.equal(a, b)


def test_soft_ce_vocab_shards_reproduce_the_full_vocabulary(cuda_device):
    """The soft cross-entropy over a vocabulary-parallel group, on one GPU: forward per weight slice, three [T] vectors
    merged, backward per slice with the global log-sum-exps; the slices' gradient shares add up to the unsharded gradient."""
    from skyrl_amd.mtp_soft_ce import softce_bwd, softce_fwd
    from skyrl_amd.vocab_shards import merge_soft_ce_shard_statistics

    B, S, H, V = 2, 150, 128, 1000
    hs, ht, w = _softce_case(B, S, H, V, 71)
    T = B * S
    hs, ht, w = hs.reshape(T, H).to(cuda_device), ht.reshape(T, H).to(cuda_device), w.to(cuda_device)
    g = torch.randn(T, generator=torch.Generator().manual_seed(72)).to(cuda_device)
    full_loss, full_ls, full_lt = softce_fwd(hs, ht, w, S, 1, 1.0)
    full_d = softce_bwd(hs, ht, w, full_ls, full_lt, g, S, 1, 1.0, 0)

    bounds = [0, 256, 333, 1000]
    outs = [softce_fwd(hs, ht, w[lo:hi].contiguous(), S, 1, 1.0) for lo, hi in zip(bounds[:-1], bounds[1:])]
    loss, ls, lt = merge_soft_ce_shard_statistics(*(torch.stack([o[k] for o in outs]) for k in range(3)))
    torch.testing.assert_close(loss, full_loss, atol=5e-5, rtol=0)
    torch.testing.assert_close(ls, full_ls, atol=2e-5, rtol=0)
    torch.testing.assert_close(lt, full_lt, atol=2e-5, rtol=0)
    d_sum = torch.zeros(T, H, dtype=torch.float32, device=cuda_device)
    for lo, hi in zip(bounds[:-1], bounds[1:]):
        d_sum += softce_bwd(hs, ht, w[lo:hi].contiguous(), ls, lt, g, S, 1, 1.0, 0).float()
    assert cos(d_sum, full_d) >= 0.9999 and rel_l2(d_sum, full_d.float()) < 1e-2


def test_opcheck_registration_of_the_soft_ce_ops(cuda_device):
    import skyrl_amd.mtp_soft_ce  # noqa: F401  (registers the ops)

    T, H, V = 128, 64, 300
    hs, ht, w = _softce_case(1, T, H, V, 5)
    hs, ht, w = hs[0].to(cuda_device), ht[0].to(cuda_device), w.to(cuda_device)
    checks = ("test_schema", "test_faketensor")
    torch.library.opcheck(torch.ops.skyrl_amd.softce_fwd.default, (hs, ht, w, T, 1, 1.0), test_utils=checks)
    _, ls, lt = torch.ops.skyrl_amd.softce_fwd(hs, ht, w, T, 1, 1.0)
    g = torch.ones(T, device=cuda_device)
    torch.library.opcheck(torch.ops.skyrl_amd.softce_bwd.default, (hs, ht, w, ls, lt, g, T, 1, 1.0, 0), test_utils=checks)


@pytest.mark.parametrize("packed", [False, True])
@pytest.mark.parametrize("compute_entropy", [False, True])
def test_fsdp_tail_action_window_only(cuda_device, packed, compute_entropy):
    """action_only=True scores only the rows the action window reads: the same action log-probabilities and in-window entropy
    as the full pass (each token's row is computed independently of the others), zeros outside, and the same gradients."""
    from skyrl_amd.model_wrapper import action_log_probs_from_hidden
    dev = cuda_device
    gen = torch.Generator().manual_seed(62)
    B, S, H, V, A, t = 4, 40, 128, 900, 11, 0.9
    seqs = torch.randint(0, V, (B, S), generator=gen).to(dev)
    am = torch.ones(B, S, dtype=torch.long)
    am[0, :9] = 0                                                # left padding
    am[2, -4:] = 0                                               # right padding inside the action window
    am = am.to(dev)
    weight = (torch.randn(V, H, generator=gen) * 3 / H ** 0.5).to(torch.bfloat16).to(dev)
    nnz = am.flatten().nonzero().flatten() if packed else None
    n_tok = int(am.sum()) if packed else B * S
    hidden = torch.randn(1 if packed else B, n_tok if packed else S, H, generator=gen).to(torch.bfloat16).to(dev)
    G = torch.randn(B, A, generator=gen).to(dev)
    Q = (torch.randn(B, S, generator=gen) * 0.1).to(dev)

    results = []
    for action_only in (False, True):
        hd, wd = hidden.clone().requires_grad_(True), weight.clone().requires_grad_(True)
        alp, out = action_log_probs_from_hidden(hd, wd, seqs, A, am, t, return_output=True, compute_entropy=compute_entropy,
                                                entropy_requires_grad=True, nnz_indices=nnz, action_only=action_only)
        loss = (alp * G).sum()
        if compute_entropy:
            loss = loss + (out["entropy"][:, -A - 1:-1] * Q[:, -A - 1:-1]).sum()
        loss.backward()
        results.append((alp.detach(), out.get("entropy"), hd.grad, wd.grad))
    (alp0, ent0, dh0, dw0), (alp1, ent1, dh1, dw1) = results
    torch.testing.assert_close(alp1, alp0, rtol=0, atol=1e-6)
    if packed:
        assert bool((alp1[2, -3:] == 0).all())                   # window positions that hold padding
    if compute_entropy:
        assert ent1.shape == (B, S)
        torch.testing.assert_close(ent1.detach()[:, -A - 1:-1], ent0.detach()[:, -A - 1:-1], rtol=0, atol=1e-6)
        outside = torch.ones(S, dtype=torch.bool, device=dev)
        outside[-A - 1:-1] = False
        assert bool((ent1.detach()[:, outside] == 0).all())
    assert cos(dh1, dh0) >= 0.9999 and cos(dw1, dw0) >= 0.9999
    assert bool((dh1.reshape(-1, H).float().abs().sum(-1) > 0).sum() <= B * A)   # only window rows receive a gradient


def test_frozen_lm_head_skips_the_weight_gradient(cuda_device):
    """A weight that takes no gradient (adapter training with a frozen LM head): the backward computes dHidden alone -- the
    same dHidden bit for bit (the dHidden tiles do not depend on what else the launch carries) -- through the C ABI with
    d_weight = NULL, the functional op and both autograd adapters."""
    T, H, V, t = 300, 128, 1000, 0.7
    hidden, weight, labels, g, q = _rand(T, H, V, seed=41)
    h, w, y, gd, qd = (x.to(cuda_device) for x in (hidden, weight, labels, g, q))
    lp, ent, lse, pz = ops.lmhead_fwd(h, w, y, 1.0 / t, True)
    for chunk in (0, 256):
        dh_full, _ = ops.lmhead_bwd(h, w, y, lse, pz, gd, qd, 1.0 / t, chunk)
        assert torch.equal(ops.lmhead_bwd_hidden(h, w, y, lse, pz, gd, qd, 1.0 / t, chunk), dh_full)
    # autograd: the verl-style function and the SkyRL adapter
    for frozen in (False, True):
        hd = h.clone().requires_grad_(True)
        wd = w.clone().requires_grad_(not frozen)
        out_lp, out_ent = linear_cross_entropy(hd, wd, y, t, "none", None)
        ((out_lp * gd).sum() + (out_ent * qd).sum()).backward()
        if frozen:
            assert wd.grad is None and torch.equal(hd.grad, kept)
        else:
            kept = hd.grad.clone()
            assert wd.grad is not None
    hd = h.clone().requires_grad_(True)
    out = FusedLinearLogprobHip.apply(hd[None], w, y[None], 0, V, 1024, None, False)
    (out[0] * gd).sum().backward()
    assert hd.grad is not None and w.grad is None
    # the kernel profile of a frozen-head backward has no hidden transposition and GEMM launches of dHidden tiles only
    lib = _lib.load()
    handle = lib.skyrl_lmhead_profile_begin()
    ops.lmhead_bwd_hidden(h, w, y, lse, pz, gd, qd, 1.0 / t, 0)
    import ctypes
    n = lib.skyrl_lmhead_num_kernel_kinds()
    ms, cnt = (ctypes.c_double * n)(), (ctypes.c_int64 * n)()
    assert lib.skyrl_lmhead_profile_end(handle, ms, cnt) == 0
    names = [lib.skyrl_lmhead_kernel_name(k).decode() for k in range(n)]
    assert cnt[names.index("transpose_bf16")] == 1               # weight^T only (V = 1000 is not a multiple of 64)


def test_entry_points_are_reentrant_across_threads_and_streams(cuda_device):
    """Two host threads, each with its own stream, inputs and workspaces, run forward + backward steps at the same time; every
    result equals the one a single thread gets (the library keeps no state between calls apart from the per-thread profile)."""
    import threading

    T, H, V = 500, 128, 3000
    cases = []
    for seed in (101, 102):
        hidden, weight, labels, g, q = _rand(T, H, V, seed=seed)
        cases.append([x.to(cuda_device) for x in (hidden, weight, labels, g, q)])

    def run(case):
        h, w, y, g, q = case
        lp, ent, lse, pz = ops.lmhead_fwd(h, w, y, 0.9, True)
        dh, dw = ops.lmhead_bwd(h, w, y, lse, pz, g, q, 0.9, 1024)
        return lp, ent, dh, dw

    want = [run(c) for c in cases]
    torch.cuda.synchronize()
    got = [[], []]
    errors = []

    def worker(k):
        try:
            stream = torch.cuda.Stream(device=cuda_device)
            with torch.cuda.stream(stream):
                for _ in range(8):
                    got[k].append(run(cases[k]))
            stream.synchronize()
        except Exception as e:  # surfaced in the main thread below
            errors.append(e)

    threads = [threading.Thread(target=worker, args=(k,)) for k in range(2)]
    for th in threads:
        th.start()
    for th in threads:
        th.join(timeout=100)
    assert not errors, errors
    assert not any(th.is_alive() for th in threads)
    torch.cuda.synchronize()
    for k in range(2):
        assert len(got[k]) == 8
        for outs in got[k]:
            for a, b in zip(outs, want[k]):
                assert torch.equal(a, b)


def test_soft_ce_extreme_logits(cuda_device):
    """Logits of the order of +-150 (a near one-hot teacher, a confident and often wrong student): losses of tens to hundreds
    of nats without overflow, against fp64; the tolerance scales with the loss, as the fp32 accumulation error does."""
    from skyrl_amd.mtp_soft_ce import soft_ce_from_hidden

    B, S, H, V = 2, 130, 128, 1500
    hs, ht, w = _softce_case(B, S, H, V, 81, spread=45.0)
    hs64 = hs.double().requires_grad_(True)
    ref = O.soft_ce_per_token(hs64 @ w.double().t(), torch.roll(ht.double() @ w.double().t(), -1, dims=1))
    ref.sum().backward()
    assert ref.max().item() > 100.0
    d_hs = hs.to(cuda_device).requires_grad_(True)
    got = soft_ce_from_hidden(d_hs, ht.to(cuda_device), w.to(cuda_device), shift=1)
    got.sum().backward()
    assert bool(torch.isfinite(got).all()) and bool(torch.isfinite(d_hs.grad.float()).all())
    err = (got.detach().cpu().double() - ref.detach()).abs()
    assert bool((err <= 1e-4 * ref.detach().abs() + 1e-3).all()), err.max().item()
    assert cos(d_hs.grad.float(), hs64.grad) >= GRAD_COS


def test_weight_gradient_in_bf16_equals_the_rounded_fp32_one(cuda_device):
    """SKYRL_DW_BF16: the GEMM epilogue rounds the fp32 sums to bf16 itself; bit-identical to casting the fp32 result, for one
    and for several vocabulary chunks, through the functional op and the autograd adapter (which now never holds an fp32
    [V, H] buffer)."""
    T, H, V, t = 300, 128, 1000, 0.7
    hidden, weight, labels, g, q = _rand(T, H, V, seed=43)
    h, w, y, gd, qd = (x.to(cuda_device) for x in (hidden, weight, labels, g, q))
    lp, ent, lse, pz = ops.lmhead_fwd(h, w, y, 1.0 / t, True)
    for chunk in (0, 256):
        dh32, dw32 = ops.lmhead_bwd(h, w, y, lse, pz, gd, qd, 1.0 / t, chunk)
        dh16, dw16 = ops.lmhead_bwd_bf16(h, w, y, lse, pz, gd, qd, 1.0 / t, chunk)
        assert dw16.dtype == torch.bfloat16 and torch.equal(dw16, dw32.to(torch.bfloat16)) and torch.equal(dh16, dh32)
    hd, wd = h.clone().requires_grad_(True), w.clone().requires_grad_(True)
    out_lp, out_ent = linear_cross_entropy(hd, wd, y, t, "none", None)
    ((out_lp * gd).sum() + (out_ent * qd).sum()).backward()
    assert wd.grad.dtype == torch.bfloat16 and torch.equal(wd.grad, dw32.to(torch.bfloat16))
    lib = _lib.load()
    p = h.data_ptr()
    ws = torch.empty(lib.skyrl_lmhead_bwd_workspace_bytes(T, H, V, 0), dtype=torch.uint8, device=cuda_device)
    assert lib.skyrl_lmhead_bwd(p, H, w.data_ptr(), H, y.data_ptr(), lse.data_ptr(), None, gd.data_ptr(), None, T, H, V, 1.0,
                                dh32.data_ptr(), dw32.data_ptr(), 3, 0, ws.data_ptr(), ws.numel(), None) == -5


@pytest.mark.parametrize("temperature", [0.25, 0.1])
def test_entropy_of_nearly_deterministic_rows(temperature, cuda_device):
    """Low temperatures make most rows nearly deterministic: entropies of 1e-6 .. 1e-2 nats next to log-sum-exps of 50 and more.
    lse - sum p z would lose them to cancellation in fp32 (an absolute error of 1e-5); the statistic kept relative to the
    maximum does not: every entropy above 1e-5 nats is right to 1e-2 relative (the stated tolerance), smaller ones to 1e-7
    absolute; the log-probabilities and both gradients are unaffected."""
    T, H, V = 600, 256, 3000
    hidden, weight, labels, g, q = _rand(T, H, V, seed=77)
    out = run_hip(cuda_device, hidden, weight, labels, temperature, g, q, True, 1024)
    ex = O.exact_fwd_bwd(hidden, weight, labels, temperature, g, q)
    ref_ent = ex["entropy"].double()
    assert float((ref_ent < 1e-2).float().mean()) > 0.05 and float(ref_ent.min()) < 1e-3     # the case is what it says
    err = (out["entropy"].double() - ref_ent).abs()
    assert float((err / ref_ent.clamp_min(1e-5)).max()) <= 1e-2, float((err / ref_ent.clamp_min(1e-5)).max())
    assert float(err[ref_ent < 1e-5].max() if bool((ref_ent < 1e-5).any()) else 0.0) <= 1e-7
    assert bool((out["entropy"] >= -1e-7).all())
    # sum p z, which the backward takes back, is still lse - entropy
    assert torch.allclose(out["pz"].double(), (ex["logprobs"].double() * 0 + out["lse"].double() - out["entropy"].double()), atol=1e-5)
    assert (out["logprobs"].double() - ex["logprobs"].double()).abs().max().item() <= 1e-3
    check_grads(out["d_hidden"], out["d_weight"], ex, f"t={temperature}")
