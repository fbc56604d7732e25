"""GPU parity of the fused off-policy correction (skyrl_off_policy_correction, skyrl_amd/off_policy_correction.py) against the
oracle's restatement of off_policy_correction_utils.py:24-391, and of the policy losses that end with it (ppo_utils.py:581,
653, 722, 815, 857, 929) against the oracle's loss followed by the oracle's correction.

Masks and counts are compared exactly (ratios within 1e-4 of a threshold are moved away first, so that fp32 and fp64 decide
alike); weights and metrics to fp32 accuracy.
"""

from __future__ import annotations

import itertools
from types import SimpleNamespace

import pytest
import torch

from oracle import lmhead_oracle as O
from skyrl_amd import off_policy_correction as OPC
from skyrl_amd import policy_loss as PL

pytestmark = pytest.mark.gpu

ERR_NULL, ERR_SHAPE, ERR_ARG = -1, -2, -5   # include/skyrl_lmhead.h
THRESHOLDS = (0.5, 0.7, 0.9, 1.1, 1.5, 2.0, 3.0)


def _cfg(**kw):
    base = dict(tis_ratio_type=None, token_tis_ratio_clip_high=2.0, sequence_tis_ratio_clip_high=3.0, sequence_mask_metric=None,
                geo_mask_high=1.1, geo_mask_low=0.9, product_mask_high=3.0, product_mask_low=0.5,
                outlier_token_is_threshold_low=None, outlier_token_is_threshold_high=None,
                token_mask_is_threshold_low=None, token_mask_is_threshold_high=None)
    base.update(kw)
    return SimpleNamespace(**base)


def _batch(B=9, S=57, seed=5, spread=0.25):
    gen = torch.Generator().manual_seed(seed)
    rollout = torch.randn(B, S, generator=gen) * 0.7 - 1.5
    delta = torch.randn(B, S, generator=gen) * spread
    delta[1] *= 0.05                                            # a row that stays inside every bound
    delta[2, 3] = 1.4                                           # one outlier token in an otherwise quiet row
    delta[2, :3] *= 0.05
    delta[2, 4:] *= 0.05
    delta[3, 0], delta[3, 1] = 30.0, -30.0                      # beyond the +-20 clamp
    mask = (torch.rand(B, S, generator=gen) > 0.3).float()
    mask[4] = 0                                                 # a row without loss tokens
    mask[5, :6] = 0.5                                           # fractional weights
    mask[3, :2] = 1
    # keep every token ratio, every row product and every geometric mean at least 1e-4 (relative) away from every threshold
    ratio = delta.double().clamp(-20, 20).exp()
    for th in THRESHOLDS:
        near = (ratio / th - 1).abs() < 1e-4
        delta = torch.where(near, delta + 3e-4, delta)
    return rollout + delta, rollout, mask


CASES = {
    "tis_token": dict(tis_ratio_type="token", token_tis_ratio_clip_high=1.5),
    "tis_sequence": dict(tis_ratio_type="sequence", sequence_tis_ratio_clip_high=2.0),
    "outlier_high": dict(outlier_token_is_threshold_high=3.0),
    "outlier_both": dict(outlier_token_is_threshold_low=0.5, outlier_token_is_threshold_high=2.0),
    "token_mask": dict(token_mask_is_threshold_low=0.7, token_mask_is_threshold_high=1.5),
    "geometric": dict(sequence_mask_metric="geometric", geo_mask_low=0.9, geo_mask_high=1.1),
    "product": dict(sequence_mask_metric="product", product_mask_low=0.5, product_mask_high=3.0),
    "everything_token": dict(tis_ratio_type="token", token_tis_ratio_clip_high=1.5, outlier_token_is_threshold_high=3.0,
                             token_mask_is_threshold_low=0.7, token_mask_is_threshold_high=1.5,
                             sequence_mask_metric="geometric", geo_mask_low=0.9, geo_mask_high=1.1),
    "everything_sequence": dict(tis_ratio_type="sequence", sequence_tis_ratio_clip_high=2.0, outlier_token_is_threshold_low=0.5,
                                token_mask_is_threshold_low=0.7, token_mask_is_threshold_high=1.5,
                                sequence_mask_metric="product", product_mask_low=0.5, product_mask_high=3.0),
}


def _rows_are_decided_alike(old, rollout, mask, cfg):
    """Row products / geometric means (after the first two steps, in fp64) stay clear of the row thresholds."""
    c = _cfg(**{k: v for k, v in vars(cfg).items() if k.startswith(("outlier", "token_mask"))})
    m2 = O.off_policy_correction(old.double(), rollout.double(), mask.double(), c)[2] if (
        c.outlier_token_is_threshold_low is not None or c.outlier_token_is_threshold_high is not None
        or (c.token_mask_is_threshold_low is not None and c.token_mask_is_threshold_high is not None)) else mask.double()
    total = ((old.double() - rollout.double()) * m2).sum(-1)
    values = torch.cat([total.clamp(-20, 20).exp(), (total / m2.sum(-1).clamp(min=1)).clamp(-20, 20).exp()])
    return all(bool(((values / th - 1).abs() > 1e-4).all()) for th in THRESHOLDS)


@pytest.mark.parametrize("case", list(CASES))
def test_compute_off_policy_correction_matches_oracle(case, cuda_device):
    cfg = _cfg(**CASES[case])
    old, rollout, mask = _batch()
    assert _rows_are_decided_alike(old, rollout, mask, cfg)
    want_tis, want_metrics, want_mask = O.off_policy_correction(old.double(), rollout.double(), mask.double(), cfg)
    tis, metrics, new_mask = OPC.compute_off_policy_correction(old.to(cuda_device), rollout.to(cuda_device), mask.to(cuda_device), cfg)
    assert torch.equal(new_mask.cpu().double(), want_mask)
    if want_tis is None:
        assert tis is None
    else:
        assert tis.shape == want_tis.shape and torch.allclose(tis.cpu().double(), want_tis, rtol=2e-5)
    assert sorted(metrics) == sorted(want_metrics)
    for key, value in want_metrics.items():
        assert isinstance(metrics[key], float) and metrics[key] == pytest.approx(value, rel=2e-5, abs=1e-7), key
    if case.startswith("everything"):                           # every step did something
        assert 0 < want_metrics["token_mask_ratio"] < 1 and 0 < float((want_mask.sum(-1) == 0).float().mean()) < 1
    # without a host synchronisation the metrics are 0-dim tensors of the same values
    _, lazy, _ = OPC.compute_off_policy_correction(old.to(cuda_device), rollout.to(cuda_device), mask.to(cuda_device), cfg, sync_metrics=False)
    assert all(isinstance(v, torch.Tensor) and v.dim() == 0 and v.item() == metrics[k] for k, v in lazy.items())
    # the wrapper on a per-token loss
    loss = torch.randn(old.shape, generator=torch.Generator().manual_seed(1))
    want_loss, want_mask2, _ = O.apply_off_policy_correction(loss.double(), old.double(), rollout.double(), mask.double(), cfg)
    got_loss, got_mask2, _ = OPC.apply_off_policy_correction(loss.to(cuda_device), old.to(cuda_device), rollout.to(cuda_device),
                                                            mask.to(cuda_device), cfg)
    assert torch.allclose(got_loss.cpu().double(), want_loss, rtol=2e-5, atol=1e-7) and torch.equal(got_mask2.cpu().double(), want_mask2)


def test_off_policy_correction_switches_and_errors(cuda_device):
    old, rollout, mask = (t.to(cuda_device) for t in _batch())
    assert not OPC.off_policy_correction_enabled(_cfg())
    assert not OPC.off_policy_correction_enabled(_cfg(token_mask_is_threshold_low=0.5))          # one bound alone is off
    assert OPC.off_policy_correction_enabled(_cfg(outlier_token_is_threshold_low=0.5))
    tis, metrics, same = OPC.compute_off_policy_correction(old, rollout, mask, _cfg())
    assert tis is None and metrics == {} and same is mask
    loss, same, metrics = OPC.apply_off_policy_correction(old, old, None, mask, _cfg(tis_ratio_type="token"))
    assert loss is old and same is mask and metrics == {}
    with pytest.raises(ValueError):
        OPC.compute_off_policy_correction(old, rollout, mask, _cfg(tis_ratio_type="rows"))
    with pytest.raises(ValueError):
        OPC.compute_off_policy_correction(old, rollout, mask, _cfg(sequence_mask_metric="median"))
    with pytest.raises(RuntimeError):
        OPC.compute_off_policy_correction(old.cpu(), rollout.cpu(), mask.cpu(), _cfg(tis_ratio_type="token"))
    # no mask at all: every token counts
    tis, metrics, new_mask = OPC.compute_off_policy_correction(old, rollout, None, _cfg(tis_ratio_type="token", token_mask_is_threshold_low=0.7,
                                                                                     token_mask_is_threshold_high=1.5))
    want = O.off_policy_correction(old.cpu().double(), rollout.cpu().double(), torch.ones(old.shape, dtype=torch.float64),
                                   _cfg(tis_ratio_type="token", token_mask_is_threshold_low=0.7, token_mask_is_threshold_high=1.5))
    assert torch.equal(new_mask.cpu().double(), want[2]) and metrics["token_mask_ratio"] == pytest.approx(want[1]["token_mask_ratio"])
    torch.library.opcheck(OPC.off_policy_correction_terms, (old, rollout, mask, 1, 1.5, 2, 0.5, 3.0, None, 2.0, 0.7, 1.5),
                          test_utils=("test_schema", "test_faketensor"))


def _loss_config(kind, correction):
    return SimpleNamespace(policy_loss_type={"dppo_tv": "dppo"}.get(kind, kind), eps_clip_low=0.2, eps_clip_high=0.25, clip_ratio_c=3.0,
                           loss_reduction="sequence_mean", sapo=SimpleNamespace(tau_pos=1.0, tau_neg=1.05),
                           cispo=SimpleNamespace(cispo_eps_clip_low=0.3, cispo_eps_clip_high=0.5, cispo_anchor="old"),
                           dppo=SimpleNamespace(dppo_type="binary_tv", delta_low=0.06, delta_high=0.05),
                           off_policy_correction=correction)


@pytest.mark.parametrize("kind", ["regular", "dual_clip", "sapo", "gspo", "cispo", "dppo_tv"])
@pytest.mark.parametrize("case", ["everything_token", "everything_sequence"])
def test_policy_losses_end_with_the_correction(kind, case, cuda_device):
    """loss = sum(per-token loss * tis * new mask) and the clip statistic over the ORIGINAL mask, as in the reference; value,
    metrics of both parts, and the gradient -- which vanishes exactly on the tokens the correction removed."""
    correction = _cfg(**CASES[case])
    old, rollout, mask = _batch(seed=11)
    assert _rows_are_decided_alike(old, rollout, mask, correction)
    gen = torch.Generator().manual_seed(3)
    lp = (old + torch.randn(old.shape, generator=gen) * 0.3).clamp(max=-0.02)
    adv = torch.randn(old.shape, generator=gen)
    cfg = _loss_config(kind, correction)
    plain = _loss_config(kind, _cfg())
    x = lp.double().requires_grad_(True)
    tis, want_extra, new_mask = O.off_policy_correction(old.double(), rollout.double(), mask.double(), correction)
    factor = new_mask / mask.double().clamp(min=1e-30) * (1.0 if tis is None else tis)        # tis * keep on the original mask
    factor = torch.where(mask.double() > 0, factor, torch.zeros_like(factor))
    if kind in ("regular", "dual_clip"):
        per_token = lambda m: O.ppo_policy_loss(x, old.double(), adv.double(), 0.2, 0.25, 3.0, kind == "dual_clip", m)  # noqa: E731
    elif kind == "gspo":
        row = O.masked_mean(x - old.double(), mask.double(), dim=-1).unsqueeze(-1)
        r = torch.clamp(x - x.detach() + row.detach(), max=10).exp()
        a64 = adv.double()
        ref_loss = (-torch.min(r * a64, r.clamp(0.8, 1.25) * a64) * factor * mask.double()).sum()
        ref_clip = O.gspo_policy_loss(x, old.double(), adv.double(), 0.2, 0.25, mask.double())[1]
        per_token = None
    elif kind == "dppo_tv":
        per_token = lambda m: O.dppo_policy_loss(x, rollout.double(), adv.double(), "binary_tv", 0.06, 0.05, m)  # noqa: E731
    else:
        fn = {"sapo": O.sapo_policy_loss, "cispo": O.cispo_policy_loss}[kind]
        lo, hi = (1.0, 1.05) if kind == "sapo" else (0.3, 0.5)
        per_token = lambda m: fn(x, old.double(), adv.double(), lo, hi, m)  # noqa: E731
    if per_token is not None:
        ref_loss, ref_clip = per_token(mask.double() * factor)[0], per_token(mask.double())[1]
    ref_loss.backward()
    fn = {"regular": PL.ppo_policy_loss, "dual_clip": PL.ppo_policy_loss, "sapo": PL.sapo_policy_loss, "gspo": PL.gspo_policy_loss,
          "cispo": PL.compute_policy_loss_cispo, "dppo_tv": PL.dppo_policy_loss}[kind]
    to = lambda t: t.to(cuda_device)  # noqa: E731
    d = to(lp).requires_grad_(True)
    loss, metrics = fn(d, to(old), to(adv), cfg, to(mask), to(rollout))
    loss.backward()
    scale = max(abs(ref_loss.item()), float(x.grad.abs().max()), 1e2)
    assert abs(loss.item() - ref_loss.item()) <= 2e-5 * scale, (loss.item(), ref_loss.item())
    if kind != "sapo":
        assert metrics["clip_ratio"] == pytest.approx(float(ref_clip), abs=1e-6)
    for key, value in want_extra.items():
        assert metrics[key] == pytest.approx(value, rel=2e-5, abs=1e-7), key
    err = (d.grad.double().cpu() - x.grad).abs().max().item()
    assert err <= 2e-5 * max(1.0, x.grad.abs().max().item()), err
    removed = (new_mask == 0) & (mask > 0)
    assert bool(removed.any()) and bool((d.grad.cpu()[removed] == 0).all())
    # without rollout log-probabilities, or with nothing switched on, the loss is the uncorrected one
    a, _ = fn(to(lp), to(old), to(adv), cfg, to(mask), None) if kind != "dppo_tv" else fn(to(lp), to(rollout), to(adv), plain, to(mask), None)
    b, _ = fn(to(lp), to(old), to(adv), plain, to(mask), to(rollout)) if kind != "dppo_tv" else fn(to(lp), to(rollout), to(adv), plain, to(mask), to(rollout))
    assert a.item() == pytest.approx(b.item(), rel=1e-6) or kind == "dppo_tv"
    assert abs(a.item() - loss.item()) > 1e-3


def test_actor_loss_ends_with_the_correction(cuda_device):
    correction = _cfg(**CASES["everything_token"])
    old, rollout, mask = _batch(seed=11)
    gen = torch.Generator().manual_seed(3)
    lp = (old + torch.randn(old.shape, generator=gen) * 0.3).clamp(max=-0.02)
    adv = torch.randn(old.shape, generator=gen)
    cfg = _loss_config("regular", correction)
    cfg.use_kl_loss, cfg.use_entropy_loss = False, False
    to = lambda t: t.to(cuda_device)  # noqa: E731
    d1, d2 = to(lp).requires_grad_(True), to(lp).requires_grad_(True)
    want, want_metrics = PL.ppo_policy_loss(d1, to(old), to(adv), cfg, to(mask), to(rollout))
    got, metrics = PL.actor_loss(d2, to(old), to(adv), cfg, to(mask), rollout_logprobs=to(rollout))
    want.backward()
    got.backward()
    assert got.item() == pytest.approx(want.item(), rel=1e-6) and torch.allclose(d1.grad, d2.grad, rtol=1e-6, atol=1e-9)
    assert metrics["clip_ratio"].item() == pytest.approx(want_metrics["clip_ratio"], abs=1e-7)
    assert metrics["token_mask_ratio"].item() == pytest.approx(want_metrics["token_mask_ratio"])
    # the supervised losses are never corrected (ppo_utils.py:1056-1142)
    cfg.policy_loss_type = "cross_entropy"
    a, m = PL.actor_loss(to(lp), to(old), to(adv), cfg, to(mask), rollout_logprobs=to(rollout))
    assert "token_mask_ratio" not in m and a.item() == pytest.approx(float(-(lp * mask).sum()), rel=1e-5)


@pytest.mark.filterwarnings("ignore:std\\(\\)")   # one element: Tensor.std() is NaN and says so
@pytest.mark.parametrize("rows,cols", [(1, 1), (1, 7), (3, 1), (2, 255), (5, 256), (4, 257), (1, 5000), (33, 1023), (7, 2049)])
def test_off_policy_correction_row_shapes(rows, cols, cuda_device):
    """Rows shorter than, equal to and longer than a workgroup's sweep, with every step on; every row is its own case."""
    gen = torch.Generator().manual_seed(rows * 10007 + cols)
    rollout = torch.randn(rows, cols, generator=gen) * 0.5 - 1.0
    delta = torch.randn(rows, cols, generator=gen) * (0.3 / max(1.0, cols ** 0.5))        # row sums of order 0.3
    delta[0, 0] += 0.8
    mask = (torch.rand(rows, cols, generator=gen) > 0.25).float()
    mask[0, 0] = 1
    ratio = delta.double().exp()
    for th in THRESHOLDS:
        delta = torch.where((ratio / th - 1).abs() < 1e-4, delta + 3e-4, delta)
    for name in ("everything_token", "everything_sequence"):
        cfg = _cfg(**CASES[name])
        old = rollout + delta
        if not _rows_are_decided_alike(old, rollout, mask, cfg):
            old = rollout + delta * 1.01
            assert _rows_are_decided_alike(old, rollout, mask, cfg)
        want_tis, want_metrics, want_mask = O.off_policy_correction(old.double(), rollout.double(), mask.double(), cfg)
        tis, metrics, new_mask = OPC.compute_off_policy_correction(old.to(cuda_device), rollout.to(cuda_device), mask.to(cuda_device), cfg)
        assert torch.equal(new_mask.cpu().double(), want_mask), name
        assert torch.allclose(tis.cpu().double(), want_tis, rtol=2e-5), name
        for key, value in want_metrics.items():
            assert metrics[key] == pytest.approx(value, rel=5e-5, abs=1e-6, nan_ok=True), (name, key)


def test_off_policy_correction_leading_dimensions_and_dtypes(cuda_device):
    """[B, G, S] inputs are rows of S; bf16 / fp64 inputs are read as fp32 and the weight comes back in the inputs' dtype."""
    old, rollout, mask = _batch(B=12, S=40, seed=21)
    cfg = _cfg(**CASES["everything_token"])
    flat = OPC.compute_off_policy_correction(old.to(cuda_device), rollout.to(cuda_device), mask.to(cuda_device), cfg)
    cube = OPC.compute_off_policy_correction(*(t.reshape(3, 4, 40).to(cuda_device) for t in (old, rollout, mask)), cfg)
    assert cube[0].shape == (3, 4, 40) and torch.equal(cube[0].reshape(12, 40), flat[0]) and torch.equal(cube[2].reshape(12, 40), flat[2])
    assert cube[1] == flat[1]
    seq = OPC.compute_off_policy_correction(*(t.reshape(3, 4, 40).to(cuda_device) for t in (old, rollout, mask)), _cfg(**CASES["tis_sequence"]))
    assert seq[0].shape == (3, 4, 1)
    wide = OPC.compute_off_policy_correction(old.double().to(cuda_device), rollout.double().to(cuda_device), mask.double().to(cuda_device), cfg)
    assert wide[0].dtype == torch.float64 and wide[2].dtype == torch.float64 and torch.equal(wide[2].float(), flat[2])
    # a non-contiguous view gives what its contiguous copy gives
    view = OPC.compute_off_policy_correction(old.to(cuda_device).t().contiguous().t(), rollout.to(cuda_device), mask.to(cuda_device), cfg)
    assert torch.equal(view[0], flat[0]) and view[1] == flat[1]


def test_off_policy_c_abi_argument_errors(cuda_device):
    import ctypes

    from skyrl_amd import _lib
    lib = _lib.load()
    rows, cols = 4, 16
    old = torch.zeros(rows, cols, device=cuda_device)
    out = torch.empty(rows, cols, device=cuda_device)
    metrics = torch.empty(16, device=cuda_device)
    stats = torch.empty(rows * 20, device=cuda_device)
    f = lambda v: ctypes.byref(ctypes.c_float(v))  # noqa: E731

    def call(old_p=old.data_ptr(), roll_p=old.data_ptr(), r=rows, c=cols, tis=1, cap=2.0, seq=0, lo=0.0, hi=0.0, ol=None, oh=None,
             tl=None, th=None, metrics_p=metrics.data_ptr(), stats_p=stats.data_ptr()):
        return lib.skyrl_off_policy_correction(old_p, roll_p, None, r, c, tis, cap, seq, lo, hi, ol, oh, tl, th, out.data_ptr(), None, None,
                                               metrics_p, stats_p, torch.cuda.current_stream(cuda_device).cuda_stream)

    assert call() == 0                                           # optional outputs may be left out
    torch.cuda.synchronize()
    assert bool((out == 1).all()) and metrics[0].item() == 1.0   # equal log-probabilities: ratio 1, nothing removed
    assert call(old_p=None) == ERR_NULL and call(roll_p=None) == ERR_NULL
    assert call(metrics_p=None) == ERR_NULL and call(stats_p=None) == ERR_NULL
    assert call(r=0) == ERR_SHAPE and call(c=0) == ERR_SHAPE
    assert call(r=1 << 31) == ERR_SHAPE
    assert call(tis=3) == ERR_ARG and call(seq=-1) == ERR_ARG
    assert call(cap=float("nan")) == ERR_ARG and call(seq=1, lo=float("inf")) == ERR_ARG
    assert call(oh=f(float("nan"))) == ERR_ARG and call(tl=f(float("inf")), th=f(1.0)) == ERR_ARG
    assert call(tis=0, cap=float("nan")) == 0                    # a cap that nothing reads is not checked
    torch.cuda.synchronize()


def test_off_policy_correction_full_size_properties(cuda_device):
    """4.2 M tokens (1024 rows of 4096): what must hold whatever the data -- keep is 0 or 1 and constant 0 on a removed row,
    weight = tis * keep, the token weight is min(ratio, cap) bit for bit, the metrics agree with torch reductions of the
    outputs, a second call returns the same bits, and applying the thinned mask again removes nothing more."""
    rows, cols = 1024, 4096
    gen = torch.Generator(device=cuda_device).manual_seed(77)
    rollout = torch.randn(rows, cols, device=cuda_device, generator=gen) * 0.7 - 1.5
    old = rollout + torch.randn(rows, cols, device=cuda_device, generator=gen) * 0.02
    old[::7, 5] += 1.0                                           # outlier tokens in every seventh row
    mask = (torch.rand(rows, cols, device=cuda_device, generator=gen) > 0.4).float()
    mask[::7, 5] = 1
    cfg = _cfg(tis_ratio_type="token", token_tis_ratio_clip_high=1.02, outlier_token_is_threshold_high=2.0,
               token_mask_is_threshold_low=0.97, token_mask_is_threshold_high=1.03)
    keep, tis, weight, m = OPC.off_policy_correction_terms(old, rollout, mask, 1, 1.02, 0, 0.0, 0.0, None, 2.0, 0.97, 1.03)
    assert bool(((keep == 0) | (keep == 1)).all()) and torch.equal(weight, tis * keep)
    ratio = (old - rollout).clamp(-20, 20).exp()
    assert torch.allclose(tis, ratio.clamp(max=1.02), rtol=2e-6)
    assert bool((keep[::7] == 0).all())                          # rows with an outlier token are removed whole
    other = torch.ones(rows, dtype=torch.bool, device=cuda_device)
    other[::7] = False
    inside = ((ratio >= 0.97) & (ratio <= 1.03)).float()
    clear = ((ratio / 0.97 - 1).abs() > 1e-5) & ((ratio / 1.03 - 1).abs() > 1e-5) & (mask > 0)   # two exp() may differ in the last bit
    assert torch.equal(keep[other][clear[other]], inside[other][clear[other]])
    assert bool((keep[other][mask[other] == 0] == 1).all())     # tokens outside the mask are not judged
    metrics = OPC.compute_off_policy_correction(old, rollout, mask, cfg)[1]
    assert metrics["outlier_seq_masked_ratio"] == pytest.approx(len(range(0, rows, 7)) / rows)
    assert metrics["is_ratio_max"] == pytest.approx(float((ratio * mask).max()), rel=1e-5)
    assert metrics["is_ratio_mean"] == pytest.approx(float((ratio.double() * mask).sum() / mask.sum()), rel=1e-5)
    kept_rows = mask[other].double()
    assert metrics["token_mask_ratio"] == pytest.approx(float(((1 - inside[other].double()) * kept_rows).sum() / kept_rows.sum().clamp(min=1)), rel=1e-4)
    again = OPC.off_policy_correction_terms(old, rollout, mask, 1, 1.02, 0, 0.0, 0.0, None, 2.0, 0.97, 1.03)
    assert all(torch.equal(a, b) for a, b in zip((keep, tis, weight, m), again))
    twice = OPC.off_policy_correction_terms(old, rollout, mask * keep, 1, 1.02, 0, 0.0, 0.0, None, 2.0, 0.97, 1.03)
    assert torch.equal(twice[0] * mask * keep, mask * keep)


def test_off_policy_correction_replays_from_a_hip_graph(cuda_device):
    """The two launches hold no memset and no allocation of the library's own: captured once, replayed on new data with eager
    work and synchronisations in between, every replay equals the eager result bit for bit."""
    old0, rollout0, mask0 = (t.to(cuda_device) for t in _batch(B=16, S=300, seed=31))
    args = (1, 1.5, 1, 0.9, 1.1, None, 3.0, 0.7, 1.5)
    old, rollout, mask = old0.clone(), rollout0.clone(), mask0.clone()
    side = torch.cuda.Stream(device=cuda_device)
    side.wait_stream(torch.cuda.current_stream(cuda_device))
    with torch.cuda.stream(side):
        for _ in range(2):
            OPC.off_policy_correction_terms(old, rollout, mask, *args)
    torch.cuda.current_stream(cuda_device).wait_stream(side)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        captured = OPC.off_policy_correction_terms(old, rollout, mask, *args)
    for seed in (32, 33, 34):
        o, r, k = (t.to(cuda_device) for t in _batch(B=16, S=300, seed=seed))
        old.copy_(o), rollout.copy_(r), mask.copy_(k)
        graph.replay()
        torch.cuda.synchronize()
        eager = OPC.off_policy_correction_terms(o, r, k, *args)
        torch.cuda.synchronize()
        assert all(torch.equal(a, b) for a, b in zip(captured, eager)), seed


def test_nan_log_probabilities_reach_weights_and_metrics(cuda_device):
    """torch.clamp passes a NaN on, so the reference's ratio of a NaN log-probability is NaN and shows in the importance
    weight of its token, in the ratio statistics and in the sequence-level decisions of its row
    (utils/off_policy_correction_utils.py: _safe_exp_delta and its callers).  The kernel's clamp must not swallow it."""
    cfg = _cfg(tis_ratio_type="token", token_tis_ratio_clip_high=1.5)
    old, rollout, mask = _batch()
    old[6, 10] = float("nan")
    mask[6, 10] = 1.0
    want_tis, want_metrics, _ = O.off_policy_correction(old.double(), rollout.double(), mask.double(), cfg)
    tis, metrics, _ = OPC.compute_off_policy_correction(old.to(cuda_device), rollout.to(cuda_device), mask.to(cuda_device), cfg)
    assert bool(torch.isnan(want_tis[6, 10])) and bool(torch.isnan(tis[6, 10]))
    clean = torch.ones_like(mask, dtype=torch.bool)
    clean[6, 10] = False
    assert torch.allclose(tis.cpu().double()[clean], want_tis[clean], rtol=2e-5)
    for key in ("is_ratio_mean", "is_ratio_std", "is_ratio_max", "is_ratio_min"):
        assert want_metrics[key] != want_metrics[key] and metrics[key] != metrics[key], key   # NaN on both sides


def test_ratio_spread_far_below_its_mean(cuda_device):
    """Ratios within 1e-4 of 1: the standard deviation of the ratios is four orders of magnitude below their mean, where sums of x
    and x^2 in fp32 would cancel to nothing (the kernel sums x - 1 instead)."""
    cfg = _cfg(tis_ratio_type="token", token_tis_ratio_clip_high=2.0)
    gen = torch.Generator().manual_seed(9)
    B, S = 64, 2048
    rollout = torch.randn(B, S, generator=gen) * 0.7 - 1.5
    old = rollout + torch.randn(B, S, generator=gen) * 1e-4
    mask = torch.ones(B, S)
    _, want, _ = O.off_policy_correction(old.double(), rollout.double(), mask.double(), cfg)
    _, got, _ = OPC.compute_off_policy_correction(old.to(cuda_device), rollout.to(cuda_device), mask.to(cuda_device), cfg)
    assert 5e-5 < want["is_ratio_std"] < 2e-4
    # the inputs are fp32: the log-ratios themselves carry 2e-7 of rounding, 2e-3 of this spread
    assert got["is_ratio_std"] == pytest.approx(want["is_ratio_std"], rel=1e-2)
    assert got["is_ratio_mean"] == pytest.approx(want["is_ratio_mean"], rel=1e-6)
