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
