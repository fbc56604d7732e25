"""The reference's own unit-test vectors for the consumers of the LM head's log-probabilities, run against the oracle (on the
CPU) and against the HIP path (marked ``gpu``).

``tests/golden/reference_unit_test_cases.json`` holds inputs and expected outputs transcribed from
tests/train/algorithms/test_off_policy_correction.py, tests/train/algorithms/test_losses.py and
tests/backends/skyrl_train/utils/test_ppo_utils.py of the SkyRL tree (each case names its lines).  Where the reference's test
states its expectation as numbers they are used as they stand; where it derives it from the inputs (SAPO's gate, GSPO's
sequence weight, DPPO's masked surrogate) the same derivation is done here token by token with ``math``, not with the
function under test.  The reference's tolerances are kept.
"""

from __future__ import annotations

import json
import math
import os
from types import SimpleNamespace

import pytest
import torch

from oracle import lmhead_oracle as O

CASES = json.load(open(os.path.join(os.path.dirname(__file__), "golden", "reference_unit_test_cases.json")))
OPC_CASES = {c["name"]: c for c in CASES["off_policy_correction"]}
LOSS_CASES = {c["name"]: c for c in CASES["policy_losses"]}
KL_CASES = {c["name"]: c for c in CASES["approx_kl"]}
NULL_CORRECTION = SimpleNamespace(**CASES["off_policy_correction_defaults"])


def _tensor(rows, dtype, device):
    return torch.tensor([[float(v) for v in row] for row in rows], dtype=dtype, device=device)


# ----------------------------------------------------------------------------------------------------------------------
# off-policy correction
# ----------------------------------------------------------------------------------------------------------------------
def _check_off_policy_case(case, fn, dtype, device):
    cfg = SimpleNamespace(**{**CASES["off_policy_correction_defaults"], **case["config"]})
    old, rollout, mask = (_tensor(case[k], dtype, device) for k in ("old", "rollout", "mask"))
    tis, metrics, new_mask = fn(old, rollout, mask, cfg)
    exp = case["expect"]
    tol = CASES["tis_tolerance"]
    if "tis" in exp:
        want = _tensor(exp["tis"], dtype, device)
        assert tis.shape == want.shape and torch.allclose(tis, want, rtol=tol["rtol"], atol=tol["atol"]), (tis, want)
    if exp.get("tis_is_none"):
        assert tis is None
    if "new_mask" in exp:
        assert torch.equal(new_mask.cpu().double(), _tensor(exp["new_mask"], torch.float64, "cpu")), new_mask
    if exp.get("metrics_empty"):
        assert metrics == {}
    for key, value in exp.get("metrics_exact", {}).items():
        assert float(metrics[key]) == value, (key, metrics[key])
    for key, (value, tol_abs) in exp.get("metrics_abs", {}).items():
        assert abs(float(metrics[key]) - value) < tol_abs, (key, metrics[key])
    for key in exp.get("metric_keys", []):
        assert key in metrics


@pytest.mark.parametrize("name", list(OPC_CASES))
def test_oracle_reproduces_the_reference_off_policy_cases(name):
    """In fp32, as the reference's tests run it; in fp64 too unless the case rests on fp32 rounding (a ratio that equals its
    threshold only after ``exp`` is rounded to fp32)."""
    case = OPC_CASES[name]
    _check_off_policy_case(case, O.off_policy_correction, torch.float32, "cpu")
    if not case["expect"].get("fp32_only"):
        _check_off_policy_case(case, O.off_policy_correction, torch.float64, "cpu")


@pytest.mark.gpu
@pytest.mark.parametrize("name", list(OPC_CASES))
def test_hip_reproduces_the_reference_off_policy_cases(name, cuda_device):
    from skyrl_amd import off_policy_correction as OPC
    _check_off_policy_case(OPC_CASES[name], OPC.compute_off_policy_correction, torch.float32, cuda_device)


def test_reference_off_policy_error_cases():
    """test_off_policy_correction.py:599-624: unknown step names raise ValueError with the reference's wording."""
    old, rollout, mask = (_tensor(v, torch.float32, "cpu") for v in ([[-1.0] * 3], [[-1.5] * 3], [[1.0] * 3]))
    with pytest.raises(ValueError, match="Unknown tis_ratio_type"):
        O.off_policy_correction(old, rollout, mask, SimpleNamespace(**{**CASES["off_policy_correction_defaults"], "tis_ratio_type": "invalid"}))
    with pytest.raises(ValueError, match="Unknown sequence_mask_metric"):
        O.off_policy_correction(old, rollout, mask, SimpleNamespace(**{**CASES["off_policy_correction_defaults"], "sequence_mask_metric": "invalid"}))


@pytest.mark.gpu
def test_hip_reference_off_policy_error_cases_and_loss_integration(cuda_device):
    """The same two errors from the product, and test_ppo_policy_loss_with_off_policy_correction (:533-596): the token-level
    weight changes the regular PPO loss."""
    from skyrl_amd import off_policy_correction as OPC
    from skyrl_amd import policy_loss as PL
    old, rollout, mask = (_tensor(v, torch.float32, cuda_device) for v in ([[-1.0] * 3], [[-1.5] * 3], [[1.0] * 3]))
    with pytest.raises(ValueError, match="Unknown tis_ratio_type"):
        OPC.compute_off_policy_correction(old, rollout, mask, SimpleNamespace(**{**CASES["off_policy_correction_defaults"], "tis_ratio_type": "invalid"}))
    with pytest.raises(ValueError, match="Unknown sequence_mask_metric"):
        OPC.compute_off_policy_correction(old, rollout, mask,
                                          SimpleNamespace(**{**CASES["off_policy_correction_defaults"], "sequence_mask_metric": "invalid"}))
    t = lambda rows: _tensor(rows, torch.float32, cuda_device)  # noqa: E731
    adv, old, lp, rollout, mask = t([[1.0, -1.0, 0.5]]), t([[-1.0] * 3]), t([[-1.1, -0.9, -1.0]]), t([[-1.05] * 3]), t([[1.0] * 3])
    correction = SimpleNamespace(**{**CASES["off_policy_correction_defaults"], "tis_ratio_type": "token", "token_tis_ratio_clip_high": 2.0,
                                    "outlier_token_is_threshold_low": 1e-4, "outlier_token_is_threshold_high": 100.0})
    base = dict(policy_loss_type="regular", eps_clip_low=0.2, eps_clip_high=0.2, clip_ratio_c=3.0)
    with_c, _ = PL.ppo_policy_loss(lp, old, adv, SimpleNamespace(**base, off_policy_correction=correction), mask, rollout)
    without, _ = PL.ppo_policy_loss(lp, old, adv, SimpleNamespace(**base, off_policy_correction=NULL_CORRECTION), mask, rollout)
    assert not torch.allclose(with_c, without, rtol=1e-3)
    # every token's weight is exp(0.05): the corrected loss is the plain one times it
    assert with_c.item() == pytest.approx(without.item() * math.exp(0.05), rel=1e-5)


# ----------------------------------------------------------------------------------------------------------------------
# policy losses
# ----------------------------------------------------------------------------------------------------------------------
def _loss_config(case):
    cfg = dict(policy_loss_type=case["loss_type"], eps_clip_low=0.2, eps_clip_high=0.2, clip_ratio_c=3.0, off_policy_correction=NULL_CORRECTION)
    for key, value in case["config"].items():
        cfg[key] = SimpleNamespace(**value) if isinstance(value, dict) else value
    return SimpleNamespace(**cfg)


def _oracle_loss(case, lp, old, adv, mask, rollout):
    """``(loss, metrics)`` of the oracle under the product's calling convention."""
    cfg, kind = _loss_config(case), case["loss_type"]
    if kind in ("regular", "dual_clip"):
        loss, clip = O.ppo_policy_loss(lp, old, adv, cfg.eps_clip_low, cfg.eps_clip_high, cfg.clip_ratio_c, kind == "dual_clip", mask)
    elif kind == "cispo":
        anchor = rollout if cfg.cispo.cispo_anchor == "rollout" else old
        loss, clip = O.cispo_policy_loss(lp, anchor, adv, cfg.cispo.cispo_eps_clip_low, cfg.cispo.cispo_eps_clip_high, mask)
        return loss, {"clip_ratio": float(clip), **O.cispo_ratio_diagnostics(lp, anchor, cfg.cispo.cispo_eps_clip_low, cfg.cispo.cispo_eps_clip_high, mask)}
    elif kind == "gspo":
        loss, clip = O.gspo_policy_loss(lp, old, adv, cfg.eps_clip_low, cfg.eps_clip_high, mask)
    elif kind == "sapo":
        loss, clip = O.sapo_policy_loss(lp, old, adv, cfg.sapo.tau_pos, cfg.sapo.tau_neg, mask)
    elif kind == "dppo":
        loss, clip = O.dppo_policy_loss(lp, rollout if rollout is not None else old, adv, cfg.dppo.dppo_type, cfg.dppo.delta_low, cfg.dppo.delta_high, mask)
    elif kind == "clip_cov":
        loss, clip, _ = O.clip_cov_policy_loss(lp, old, adv, cfg.eps_clip_low, cfg.eps_clip_high, cfg.clip_cov.clip_ratio, cfg.clip_cov.clip_cov_lb,
                                               cfg.clip_cov.clip_cov_ub, mask)
    elif kind == "kl_cov":
        loss, _ = O.kl_cov_policy_loss(lp, old, adv, cfg.kl_cov.kl_cov_frac, cfg.kl_cov.ppo_kl_coef, mask)
        clip = 0.0
    else:
        raise AssertionError(kind)
    return loss, {"clip_ratio": float(clip)}


def _product_loss(case, lp, old, adv, mask, rollout):
    from skyrl_amd import policy_loss as PL
    fn = PL.get_policy_loss(case["loss_type"])
    return fn(lp, old, adv, _loss_config(case), mask, rollout)


def _hand_expectation(case):
    """What the reference's test derives from the inputs, token by token with ``math``."""
    exp, lp, old, adv = case["expect"], case["log_probs"], case["old_log_probs"], case["advantages"]
    mask = case.get("loss_mask") or [[1.0] * len(r) for r in lp]
    rollout = case.get("rollout_logprobs")
    clamp = lambda v, lo, hi: min(max(v, lo), hi)  # noqa: E731
    total = 0.0
    if exp.get("formula") == "cispo":          # test_losses.py:159-160
        for b, row in enumerate(lp):
            for s, x in enumerate(row):
                total += -clamp(math.exp(x - rollout[b][s]), 0.8, 1.2) * adv[b][s] * x
        return total
    if exp.get("formula") == "sapo":           # :576-594
        for b, row in enumerate(lp):
            for s, x in enumerate(row):
                tau = 1.0 if adv[b][s] > 0 else 2.0
                ratio = math.exp(clamp(x - old[b][s], -20.0, 20.0))
                total += -(1.0 / (1.0 + math.exp(-tau * (ratio - 1.0)))) * (4.0 / tau) * adv[b][s]
        return total
    if exp.get("formula") == "gspo_and_regular":   # :352-376: the row's masked mean log-ratio is every token's log-weight
        token = 0.0
        for b, row in enumerate(lp):
            n = sum(mask[b])
            seq = math.exp(sum((x - old[b][s]) * mask[b][s] for s, x in enumerate(row)) / max(n, 1.0))
            for s, x in enumerate(row):
                a = adv[b][s]
                total += -min(seq * a, clamp(seq, 0.8, 1.2) * a)
                r = math.exp(x - old[b][s])
                token += -min(r * a, clamp(r, 0.8, 1.2) * a) * mask[b][s]
        return total, token
    if "kept_mask" in exp and exp["kept_mask"] is not None:      # :726-729
        for b, row in enumerate(lp):
            for s, x in enumerate(row):
                total += -math.exp(x - old[b][s]) * adv[b][s] * exp["kept_mask"][b][s]
        return total
    return None


def _check_loss_case(case, fn, dtype, device):
    t = lambda key: None if case.get(key) is None else _tensor(case[key], dtype, device)  # noqa: E731
    lp, old, adv, mask, rollout = t("log_probs"), t("old_log_probs"), t("advantages"), t("loss_mask"), t("rollout_logprobs")
    exp = case["expect"]
    if "seed" in case:
        torch.manual_seed(case["seed"])
    loss, metrics = fn(case, lp, old, adv, mask, rollout)
    loss = float(loss)
    if "loss" in exp:
        assert loss == pytest.approx(exp["loss"], abs=exp["loss_abs"])
        assert loss == pytest.approx(sum(sum(r) for r in exp["per_token"]), rel=exp["per_token_rtol"])
    hand = _hand_expectation(case)
    if exp.get("formula") == "gspo_and_regular":
        want_seq, want_token = hand
        assert loss == pytest.approx(want_seq, rel=exp["rtol"], abs=1e-8)
        regular, _ = fn({**case, "loss_type": "regular"}, lp, old, adv, mask, rollout)
        assert float(regular) == pytest.approx(want_token, rel=exp["rtol"], abs=1e-8)
        assert abs(float(regular) - loss) > 1e-3 * abs(loss)                       # :412-414
    elif hand is not None:
        assert loss == pytest.approx(hand, rel=exp.get("rtol", 1e-3), abs=exp.get("atol", 1e-8))
    for key in exp.get("metric_keys", []):
        assert key in metrics
    if exp.get("formula") == "cispo":          # :171-175
        ratios = [math.exp(x - r) for x, r in zip(case["log_probs"][0], case["rollout_logprobs"][0])]
        assert float(metrics["cispo/ratio_mean"]) == pytest.approx(sum(ratios) / 3, rel=1e-3)
        assert float(metrics["cispo/ratio_clamped_mean"]) == pytest.approx(sum(min(max(r, 0.8), 1.2) for r in ratios) / 3, rel=1e-3)
        assert float(metrics["cispo/ratio_max"]) == pytest.approx(max(ratios), rel=1e-3)
        old_anchor = {**case, "config": {"cispo": {**case["config"]["cispo"], "cispo_anchor": "old"}}}
        assert abs(float(fn(old_anchor, lp, old, adv, mask, rollout)[0]) - loss) > 1e-3          # :178-192
    for key, (value, rel) in exp.get("metrics_rel", {}).items():
        assert float(metrics[key]) > 0.0 and float(metrics[key]) == pytest.approx(value, rel=rel), key
    if "clip_ratio" in exp:
        assert float(metrics["clip_ratio"]) == exp["clip_ratio"]
    if exp.get("clip_ratio_positive") is True:
        assert float(metrics["clip_ratio"]) > 0.0
    elif exp.get("clip_ratio_positive") is False:
        assert float(metrics["clip_ratio"]) == pytest.approx(0.0, abs=1e-6)
    if exp.get("rollout_changes_loss"):        # :703-720
        assert abs(float(fn(case, lp, old, adv, mask, None)[0]) - loss) > 1e-6
    if exp.get("finite"):
        assert math.isfinite(loss)
    if exp.get("clip_ratio_in_unit_interval"):
        assert 0.0 <= float(metrics["clip_ratio"]) <= 1.0
    if "differs_from_regular_rtol" in exp:
        regular = float(fn({**case, "loss_type": "regular", "config": {"eps_clip_low": 0.2, "eps_clip_high": 0.2}}, lp, old, adv, mask, rollout)[0])
        assert abs(regular - loss) > exp["differs_from_regular_rtol"] * abs(regular)


@pytest.mark.parametrize("name", list(LOSS_CASES))
def test_oracle_reproduces_the_reference_loss_cases(name):
    _check_loss_case(LOSS_CASES[name], _oracle_loss, torch.float32, "cpu")
    _check_loss_case(LOSS_CASES[name], _oracle_loss, torch.float64, "cpu")


@pytest.mark.gpu
@pytest.mark.parametrize("name", list(LOSS_CASES))
def test_hip_reproduces_the_reference_loss_cases(name, cuda_device):
    _check_loss_case(LOSS_CASES[name], _product_loss, torch.float32, cuda_device)


@pytest.mark.gpu
def test_hip_reference_cispo_argument_errors(cuda_device):
    """test_losses.py:236-271: the rollout anchor needs rollout log-probabilities (AssertionError) and refuses a TIS weight on
    top (ValueError naming the double count)."""
    from skyrl_amd import policy_loss as PL
    one = lambda v: torch.tensor([[v]], device=cuda_device)  # noqa: E731
    cfg = SimpleNamespace(policy_loss_type="cispo", cispo=SimpleNamespace(cispo_eps_clip_low=1.0, cispo_eps_clip_high=4.0, cispo_anchor="rollout"),
                          off_policy_correction=NULL_CORRECTION)
    with pytest.raises(AssertionError):
        PL.compute_policy_loss_cispo(one(-1.0), one(-1.0), one(1.0), cfg, None, None)
    cfg.off_policy_correction = SimpleNamespace(**{**CASES["off_policy_correction_defaults"], "tis_ratio_type": "token"})
    with pytest.raises(ValueError, match="double-count"):
        PL.compute_policy_loss_cispo(one(-1.0), one(-1.0), one(1.0), cfg, None, one(-1.2))


# ----------------------------------------------------------------------------------------------------------------------
# approximate KL
# ----------------------------------------------------------------------------------------------------------------------
def _check_kl_cases(fn, dtype, device):
    c = KL_CASES["estimators"]                 # test_ppo_utils.py:57-76
    lp, base, mask = (_tensor(c[k], dtype, device) for k in ("log_probs", "log_probs_base", "mask"))
    d = [x - y for x, y in zip(c["log_probs"][0], c["log_probs_base"][0])]
    m = c["mask"][0]
    hand = {"k1": [di * mi for di, mi in zip(d, m)], "abs": [abs(di) * mi for di, mi in zip(d, m)],
            "k2": [0.5 * di * di * mi for di, mi in zip(d, m)], "k3": [(math.exp(-di) - 1 + di) * mi for di, mi in zip(d, m)]}
    for kind, want in hand.items():
        got = fn(lp, base, mask, kind)
        assert torch.allclose(got.cpu().double(), torch.tensor([want], dtype=torch.float64), atol=c["atol"]), kind
    c = KL_CASES["applies_loss_mask"]          # :78-98: a masked position is 0 even when its input is NaN; soft masks scale
    lp, base, mask = (_tensor(c[k], dtype, device) for k in ("log_probs", "log_probs_base", "mask"))
    for kind in ("k1", "k2", "k3", "abs"):
        kld = fn(lp, base, mask, kind)
        assert bool(torch.isfinite(kld).all()) and kld[0, 3].item() == 0.0, kind
        mean = (kld * mask).sum() / mask.sum().clamp(min=1.0)
        assert bool(torch.isfinite(mean))
        unmasked = fn(lp, base, None, kind)
        assert torch.allclose(kld[:, :3], unmasked[:, :3] * mask[:, :3], atol=c["atol"]), kind


def test_oracle_reproduces_the_reference_approx_kl_cases():
    _check_kl_cases(O.compute_approx_kl, torch.float32, "cpu")
    _check_kl_cases(O.compute_approx_kl, torch.float64, "cpu")


@pytest.mark.gpu
def test_hip_reproduces_the_reference_approx_kl_cases(cuda_device):
    from skyrl_amd import policy_loss as PL
    _check_kl_cases(lambda lp, base, mask, kind: PL.compute_approx_kl(lp, base, mask, kl_estimator_type=kind), torch.float32, cuda_device)


# ----------------------------------------------------------------------------------------------------------------------
# MTP draft loss: the reference's helper and end-to-end cases (tests/backends/skyrl_train/mtp/test_soft_ce.py)
# ----------------------------------------------------------------------------------------------------------------------
def test_unpadded_vocab_shard_width_reference_cases():
    """test_soft_ce.py:285-297, the six known answers."""
    from skyrl_amd.mtp_soft_ce import unpadded_vocab_shard_width
    assert unpadded_vocab_shard_width(None, 128, 0) == 128
    assert unpadded_vocab_shard_width(256, 128, 0) == 128 and unpadded_vocab_shard_width(256, 128, 1) == 128
    assert unpadded_vocab_shard_width(250, 128, 0) == 128 and unpadded_vocab_shard_width(250, 128, 1) == 122
    assert unpadded_vocab_shard_width(100, 128, 1) == 0


@pytest.mark.gpu
def test_hip_left_padded_draft_loss_is_the_teacher_entropy(cuda_device):
    """test_soft_ce.py:248-282 from hidden states: a left-padded row whose padding holds zeros (uniform logits), a student
    aligned with the rolled teacher.  The draft loss over ``shift_mask_for_mtp``'s mask is the teacher's entropy over the
    positions whose own token and target are real -- the uniform padding must not leak in -- and stays below ln V.  Then the
    padded-vocabulary case: junk weight rows behind the true vocabulary change nothing once ``weight[:width]`` is passed."""
    from skyrl_amd import mtp_soft_ce as M
    gen = torch.Generator().manual_seed(0)
    V, H, pad, real = 320, 128, 2, 6
    seq = pad + real
    weight = (torch.randn(V, H, generator=gen) * 0.3).bfloat16()
    policy_hidden = torch.zeros(1, seq, H)
    policy_hidden[:, pad:] = torch.randn(1, real, H, generator=gen)
    policy_hidden = policy_hidden.bfloat16()
    mask = torch.zeros(1, seq)
    mask[:, pad:] = 1.0
    student_hidden = torch.roll(policy_hidden, -1, dims=1)         # aligned with the depth-0 teacher
    layer_mask = M.shift_mask_for_mtp(mask, 0)
    assert layer_mask.tolist() == [[0.0, 0.0, 1.0, 1.0, 1.0, 1.0, 1.0, 0.0]]
    to = lambda t: t.to(cuda_device)  # noqa: E731
    loss = M.draft_soft_ce_from_hidden(to(student_hidden), to(policy_hidden), to(weight), to(layer_mask), mtp_layer_number=0)
    teacher_logits = torch.roll(policy_hidden.double() @ weight.double().t(), -1, dims=1)
    dist = torch.distributions.Categorical(logits=teacher_logits)
    entropy = dist.entropy()
    want = (entropy * layer_mask.double()).sum() / layer_mask.sum()
    assert loss.item() == pytest.approx(want.item(), abs=1e-4)
    assert loss.item() < entropy[layer_mask.bool()].max().item() + 1e-4 and loss.item() < math.log(V)
    # the rolled mask alone (without the source-side AND) would have let a padding position in: a different value at this tolerance
    leaked = (entropy * torch.roll(mask, -1, 1).double()).sum() / torch.roll(mask, -1, 1).sum()
    assert abs(leaked.item() - want.item()) > 1e-3
    # a vocabulary padded from 300 to 320 rows: the tail rows hold junk and are sliced away
    width = M.unpadded_vocab_shard_width(300, V, 0)
    assert width == 300
    clean = M.draft_soft_ce_from_hidden(to(student_hidden), to(policy_hidden), to(weight[:width].contiguous()), to(layer_mask), mtp_layer_number=0)
    junk = weight.clone()
    junk[width:] = 7.0
    padded = M.draft_soft_ce_from_hidden(to(student_hidden), to(policy_hidden), to(junk)[:width], to(layer_mask), mtp_layer_number=0)
    assert padded.item() == clean.item()
    topk = M.draft_soft_ce_topk_from_hidden(to(student_hidden), to(policy_hidden), to(junk)[:width], to(layer_mask), k=width, roll_shift=1)
    assert topk.item() == pytest.approx(clean.item(), abs=1e-4)    # k = V: the full soft cross-entropy


@pytest.mark.gpu
def test_hip_draft_losses_reject_an_attached_teacher(cuda_device):
    """test_soft_ce.py:196-212: both draft losses assert that the caller detached the teacher."""
    from skyrl_amd import mtp_soft_ce as M
    student = torch.randn(1, 3, 64, device=cuda_device).bfloat16().requires_grad_(True)
    teacher = torch.randn(1, 3, 64, device=cuda_device).bfloat16().requires_grad_(True)
    weight = torch.randn(256, 64, device=cuda_device).bfloat16()
    mask = torch.ones(1, 3, device=cuda_device)
    for call in (lambda t: M.draft_soft_ce_from_hidden(student, t, weight, mask),
                 lambda t: M.draft_soft_ce_topk_from_hidden(student, t, weight, mask, k=3)):
        with pytest.raises(AssertionError, match="must be detached"):
            call(teacher)
        assert bool(torch.isfinite(call(teacher.detach())))


# ----------------------------------------------------------------------------------------------------------------------
# the FSDP wrapper's forward tail on the reference's own padded layouts (tests/backends/skyrl_train/gpu/gpu_ci/
# test_model_wrapper.py:24-33, 200-245): padding on both sides, the last action slot a padding token
# ----------------------------------------------------------------------------------------------------------------------
WRAPPER_V, WRAPPER_EOS, WRAPPER_PAD = 1000, 999, 0
WRAPPER_LAYOUTS = {
    "one_row": ([[WRAPPER_PAD] * 3 + [10, 14, 200, 3, 40, WRAPPER_EOS] + [WRAPPER_PAD]], [[0] * 3 + [1] * 6 + [0]]),
    "two_rows": ([[WRAPPER_PAD] * 3 + [10, 14, 200, 3, 40, WRAPPER_EOS] + [WRAPPER_PAD],
                  [WRAPPER_PAD, 12, 13, 220, 998, 3, 40, WRAPPER_EOS] + [WRAPPER_PAD] * 2], [[0] * 3 + [1] * 6 + [0], [0] + [1] * 7 + [0] * 2]),
}


def _marker_logits(next_tokens, V):
    """Logits whose log-probability of ``next_tokens[p]`` at position ``p`` is a known function of that token: zeros except a
    peak ``a = token / 200`` at the token's own column, so log p = a - ln(V - 1 + e^a)."""
    z = torch.zeros(len(next_tokens), V, dtype=torch.float64)
    for p, tok in enumerate(next_tokens):
        z[p, tok] = tok / 200.0
    return z


def _marker_value(tok, V):
    a = tok / 200.0
    return a - math.log(V - 1 + math.exp(a))


@pytest.mark.gpu
@pytest.mark.parametrize("layout", list(WRAPPER_LAYOUTS))
@pytest.mark.parametrize("from_hidden", [False, True])
def test_hip_wrapper_tail_on_the_reference_layouts(layout, from_hidden, cuda_device):
    """The reference mocks the per-position log-probability as "the next token's id" and expects the wrapper to hand back the
    action tokens themselves, with and without sample packing (test_model_wrapper.py:36-103).  Without mocking: logits built
    so that the log-probability of the next token is a known function of its id; the wrapper must return that function of the
    last ``num_actions`` tokens.  The last action slot is the padding token behind EOS: without packing its label is that
    padding token, with packing the roll wraps to the first real token of the stream -- as in the reference.  Then
    test_actor_entropy_consistency_sample_packing (:200-245): entropy with and without packing agrees on the real tokens."""
    from skyrl_amd.model_wrapper import action_log_probs_from_hidden, action_log_probs_from_logits
    ids, am = (torch.tensor(v) for v in WRAPPER_LAYOUTS[layout])
    B, S = ids.shape
    A, V = 4, WRAPPER_V
    nnz = am.flatten().nonzero().flatten()
    dev = cuda_device
    results = {}
    for packed in (False, True):
        stream = ids.reshape(-1)[nnz][None] if packed else ids
        rolled = torch.roll(stream, -1, dims=1)
        logits = torch.stack([_marker_logits(r.tolist(), V) for r in rolled])              # [rows, positions, V]
        if from_hidden:   # an identity-like head: hidden = logits padded to H = 1024 columns, weight = the matching unit rows
            H = 1024
            hidden = torch.zeros(*logits.shape[:2], H, dtype=torch.float64)
            hidden[..., :V] = logits
            weight = torch.zeros(V, H, dtype=torch.float64)
            weight[torch.arange(V), torch.arange(V)] = 1.0
            alp, out = action_log_probs_from_hidden(hidden.bfloat16().to(dev), weight.bfloat16().to(dev), ids.to(dev), A, am.to(dev), 1.0,
                                                    return_output=True, compute_entropy=True, entropy_requires_grad=False,
                                                    nnz_indices=nnz.to(dev) if packed else None)
            tol = 2e-2                                                                     # the peaks a = token / 200 rounded to bf16
        else:
            alp, out = action_log_probs_from_logits(logits.float().to(dev), ids.to(dev), A, am.to(dev), 1.0, return_output=True,
                                                    compute_entropy=True, entropy_requires_grad=False,
                                                    nnz_indices=nnz.to(dev) if packed else None)
            tol = 1e-5
        assert alp.shape == (B, A)
        for b in range(B):
            for j in range(A):
                pos = S - A - 1 + j                                                        # the position that scores action j
                if packed and not bool(am[b, pos]):
                    want = 0.0                                                             # padding put back as zeros
                elif packed:
                    k = int((nnz == b * S + pos).nonzero())                               # its place in the packed stream
                    want = _marker_value(int(rolled[0, k]), V)
                else:
                    want = _marker_value(int(ids[b, pos + 1]), V)
                assert alp[b, j].item() == pytest.approx(want, abs=tol), (packed, b, j)
        results[packed] = out["entropy"].float().cpu()
        # cross-check with the oracle's statement of the tail on the same logits
        want_alp, want_ent = O.hf_wrapper_tail(logits, ids, A, am.double(), 1.0, nnz_indices=nnz if packed else None)
        assert (alp.cpu().double() - want_alp).abs().max().item() <= tol
        assert (results[packed].double() - want_ent).abs().max().item() <= (5e-2 if from_hidden else 1e-5)
    # wherever both runs scored the same next token -- every real token but the last of each row -- the entropies agree;
    # padding positions are zero in both
    real = am.bool()
    same_label = real & torch.roll(am, -1, dims=1).bool()
    same_label[:, -1] = False
    assert torch.allclose(results[False][same_label], results[True][same_label], atol=5e-2 if from_hidden else 1e-5)
    assert bool((results[True][~real] == 0).all()) and bool((results[False][~real] == 0).all())
