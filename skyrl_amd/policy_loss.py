"""Losses on the fused path's log-probabilities and entropies: value, statistics and gradient from one HIP kernel each.

Mirrors of the reference's functions (skyrl/backends/skyrl_train/utils/ppo_utils.py unless noted), same positional arguments
and results:

* ``ppo_policy_loss``           :555-588  (policy loss types "regular" and "dual_clip") -> ``(loss, {"clip_ratio": ...})``
* ``cross_entropy_loss``        :1056-1092 -> ``(loss, {"clip_ratio": 0.0})``
* ``importance_sampling_loss``  :1095-1142 -> ``(loss, {"importance_ratio": ...})``
* ``sapo_policy_loss``          :590-660, ``gspo_policy_loss`` :663-729, ``compute_policy_loss_cispo`` :732-821,
  ``rollout_is_policy_loss`` :824-863, ``dppo_policy_loss`` :866-935 -> ``(loss, {"clip_ratio": ...})``
* ``compute_approx_kl``         :88-126    -> per-token KL estimate ``[B, S]``
* ``masked_mean``               torch_utils.py:180-184

plus ``actor_loss``, the whole per-micro-batch loss of the policy worker (policy loss + KL term - entropy term,
workers/worker.py:989-1089) with both upstream gradients of the LM head from two launches (three with an entropy gradient), and ``approx_kl_loss``, the
reduction the trainer applies to the KL estimate (``masked_mean(kl, mask, dim=-1).mean()``,
workers/worker.py:1071-1077) fused with the estimate and its gradient.  The losses are reduced as ``reduce_loss`` does
(masked sum, :1145-1149; the reference folds the kind of mean into the advantages beforehand, :1152-1181).  The reference
computes each with a chain of elementwise torch kernels and lets autograd derive the gradient; here one kernel produces
value, statistics and gradient, so the upstream gradient of ``skyrl_lmhead_bwd`` is ready without another pass over the
``[B, S]`` tensors and, with ``sync_metrics=False``, without a host synchronisation.

Off-policy correction (``apply_off_policy_correction``, off_policy_correction_utils.py:351-391): the six losses that end with
it in the reference (regular / dual clip, SAPO, GSPO, CISPO, rollout-IS, DPPO) end with it here -- when the config
switches a correction on and ``rollout_logprobs`` are given, ``skyrl_amd.off_policy_correction`` computes the truncated
importance weight and the thinned mask in two launches and their product joins ``loss_weight``; the metrics of the
correction are added to the loss's metrics under the reference's names.  A weight computed elsewhere can still be passed as
``loss_weight``.
The two covariance-based types pick their tokens from the whole batch exactly as the reference does -- ``clip_cov`` a random
subset drawn with ``torch.randperm`` on the host's generator, ``kl_cov`` a top-k computed on the CPU -- and hand the
per-token decision to the same fused kernel (``compute_policy_loss_clip_cov``, ``compute_policy_loss_kl_cov``, :938-1053).
"""

from __future__ import annotations

from typing import Any, Dict, Optional, Tuple

import torch

from . import _lib
from .ops import _require_device

__all__ = ["ppo_policy_loss", "cross_entropy_loss", "importance_sampling_loss", "sapo_policy_loss", "gspo_policy_loss",
           "compute_policy_loss_cispo", "rollout_is_policy_loss", "dppo_policy_loss", "compute_approx_kl", "approx_kl_loss",
           "masked_mean", "actor_loss", "ppo_policy_loss_terms", "compute_policy_loss_clip_cov", "compute_policy_loss_kl_cov",
           "POLICY_LOSS_FUNCTIONS", "get_policy_loss"]

LOSS_REGULAR, LOSS_DUAL_CLIP, LOSS_CROSS_ENTROPY, LOSS_IMPORTANCE_SAMPLING = 0, 1, 2, 3
LOSS_GSPO, LOSS_SAPO, LOSS_CISPO, LOSS_ROLLOUT_IS, LOSS_DPPO_TV, LOSS_DPPO_KL = 4, 5, 6, 7, 8, 9
LOSS_CLIP_COV, LOSS_KL_COV = 10, 11


def _get(obj: Any, name: str, default: Any = None) -> Any:
    """Field of a config given as an object or as a mapping."""
    if obj is None:
        return default
    if isinstance(obj, dict):
        return obj.get(name, default)
    return getattr(obj, name, default)


def _with_off_policy_correction(config: Any, old_log_probs, rollout_logprobs, loss_mask, loss_weight, sync_metrics: bool):
    """The reference's losses end with ``apply_off_policy_correction(loss, old_log_probs, rollout_logprobs, loss_mask,
    config.off_policy_correction)`` (ppo_utils.py:581, 653, 722, 815, 857, 929): the per-token loss times the truncated
    importance weight, summed over the thinned mask, while their clip statistic was counted with the original mask.  Here
    the correction's per-token factor ``tis * keep`` joins ``loss_weight`` and the original mask stays the kernel's mask.
    Returns ``(loss_weight, the correction's metrics)``; nothing changes when the reference would not correct."""
    from .off_policy_correction import correction_weight

    weight, metrics = correction_weight(config, old_log_probs, rollout_logprobs, loss_mask, sync_metrics)
    if weight is None:
        return loss_weight, metrics
    return (weight if loss_weight is None else loss_weight.to(torch.float32) * weight), metrics


KL_ESTIMATORS = {"k1": 0, "abs": 1, "k2": 2, "k3": 3}
_LOSS_PARTIALS = 256  # SKYRL_POLICY_LOSS_PARTIALS of the header


def _flat_f32(name: str, t: Optional[torch.Tensor], numel: int) -> Optional[torch.Tensor]:
    if t is None:
        return None
    if t.numel() != numel:
        raise ValueError(f"{name} has {t.numel()} elements, log_probs has {numel}")
    return t.detach().reshape(-1).to(torch.float32).contiguous()


@torch.library.custom_op("skyrl_amd::ppo_policy_loss", mutates_args=())
def ppo_policy_loss_terms(
    log_probs: torch.Tensor,
    old_log_probs: Optional[torch.Tensor],
    advantages: Optional[torch.Tensor],
    loss_mask: Optional[torch.Tensor],
    loss_weight: Optional[torch.Tensor],
    eps_clip_low: float,
    eps_clip_high: float,
    clip_ratio_c: float,
    loss_type: int,
) -> Tuple[torch.Tensor, torch.Tensor]:
    """``(sums, grad)``: sums = [sum loss*mask*weight, statistic, sum mask] (fp32 [3]; the statistic is the number of clipped
    tokens, or the sum of importance ratios for LOSS_IMPORTANCE_SAMPLING); grad = d sums[0] / d log_probs (fp32, flat).
    All inputs are flat contiguous fp32 tensors of one length; LOSS_CROSS_ENTROPY reads neither old_log_probs nor
    advantages."""
    dev = _require_device(log_probs)
    if loss_type != LOSS_CROSS_ENTROPY and (old_log_probs is None or advantages is None):
        raise ValueError("this loss type needs old_log_probs and advantages")
    n = log_probs.numel()
    for name, t in (("log_probs", log_probs), ("old_log_probs", old_log_probs), ("advantages", advantages),
                    ("loss_mask", loss_mask), ("loss_weight", loss_weight)):
        if t is None:
            continue
        if t.dtype != torch.float32 or t.dim() != 1 or t.numel() != n or not t.is_contiguous():
            raise ValueError(f"{name} must be a contiguous fp32 vector of {n} elements, got {t.dtype} {tuple(t.shape)}")
    if n == 0:
        return torch.zeros(3, dtype=torch.float32, device=dev), torch.empty(0, dtype=torch.float32, device=dev)
    sums = torch.empty(3, dtype=torch.float32, device=dev)
    grad = torch.empty(n, dtype=torch.float32, device=dev)
    partials = torch.empty(3 * _LOSS_PARTIALS, dtype=torch.float32, device=dev)   # per-workgroup sums of the kernel
    ptr = lambda t: None if t is None else t.data_ptr()  # noqa: E731
    with torch.cuda.device(dev):
        st = _lib.load().skyrl_ppo_policy_loss(
            log_probs.data_ptr(), ptr(old_log_probs), ptr(advantages), ptr(loss_mask), ptr(loss_weight), n,
            float(eps_clip_low), float(eps_clip_high), float(clip_ratio_c), int(loss_type), sums.data_ptr(),
            grad.data_ptr(), partials.data_ptr(), torch.cuda.current_stream(dev).cuda_stream)
    _lib.check(st, "skyrl_ppo_policy_loss")
    return sums, grad


@ppo_policy_loss_terms.register_fake
def _(log_probs, old_log_probs, advantages, loss_mask, loss_weight, eps_clip_low, eps_clip_high, clip_ratio_c, loss_type):
    return log_probs.new_empty(3, dtype=torch.float32), log_probs.new_empty(log_probs.numel(), dtype=torch.float32)


class _PolicyLoss(torch.autograd.Function):
    @staticmethod
    def forward(ctx, log_probs, old_log_probs, advantages, loss_mask, loss_weight, eps_low, eps_high, clip_c, loss_type):
        n = log_probs.numel()
        sums, grad = ppo_policy_loss_terms(
            _flat_f32("log_probs", log_probs, n), _flat_f32("old_log_probs", old_log_probs, n),
            _flat_f32("advantages", advantages, n), _flat_f32("loss_mask", loss_mask, n),
            _flat_f32("loss_weight", loss_weight, n), eps_low, eps_high, clip_c, loss_type)
        ctx.save_for_backward(grad)
        ctx.shape, ctx.dtype = log_probs.shape, log_probs.dtype
        ctx.mark_non_differentiable(sums)
        return sums[0].clone(), sums

    @staticmethod
    def backward(ctx, grad_loss, _grad_sums):
        (grad,) = ctx.saved_tensors
        return (grad * grad_loss).reshape(ctx.shape).to(ctx.dtype), None, None, None, None, None, None, None, None


def ppo_policy_loss(
    log_probs: torch.Tensor,
    old_log_probs: torch.Tensor,
    advantages: torch.Tensor,
    config: Any,
    loss_mask: Optional[torch.Tensor] = None,
    rollout_logprobs: Optional[torch.Tensor] = None,
    *,
    loss_weight: Optional[torch.Tensor] = None,
    sync_metrics: bool = True,
) -> Tuple[torch.Tensor, Dict[str, Any]]:
    """Same contract as the reference's ``ppo_policy_loss`` (ppo_utils.py:555-588).

    ``config`` needs ``policy_loss_type`` ("regular" or "dual_clip"), ``eps_clip_low``, ``eps_clip_high`` and, for dual clip,
    ``clip_ratio_c``.  Returns the loss (a scalar that back-propagates into ``log_probs``) and ``{"clip_ratio": value}``;
    the value is a Python float as in the reference, or a 0-dim tensor when ``sync_metrics=False`` (no host synchronisation).
    """
    loss_type = getattr(config, "policy_loss_type", "regular")
    assert loss_type in ["regular", "dual_clip"], "loss_type must be either 'regular' or 'dual_clip'"
    loss_weight, extra = _with_off_policy_correction(config, old_log_probs, rollout_logprobs, loss_mask, loss_weight, sync_metrics)
    dual = loss_type == "dual_clip"
    loss, sums = _PolicyLoss.apply(log_probs, old_log_probs, advantages, loss_mask, loss_weight, float(config.eps_clip_low),
                                   float(config.eps_clip_high), float(getattr(config, "clip_ratio_c", 0.0)) if dual else 0.0,
                                   LOSS_DUAL_CLIP if dual else LOSS_REGULAR)
    clip_ratio = sums[1] / sums[2].clamp(min=1.0)
    return loss, {"clip_ratio": clip_ratio.item() if sync_metrics else clip_ratio, **extra}


def cross_entropy_loss(
    log_probs: torch.Tensor,
    old_log_probs: Optional[torch.Tensor],
    advantages: Optional[torch.Tensor],
    config: Any,
    loss_mask: Optional[torch.Tensor] = None,
    rollout_logprobs: Optional[torch.Tensor] = None,
) -> Tuple[torch.Tensor, Dict[str, Any]]:
    """Supervised negative log-likelihood, ``-(log_probs * loss_mask).sum()`` (reference ``cross_entropy_loss``,
    ppo_utils.py:1056-1092); ``old_log_probs``, ``advantages``, ``config`` and ``rollout_logprobs`` are ignored as there."""
    loss, _ = _PolicyLoss.apply(log_probs, None, None, loss_mask, None, 0.0, 0.0, 0.0, LOSS_CROSS_ENTROPY)
    return loss, {"clip_ratio": 0.0}


def importance_sampling_loss(
    log_probs: torch.Tensor,
    old_log_probs: torch.Tensor,
    advantages: torch.Tensor,
    config: Any,
    loss_mask: Optional[torch.Tensor] = None,
    rollout_logprobs: Optional[torch.Tensor] = None,
    *,
    sync_metrics: bool = True,
) -> Tuple[torch.Tensor, Dict[str, Any]]:
    """``-(exp(log_probs - old_log_probs) * advantages * loss_mask).sum()`` and the masked mean importance ratio (reference
    ``importance_sampling_loss``, ppo_utils.py:1095-1142; no clamp of the log-ratio, no clamp of the mask count)."""
    loss, sums = _PolicyLoss.apply(log_probs, old_log_probs, advantages, loss_mask, None, 0.0, 0.0, 0.0,
                                   LOSS_IMPORTANCE_SAMPLING)
    ratio = sums[1] / sums[2]
    return loss, {"importance_ratio": ratio.item() if sync_metrics else ratio}


def _type_parameters(config: Any, name: str, rollout_logprobs: Optional[torch.Tensor], old_log_probs):
    """``(loss_type, a, b, c, behaviour log-probabilities)`` of a policy-loss type as the kernels take them: the two bounds
    (or temperatures, or thresholds), the dual-clip constant, and the log-probabilities its ratio is anchored on."""
    if name in ("regular", "dual_clip", "gspo"):
        dual = name == "dual_clip"
        return ({"regular": LOSS_REGULAR, "dual_clip": LOSS_DUAL_CLIP, "gspo": LOSS_GSPO}[name], float(config.eps_clip_low),
                float(config.eps_clip_high), float(getattr(config, "clip_ratio_c", 0.0)) if dual else 0.0, old_log_probs)
    if name in ("cross_entropy", "importance_sampling"):
        return (LOSS_CROSS_ENTROPY if name == "cross_entropy" else LOSS_IMPORTANCE_SAMPLING), 0.0, 0.0, 0.0, old_log_probs
    if name == "sapo":
        sapo = _get(config, "sapo")
        return LOSS_SAPO, float(_get(sapo, "tau_pos", 1.0)), float(_get(sapo, "tau_neg", 1.05)), 0.0, old_log_probs
    if name == "cispo":
        cispo = _get(config, "cispo")
        behaviour = old_log_probs
        if _get(cispo, "cispo_anchor", "old") == "rollout":
            assert rollout_logprobs is not None, "rollout_logprobs are required for cispo with cispo_anchor='rollout'"
            tis = _get(_get(config, "off_policy_correction"), "tis_ratio_type")
            if tis is not None:
                raise ValueError("cispo_anchor='rollout' is already rollout-anchored and performs the off-policy correction; "
                                 f"TIS (tis_ratio_type={tis!r}) would double-count it. Set "
                                 "off_policy_correction.tis_ratio_type=None.")
            behaviour = rollout_logprobs
        return (LOSS_CISPO, float(_get(cispo, "cispo_eps_clip_low", 1.0)), float(_get(cispo, "cispo_eps_clip_high", 4.0)), 0.0,
                behaviour)
    if name == "rollout_is":
        assert rollout_logprobs is not None, "rollout_logprobs are required for rollout_is"
        return LOSS_ROLLOUT_IS, float(config.eps_clip_low), float(config.eps_clip_high), 0.0, rollout_logprobs
    if name == "dppo":
        dppo = _get(config, "dppo")
        kind = _get(dppo, "dppo_type", "binary_tv")
        if kind not in ("binary_tv", "binary_kl"):
            raise ValueError(f"Unknown DPPO type: {kind}. Must be 'binary_tv' or 'binary_kl'.")
        return (LOSS_DPPO_TV if kind == "binary_tv" else LOSS_DPPO_KL, float(_get(dppo, "delta_low", 0.2)),
                float(_get(dppo, "delta_high", 0.2)), 0.0, rollout_logprobs if rollout_logprobs is not None else old_log_probs)
    raise NotImplementedError(f"policy_loss_type {name!r} is not part of the fused losses; fused types: "
                              f"{sorted(_POLICY_LOSS_NAMES)}")


_POLICY_LOSS_NAMES = ("regular", "dual_clip", "cross_entropy", "importance_sampling", "gspo", "sapo", "cispo", "rollout_is",
                      "dppo")


def _elementwise_loss(name: str, log_probs, old_log_probs, advantages, config, loss_mask, rollout_logprobs, loss_weight,
                      sync_metrics: bool, read_clip_ratio: bool = True):
    loss_type, a, b, c, behaviour = _type_parameters(config, name, rollout_logprobs, old_log_probs)
    loss_weight, extra = _with_off_policy_correction(config, old_log_probs, rollout_logprobs, loss_mask, loss_weight, sync_metrics)
    loss, sums = _PolicyLoss.apply(log_probs, behaviour, advantages, loss_mask, loss_weight, a, b, c, loss_type)
    if not read_clip_ratio:  # a loss whose clip statistic is a constant: no device value, no read-back
        return loss, dict(extra)
    clip_ratio = sums[1] / sums[2].clamp(min=1.0)
    return loss, {"clip_ratio": clip_ratio.item() if sync_metrics else clip_ratio, **extra}


def sapo_policy_loss(log_probs, old_log_probs, advantages, config, loss_mask=None, rollout_logprobs=None, *,
                     loss_weight=None, sync_metrics: bool = True) -> Tuple[torch.Tensor, Dict[str, Any]]:
    """Soft adaptive policy optimisation (reference ``sapo_policy_loss``, ppo_utils.py:590-660): the gate
    ``sigmoid(tau (r - 1)) 4 / tau`` replaces the clipped ratio, ``tau = config.sapo.tau_pos`` where the advantage is
    positive, ``tau_neg`` elsewhere.  ``clip_ratio`` is 0.0 as in the reference (a constant: nothing is read back for it);
    ``sync_metrics=False`` leaves the off-policy-correction metrics as 0-dim tensors, so that nothing waits for the device."""
    loss, metrics = _elementwise_loss("sapo", log_probs, old_log_probs, advantages, config, loss_mask, rollout_logprobs, loss_weight,
                                      sync_metrics, read_clip_ratio=False)
    metrics["clip_ratio"] = 0.0
    return loss, metrics


def compute_policy_loss_cispo(log_probs, old_log_probs, advantages, config, loss_mask=None, rollout_logprobs=None, *,
                              loss_weight=None, sync_metrics: bool = True) -> Tuple[torch.Tensor, Dict[str, Any]]:
    """Clipped importance-weight policy optimisation (reference ``compute_policy_loss_cispo``, ppo_utils.py:732-821):
    ``-A stopgrad(clamp(r, 1 - cispo_eps_clip_low, 1 + cispo_eps_clip_high)) log_probs`` with the ratio anchored as
    ``config.cispo.cispo_anchor`` says.  Returns ``clip_ratio`` and the reference's four ``cispo/ratio_*`` diagnostics
    (:790-815: masked means of the ratio and of the clamped ratio, extremes over the unmasked tokens), which are monitoring
    values outside the loss kernel; as floats, or as 0-dim tensors with ``sync_metrics=False`` (the extremes are then taken
    with the masked tokens neutralised instead of selected, so nothing waits for a count)."""
    loss, metrics = _elementwise_loss("cispo", log_probs, old_log_probs, advantages, config, loss_mask, rollout_logprobs,
                                      loss_weight, sync_metrics)
    _, lo, hi, _, behaviour = _type_parameters(config, "cispo", rollout_logprobs, old_log_probs)
    with torch.no_grad():
        ratio = torch.clamp(log_probs.detach().float() - behaviour.float(), -20.0, 20.0).exp()
        clamped = ratio.clamp(1.0 - lo, 1.0 + hi)
        if loss_mask is None:
            mean, cmean, rmax, rmin = ratio.mean(), clamped.mean(), ratio.max(), ratio.min()
        else:
            m = loss_mask.float()
            count = m.sum()
            denom = count.clamp(min=1.0)
            mean, cmean = (ratio * m).sum() / denom, (clamped * m).sum() / denom
            active = m > 0
            some = count > 0   # an empty mask: the extremes over all tokens, as the reference's else branch
            rmax = torch.where(some, torch.where(active, ratio, ratio.new_full((), -torch.inf)).max(), ratio.max())
            rmin = torch.where(some, torch.where(active, ratio, ratio.new_full((), torch.inf)).min(), ratio.min())
    extra = {"cispo/ratio_mean": mean, "cispo/ratio_clamped_mean": cmean, "cispo/ratio_max": rmax, "cispo/ratio_min": rmin}
    metrics.update({k: (v.item() if sync_metrics else v) for k, v in extra.items()})
    return loss, metrics


def compute_policy_loss_clip_cov(log_probs, old_log_probs, advantages, config, loss_mask=None, rollout_logprobs=None
                                 ) -> Tuple[torch.Tensor, Dict[str, Any]]:
    """Clip-Cov (reference ``compute_policy_loss_clip_cov``, ppo_utils.py:938-999): the clipped surrogate on the unclamped
    ratio, with the loss of a random subset of tokens removed -- tokens the clip did not catch whose covariance term
    ``(A - mean A)(logp - mean logp)`` lies inside ``(clip_cov_lb, clip_cov_ub)``, ``max(int(clip_ratio * sum mask), 1)`` of them,
    drawn with ``torch.randperm`` on the global CPU generator exactly as the reference draws them (same generator state, same
    tokens).  The selection is batch-level host logic there and here (it reads a count and a permutation back); value,
    gradient and sums then come from the fused kernel with the selection as its per-token weight.  ``loss_mask`` is required,
    as in the reference."""
    cc = _get(config, "clip_cov")
    ratio_frac, lb, ub = float(_get(cc, "clip_ratio")), float(_get(cc, "clip_cov_lb")), float(_get(cc, "clip_cov_ub"))
    eps_low, eps_high = float(config.eps_clip_low), float(config.eps_clip_high)
    with torch.no_grad():
        lp, old, adv, mask = log_probs.detach(), old_log_probs, advantages, loss_mask
        r = torch.exp(lp - old)
        pg1 = -adv * r
        pg2 = -adv * torch.clamp(r, 1 - eps_low, 1 + eps_high)
        clip_by_origin = (pg2 > pg1) & (mask > 0)
        denom = mask.sum().clamp(min=1.0)
        cov_all = (adv - (adv * mask).sum() / denom) * (lp - (lp * mask).sum() / denom)
        cov_all[mask == 0] = -torch.inf
        cov_all[clip_by_origin] = -torch.inf
        clip_num = max(int(ratio_frac * mask.sum().item()), 1)
        candidates = torch.nonzero((cov_all < ub) & (cov_all > lb) & (mask > 0))
        corr = torch.ones_like(adv, dtype=torch.float32)
        if len(candidates) > 0:
            perm = torch.randperm(len(candidates))
            chosen = candidates[perm[: min(clip_num, len(candidates))].to(candidates.device)]
            corr[tuple(chosen[:, k] for k in range(chosen.shape[1]))] = 0
        clip_frac = ((corr == 0).float() * mask).sum() / denom
    loss, _ = _PolicyLoss.apply(log_probs, old_log_probs, advantages, loss_mask, corr, eps_low, eps_high, 0.0, LOSS_CLIP_COV)
    return loss, {"clip_ratio": clip_frac.item()}


def compute_policy_loss_kl_cov(log_probs, old_log_probs, advantages, config, loss_mask=None, rollout_logprobs=None
                               ) -> Tuple[torch.Tensor, Dict[str, Any]]:
    """KL-Cov (reference ``compute_policy_loss_kl_cov``, ppo_utils.py:1002-1053): the importance-sampling surrogate, plus
    ``ppo_kl_coef * |logp - old|`` on the ``max(1, int(n * kl_cov_frac))`` unmasked tokens with the largest covariance term.
    The top-k is taken on the CPU from the unmasked values, as the reference takes it (:1027-1036), so that ties and rounding
    fall the same way; the selector then goes to the fused kernel, which returns value and gradient."""
    kc = _get(config, "kl_cov")
    frac, coef = float(_get(kc, "kl_cov_frac")), float(_get(kc, "ppo_kl_coef"))
    with torch.no_grad():
        valid = loss_mask > 0
        idx = torch.nonzero(valid.reshape(-1), as_tuple=True)[0]
        adv_v = advantages[valid].detach().reshape(-1).cpu()
        lp_v = log_probs[valid].detach().reshape(-1).cpu()
        selector = torch.zeros(advantages.numel(), dtype=torch.float32, device=log_probs.device)
        if len(adv_v) > 0:
            cov = (adv_v - adv_v.mean()) * (lp_v - lp_v.mean())
            k = max(1, int(len(cov) * frac))
            top = torch.topk(cov, min(k, len(cov)), largest=True).indices
            selector[idx[top.to(idx.device)]] = 1.0
    loss, _ = _PolicyLoss.apply(log_probs, old_log_probs, advantages, loss_mask, selector.reshape(advantages.shape), 0.0, 0.0, coef,
                                LOSS_KL_COV)
    return loss, {"clip_ratio": 0.0}   # not applicable to KL-Cov: the reference reports 0.0 (:1052)


def rollout_is_policy_loss(log_probs, old_log_probs, advantages, config, loss_mask=None, rollout_logprobs=None, *,
                           loss_weight=None, sync_metrics: bool = True) -> Tuple[torch.Tensor, Dict[str, Any]]:
    """Calibrated importance-weighted policy gradient on the rollout log-probabilities (reference
    ``rollout_is_policy_loss``, ppo_utils.py:824-863): the weight is the ratio inside the open interval
    ``(1 - eps_clip_low, 1 + eps_clip_high)`` and zero outside; ``old_log_probs`` is not read."""
    return _elementwise_loss("rollout_is", log_probs, old_log_probs, advantages, config, loss_mask, rollout_logprobs,
                             loss_weight, sync_metrics)


def dppo_policy_loss(log_probs, old_log_probs, advantages, config, loss_mask=None, rollout_logprobs=None, *,
                     loss_weight=None, sync_metrics: bool = True) -> Tuple[torch.Tensor, Dict[str, Any]]:
    """Divergence proximal policy optimisation (reference ``dppo_policy_loss``, ppo_utils.py:866-935): the unclipped
    surrogate times a binary trust-region mask (``config.dppo.dppo_type`` "binary_tv" or "binary_kl", thresholds
    ``delta_low`` / ``delta_high``); the rollout log-probabilities are the behaviour policy when given."""
    return _elementwise_loss("dppo", log_probs, old_log_probs, advantages, config, loss_mask, rollout_logprobs, loss_weight,
                             sync_metrics)


def gspo_policy_loss(log_probs, old_log_probs, advantages, config, loss_mask=None, rollout_logprobs=None, *,
                     loss_weight=None, sync_metrics: bool = True) -> Tuple[torch.Tensor, Dict[str, Any]]:
    """Group sequence policy optimisation, token-level variant (reference ``gspo_policy_loss``, ppo_utils.py:663-729): the
    clipped surrogate with every token's ratio replaced by its sequence's, ``exp(min(masked row mean of the log-ratio,
    10))``.  ``log_probs`` is ``[B, S]``; the rows are the sequences."""
    if log_probs.dim() < 2:
        raise ValueError("gspo_policy_loss needs [B, S] inputs: the importance weight is a row mean")
    loss_weight, extra = _with_off_policy_correction(config, old_log_probs, rollout_logprobs, loss_mask, loss_weight, sync_metrics)
    scalars = (LOSS_GSPO, float(config.eps_clip_low), float(config.eps_clip_high), 0.0, 3, 1.0, 1.0, 0.0, 0.0)
    loss, out6 = _ActorLoss.apply(log_probs, None, (old_log_probs, advantages, loss_mask, loss_weight, None), scalars)
    clip_ratio = out6[2] / out6[3].clamp(min=1.0)
    return loss, {"clip_ratio": clip_ratio.item() if sync_metrics else clip_ratio, **extra}


# ----------------------------------------------------------------------------------------------------------------------
# approximate KL and masked mean
# ----------------------------------------------------------------------------------------------------------------------
def _rows_cols(t: torch.Tensor) -> Tuple[int, int]:
    if t.dim() == 0:
        return 1, 1
    cols = t.shape[-1]
    return (t.numel() // cols if cols else 0), cols


def _same_f32(name: str, t: Optional[torch.Tensor], like: torch.Tensor) -> Optional[torch.Tensor]:
    if t is None:
        return None
    if t.shape != like.shape:
        raise ValueError(f"{name} has shape {tuple(t.shape)}, expected {tuple(like.shape)}")
    return t.detach().to(torch.float32).contiguous()


@torch.library.custom_op("skyrl_amd::approx_kl", mutates_args=())
def _approx_kl(log_probs: torch.Tensor, log_probs_base: torch.Tensor, loss_mask: Optional[torch.Tensor], estimator: int,
               grad_mode: int) -> Tuple[torch.Tensor, torch.Tensor, torch.Tensor, torch.Tensor]:
    """``(kld, row_mean, mean, grad)`` for contiguous fp32 ``[rows, cols]`` inputs; grad_mode 1: elementwise derivative of
    kld, 2: derivative of ``mean``; 0: grad is empty."""
    dev = _require_device(log_probs, log_probs_base)
    rows, cols = log_probs.shape
    kld = torch.empty_like(log_probs)
    row_mean = torch.empty(rows, dtype=torch.float32, device=dev)
    mean = torch.empty((), dtype=torch.float32, device=dev)
    grad = torch.empty_like(log_probs) if grad_mode else torch.empty(0, dtype=torch.float32, device=dev)
    with torch.cuda.device(dev):
        st = _lib.load().skyrl_approx_kl(
            log_probs.data_ptr(), log_probs_base.data_ptr(), None if loss_mask is None else loss_mask.data_ptr(), rows, cols,
            int(estimator), kld.data_ptr(), row_mean.data_ptr(), mean.data_ptr(), int(grad_mode),
            grad.data_ptr() if grad_mode else None, torch.cuda.current_stream(dev).cuda_stream)
    _lib.check(st, "skyrl_approx_kl")
    return kld, row_mean, mean, grad


@_approx_kl.register_fake
def _(log_probs, log_probs_base, loss_mask, estimator, grad_mode):
    rows = log_probs.shape[0]
    return (torch.empty_like(log_probs), log_probs.new_empty(rows), log_probs.new_empty(()),
            torch.empty_like(log_probs) if grad_mode else log_probs.new_empty(0))


def _kl_operands(log_probs, log_probs_base, loss_mask, kl_estimator_type):
    if kl_estimator_type not in KL_ESTIMATORS:
        raise ValueError(f"Invalid KL estimator type: {kl_estimator_type}")
    rows, cols = _rows_cols(log_probs)
    lp = log_probs.detach().to(torch.float32).contiguous().reshape(rows, cols)
    base = _same_f32("log_probs_base", log_probs_base, log_probs).reshape(rows, cols)
    mask = _same_f32("loss_mask", loss_mask, log_probs)
    return lp, base, None if mask is None else mask.reshape(rows, cols), KL_ESTIMATORS[kl_estimator_type]


class _ApproxKL(torch.autograd.Function):
    """grad_mode 1: returns the per-token estimate; grad_mode 2: returns the trainer's scalar reduction of it."""

    @staticmethod
    def forward(ctx, log_probs, log_probs_base, loss_mask, kl_estimator_type, grad_mode):
        lp, base, mask, est = _kl_operands(log_probs, log_probs_base, loss_mask, kl_estimator_type)
        kld, _, mean, grad = _approx_kl(lp, base, mask, est, grad_mode)
        ctx.save_for_backward(grad)
        ctx.shape, ctx.dtype = log_probs.shape, log_probs.dtype
        return kld.reshape(log_probs.shape) if grad_mode == 1 else mean

    @staticmethod
    def backward(ctx, grad_out):
        (grad,) = ctx.saved_tensors
        d = grad.reshape(ctx.shape) * grad_out  # only the dependence on log_probs is tracked, as the trainer needs it
        return d.to(ctx.dtype), None, None, None, None


def compute_approx_kl(
    log_probs: torch.Tensor,
    log_probs_base: torch.Tensor,
    loss_mask: Optional[torch.Tensor] = None,
    kl_estimator_type: str = "k3",
) -> torch.Tensor:
    """Per-token KL estimate, same contract as the reference's ``compute_approx_kl`` (ppo_utils.py:88-126): estimators
    ``k1``, ``abs``, ``k2``, ``k3``; masked positions are exactly 0.  fp32 result of the shape of ``log_probs``;
    differentiable with respect to ``log_probs`` (the base policy's log-probabilities are treated as constants)."""
    if kl_estimator_type not in KL_ESTIMATORS:
        raise ValueError(f"Invalid KL estimator type: {kl_estimator_type}")
    if log_probs.numel() == 0:  # nothing to launch: the empty estimate, attached to log_probs as any other
        return (log_probs - log_probs_base.detach()).to(torch.float32)
    return _ApproxKL.apply(log_probs, log_probs_base, loss_mask, kl_estimator_type, 1)


def approx_kl_loss(
    log_probs: torch.Tensor,
    log_probs_base: torch.Tensor,
    loss_mask: Optional[torch.Tensor] = None,
    kl_estimator_type: str = "k3",
) -> torch.Tensor:
    """``masked_mean(compute_approx_kl(...), loss_mask, dim=-1).mean()`` -- the KL loss term of the trainer
    (workers/worker.py:1071-1077) -- from one kernel, with its gradient with respect to ``log_probs``."""
    if log_probs.numel() == 0:  # nothing to launch: the reference's expression on the empty estimate (no rows: NaN; no columns: 0)
        kld = compute_approx_kl(log_probs, log_probs_base, loss_mask, kl_estimator_type)
        return masked_mean(kld, loss_mask, dim=-1).mean()
    return _ApproxKL.apply(log_probs, log_probs_base, loss_mask, kl_estimator_type, 2)


@torch.library.custom_op("skyrl_amd::masked_mean", mutates_args=())
def _masked_mean(values: torch.Tensor, mask: Optional[torch.Tensor], want_grad: bool) -> Tuple[torch.Tensor, torch.Tensor]:
    """``(means [rows], dvalues [rows, cols] or empty)`` for contiguous fp32 ``[rows, cols]`` inputs."""
    dev = _require_device(values)
    rows, cols = values.shape
    means = torch.empty(rows, dtype=torch.float32, device=dev)
    dv = torch.empty_like(values) if want_grad else torch.empty(0, dtype=torch.float32, device=dev)
    with torch.cuda.device(dev):
        st = _lib.load().skyrl_masked_mean(values.data_ptr(), None if mask is None else mask.data_ptr(), rows, cols,
                                           means.data_ptr(), dv.data_ptr() if want_grad else None,
                                           torch.cuda.current_stream(dev).cuda_stream)
    _lib.check(st, "skyrl_masked_mean")
    return means, dv


@_masked_mean.register_fake
def _(values, mask, want_grad):
    return values.new_empty(values.shape[0]), torch.empty_like(values) if want_grad else values.new_empty(0)


class _MaskedMean(torch.autograd.Function):
    @staticmethod
    def forward(ctx, tensor, mask, rows, cols, out_shape):
        v = tensor.detach().to(torch.float32).contiguous().reshape(rows, cols)
        m = None if mask is None else mask.detach().to(torch.float32).expand_as(tensor).contiguous().reshape(rows, cols)
        means, dv = _masked_mean(v, m, bool(ctx.needs_input_grad[0]))
        ctx.save_for_backward(dv)
        ctx.shape, ctx.dtype, ctx.rows = tensor.shape, tensor.dtype, rows
        return means.reshape(out_shape)

    @staticmethod
    def backward(ctx, grad_out):
        (dv,) = ctx.saved_tensors
        d = dv * grad_out.reshape(ctx.rows, 1).to(torch.float32)
        return d.reshape(ctx.shape).to(ctx.dtype), None, None, None, None


def masked_mean(tensor: torch.Tensor, mask: Optional[torch.Tensor], dim: Optional[int] = None) -> torch.Tensor:
    """``(tensor * mask).sum(dim) / mask.sum(dim).clamp(min=1)``; ``mask=None``: the plain mean (reference ``masked_mean``,
    torch_utils.py:180-184).  ``dim`` is ``None`` (everything) or the last dimension; fp32 result; differentiable with respect
    to ``tensor``."""
    if tensor.numel() == 0:  # nothing to launch: the reference's expression itself, which is shape arithmetic on an empty tensor
        t = tensor.to(torch.float32)
        if mask is None:
            return t.mean() if dim is None else t.mean(dim=dim)
        m = mask.to(torch.float32)
        if dim is None:
            return (t * m).sum() / m.sum().clamp(min=1.0)
        return (t * m).sum(dim=dim) / m.sum(dim=dim).clamp(min=1.0)
    if dim is None:
        return _MaskedMean.apply(tensor, mask, 1, tensor.numel(), ())
    if dim not in (-1, tensor.dim() - 1):
        raise NotImplementedError("masked_mean reduces everything (dim=None) or the last dimension")
    rows, cols = _rows_cols(tensor)
    return _MaskedMean.apply(tensor, mask, rows, cols, tensor.shape[:-1])


# ----------------------------------------------------------------------------------------------------------------------
# the assembled actor loss
# ----------------------------------------------------------------------------------------------------------------------
@torch.library.custom_op("skyrl_amd::actor_loss", mutates_args=())
def _actor_loss(log_probs: torch.Tensor, old_log_probs: Optional[torch.Tensor], advantages: Optional[torch.Tensor],
                loss_mask: Optional[torch.Tensor], loss_weight: Optional[torch.Tensor], base_log_probs: Optional[torch.Tensor],
                entropy: Optional[torch.Tensor], loss_type: int, eps_clip_low: float, eps_clip_high: float, clip_ratio_c: float,
                kl_estimator: int, policy_scale: float, term_scale: float, kl_coef: float, entropy_coef: float,
                ) -> Tuple[torch.Tensor, torch.Tensor, torch.Tensor]:
    """``(out6, dlogprobs, dentropy)`` for contiguous fp32 ``[rows, cols]`` inputs; ``dentropy`` is empty without ``entropy``."""
    dev = _require_device(log_probs)
    rows, cols = log_probs.shape
    for name, t in (("old_log_probs", old_log_probs), ("advantages", advantages), ("loss_mask", loss_mask),
                    ("loss_weight", loss_weight), ("base_log_probs", base_log_probs), ("entropy", entropy)):
        if t is not None and (t.dtype != torch.float32 or t.shape != log_probs.shape or not t.is_contiguous()):
            raise ValueError(f"{name} must be a contiguous fp32 tensor of shape {tuple(log_probs.shape)}")
    out6 = torch.empty(6, dtype=torch.float32, device=dev)
    row_sums = torch.empty((rows, 6), dtype=torch.float32, device=dev)
    dlp = torch.empty_like(log_probs)
    dent = torch.empty_like(log_probs) if entropy is not None else torch.empty(0, dtype=torch.float32, device=dev)
    ptr = lambda t: None if t is None else t.data_ptr()  # noqa: E731
    with torch.cuda.device(dev):
        st = _lib.load().skyrl_actor_loss(
            log_probs.data_ptr(), ptr(old_log_probs), ptr(advantages), ptr(loss_mask), ptr(loss_weight), ptr(base_log_probs),
            ptr(entropy), rows, cols, int(loss_type), float(eps_clip_low), float(eps_clip_high), float(clip_ratio_c),
            int(kl_estimator), float(policy_scale), float(term_scale), float(kl_coef), float(entropy_coef), row_sums.data_ptr(),
            out6.data_ptr(), dlp.data_ptr(), dent.data_ptr() if entropy is not None else None,
            torch.cuda.current_stream(dev).cuda_stream)
    _lib.check(st, "skyrl_actor_loss")
    return out6, dlp, dent


@_actor_loss.register_fake
def _(log_probs, old_log_probs, advantages, loss_mask, loss_weight, base_log_probs, entropy, loss_type, eps_clip_low,
      eps_clip_high, clip_ratio_c, kl_estimator, policy_scale, term_scale, kl_coef, entropy_coef):
    return (log_probs.new_empty(6), torch.empty_like(log_probs),
            torch.empty_like(log_probs) if entropy is not None else log_probs.new_empty(0))


class _ActorLoss(torch.autograd.Function):
    @staticmethod
    def forward(ctx, log_probs, entropy, consts, scalars):
        old, adv, mask, weight, base = consts
        rows, cols = _rows_cols(log_probs)
        flat = lambda t: None if t is None else t.detach().to(torch.float32).contiguous().reshape(rows, cols)  # noqa: E731
        for name, t in (("old_log_probs", old), ("advantages", adv), ("loss_mask", mask), ("loss_weight", weight),
                        ("base_log_probs", base), ("entropy", entropy)):
            if t is not None and t.shape != log_probs.shape:
                raise ValueError(f"{name} has shape {tuple(t.shape)}, expected {tuple(log_probs.shape)}")
        out6, dlp, dent = _actor_loss(flat(log_probs), flat(old), flat(adv), flat(mask), flat(weight), flat(base), flat(entropy),
                                      *scalars)
        ctx.save_for_backward(dlp, dent)
        ctx.lp_meta = (log_probs.shape, log_probs.dtype)
        ctx.ent_meta = None if entropy is None else (entropy.shape, entropy.dtype)
        ctx.mark_non_differentiable(out6)
        return out6[0].clone(), out6

    @staticmethod
    def backward(ctx, grad_loss, _grad_out6):
        dlp, dent = ctx.saved_tensors
        shape, dtype = ctx.lp_meta
        g_lp = (dlp * grad_loss).reshape(shape).to(dtype)
        g_ent = None
        if ctx.ent_meta is not None:
            g_ent = (dent * grad_loss).reshape(ctx.ent_meta[0]).to(ctx.ent_meta[1])
        return g_lp, g_ent, None, None


def actor_loss(
    log_probs: torch.Tensor,
    old_log_probs: Optional[torch.Tensor],
    advantages: Optional[torch.Tensor],
    config: Any,
    loss_mask: Optional[torch.Tensor] = None,
    *,
    base_log_probs: Optional[torch.Tensor] = None,
    entropy: Optional[torch.Tensor] = None,
    loss_weight: Optional[torch.Tensor] = None,
    rollout_logprobs: Optional[torch.Tensor] = None,
    policy_scale: float = 1.0,
    term_scale: float = 1.0,
) -> Tuple[torch.Tensor, Dict[str, torch.Tensor]]:
    """The loss the policy worker back-propagates for one micro-batch, assembled in two kernel launches (three when the entropy takes a gradient) together with
    both upstream gradients of the fused LM head (reference: workers/worker.py:989-1089):

        ``policy_loss * policy_scale + (kl_loss * config.kl_loss_coef - entropy * config.entropy_loss_coef) * term_scale``

    ``config`` is the algorithm config: ``policy_loss_type`` (regular, dual_clip, cross_entropy, importance_sampling, gspo,
    sapo, cispo, rollout_is, dppo) with that type's parameters (``eps_clip_low`` / ``eps_clip_high`` / ``clip_ratio_c``,
    ``sapo``, ``cispo``, ``dppo``), ``use_kl_loss`` + ``kl_loss_coef`` + ``kl_estimator_type``, ``use_entropy_loss`` +
    ``entropy_loss_coef``.  ``rollout_logprobs`` are read by the types anchored on them.  The KL term needs ``base_log_probs``; the entropy term needs ``entropy``
    (``[B, S]``, e.g. from ``action_log_probs_from_hidden(..., compute_entropy=True)``) and sends a gradient into it.
    ``policy_scale`` is the worker's ``grad_sum_correction_factor``, ``term_scale`` its ``microbatch_weight``.

    Returns the loss and a dict of 0-dim tensors (no host synchronisation): ``policy_loss``, ``policy_kl``, ``policy_entropy``
    and ``clip_ratio`` (``importance_ratio`` for the importance-sampling loss).
    """
    name = getattr(config, "policy_loss_type", "regular")
    if log_probs.numel() == 0:
        raise ValueError(f"actor_loss needs at least one token, got log_probs of shape {tuple(log_probs.shape)}: the mean over "
                         "the rows of an empty micro-batch is undefined (the reference's KL and entropy terms are NaN there)")
    loss_type, a, b, c, behaviour = _type_parameters(config, name, rollout_logprobs, old_log_probs)
    extra: Dict[str, Any] = {}
    if name not in ("cross_entropy", "importance_sampling"):   # the two losses the reference never corrects (:1056-1142)
        loss_weight, extra = _with_off_policy_correction(config, old_log_probs, rollout_logprobs, loss_mask, loss_weight, False)
    use_kl = bool(getattr(config, "use_kl_loss", False))
    if use_kl and base_log_probs is None:
        raise ValueError("use_kl_loss needs base_log_probs")
    use_ent = bool(getattr(config, "use_entropy_loss", False))
    if use_ent and entropy is None:
        raise ValueError("use_entropy_loss needs the per-token entropy")
    estimator = getattr(config, "kl_estimator_type", "k3")
    if use_kl and estimator not in KL_ESTIMATORS:
        raise ValueError(f"Invalid KL estimator type: {estimator}")
    scalars = (loss_type, a, b, c, KL_ESTIMATORS.get(estimator, 3), float(policy_scale), float(term_scale),
               float(config.kl_loss_coef) if use_kl else 0.0, float(config.entropy_loss_coef) if use_ent else 0.0)
    consts = (behaviour, advantages, loss_mask, loss_weight, base_log_probs if use_kl else None)
    # The entropy is reduced for the metric even when it is not part of the loss, as the worker does.
    loss, out6 = _ActorLoss.apply(log_probs, entropy, consts, scalars)
    stat = out6[2] / (out6[3] if loss_type == LOSS_IMPORTANCE_SAMPLING else out6[3].clamp(min=1.0))
    metrics = {"policy_loss": out6[1], "policy_kl": out6[4], "policy_entropy": out6[5],
               ("importance_ratio" if loss_type == LOSS_IMPORTANCE_SAMPLING else "clip_ratio"): stat, **extra}
    return loss, metrics


# The names under which the reference registers its policy losses (``PolicyLossRegistry.repopulate_registry``,
# ppo_utils.py:497-515), each with the function of this module that has the same signature:
# ``PolicyLossRegistry.register(name, POLICY_LOSS_FUNCTIONS[name])`` puts the fused loss in the reference's place.
POLICY_LOSS_FUNCTIONS = {
    "regular": ppo_policy_loss,
    "dual_clip": ppo_policy_loss,
    "gspo": gspo_policy_loss,
    "cispo": compute_policy_loss_cispo,
    "clip_cov": compute_policy_loss_clip_cov,
    "kl_cov": compute_policy_loss_kl_cov,
    "sapo": sapo_policy_loss,
    "cross_entropy": cross_entropy_loss,
    "importance_sampling": importance_sampling_loss,
    "dppo": dppo_policy_loss,
    "rollout_is": rollout_is_policy_loss,
}


def get_policy_loss(name: str):
    """The fused loss registered under ``name`` in the reference (``PolicyLossRegistry.get``, ppo_utils.py:444-452)."""
    if name not in POLICY_LOSS_FUNCTIONS:
        raise ValueError(f"Unknown policy loss '{name}'. Available: {sorted(POLICY_LOSS_FUNCTIONS)}")
    return POLICY_LOSS_FUNCTIONS[name]
