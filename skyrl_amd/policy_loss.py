"""PPO policy loss on the fused path's log-probabilities: loss, clip statistics and d loss / d log-probs in one HIP kernel.

Mirrors ``ppo_policy_loss`` of the reference (skyrl/backends/skyrl_train/utils/ppo_utils.py:555-588; policy loss types
"regular" and "dual_clip"): the same positional arguments, the same ``(loss, {"clip_ratio": ...})`` result, the loss reduced
as ``reduce_loss`` does (masked sum, ppo_utils.py:1145-1149; the reference folds the kind of mean into the advantages
beforehand, ppo_utils.py:1152-1181).  The reference computes it with about fifteen elementwise torch kernels and lets
autograd derive the gradient; here one kernel produces the loss sum, the clip counts and the gradient, so the upstream
gradient of ``skyrl_lmhead_bwd`` is ready without another pass over the ``[B, S]`` tensors and, with
``sync_metrics=False``, without a host synchronisation.

Off-policy correction (``apply_off_policy_correction``, off_policy_correction_utils.py:351-385) multiplies the per-token
loss by an importance ratio that does not depend on the policy's log-probabilities: pass that ratio as ``loss_weight``.
Computing it from ``rollout_logprobs`` is outside this module, so ``rollout_logprobs`` must be ``None``.
"""

from __future__ import annotations

from typing import Any, Dict, Optional, Tuple

import torch

from . import _lib
from .ops import _require_device

__all__ = ["ppo_policy_loss", "ppo_policy_loss_terms"]


def _flat_f32(name: str, t: Optional[torch.Tensor], numel: int) -> Optional[torch.Tensor]:
    if t is None:
        return None
    if t.numel() != numel:
        raise ValueError(f"{name} has {t.numel()} elements, log_probs has {numel}")
    return t.detach().reshape(-1).to(torch.float32).contiguous()


@torch.library.custom_op("skyrl_amd::ppo_policy_loss", mutates_args=())
def ppo_policy_loss_terms(
    log_probs: torch.Tensor,
    old_log_probs: torch.Tensor,
    advantages: torch.Tensor,
    loss_mask: Optional[torch.Tensor],
    loss_weight: Optional[torch.Tensor],
    eps_clip_low: float,
    eps_clip_high: float,
    clip_ratio_c: float,
    dual_clip: bool,
) -> Tuple[torch.Tensor, torch.Tensor]:
    """``(sums, grad)``: sums = [sum loss*mask*weight, sum clipped*mask, sum mask] (fp32 [3]); grad = d sums[0] / d log_probs
    (fp32, flat).  All inputs are flat contiguous fp32 tensors of one length."""
    dev = _require_device(log_probs, old_log_probs, advantages)
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
    ptr = lambda t: None if t is None else t.data_ptr()  # noqa: E731
    with torch.cuda.device(dev):
        st = _lib.load().skyrl_ppo_policy_loss(
            log_probs.data_ptr(), old_log_probs.data_ptr(), advantages.data_ptr(), ptr(loss_mask), ptr(loss_weight), n,
            float(eps_clip_low), float(eps_clip_high), float(clip_ratio_c), int(bool(dual_clip)), sums.data_ptr(),
            grad.data_ptr(), torch.cuda.current_stream(dev).cuda_stream)
    _lib.check(st, "skyrl_ppo_policy_loss")
    return sums, grad


@ppo_policy_loss_terms.register_fake
def _(log_probs, old_log_probs, advantages, loss_mask, loss_weight, eps_clip_low, eps_clip_high, clip_ratio_c, dual_clip):
    return log_probs.new_empty(3, dtype=torch.float32), log_probs.new_empty(log_probs.numel(), dtype=torch.float32)


class _PolicyLoss(torch.autograd.Function):
    @staticmethod
    def forward(ctx, log_probs, old_log_probs, advantages, loss_mask, loss_weight, eps_low, eps_high, clip_c, dual):
        n = log_probs.numel()
        sums, grad = ppo_policy_loss_terms(
            _flat_f32("log_probs", log_probs, n), _flat_f32("old_log_probs", old_log_probs, n),
            _flat_f32("advantages", advantages, n), _flat_f32("loss_mask", loss_mask, n),
            _flat_f32("loss_weight", loss_weight, n), eps_low, eps_high, clip_c, dual)
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
    if rollout_logprobs is not None:
        raise NotImplementedError(
            "off-policy correction from rollout_logprobs is not part of the fused loss; compute the importance ratio with "
            "the trainer's own helper and pass it as loss_weight")
    dual = loss_type == "dual_clip"
    loss, sums = _PolicyLoss.apply(log_probs, old_log_probs, advantages, loss_mask, loss_weight, float(config.eps_clip_low),
                                   float(config.eps_clip_high), float(getattr(config, "clip_ratio_c", 0.0)) if dual else 0.0,
                                   dual)
    clip_ratio = sums[1] / sums[2].clamp(min=1.0)
    return loss, {"clip_ratio": clip_ratio.item() if sync_metrics else clip_ratio}
