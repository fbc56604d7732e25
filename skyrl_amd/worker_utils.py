"""Per-micro-batch drift statistics between the train step's and the rollout engine's log-probabilities, in two launches.

Same name, arguments, keys and values as ``compute_minibatch_rollout_logprob_diff_metrics`` of
``skyrl/backends/skyrl_train/workers/worker_utils.py`` (:26-58), which both trainers call after every micro-batch's loss
(``workers/worker.py:1124-1126``, ``megatron_model_wrapper.py:982-984``).  The reference runs nine elementwise and reduction
kernels and four ``.item()`` read-backs; here one sweep gathers all four statistics, and with ``sync_metrics=False`` they stay
0-dim tensors (no host synchronisation).
"""

from __future__ import annotations

from typing import Any, Dict, Optional

import torch

from . import _lib
from .ops import _require_device

__all__ = ["compute_minibatch_rollout_logprob_diff_metrics", "logprob_diff_terms", "MINIBATCH_ROLLOUT_LOGPROB_DIFF_PREFIX",
           "MINIBATCH_ROLLOUT_LOGPROB_DIFF_MEAN_KEY", "MINIBATCH_ROLLOUT_LOGPROB_DIFF_SQ_MEAN_KEY",
           "MINIBATCH_ROLLOUT_LOGPROB_DIFF_MAX_KEY", "MINIBATCH_ROLLOUT_LOGPROB_DIFF_MIN_KEY"]

MINIBATCH_ROLLOUT_LOGPROB_DIFF_PREFIX = "minibatch_rollout_logprobs_abs_diff"
MINIBATCH_ROLLOUT_LOGPROB_DIFF_MEAN_KEY = f"{MINIBATCH_ROLLOUT_LOGPROB_DIFF_PREFIX}_mean"
MINIBATCH_ROLLOUT_LOGPROB_DIFF_SQ_MEAN_KEY = f"{MINIBATCH_ROLLOUT_LOGPROB_DIFF_PREFIX}_sq_mean"
MINIBATCH_ROLLOUT_LOGPROB_DIFF_MAX_KEY = f"{MINIBATCH_ROLLOUT_LOGPROB_DIFF_PREFIX}_max"
MINIBATCH_ROLLOUT_LOGPROB_DIFF_MIN_KEY = f"{MINIBATCH_ROLLOUT_LOGPROB_DIFF_PREFIX}_min"

_PARTIALS = 5 * 256   # 5 * SKYRL_POLICY_LOSS_PARTIALS of the header


@torch.library.custom_op("skyrl_amd::logprob_diff_metrics", mutates_args=())
def logprob_diff_terms(log_probs: torch.Tensor, rollout_logprobs: torch.Tensor, loss_mask: Optional[torch.Tensor]) -> torch.Tensor:
    """``[mean, mean of squares, max, min]`` of ``|log_probs - rollout_logprobs|`` over the masked tokens, fp32 ``[4]``, for
    contiguous fp32 inputs of one shape."""
    dev = _require_device(log_probs, rollout_logprobs)
    for name, t in (("log_probs", log_probs), ("rollout_logprobs", rollout_logprobs), ("loss_mask", loss_mask)):
        if t is not None and (t.dtype != torch.float32 or t.shape != log_probs.shape or not t.is_contiguous()):
            raise ValueError(f"{name} must be a contiguous fp32 tensor of shape {tuple(log_probs.shape)}, got {t.dtype} {tuple(t.shape)}")
    if log_probs.numel() == 0:
        raise ValueError("the statistics of an empty micro-batch are undefined (Tensor.max() raises as well)")
    out = torch.empty(4, dtype=torch.float32, device=dev)
    partials = torch.empty(_PARTIALS, dtype=torch.float32, device=dev)
    with torch.cuda.device(dev):
        st = _lib.load().skyrl_logprob_diff_metrics(
            log_probs.data_ptr(), rollout_logprobs.data_ptr(), None if loss_mask is None else loss_mask.data_ptr(), log_probs.numel(),
            out.data_ptr(), partials.data_ptr(), torch.cuda.current_stream(dev).cuda_stream)
    _lib.check(st, "skyrl_logprob_diff_metrics")
    return out


@logprob_diff_terms.register_fake
def _(log_probs, rollout_logprobs, loss_mask):
    return log_probs.new_empty(4, dtype=torch.float32)


def compute_minibatch_rollout_logprob_diff_metrics(action_log_probs: torch.Tensor, rollout_logprobs: Optional[torch.Tensor],
                                                   loss_mask: Optional[torch.Tensor], *, sync_metrics: bool = True
                                                   ) -> Dict[str, Any]:
    """Reference ``compute_minibatch_rollout_logprob_diff_metrics`` (:34-58): ``{}`` without rollout log-probabilities, else the
    four ``minibatch_rollout_logprobs_abs_diff_*`` statistics (floats; 0-dim tensors with ``sync_metrics=False``)."""
    if rollout_logprobs is None:
        return {}
    flat = lambda t: None if t is None else t.detach().to(torch.float32).expand(action_log_probs.shape).contiguous()  # noqa: E731
    out = logprob_diff_terms(flat(action_log_probs), flat(rollout_logprobs), flat(loss_mask))
    values = out.tolist() if sync_metrics else out.unbind(0)   # one read-back for the four
    return dict(zip((MINIBATCH_ROLLOUT_LOGPROB_DIFF_MEAN_KEY, MINIBATCH_ROLLOUT_LOGPROB_DIFF_SQ_MEAN_KEY,
                     MINIBATCH_ROLLOUT_LOGPROB_DIFF_MAX_KEY, MINIBATCH_ROLLOUT_LOGPROB_DIFF_MIN_KEY), values))
