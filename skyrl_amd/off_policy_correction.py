"""Off-policy correction from the rollout engine's log-probabilities, fused into two kernel launches.

Same names, arguments and results as ``skyrl/backends/skyrl_train/utils/off_policy_correction_utils.py``:

* ``off_policy_correction_enabled(off_policy_correction)`` (:9-21);
* ``compute_off_policy_correction(old_log_probs, rollout_logprobs, loss_mask, off_policy_correction)`` ->
  ``(tis_ratio | None, metrics, loss_mask)`` (:257-348): the truncated importance weight (``"token"``: ``[B, S]``, ``"sequence"``:
  ``[B, 1]``), the metrics of every switched-on step under the reference's names, and the thinned loss mask;
* ``apply_off_policy_correction(loss, old_log_probs, rollout_logprobs, loss_mask, off_policy_correction)`` ->
  ``(loss, loss_mask, metrics)`` (:351-391) for a per-token loss tensor.

The reference runs four helper functions of a dozen elementwise kernels each, with a ``.item()`` per metric; here one row
kernel does all steps in their order and a one-workgroup kernel adds the rows' statistics, and with ``sync_metrics=False`` the
metrics stay 0-dim tensors (no host synchronisation).  The correction reads ``old_log_probs`` and ``rollout_logprobs`` only and
carries no gradient.  The fused policy losses of ``skyrl_amd.policy_loss`` call ``correction_weight`` themselves when the
config switches a correction on and ``rollout_logprobs`` are given, as the reference's losses call ``apply_off_policy_correction``.
"""

from __future__ import annotations

import ctypes
from typing import Any, Dict, Optional, Tuple

import torch

from . import _lib
from .ops import _require_device

__all__ = ["off_policy_correction_enabled", "compute_off_policy_correction", "apply_off_policy_correction", "correction_weight",
           "off_policy_correction_terms"]

_ROW_STATS, _METRICS = 20, 16   # SKYRL_OFF_POLICY_ROW_STATS, SKYRL_OFF_POLICY_METRICS of the header
_TIS = {None: 0, "token": 1, "sequence": 2}
_SEQ = {None: 0, "geometric": 1, "product": 2}


def _get(obj: Any, name: str, default: Any = None) -> Any:
    if obj is None:
        return default
    if isinstance(obj, dict):
        return obj.get(name, default)
    return getattr(obj, name, default)


def off_policy_correction_enabled(off_policy_correction: Any) -> bool:
    """Whether any off-policy correction (TIS, sequence / outlier / token masking) is active (reference :9-21)."""
    c = off_policy_correction
    return (_get(c, "tis_ratio_type") is not None or _get(c, "sequence_mask_metric") is not None
            or _get(c, "outlier_token_is_threshold_low") is not None or _get(c, "outlier_token_is_threshold_high") is not None
            or (_get(c, "token_mask_is_threshold_low") is not None and _get(c, "token_mask_is_threshold_high") is not None))


@torch.library.custom_op("skyrl_amd::off_policy_correction", mutates_args=())
def off_policy_correction_terms(old_log_probs: torch.Tensor, rollout_logprobs: torch.Tensor, loss_mask: Optional[torch.Tensor],
                                tis_type: int, tis_cap: float, seq_metric: int, seq_low: float, seq_high: float,
                                outlier_low: Optional[float], outlier_high: Optional[float], token_low: Optional[float],
                                token_high: Optional[float]) -> Tuple[torch.Tensor, torch.Tensor, torch.Tensor, torch.Tensor]:
    """``(keep, tis, weight, metrics)`` for contiguous fp32 ``[rows, cols]`` inputs: ``keep`` in {0, 1}, ``tis`` the truncated
    importance weight (a row's value repeated for the sequence type, ones without TIS), ``weight = tis * keep``, ``metrics``
    the sixteen floats the header lists."""
    dev = _require_device(old_log_probs, rollout_logprobs)
    if old_log_probs.dim() != 2:
        raise ValueError(f"expected [rows, cols] inputs, got {tuple(old_log_probs.shape)}")
    rows, cols = old_log_probs.shape
    for name, t in (("old_log_probs", old_log_probs), ("rollout_logprobs", rollout_logprobs), ("loss_mask", loss_mask)):
        if t is not None and (t.dtype != torch.float32 or t.shape != (rows, cols) or not t.is_contiguous()):
            raise ValueError(f"{name} must be a contiguous fp32 [{rows}, {cols}] tensor, got {t.dtype} {tuple(t.shape)}")
    keep, tis, weight = (torch.empty((rows, cols), dtype=torch.float32, device=dev) for _ in range(3))
    metrics = torch.zeros(_METRICS, dtype=torch.float32, device=dev)
    if rows == 0 or cols == 0:
        return keep, tis, weight, metrics
    row_stats = torch.empty(rows * _ROW_STATS, dtype=torch.float32, device=dev)
    ref = lambda v: None if v is None else ctypes.byref(ctypes.c_float(float(v)))  # noqa: E731
    with torch.cuda.device(dev):
        st = _lib.load().skyrl_off_policy_correction(
            old_log_probs.data_ptr(), rollout_logprobs.data_ptr(), None if loss_mask is None else loss_mask.data_ptr(), rows, cols,
            int(tis_type), float(tis_cap), int(seq_metric), float(seq_low), float(seq_high), ref(outlier_low), ref(outlier_high),
            ref(token_low), ref(token_high), keep.data_ptr(), tis.data_ptr(), weight.data_ptr(), metrics.data_ptr(),
            row_stats.data_ptr(), torch.cuda.current_stream(dev).cuda_stream)
    _lib.check(st, "skyrl_off_policy_correction")
    return keep, tis, weight, metrics


@off_policy_correction_terms.register_fake
def _(old_log_probs, rollout_logprobs, loss_mask, tis_type, tis_cap, seq_metric, seq_low, seq_high, outlier_low, outlier_high,
      token_low, token_high):
    e = lambda: torch.empty_like(old_log_probs, dtype=torch.float32)  # noqa: E731
    return e(), e(), e(), old_log_probs.new_empty(_METRICS, dtype=torch.float32)


def _run(old_log_probs, rollout_logprobs, loss_mask, cfg, sync_metrics: bool):
    """``(keep, tis, weight, metrics dict, tis type)`` in the inputs' shape, for a config that switches something on."""
    tis_type = _get(cfg, "tis_ratio_type")
    seq_metric = _get(cfg, "sequence_mask_metric")
    if tis_type not in _TIS:
        raise ValueError(f"Unknown tis_ratio_type: {tis_type}")
    if seq_metric not in _SEQ:
        raise ValueError(f"Unknown sequence_mask_metric: {seq_metric}")
    tis_cap = {None: 0.0, "token": _get(cfg, "token_tis_ratio_clip_high"), "sequence": _get(cfg, "sequence_tis_ratio_clip_high")}[tis_type]
    if tis_cap is None:
        raise ValueError(f"tis_ratio_type={tis_type!r} needs off_policy_correction.{tis_type}_tis_ratio_clip_high")
    prefix = {None: None, "geometric": "geo", "product": "product"}[seq_metric]
    seq_low = 0.0 if prefix is None else _get(cfg, f"{prefix}_mask_low")
    seq_high = 0.0 if prefix is None else _get(cfg, f"{prefix}_mask_high")
    if seq_low is None or seq_high is None:
        raise ValueError(f"sequence_mask_metric={seq_metric!r} needs off_policy_correction.{prefix}_mask_low and {prefix}_mask_high")
    out_low, out_high = _get(cfg, "outlier_token_is_threshold_low"), _get(cfg, "outlier_token_is_threshold_high")
    tok_low, tok_high = _get(cfg, "token_mask_is_threshold_low"), _get(cfg, "token_mask_is_threshold_high")
    shape = old_log_probs.shape
    cols = shape[-1] if old_log_probs.dim() else 1
    rows = 1
    for extent in shape[:-1]:
        rows *= int(extent)
    flat = lambda t: None if t is None else t.detach().reshape(rows, cols).to(torch.float32).contiguous()  # noqa: E731
    keep, tis, weight, m = off_policy_correction_terms(
        flat(old_log_probs), flat(rollout_logprobs), flat(loss_mask), _TIS[tis_type], float(tis_cap), _SEQ[seq_metric],
        float(seq_low), float(seq_high), out_low, out_high, tok_low if tok_high is not None else None,
        tok_high if tok_low is not None else None)
    host = m.tolist() if sync_metrics else None                  # one read-back for all metrics
    val = (lambda i: host[i]) if sync_metrics else (lambda i: m[i])
    metrics: Dict[str, Any] = {"is_ratio_mean": val(0), "is_ratio_std": val(1), "is_ratio_max": val(2), "is_ratio_min": val(3)}
    if out_low is not None or out_high is not None:
        metrics.update({"outlier_seq_masked_ratio": val(4), "outlier_seq_over_high_ratio": val(5),
                        "outlier_seq_under_low_ratio": val(6)})
    if tok_low is not None and tok_high is not None:
        metrics["token_mask_ratio"] = val(7)
    if tis_type == "token":
        metrics["tis_token_clip_high_ratio"] = val(8)
    elif tis_type == "sequence":
        metrics["tis_seq_clip_high_ratio"] = val(9)
    if seq_metric is not None:
        name = "geo_sequence_mask" if seq_metric == "geometric" else "product_sequence_mask"
        metrics.update({f"{name}_masked_ratio": val(10), f"{name}_over_high_ratio": val(11), f"{name}_under_low_ratio": val(12)})
    return keep.reshape(shape), tis.reshape(shape), weight.reshape(shape), metrics, tis_type


def compute_off_policy_correction(old_log_probs: torch.Tensor, rollout_logprobs: torch.Tensor, loss_mask: torch.Tensor,
                                  off_policy_correction: Any, *, sync_metrics: bool = True
                                  ) -> Tuple[Optional[torch.Tensor], Dict[str, Any], torch.Tensor]:
    """Reference ``compute_off_policy_correction`` (:257-348): ``(tis_ratio, metrics, loss_mask)``; ``(None, {}, loss_mask)``
    when the config switches nothing on."""
    if not off_policy_correction_enabled(off_policy_correction):
        return None, {}, loss_mask
    keep, tis, _, metrics, tis_type = _run(old_log_probs, rollout_logprobs, loss_mask, off_policy_correction, sync_metrics)
    new_mask = keep.to(old_log_probs.dtype) if loss_mask is None else loss_mask * keep.to(loss_mask.dtype)
    tis_ratio = None
    if tis_type == "token":
        tis_ratio = tis.to(old_log_probs.dtype)
    elif tis_type == "sequence":
        tis_ratio = tis[..., :1].to(old_log_probs.dtype)
    return tis_ratio, metrics, new_mask


def apply_off_policy_correction(loss: torch.Tensor, old_log_probs: torch.Tensor, rollout_logprobs: Optional[torch.Tensor],
                                loss_mask: torch.Tensor, off_policy_correction: Any, *, sync_metrics: bool = True
                                ) -> Tuple[torch.Tensor, torch.Tensor, Dict[str, Any]]:
    """Reference ``apply_off_policy_correction`` (:351-391): the per-token loss times the TIS weight, the thinned mask, the
    metrics; everything unchanged without ``rollout_logprobs``."""
    metrics: Dict[str, Any] = {}
    if rollout_logprobs is not None:
        tis_ratio, metrics, loss_mask = compute_off_policy_correction(old_log_probs, rollout_logprobs, loss_mask,
                                                                      off_policy_correction, sync_metrics=sync_metrics)
        if tis_ratio is not None:
            loss = loss * tis_ratio
    return loss, loss_mask, metrics


def correction_weight(config: Any, old_log_probs: torch.Tensor, rollout_logprobs: Optional[torch.Tensor],
                      loss_mask: Optional[torch.Tensor], sync_metrics: bool = True) -> Tuple[Optional[torch.Tensor], Dict[str, Any]]:
    """What a fused policy loss needs of the correction: the per-token factor ``tis * keep`` to multiply its loss with next to
    the ORIGINAL ``loss_mask`` (the reference counts its clip statistic with the original mask and sums the loss with the
    thinned one), and the metrics.  ``(None, {})`` when the reference would not correct (no ``rollout_logprobs``, or nothing
    switched on, :285-305, 388-391)."""
    cfg = _get(config, "off_policy_correction")
    if rollout_logprobs is None or cfg is None or not off_policy_correction_enabled(cfg):
        return None, {}
    _, _, weight, metrics, _ = _run(old_log_probs, rollout_logprobs, loss_mask, cfg, sync_metrics)
    return weight, metrics
