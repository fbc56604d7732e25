import json, math
import numpy as np
SRC = "tests/train/algorithms/test_off_policy_correction.py"
def c(name, lines, old, rollout, mask, cfg, **exp):
    return dict(name=name, source=f"{SRC}:{lines}", old=old, rollout=rollout, mask=mask, config=cfg, expect=exp)
ones3 = [[1.0, 1.0, 1.0]]
m1 = [[-1.0, -1.0, -1.0]]
f32 = lambda x: float(np.float32(x))
opc = [
 c("tis_token_level", "21-43", [[-1.0, -1.5, -0.5]], [[-1.5, -1.0, -1.5]], ones3, dict(tis_ratio_type="token", token_tis_ratio_clip_high=2.0),
   tis=[[1.6487, 0.6065, 2.0]], metrics_abs={"tis_token_clip_high_ratio": [1 / 3, 0.01]}),
 c("tis_sequence_level", "46-69", [[-1.0, -1.5, -0.5]], [[-1.5, -1.0, -1.5]], ones3, dict(tis_ratio_type="sequence", sequence_tis_ratio_clip_high=5.0),
   tis=[[2.7183]], metrics_exact={"tis_seq_clip_high_ratio": 0.0}),
 c("tis_sequence_level_with_cap", "72-95", m1, [[-2.0, -2.0, -2.0]], ones3, dict(tis_ratio_type="sequence", sequence_tis_ratio_clip_high=5.0),
   tis=[[5.0]], metrics_exact={"tis_seq_clip_high_ratio": 1.0}),
 c("tis_sequence_with_mask", "98-121", [[-1.0, -1.5, -0.5]], [[-1.5, -1.0, -1.5]], [[1.0, 0.0, 1.0]], dict(tis_ratio_type="sequence", sequence_tis_ratio_clip_high=10.0),
   tis=[[math.exp(1.5)]], metrics_exact={"tis_seq_clip_high_ratio": 0.0}),
 c("sequence_mask_geometric", "124-148", [[-1.0, -1.1, -1.0]], [[-1.1, -1.0, -1.0]], ones3, dict(sequence_mask_metric="geometric", geo_mask_high=1.1, geo_mask_low=0.9),
   new_mask=ones3, metrics_exact={"geo_sequence_mask_masked_ratio": 0.0, "geo_sequence_mask_over_high_ratio": 0.0, "geo_sequence_mask_under_low_ratio": 0.0}),
 c("sequence_mask_geometric_rejects", "151-175", m1, [[-1.5, -1.5, -1.5]], ones3, dict(sequence_mask_metric="geometric", geo_mask_high=1.1, geo_mask_low=0.9),
   new_mask=[[0.0, 0.0, 0.0]], metrics_exact={"geo_sequence_mask_masked_ratio": 1.0, "geo_sequence_mask_over_high_ratio": 1.0, "geo_sequence_mask_under_low_ratio": 0.0}),
 c("sequence_mask_product", "178-202", [[-1.0, -1.1, -1.2]], [[-1.2, -1.2, -1.2]], ones3, dict(sequence_mask_metric="product", product_mask_high=2.0, product_mask_low=0.5),
   new_mask=ones3, metrics_exact={"product_sequence_mask_masked_ratio": 0.0, "product_sequence_mask_over_high_ratio": 0.0, "product_sequence_mask_under_low_ratio": 0.0}),
 c("sequence_mask_product_rejects", "205-229", m1, [[-2.0, -2.0, -2.0]], ones3, dict(sequence_mask_metric="product", product_mask_high=2.0, product_mask_low=0.5),
   new_mask=[[0.0, 0.0, 0.0]], metrics_exact={"product_sequence_mask_masked_ratio": 1.0, "product_sequence_mask_over_high_ratio": 1.0, "product_sequence_mask_under_low_ratio": 0.0}),
 c("outlier_masks_by_token_bounds", "232-256", m1, [[-1.0, -1.0, -6.0]], ones3, dict(outlier_token_is_threshold_low=1e-4, outlier_token_is_threshold_high=100.0),
   new_mask=[[0.0, 0.0, 0.0]], metrics_exact={"outlier_seq_masked_ratio": 1.0, "outlier_seq_over_high_ratio": 1.0, "outlier_seq_under_low_ratio": 0.0}),
 c("outlier_accepts_in_bounds", "259-283", [[-1.0, -1.5, -1.0]], [[-1.5, -1.0, -1.0]], ones3, dict(outlier_token_is_threshold_low=1e-4, outlier_token_is_threshold_high=100.0),
   new_mask=ones3, metrics_exact={"outlier_seq_masked_ratio": 0.0, "outlier_seq_over_high_ratio": 0.0, "outlier_seq_under_low_ratio": 0.0}),
 c("outlier_respects_loss_mask", "286-307", m1, [[-1.0, -1.0, -6.0]], [[1.0, 1.0, 0.0]], dict(outlier_token_is_threshold_low=1e-4, outlier_token_is_threshold_high=100.0),
   new_mask=[[1.0, 1.0, 0.0]], metrics_exact={"outlier_seq_masked_ratio": 0.0}),
 c("outlier_null_thresholds", "310-333", m1, [[-1.0, -1.0, -6.0]], ones3, dict(outlier_token_is_threshold_low=None, outlier_token_is_threshold_high=None),
   new_mask=ones3, tis_is_none=True, metrics_empty=True),
 c("outlier_only_high_threshold", "336-358", m1, [[-1.0, -1.0, -6.0]], ones3, dict(outlier_token_is_threshold_low=None, outlier_token_is_threshold_high=100.0),
   new_mask=[[0.0, 0.0, 0.0]], metrics_exact={"outlier_seq_masked_ratio": 1.0, "outlier_seq_over_high_ratio": 1.0, "outlier_seq_under_low_ratio": 0.0}),
 c("outlier_only_low_threshold", "361-383", [[-1.0, -1.0, -11.0]], m1, ones3, dict(outlier_token_is_threshold_low=1e-4, outlier_token_is_threshold_high=None),
   new_mask=[[0.0, 0.0, 0.0]], metrics_exact={"outlier_seq_masked_ratio": 1.0, "outlier_seq_over_high_ratio": 0.0, "outlier_seq_under_low_ratio": 1.0}),
 c("null_configs", "386-405", m1, [[-2.0, -2.0, -2.0]], ones3, dict(tis_ratio_type=None, sequence_mask_metric=None), tis_is_none=True, metrics_empty=True),
 c("pipeline_tis_only", "408-436", m1, [[-1.5, -1.5, -1.5]], ones3,
   dict(tis_ratio_type="token", token_tis_ratio_clip_high=2.0, sequence_mask_metric=None, outlier_token_is_threshold_low=1e-4, outlier_token_is_threshold_high=100.0),
   tis=[[math.exp(0.5)] * 3], metric_keys=["is_ratio_mean", "tis_token_clip_high_ratio"]),
 c("pipeline_sequence_mask_only", "439-467", m1, m1, ones3,
   dict(tis_ratio_type=None, sequence_mask_metric="geometric", geo_mask_high=1.1, geo_mask_low=0.9, outlier_token_is_threshold_low=1e-4, outlier_token_is_threshold_high=100.0),
   tis_is_none=True, new_mask=ones3, metric_keys=["is_ratio_mean", "geo_sequence_mask_masked_ratio"]),
 c("pipeline_both_enabled", "470-501", m1, [[-1.1, -1.1, -1.1]], ones3,
   dict(tis_ratio_type="token", token_tis_ratio_clip_high=2.0, sequence_mask_metric="geometric", geo_mask_high=1.2, geo_mask_low=0.8, outlier_token_is_threshold_low=1e-4, outlier_token_is_threshold_high=100.0),
   tis=[[math.exp(0.1)] * 3], metric_keys=["tis_token_clip_high_ratio", "geo_sequence_mask_masked_ratio"]),
 c("pipeline_sequence_mask_zeros_loss", "504-530", m1, [[-2.0, -2.0, -2.0]], ones3,
   dict(tis_ratio_type=None, sequence_mask_metric="geometric", geo_mask_high=1.1, geo_mask_low=0.9, outlier_token_is_threshold_low=1e-4, outlier_token_is_threshold_high=100.0),
   new_mask=[[0.0, 0.0, 0.0]], metrics_exact={"geo_sequence_mask_masked_ratio": 1.0}),
 c("token_mask_all_in_bounds", "632-647", [[-1.0, -1.1, -1.0]], [[-1.1, -1.0, -1.0]], ones3, dict(token_mask_is_threshold_low=0.5, token_mask_is_threshold_high=2.0),
   new_mask=ones3, metrics_exact={"token_mask_ratio": 0.0}),
 c("token_mask_masks_high_ratio_tokens", "650-666", m1, [[-1.0, -1.0, -3.0]], ones3, dict(token_mask_is_threshold_low=0.5, token_mask_is_threshold_high=2.0),
   new_mask=[[1.0, 1.0, 0.0]], metrics_abs={"token_mask_ratio": [1 / 3, 0.01]}),
 c("token_mask_masks_low_ratio_tokens", "669-685", [[-1.0, -1.0, -3.0]], m1, ones3, dict(token_mask_is_threshold_low=0.5, token_mask_is_threshold_high=2.0),
   new_mask=[[1.0, 1.0, 0.0]], metrics_abs={"token_mask_ratio": [1 / 3, 0.01]}),
 c("token_mask_ignores_already_masked_tokens", "688-707", m1, [[-1.0, -1.0, -6.0]], [[1.0, 1.0, 0.0]], dict(token_mask_is_threshold_low=0.5, token_mask_is_threshold_high=2.0),
   new_mask=[[1.0, 1.0, 0.0]], metrics_exact={"token_mask_ratio": 0.0}),
 c("token_mask_multi_sequence_batch", "710-728", [[-1.0, -1.0], [-3.0, -1.0]], [[-1.0, -3.0], [-1.0, -1.0]], [[1.0, 1.0], [1.0, 1.0]],
   dict(token_mask_is_threshold_low=0.5, token_mask_is_threshold_high=2.0), new_mask=[[1.0, 0.0], [0.0, 1.0]], metrics_abs={"token_mask_ratio": [0.5, 0.01]}),
 c("token_mask_boundary_values", "731-748", [[0.0, 0.0]], [[f32(-np.log(np.float32(0.5))), f32(-np.log(np.float32(2.0)))]], [[1.0, 1.0]],
   dict(token_mask_is_threshold_low=0.5, token_mask_is_threshold_high=2.0), new_mask=[[1.0, 1.0]], metrics_exact={"token_mask_ratio": 0.0}, fp32_only=True),
 c("pipeline_with_token_mask", "751-776", m1, [[-1.0, -1.0, -3.0]], ones3,
   dict(tis_ratio_type=None, token_tis_ratio_clip_high=None, sequence_mask_metric=None, outlier_token_is_threshold_low=None, outlier_token_is_threshold_high=None,
        token_mask_is_threshold_low=0.5, token_mask_is_threshold_high=2.0),
   tis_is_none=True, new_mask=[[1.0, 1.0, 0.0]], metrics_abs={"token_mask_ratio": [1 / 3, 0.01]}),
]
LS = "tests/train/algorithms/test_losses.py"
base3 = dict(advantages=[[1.0, -1.0, -4.0]], old_log_probs=[[-1.0, -1.0, -3.0]], log_probs=[[-1.69315, -1.0, -0.69741]])
losses = [
 dict(name="dual_clip", source=f"{LS}:33-82", **base3, loss_type="dual_clip", config=dict(eps_clip_low=0.2, eps_clip_high=0.2, clip_ratio_c=3.0),
      expect=dict(per_token=[[-0.5, 1.0, 12.0]], per_token_rtol=1e-3, loss=12.5, loss_abs=1e-4)),
 dict(name="cispo", source=f"{LS}:85-136", **base3, loss_type="cispo", config=dict(cispo=dict(cispo_eps_clip_low=0.2, cispo_eps_clip_high=0.2, cispo_anchor="old")),
      expect=dict(per_token=[[1.35452, -1.0, -3.347568]], per_token_rtol=1e-3, loss=-2.9930, loss_abs=1e-4)),
 dict(name="cispo_rollout_anchor", source=f"{LS}:139-193", **base3, rollout_logprobs=[[-1.30685, -1.5, -1.0]], loss_type="cispo",
      config=dict(cispo=dict(cispo_eps_clip_low=0.2, cispo_eps_clip_high=0.2, cispo_anchor="rollout")),
      expect=dict(formula="cispo", metric_keys=["clip_ratio", "cispo/ratio_mean", "cispo/ratio_clamped_mean", "cispo/ratio_max", "cispo/ratio_min"])),
 dict(name="cispo_ratio_min_max_ignore_masked_tokens", source=f"{LS}:196-233", **base3, loss_mask=[[1.0, 0.0, 1.0]], loss_type="cispo",
      config=dict(cispo=dict(cispo_eps_clip_low=0.2, cispo_eps_clip_high=0.2, cispo_anchor="old")),
      expect=dict(metrics_rel={"cispo/ratio_min": [math.exp(-0.69315), 1e-3], "cispo/ratio_max": [math.exp(2.30259), 1e-3]})),
 dict(name="gspo_importance_sampling_levels", source=f"{LS}:280-426", loss_type="gspo",
      advantages=[[1.5, 2.0, 1.0, 0.8, 0.5, 0.0, 0.0, 0.0], [3.0, 1.5, 0.0, 0.0, 0.0, 0.0, 0.0, 0.0], [0.5, 0.8, 1.2, 2.5, 0.0, 0.0, 0.0, 0.0]],
      old_log_probs=[[-1.0] * 8] * 3,
      log_probs=[[0.2, -2.5, -0.3, 0.1, -1.8, -1.0, -1.0, -1.0], [0.8, -0.2, -1.0, -1.0, -1.0, -1.0, -1.0, -1.0], [-0.5, 0.3, -1.7, 0.4, -1.0, -1.0, -1.0, -1.0]],
      loss_mask=[[1.0] * 5 + [0.0] * 3, [1.0] * 2 + [0.0] * 6, [1.0] * 4 + [0.0] * 4],
      config=dict(eps_clip_low=0.2, eps_clip_high=0.2, clip_ratio_c=3.0), expect=dict(formula="gspo_and_regular", rtol=1e-5)),
 dict(name="clip_cov", source=f"{LS}:429-486", loss_type="clip_cov", seed=42,
      advantages=[[2.0, -1.0, 1.5, 0.8], [1.0, 0.5, -2.0, 1.2]], old_log_probs=[[-1.0] * 4] * 2,
      log_probs=[[-0.5, -1.5, -0.8, -1.2], [-1.3, -0.7, -1.8, -0.9]], loss_mask=[[1.0] * 4, [1.0, 1.0, 1.0, 0.0]],
      config=dict(eps_clip_low=0.2, eps_clip_high=0.2, clip_cov=dict(clip_ratio=0.5, clip_cov_lb=-5.0, clip_cov_ub=5.0)),
      expect=dict(finite=True, clip_ratio_in_unit_interval=True, differs_from_regular_rtol=1e-3)),
 dict(name="kl_cov", source=f"{LS}:489-544", loss_type="kl_cov", seed=42,
      advantages=[[1.5, -0.5, 2.0, 0.8], [0.5, 1.0, -1.5, 1.2]], old_log_probs=[[-1.0] * 4] * 2,
      log_probs=[[-0.8, -1.2, -0.6, -1.1], [-1.1, -0.9, -1.4, -0.7]], loss_mask=[[1.0] * 4, [1.0, 1.0, 1.0, 0.0]],
      config=dict(eps_clip_low=0.2, eps_clip_high=0.2, kl_cov=dict(kl_cov_frac=0.5, ppo_kl_coef=1.0)),
      expect=dict(finite=True, clip_ratio=0.0, differs_from_regular_rtol=1e-3)),
 dict(name="sapo_basic", source=f"{LS}:547-604", loss_type="sapo", advantages=[[1.0, -1.0, 0.5]], old_log_probs=[[-1.0, -1.0, -1.0]],
      log_probs=[[-1.5, -0.8, -1.1]], config=dict(sapo=dict(tau_pos=1.0, tau_neg=2.0)), expect=dict(formula="sapo", rtol=1e-5, clip_ratio=0.0)),
]
dppo = [
 ("tv_pos_adv_masked", "binary_tv", 0.2, 0.2, [[-1.0, -1.0, -1.0]], [[-0.3, -2.0, -0.9]], [[1.0, -1.0, 1.0]], None, [[0.0, 0.0, 1.0]], True),
 ("tv_wrong_direction_not_masked", "binary_tv", 0.2, 0.2, [[-1.0, -1.0]], [[-2.0, -0.3]], [[1.0, -1.0]], None, [[1.0, 1.0]], False),
 ("tv_uses_rollout_logprobs", "binary_tv", 0.2, 0.2, [[-1.0, -1.0]], [[-0.3, -0.95]], [[1.0, 1.0]], [[-0.35, -1.0]], None, None),
 ("kl_masked", "binary_kl", 0.05, 0.05, [[-1.0, -1.0]], [[-0.1, -0.95]], [[1.0, 1.0]], None, None, True),
 ("kl_no_masking_within_delta", "binary_kl", 0.5, 0.5, [[-1.0, -1.0]], [[-1.01, -0.99]], [[1.0, -1.0]], None, [[1.0, 1.0]], False),
]
for name, typ, lo, hi, old, new, adv, roll, mask, clip in dppo:
    losses.append(dict(name="dppo_" + name, source=f"{LS}:607-734", loss_type="dppo", advantages=adv, old_log_probs=old, log_probs=new,
                       rollout_logprobs=roll, config=dict(dppo=dict(dppo_type=typ, delta_low=lo, delta_high=hi)),
                       expect=dict(kept_mask=mask, clip_ratio_positive=clip, rtol=1e-4, atol=1e-6,
                                   rollout_changes_loss=(name == "tv_uses_rollout_logprobs"))))
KL = "tests/backends/skyrl_train/utils/test_ppo_utils.py"
approx_kl = [
 dict(name="estimators", source=f"{KL}:38-76", log_probs=[[0.2, 0.3, 0.5]], log_probs_base=[[0.1, 0.2, 0.4]], mask=[[1.0, 1.0, 0.0]], atol=1e-4),
 dict(name="applies_loss_mask", source=f"{KL}:78-98", log_probs=[[0.2, 0.3, 0.5, 0.7]], log_probs_base=[[0.1, 0.2, 0.4, "nan"]], mask=[[1.0, 0.5, 0.25, 0.0]], atol=1e-6),
]
doc = {
 "_about": "Inputs and expected outputs of the reference's own unit tests for the consumers of the fused LM head's log-probabilities: "
           "off-policy correction, policy losses, approximate KL.  Data only (transcribed from the test files named in each case's "
           "'source'); the reference's helper-level cases are stated as configurations of compute_off_policy_correction that switch "
           "that one step on.  'config' holds the fields a case sets; the others take 'off_policy_correction_defaults' "
           "(skyrl/train/config/config.py:793-818).",
 "off_policy_correction_defaults": dict(tis_ratio_type=None, token_tis_ratio_clip_high=2.0, sequence_tis_ratio_clip_high=5.0, sequence_mask_metric=None,
        geo_mask_high=1.01, geo_mask_low=0.99, product_mask_high=2.0, product_mask_low=0.5, outlier_token_is_threshold_low=None,
        outlier_token_is_threshold_high=None, token_mask_is_threshold_low=None, token_mask_is_threshold_high=None),
 "tis_tolerance": {"rtol": 1e-3, "atol": 1e-4},
 "off_policy_correction": opc, "policy_losses": losses, "approx_kl": approx_kl,
}
json.dump(doc, open(__file__.rsplit("/", 1)[0] + "/reference_unit_test_cases.json", "w"), indent=1)
print(len(opc), len(losses), len(approx_kl))
