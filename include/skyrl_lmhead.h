/*
 * C ABI of the MI355X (gfx950) fused LM-head log-probability path.
 *
 * One shared library, plain pointers and sizes, no C++ or torch types in any signature.  Every device
 * pointer is memory the caller owns (in practice a torch tensor's data_ptr()); the library never frees or
 * keeps it after the call returns.  All work is enqueued asynchronously on the HIP stream passed in
 * (hipStream_t as void*, NULL = the default stream).  The library allocates nothing: scratch comes in as
 * `workspace`, sized by the *_workspace_bytes queries, so a caller can observe that no T x V buffer exists.
 *
 * Math (T tokens, H hidden, V vocab; z = (hidden . weight^T) * rcp_temperature):
 *     lse_t      = log sum_v exp z_tv
 *     logprob_t  = z_{t,label_t} - lse_t            (0 when label_t is outside [0, V))
 *     pz_t       = sum_v softmax(z_t)_v * z_tv
 *     entropy_t  = lse_t - pz_t
 *     dz_tv      = ( g_t * (1[v == label_t] - p_tv) - q_t * p_tv * (z_tv - pz_t) ) * rcp_temperature
 *     d_hidden   = dz . weight     (bf16)            d_weight = dz^T . hidden   (fp32)
 * with g = dlogprobs, q = dentropy.  dz is rounded to bf16 once before the two gradient GEMMs, as the
 * reference does (model_utils.py:413); all accumulation is fp32.
 *
 * Reference interfaces these entry points stand in for (paths under the SkyRL tree,
 * skyrl/backends/skyrl_train/distributed/megatron/):
 *   skyrl_lmhead_fwd  <- efficient_entropy_forward            fused_linear_logprob_triton.py:614-803
 *                        FusedLinearChunkedDistributedLogprob.forward            model_utils.py:302-359
 *                        _fused_vocab_parallel_entropy_from_hidden               model_utils.py:1090-1121
 *   skyrl_lmhead_bwd  <- efficient_entropy_backward           fused_linear_logprob_triton.py:1541-1753
 *                        FusedLinearChunkedDistributedLogprob.backward           model_utils.py:361-428
 *
 * Status codes: 0 = ok; negative = argument error detected before anything was enqueued (table below);
 * positive = a hipError_t returned by the HIP runtime.
 */
#ifndef SKYRL_LMHEAD_H
#define SKYRL_LMHEAD_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define SKYRL_LMHEAD_OK 0
#define SKYRL_LMHEAD_ERR_NULL (-1)      /* a required pointer is NULL, or only some of seg_row / seg_col / seg_len are given */
#define SKYRL_LMHEAD_ERR_SHAPE (-2)     /* T, V < 1, H not a positive multiple of 64, a leading dimension < H or > 4194304 elements, a negative count */
#define SKYRL_LMHEAD_ERR_ALIGN (-3)     /* a pointer is not 16-byte aligned or a leading dimension is not a multiple of 8 */
#define SKYRL_LMHEAD_ERR_WORKSPACE (-4) /* workspace is NULL or smaller than the matching *_workspace_bytes() */
#define SKYRL_LMHEAD_ERR_TOO_LARGE (-6) /* skyrl_lmhead_fwd_static_scratch only: V beyond SKYRL_LMHEAD_STATIC_SCRATCH_MAX_V */
#define SKYRL_LMHEAD_ERR_ARG (-5)       /* rcp_temperature not finite and positive, vocab_chunk not a multiple of 256, or both sub-sequence arrays and a mask */

/* ABI version of this header (bumped on any signature change). */
int skyrl_lmhead_version(void);

/* Human-readable text for a status code returned by this library (never NULL). */
const char* skyrl_lmhead_strerror(int status);

/* Scratch needed by skyrl_lmhead_fwd: per-vocab-tile (max, sum-exp, sum (z-max)*exp) partials of one token block,
 * 24 * min(T, 32768) * ceil(V/256) bytes (tokens rounded up to a multiple of 64) plus alignment slack.  The forward walks the
 * tokens in blocks of 32768 and merges a block's partials before the next block overwrites them, so the scratch does not
 * grow with T beyond one block (results are bit-identical to an unblocked run: block boundaries are tile boundaries).
 * (The reference allocates the same kind of buffers for all of T: `_max/_accu/_entropy_b [T, num_splits]`,
 * fused_linear_logprob_triton.py:670-672.) */
size_t skyrl_lmhead_fwd_workspace_bytes(int64_t T, int64_t H, int64_t V);

/* Scratch needed by skyrl_lmhead_bwd for a given vocab chunk width (0 = library default).  The backward walks the tokens in
 * blocks of T_b = min(T, 32768) and every scratch matrix is sized by the block:
 * hidden^T bf16 [H, T_b'+64], fp32 dHidden partial sums (T_b' x H' values, kept in the kernel's accumulator order between
 * chunks), one bf16 dz panel [T_b', chunk+64] and, only when V is not a multiple of 64, weight^T bf16 [H, V'+64] (otherwise
 * the weight is read where it is); for T > 32768 also one fp32 [V, H] matrix in which SKYRL_DW_BF16 sums dW over the blocks
 * (T_b', V', H' = T_b, V, H rounded up to 256; the 64 extra elements keep row pitches off powers of two).
 * The default chunk keeps the panel at or below 1.5 GiB, so nothing here grows with T * V.
 * (Stands in for the `d_logits [T, 9504]` scratch of the reference's default backward,
 * fused_linear_logprob_triton.py:1689-1748.) */
size_t skyrl_lmhead_bwd_workspace_bytes(int64_t T, int64_t H, int64_t V, int64_t vocab_chunk);

/*
 * Forward.  hidden: bf16 [T, ld_hidden]; weight: bf16 [V, ld_weight]; labels: int64 [T] (a value outside [0, V),
 * e.g. INT64_MAX, means "no target": logprob 0, no one-hot term in backward).
 * Outputs, all fp32 [T]: logprobs (required); entropy, row_lse, row_pz (each may be NULL).
 * row_lse (and row_pz when an entropy gradient will be applied) are what skyrl_lmhead_bwd needs back.
 * If entropy and row_pz are both NULL the sum p*z accumulation is skipped entirely.
 */
int skyrl_lmhead_fwd(const void* hidden, int64_t ld_hidden, const void* weight, int64_t ld_weight,
                     const int64_t* labels, int64_t T, int64_t H, int64_t V, float rcp_temperature,
                     float* logprobs, float* entropy, float* row_lse, float* row_pz,
                     void* workspace, size_t workspace_bytes, void* stream);

/*
 * The forward for callers that cannot allocate device memory and have no workspace to pass: code under HIP graph capture,
 * tight serving loops, harnesses that forbid hipMalloc.  It has no counterpart in the reference.  Same arguments, kernels and
 * results (bit for bit) as skyrl_lmhead_fwd, but the partial statistics go into a fixed array of
 * SKYRL_LMHEAD_STATIC_SCRATCH_BYTES (32 MiB) that lives in the library's own device image: every GPU the library runs on
 * holds one until the process ends, and the call itself performs no hipMalloc / hipFree or any other allocating call.
 * The tokens are walked in blocks whose partials fit that array (2304 tokens per block at V = 152064), so T is unlimited;
 * a vocabulary so large that one 256-token tile does not fit, V > SKYRL_LMHEAD_STATIC_SCRATCH_MAX_V, is refused with
 * SKYRL_LMHEAD_ERR_TOO_LARGE before anything is enqueued.  Nothing in the array has to start at zero (every partial is
 * written before it is read).  All calls on one GPU share that GPU's array: calls that overlap in time on one GPU -- two
 * streams, two host threads -- race; calls on one stream are ordered and safe.
 */
#define SKYRL_LMHEAD_STATIC_SCRATCH_BYTES 33554432
#define SKYRL_LMHEAD_STATIC_SCRATCH_MAX_V 1398016
int skyrl_lmhead_fwd_static_scratch(const void* hidden, int64_t ld_hidden, const void* weight, int64_t ld_weight,
                                    const int64_t* labels, int64_t T, int64_t H, int64_t V, float rcp_temperature,
                                    float* logprobs, float* entropy, float* row_lse, float* row_pz, void* stream);
/* Size of that array, as compiled into the library (equals SKYRL_LMHEAD_STATIC_SCRATCH_BYTES). */
size_t skyrl_lmhead_static_scratch_bytes(void);

/*
 * Backward.  Same hidden / weight / labels as the forward call; row_lse, row_pz from it (row_pz may be NULL
 * iff dentropy is NULL); dlogprobs fp32 [T] (required), dentropy fp32 [T] or NULL.
 * d_hidden: bf16 [T, H] contiguous, overwritten.  d_weight: [V, H] contiguous; by dw_mode fp32 overwritten (SKYRL_DW_FP32),
 * fp32 added to (SKYRL_DW_FP32_ACCUMULATE: gradient accumulation across micro-batches) or bf16 overwritten (SKYRL_DW_BF16:
 * the fp32 sums are rounded to nearest-even in the GEMM epilogue -- grad_weight in the weight dtype as model_utils.py:428
 * returns it, without an fp32 [V, H] buffer and a cast pass); NULL when the weight takes no gradient (a frozen
 * LM head, e.g. adapter training: autograd would drop grad_weight of model_utils.py:419-428 too) -- the dW product, a third
 * of the backward's work, is then not computed.  Both gradients are with respect to the unscaled weight / hidden: the
 * 1/temperature factor is already applied.
 * vocab_chunk: width of the dz panel in vocab columns (multiple of 256; 0 = library default: the width, with a panel of
 * at most 1.5 GiB, whose launches divide most evenly over the device's compute units).
 */
#define SKYRL_DW_FP32 0
#define SKYRL_DW_FP32_ACCUMULATE 1
#define SKYRL_DW_BF16 2
/*
 * Option bit, OR-ed into dw_mode of any backward entry point (no counterpart in the reference; off unless asked for):
 * softmax probabilities below 2^-24 -- the unit round-off of the fp32 in which p is formed; 1 - p rounds to 1 for them --
 * are taken as exactly zero when dz is formed.  Every product of the two gradient GEMMs is still computed; what changes is
 * the data: on peaked distributions most of the dz panel becomes zeros, and on an MI355X, whose matrix pipe is power-limited
 * on random operands, the gradient GEMMs then run at a higher clock.  The gradients differ from the exact ones by at most
 * the flushed probability mass of a row (below V * 2^-24, in practice far less) times |g| / temperature per dz row.
 */
#define SKYRL_BWD_FLUSH_TINY_DZ 0x100
int skyrl_lmhead_bwd(const void* hidden, int64_t ld_hidden, const void* weight, int64_t ld_weight,
                     const int64_t* labels, const float* row_lse, const float* row_pz,
                     const float* dlogprobs, const float* dentropy,
                     int64_t T, int64_t H, int64_t V, float rcp_temperature,
                     void* d_hidden, void* d_weight, int dw_mode, int64_t vocab_chunk,
                     void* workspace, size_t workspace_bytes, void* stream);

/*
 * The backward on the tokens that have an upstream gradient.  A token with dlogprobs == 0 (and dentropy == 0) has a zero dz
 * row: it adds nothing to d_weight and its d_hidden row is zero.  In RL micro-batches those are the prompt and padding tokens
 * the loss mask removes (loss_mask in workers/megatron/megatron_model_wrapper.py:607-985), often more than half of the batch; the
 * reference runs its three backward GEMMs over them all the same (model_utils.py:383-426).  This entry point compacts them
 * away on the device: a small kernel lists the active tokens and counts them, their hidden rows and per-token inputs are
 * gathered into the workspace, the kernels of skyrl_lmhead_bwd run on a grid sized for T whose tiles beyond the device-side
 * count return at once, and the d_hidden rows are scattered back (zero rows for the inactive tokens).  The host never learns
 * the count: no synchronisation, and the call can be captured in a HIP graph.  Arguments and results as skyrl_lmhead_bwd
 * (d_weight is bit-identical to what skyrl_lmhead_bwd computes on the compacted inputs; summing fewer zero rows may differ
 * from the dense result in the last bit); the workspace is larger by the gathered copies, 4 * T * H + 28 * T bytes.
 */
size_t skyrl_lmhead_bwd_active_rows_workspace_bytes(int64_t T, int64_t H, int64_t V, int64_t vocab_chunk);
int skyrl_lmhead_bwd_active_rows(const void* hidden, int64_t ld_hidden, const void* weight, int64_t ld_weight,
                                 const int64_t* labels, const float* row_lse, const float* row_pz,
                                 const float* dlogprobs, const float* dentropy,
                                 int64_t T, int64_t H, int64_t V, float rcp_temperature,
                                 void* d_hidden, void* d_weight, int dw_mode, int64_t vocab_chunk,
                                 void* workspace, size_t workspace_bytes, void* stream);

/*
 * fp32 operands.  The reference casts hidden to the weight's dtype and forms fp32 logits when the output weight is fp32
 * (model_utils.py:328-333; its tests cover (bf16 hidden, fp32 weight) -- "the real Megatron case" -- and (fp32, fp32),
 * tests/backends/skyrl_train/gpu/gpu_ci/megatron/test_fused_linear_logprob.py:99-103).  The matrix pipe multiplies bf16, so
 * an fp32 operand is given to it as a sum of bf16 terms, x = hi + lo with hi = bf16(x), lo = bf16(x - hi) (exact to 2^-17),
 * stacked along the contraction axis; the MFMA accumulates all terms in fp32:
 *     weight fp32, hidden bf16:   weight' = [w_hi | w_lo]         hidden' = [h | h]                 (terms = 2)
 *     weight fp32, hidden fp32:   weight' = [w_hi | w_lo | w_hi]  hidden' = [h_hi | h_hi | h_lo]    (terms = 3)
 * so that hidden' . weight'^T = h . w up to the dropped lo x lo products (below 2^-16 of each product; measured: log-probabilities
 * within 1e-5 of the fp32 product at the reference's test shapes).  Nothing is down-cast silently, and no kernel is special:
 *   skyrl_lmhead_split_operand  writes one stacked operand: src [rows, H] (fp32, or bf16 with src_is_fp32 = 0), dst bf16
 *                               [rows, terms * H] with leading dimension ld_dst, layout one of SKYRL_SPLIT_*
 *   skyrl_lmhead_fwd            is called on the stacked operands with H' = terms * H
 *   skyrl_lmhead_bwd_split      is skyrl_lmhead_bwd (active_rows = 0) or skyrl_lmhead_bwd_active_rows (active_rows = 1) on the
 *                               stacked operands: the logits are recomputed over all terms * H columns, dz is rounded to bf16
 *                               once as always, and the two gradient GEMMs use the leading H columns (the hi terms):
 *                               d_hidden bf16 [T, H], d_weight [V, H] by dw_mode.  Gradients therefore carry bf16 rounding of
 *                               dz and of the multiplied operand (2^-9 per element, inside the reference's 2e-3 tolerance).
 * Cost: the two logits GEMMs take terms times as long; the gradient GEMMs are unchanged.
 */
#define SKYRL_SPLIT_HI_LO 0
#define SKYRL_SPLIT_HI_HI 1
#define SKYRL_SPLIT_HI_LO_HI 2
#define SKYRL_SPLIT_HI_HI_LO 3
int skyrl_lmhead_split_operand(const void* src, int src_is_fp32, int64_t ld_src, int64_t rows, int64_t H, int layout,
                               void* dst, int64_t ld_dst, void* stream);
size_t skyrl_lmhead_bwd_split_workspace_bytes(int64_t T, int64_t H, int64_t terms, int64_t V, int64_t vocab_chunk,
                                              int active_rows);
int skyrl_lmhead_bwd_split(const void* hidden_terms, int64_t ld_hidden, const void* weight_terms, int64_t ld_weight,
                           const int64_t* labels, const float* row_lse, const float* row_pz,
                           const float* dlogprobs, const float* dentropy,
                           int64_t T, int64_t H, int64_t terms, int64_t V, float rcp_temperature,
                           void* d_hidden, void* d_weight, int dw_mode, int64_t vocab_chunk, int active_rows,
                           void* workspace, size_t workspace_bytes, void* stream);

/*
 * The consumer one step after the log-probabilities: the policy loss and its gradient with respect to the
 * log-probabilities in one pass -- what the reference computes with elementwise torch kernels plus autograd
 * (skyrl/backends/skyrl_train/utils/ppo_utils.py; safe_exp_delta / masked_mean of
 * skyrl/backends/skyrl_train/utils/torch_utils.py:180-192; reduce_loss of ppo_utils.py:1145-1149).  loss_type:
 *   REGULAR, DUAL_CLIP (ppo_policy_loss, ppo_utils.py:555-588):
 *     ratio = exp(clamp(logprobs - old_logprobs, -20, 20))
 *     loss  = -min(ratio * A, clamp(ratio, 1 - eps_clip_low, 1 + eps_clip_high) * A)
 *     DUAL_CLIP:  loss = A < 0 ? min(-A * clip_ratio_c, loss) : loss
 *     out3[1] = sum [clipped] * mask            (clip_ratio of the reference = out3[1] / max(out3[2], 1))
 *   CROSS_ENTROPY (cross_entropy_loss, ppo_utils.py:1056-1092):  loss = -logprobs; old_logprobs and advantages are not
 *     read and may be NULL; out3[1] = 0
 *   IMPORTANCE_SAMPLING (importance_sampling_loss, ppo_utils.py:1095-1142):  loss = -exp(logprobs - old_logprobs) * A;
 *     out3[1] = sum exp(logprobs - old_logprobs) * mask     (importance_ratio of the reference = out3[1] / out3[2])
 * All arrays fp32 [T].  loss_mask and loss_weight may be NULL (= 1); loss_weight is any factor of the loss that does not
 * depend on logprobs (the off-policy importance ratio).  out3 = { sum loss*mask*weight, (see above), sum mask }.
 * dlogprobs (may be NULL) receives d out3[0] / d logprobs, i.e. the upstream gradient skyrl_lmhead_bwd takes when the
 * loss is that sum.  The eps / clip_ratio_c arguments are ignored by the loss types that do not clip.
 * partials: fp32 scratch of 3 * SKYRL_POLICY_LOSS_PARTIALS elements for the partial sums of the workgroups; may be NULL
 * for T <= 8192 (one workgroup), ERR_WORKSPACE otherwise.  The sums are added in a fixed order: reproducible bit for bit.
 */
#define SKYRL_POLICY_LOSS_PARTIALS 256
#define SKYRL_POLICY_LOSS_REGULAR 0
#define SKYRL_POLICY_LOSS_DUAL_CLIP 1
#define SKYRL_POLICY_LOSS_CROSS_ENTROPY 2
#define SKYRL_POLICY_LOSS_IMPORTANCE_SAMPLING 3
/* Further types of the reference's registry (ppo_utils.py), same outputs; r = exp(clamp(logprobs - old_logprobs, -20, 20)):
 *   GSPO (gspo_policy_loss, :663-729; skyrl_actor_loss only, it needs rows): the clipped surrogate of REGULAR with every
 *     token's ratio replaced by its sequence's, exp(min(masked row mean of logprobs - old_logprobs, 10)), whose gradient
 *     reaches each token's own logprob with weight 1.
 *   SAPO (sapo_policy_loss, :590-660): loss = -sigmoid(tau (r - 1)) (4 / tau) A, tau = A > 0 ? eps_clip_low : eps_clip_high
 *     (the two arguments carry tau_pos and tau_neg); out3[1] = 0.
 *   CISPO (compute_policy_loss_cispo, :732-821, anchor "old"; pass the rollout log-probabilities as old_logprobs for the
 *     "rollout" anchor): loss = -A stopgrad(clamp(r, 1 - eps_clip_low, 1 + eps_clip_high)) logprobs; out3[1] counts r outside.
 *   ROLLOUT_IS (rollout_is_policy_loss, :824-863; old_logprobs = rollout log-probabilities):
 *     loss = -stopgrad(r inside the open interval (1 - eps_clip_low, 1 + eps_clip_high) ? r : 0) A logprobs; out3[1] counts outside.
 *   DPPO_TV, DPPO_KL (dppo_policy_loss, :866-935; old_logprobs = rollout log-probabilities when there are any):
 *     loss = -r A keep, keep = 0 where the probability moved too far in the advantage's direction -- TV: p - p_old >
 *     eps_clip_high (A > 0) or p_old - p > eps_clip_low (A < 0); KL: the binary KL of p_old to p exceeds the same thresholds
 *     (the two arguments carry delta_low and delta_high); out3[1] counts keep == 0.
 * The two covariance-based types (skyrl_ppo_policy_loss only).  Which tokens they single out is decided from the whole batch
 * on the host side, as the reference does (a random subset drawn with the host's generator / a top-k computed on the CPU);
 * the per-token decision comes in through loss_weight:
 *   CLIP_COV (compute_policy_loss_clip_cov, :938-999): the clipped surrogate of REGULAR on the unclamped ratio exp(logprobs -
 *     old_logprobs), times loss_weight = 0 for the tokens the covariance rule removes, 1 elsewhere; out3[1] counts clipped tokens.
 *   KL_COV (compute_policy_loss_kl_cov, :1002-1053): loss = -exp(logprobs - old_logprobs) A + clip_ratio_c |logprobs - old_logprobs|
 *     where loss_weight = 1 (the selected tokens; clip_ratio_c carries ppo_kl_coef), the plain importance-sampling term
 *     elsewhere; loss_weight does not scale the loss here; out3[1] counts selected tokens. */
#define SKYRL_POLICY_LOSS_GSPO 4
#define SKYRL_POLICY_LOSS_SAPO 5
#define SKYRL_POLICY_LOSS_CISPO 6
#define SKYRL_POLICY_LOSS_ROLLOUT_IS 7
#define SKYRL_POLICY_LOSS_DPPO_TV 8
#define SKYRL_POLICY_LOSS_DPPO_KL 9
#define SKYRL_POLICY_LOSS_CLIP_COV 10
#define SKYRL_POLICY_LOSS_KL_COV 11
int skyrl_ppo_policy_loss(const float* logprobs, const float* old_logprobs, const float* advantages,
                          const float* loss_mask, const float* loss_weight, int64_t T,
                          float eps_clip_low, float eps_clip_high, float clip_ratio_c, int loss_type,
                          float* out3, float* dlogprobs, float* partials, void* stream);

/*
 * Approximate KL divergence to a base policy per token (compute_approx_kl, ppo_utils.py:88-126), reduced as the trainer
 * reduces it for the KL loss term (workers/worker.py:1071-1077: masked_mean over dim -1, then the mean over rows), with
 * d = logprobs - base_logprobs:
 *     K1: d        ABS: |d|        K2: d^2 / 2        K3: k = clamp(-d, -20, 20); clamp(exp(k) - k - 1, -10, 10)
 *     kld[b,s]    = mask != 0 ? value * mask : 0                              (optional output, [rows, cols])
 *     row_mean[b] = sum_s kld[b,s] * mask[b,s] / max(sum_s mask[b,s], 1)      (required output, [rows])
 *     mean[0]     = sum_b row_mean[b] / rows                                  (required output)
 * logprobs, base_logprobs fp32 [rows, cols]; loss_mask fp32 [rows, cols] or NULL (= 1, plain means).
 * grad_mode 0: dlogprobs not written; 1: dlogprobs = d kld / d logprobs elementwise; 2: dlogprobs = d mean[0] / d logprobs.
 * Derivatives follow torch: clamp passes the gradient on its closed interval, |.| has derivative 0 at 0.
 */
#define SKYRL_KL_K1 0
#define SKYRL_KL_ABS 1
#define SKYRL_KL_K2 2
#define SKYRL_KL_K3 3
int skyrl_approx_kl(const float* logprobs, const float* base_logprobs, const float* loss_mask, int64_t rows, int64_t cols,
                    int estimator, float* kld, float* row_mean, float* mean, int grad_mode, float* dlogprobs, void* stream);

/*
 * The whole actor loss of a micro-batch and both upstream gradients of the LM-head backward in two launches (three with dentropy) -- what the
 * worker assembles from the policy loss, the KL term and the entropy term (skyrl/backends/skyrl_train/workers/worker.py:989-1089,
 * workers/megatron/megatron_model_wrapper.py:902-941):
 *     out6[0] = policy_scale * out6[1] + term_scale * (kl_coef * out6[4] - entropy_coef * out6[5])
 *     out6[1] = policy loss, out6[2] its statistic, out6[3] = sum mask          (as skyrl_ppo_policy_loss's out3)
 *     out6[4] = KL term: mean over rows of the masked row means of the estimate   (as skyrl_approx_kl's mean; 0 without base_logprobs)
 *     out6[5] = entropy term: sum entropy * mask / max(sum mask, 1)               (masked_mean over everything; 0 without entropy)
 *     dlogprobs = d out6[0] / d logprobs        dentropy = d out6[0] / d entropy
 * All arrays fp32 [rows, cols]; loss_mask, loss_weight, base_logprobs, entropy, dlogprobs, dentropy may be NULL (dentropy needs
 * entropy).  policy_scale is the factor the worker applies to the pre-scaled policy loss (its data-parallel size), term_scale
 * the micro-batch weight of the two mean-reduced terms.  row_sums: fp32 scratch [rows, 6].
 */
int skyrl_actor_loss(const float* logprobs, const float* old_logprobs, const float* advantages, const float* loss_mask,
                     const float* loss_weight, const float* base_logprobs, const float* entropy, int64_t rows, int64_t cols,
                     int loss_type, float eps_clip_low, float eps_clip_high, float clip_ratio_c, int kl_estimator,
                     float policy_scale, float term_scale, float kl_coef, float entropy_coef, float* row_sums, float* out6,
                     float* dlogprobs, float* dentropy, void* stream);

/*
 * masked_mean (torch_utils.py:180-184) per row of values fp32 [rows, cols]:
 *     means[b] = sum_s values * mask / max(sum_s mask, 1)          (mask NULL: the plain mean)
 * and, when dvalues is not NULL, dvalues[b,s] = d means[b] / d values[b,s] = mask / max(sum_s mask, 1).
 * The global form (dim=None, e.g. the entropy term of workers/worker.py:1062) is rows = 1, cols = the element count.
 */
int skyrl_masked_mean(const float* values, const float* mask, int64_t rows, int64_t cols, float* means, float* dvalues,
                      void* stream);

/*
 * compute_minibatch_rollout_logprob_diff_metrics (workers/worker_utils.py:34-58), the drift statistics both trainers log per
 * micro-batch (workers/worker.py:1124-1126, megatron_model_wrapper.py:982-984): over n fp32 tokens, with d = |logprobs -
 * rollout_logprobs| and m = loss_mask (NULL: every token counts, plain means),
 *     out4 = { sum d m / max(sum m, 1),  sum d^2 m / max(sum m, 1),  max d m,  min d m }.
 * partials: fp32 scratch of 5 * SKYRL_POLICY_LOSS_PARTIALS elements.  Two launches, no read-back; the sums are added in a
 * fixed order (bit-reproducible); a NaN reaches all four results, as with the torch reductions.
 */
int skyrl_logprob_diff_metrics(const float* logprobs, const float* rollout_logprobs, const float* loss_mask, int64_t n, float* out4,
                               float* partials, void* stream);

/*
 * Packed-sequence front end: the label of every token of a packed [T] stream is its successor inside its own sequence,
 *     labels[t] = tokens[cu[s] + (t - cu[s] + 1) mod (cu[s+1] - cu[s])],   s = the sequence with cu[s] <= t < cu[s+1]
 * (next_offsets / rolled_targets_full of from_parallel_hidden_to_logprobs_packed_sequences,
 * skyrl/backends/skyrl_train/distributed/megatron/model_utils.py:810-815, with _packed_sequence_indices, :920-928).
 * tokens, labels int64 [T]; cu_seqlens int64 [num_seqs + 1], non-decreasing, cu_seqlens[0] = 0.  Tokens at or beyond
 * cu_seqlens[num_seqs] (the reference indexes out of range there) get INT64_MAX, the "not in this shard" label.
 */
int skyrl_packed_next_token_labels(const int64_t* tokens, const int64_t* cu_seqlens, int64_t num_seqs, int64_t T,
                                   int64_t* labels, void* stream);

/*
 * Packed-sequence back end: packed per-token values fp32 [T] -> out fp32 [rows, cols] (cols = unpacked_seqlen - 1), every
 * element of out written (0 where no token lands); the three branches of model_utils.py:851-883.  Token t of sequence s,
 * offset o = t - cu[s]:
 *   plain (seg_* and attention_mask NULL; :880-883):  out[s, o]                        for o < cu[s+1] - cu[s] - 1
 *   sub-sequences (seg_row, seg_col, seg_len int64 [num_seqs], all three; :859-871):
 *                                                     out[seg_row[s], seg_col[s] + o]  for o < seg_len[s] - 1
 *   attention mask (uint8 [rows, cols + 1], rows == num_seqs; :873-878): the j-th non-zero column of row s takes token
 *     cu[s] + j, for every non-zero column but the last of the row.  This is the reference's
 *     out[output_mask] = probs[packed_mask] whenever each packed segment holds at least its row's real tokens minus one
 *     (otherwise the reference raises a shape error; here the tokens that do not exist read as 0).
 * Destinations outside [rows, cols] are dropped, as the reference's in-bounds masks do.  T = 0 and rows * cols = 0 are
 * valid (the pointer of an empty array may then be NULL).
 * skyrl_packed_gather_grad is the adjoint: d_packed[t] = d_out[destination of t], 0 for tokens without one.
 */
int skyrl_packed_scatter_logprobs(const float* packed, const int64_t* cu_seqlens, int64_t num_seqs, int64_t T,
                                  const int64_t* seg_row, const int64_t* seg_col, const int64_t* seg_len,
                                  const uint8_t* attention_mask, int64_t rows, int64_t cols, float* out, void* stream);
int skyrl_packed_gather_grad(const float* d_out, const int64_t* cu_seqlens, int64_t num_seqs, int64_t T,
                             const int64_t* seg_row, const int64_t* seg_col, const int64_t* seg_len,
                             const uint8_t* attention_mask, int64_t rows, int64_t cols, float* d_packed, void* stream);

/*
 * Soft cross-entropy of a draft head against the policy's own next-token distribution, from hidden states.
 * Replaces, for the full-vocabulary branch on one vocabulary shard, draft_soft_ce / _VocabParallelSoftCrossEntropy
 * (skyrl/backends/skyrl_train/mtp/soft_ce.py:123-154, 200-240) together with the two output-layer products that feed it
 * (project_mtp_hidden_to_logits, mtp/adapter.py:37-64, and the policy's own logits) and the teacher roll
 * (build_teacher_logits, soft_ce.py:22-34):
 *
 *     z_s[t] = student_hidden[t] . weight^T / temperature        z_t[t] = teacher_hidden[roll(t)] . weight^T / temperature
 *     loss[t] = -sum_v softmax(z_t[t])_v * log_softmax(z_s[t])_v
 *
 * roll(t) for t = b * seq_len + s is b * seq_len + (s + shift) mod seq_len (shift = MTP depth + 1; seq_len = T for one packed
 * row); the caller's loss mask removes the wrapped positions, as in the reference.  Neither [T, V] logits tensor exists:
 * both hidden rows of a token go through one tile of the MFMA kernel side by side.  student_hidden / teacher_hidden are
 * bf16 [T, H] with leading dimensions ld_student / ld_teacher; weight is bf16 [V, H]; T must be a multiple of seq_len.
 *
 * skyrl_softce_fwd writes loss [T] and the two row log-sum-exps [T] (fp32) that skyrl_softce_bwd takes back.
 * skyrl_softce_bwd writes d_student_hidden [T, H] bf16 = sum_v dloss[t] * (softmax(z_s) - softmax(z_t))_v / temperature *
 * weight[v] (soft_ce.py:146-151 followed by the output layer's input gradient).  The teacher and the weight get no gradient:
 * the reference detaches both (soft_ce.py:16-19, mtp/adapter.py:51-56).  Workspaces: 256-byte aligned device memory of at
 * least the queried size (0 = bad arguments); vocab_chunk as in skyrl_lmhead_bwd.  Not covered: more than one vocabulary
 * shard.
 */
size_t skyrl_softce_fwd_workspace_bytes(int64_t T, int64_t H, int64_t V);
size_t skyrl_softce_bwd_workspace_bytes(int64_t T, int64_t H, int64_t V, int64_t vocab_chunk);
int skyrl_softce_fwd(const void* student_hidden, int64_t ld_student, const void* teacher_hidden, int64_t ld_teacher,
                     const void* weight, int64_t ld_weight, int64_t T, int64_t seq_len, int64_t shift, int64_t H, int64_t V,
                     float rcp_temperature, float* loss, float* lse_student, float* lse_teacher, void* workspace,
                     size_t workspace_bytes, void* stream);
int skyrl_softce_bwd(const void* student_hidden, int64_t ld_student, const void* teacher_hidden, int64_t ld_teacher,
                     const void* weight, int64_t ld_weight, const float* lse_student, const float* lse_teacher,
                     const float* dloss, int64_t T, int64_t seq_len, int64_t shift, int64_t H, int64_t V, float rcp_temperature,
                     void* d_student_hidden, int64_t vocab_chunk, void* workspace, size_t workspace_bytes, void* stream);

/* ---- top-k draft loss from hidden states ----------------------------------------------------------------------------
 * Stands in for draft_soft_ce_topk / _VocabParallelTopkSoftCE (skyrl/backends/skyrl_train/mtp/soft_ce.py:243-341) on one
 * vocabulary shard, together with the two output-layer products in front of it: only the teacher's k largest logits of a
 * token are distilled, teacher and student renormalised over those k columns.
 *
 * skyrl_lmhead_topk_logits stands in for `teacher_logits.topk(k, dim=-1)` (:273) on logits = hidden . weight^T *
 * rcp_temperature that are never stored: values [T, k] fp32 and columns [T, k] int32, best first; among equal values the
 * lower column comes first.  1 <= k <= min(V, 1024).  The workspace (256-byte aligned, at least the queried size, 0 = bad
 * arguments) does not grow with T * V: at most 16384 tokens x 8192 candidate slots of 8 bytes.
 *
 * skyrl_softce_topk_fwd: token b * seq_len + s takes the teacher's list of token b * seq_len + (s + shift) % seq_len (the roll
 * of the [B, S, k] result, :276-279), gathers the student's logits at those columns (k dot products of student_hidden[t] with
 * weight rows, :282), and writes loss [T] = -sum_j softmax(teacher)_j log softmax(student)_j (:285-300), coef [T, k] =
 * softmax(student) - softmax(teacher) (:309) and the columns [T, k] it used -- the O(T * k) state the backward needs.
 * skyrl_softce_topk_bwd writes d_student_hidden [T, H] bf16 = dloss[t] * rcp_temperature * sum_j coef[t, j] * weight[columns
 * [t, j]] (the scatter of :309-312 followed by the output layer's input gradient).  Teacher and weight get no gradient.
 */
size_t skyrl_lmhead_topk_workspace_bytes(int64_t T, int64_t H, int64_t V, int64_t k);
int skyrl_lmhead_topk_logits(const void* hidden, int64_t ld_hidden, const void* weight, int64_t ld_weight, int64_t T, int64_t H,
                             int64_t V, int64_t k, float rcp_temperature, float* values, int32_t* columns, void* workspace,
                             size_t workspace_bytes, void* stream);
int skyrl_softce_topk_fwd(const void* student_hidden, int64_t ld_student, const void* weight, int64_t ld_weight,
                          const float* teacher_values, const int32_t* teacher_columns, int64_t T, int64_t seq_len, int64_t shift,
                          int64_t H, int64_t V, int64_t k, float rcp_temperature, float* loss, float* coef, int32_t* columns,
                          void* stream);
int skyrl_softce_topk_bwd(const void* weight, int64_t ld_weight, const float* coef, const int32_t* columns, const float* dloss,
                          int64_t T, int64_t H, int64_t V, int64_t k, float rcp_temperature, void* d_student_hidden,
                          int64_t ld_d_student, void* stream);

/* ---- off-policy correction from the rollout engine's log-probabilities -------------------------------------------------
 * Stands in for compute_off_policy_correction (skyrl/backends/skyrl_train/utils/off_policy_correction_utils.py:257-348) and
 * the four functions it combines (compute_tis_ratio :24-72, compute_outlier_token_mask :75-134, compute_token_mask :137-188,
 * compute_sequence_mask :191-254), which the policy losses apply to their per-token loss (apply_off_policy_correction,
 * :351-391; ppo_utils.py:581, 653, 722, 815, 857, 929).  It depends on old_log_probs and rollout_logprobs only, never on the
 * policy's current log-probabilities, so it carries no gradient.
 *   old_log_probs, rollout_logprobs, loss_mask: fp32 [rows, cols] (loss_mask NULL = all ones).
 *   tis_type: 0 off, 1 "token" (weight min(r, tis_cap)), 2 "sequence" (the row's product ratio, capped).
 *   seq_metric: 0 off, 1 "geometric", 2 "product", with bounds seq_low / seq_high (geo_mask_* / product_mask_*).
 *   outlier_low / outlier_high: pointers to the thresholds, NULL = not set (either alone switches the outlier filter on);
 *   token_low / token_high: the per-token hard mask, on only when both are given.
 * Outputs (each may be NULL): keep [rows, cols] in {0, 1} -- loss_mask * keep is the mask the reference returns; tis
 * [rows, cols] (a row's value repeated for "sequence"; ones when tis_type is 0); weight = tis * keep, the per-token factor
 * to hand to the policy-loss entry points as loss_weight together with the ORIGINAL loss_mask (the reference counts its
 * clip statistic with the original mask and sums the loss with the new one).  metrics: SKYRL_OFF_POLICY_METRICS floats --
 * 0 is_ratio_mean, 1 is_ratio_std, 2 is_ratio_max, 3 is_ratio_min, 4 outlier_seq_masked_ratio, 5 outlier_seq_over_high_ratio,
 * 6 outlier_seq_under_low_ratio, 7 token_mask_ratio, 8 tis_token_clip_high_ratio, 9 tis_seq_clip_high_ratio, 10-12 the
 * sequence mask's masked / over_high / under_low ratios -- added over the rows in a fixed order.  row_stats: scratch of
 * rows * SKYRL_OFF_POLICY_ROW_STATS floats.  Two launches, no synchronisation. */
#define SKYRL_OFF_POLICY_ROW_STATS 20
#define SKYRL_OFF_POLICY_METRICS 16
int skyrl_off_policy_correction(const float* old_log_probs, const float* rollout_logprobs, const float* loss_mask, int64_t rows,
                                int64_t cols, int tis_type, float tis_cap, int seq_metric, float seq_low, float seq_high,
                                const float* outlier_low, const float* outlier_high, const float* token_low,
                                const float* token_high, float* keep_out, float* tis_out, float* weight_out, float* metrics,
                                float* row_stats, void* stream);

/* ---- the same statistics from materialised logits -------------------------------------------------------------------
 * For callers that hold a [T, V] logits matrix: the FSDP worker's forward tail -- logprobs_from_logits / _v2 / _flash_attn
 * (skyrl/backends/skyrl_train/utils/torch_utils.py:115-177) and chunked_entropy_from_logits (:58-111) -- and the
 * logits-input autograd functions DistributedLogprob / ChunkedDistributedLogprob (distributed/megatron/model_utils.py:66-272)
 * and _VocabParallelEntropy (:1316-1345) on one vocabulary shard.  One pass over the matrix per call; nothing of size T * V is
 * allocated or saved (the reference keeps an fp32 softmax of the whole matrix for its backward, model_utils.py:91-104).
 *
 * logits: bf16 or fp32 (logits_dtype), row r at logits + r * ld_logits elements; rows and pitches that allow 16-byte loads
 * take the fast path, any other alignment works.  labels int64 [T] (NULL when no log-probability is wanted); a label outside
 * [0, V) gives log-probability 0 and, in the backward, no one-hot term (model_utils.py:83-99, 111-137).
 * skyrl_logits_fwd writes any of logprobs / entropy / row_lse / row_pz (fp32 [T], NULL = not wanted), computed on
 * logits * rcp_temperature (the worker divides its logits by the temperature in place first, workers/model_wrapper.py:334).
 * skyrl_logits_bwd writes dlogits (same dtype as the logits; leading dimension ld_dlogits)
 *   = ( dlogprobs * (onehot - p) - dentropy * p * (y - row_pz) ) * rcp_temperature,  p = exp(y - row_lse),  y = logits * rcp_temperature
 * dlogits may be the logits pointer itself with the same leading dimension -- the gradient then overwrites the logits, as the
 * flash-attn cross-entropy does with inplace_backward=True (torch_utils.py:131-152) -- or a buffer that does not overlap them.
 * Rows whose upstream gradients are both zero are written as zeros without being read. */
#define SKYRL_LOGITS_BF16 0
#define SKYRL_LOGITS_F32 1
int skyrl_logits_fwd(const void* logits, int logits_dtype, int64_t ld_logits, const int64_t* labels, int64_t T, int64_t V,
                     float rcp_temperature, float* logprobs, float* entropy, float* row_lse, float* row_pz, void* stream);
int skyrl_logits_bwd(const void* logits, int logits_dtype, int64_t ld_logits, const int64_t* labels, const float* row_lse,
                     const float* row_pz, const float* dlogprobs, const float* dentropy, int64_t T, int64_t V,
                     float rcp_temperature, void* dlogits, int64_t ld_dlogits, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* SKYRL_LMHEAD_H */
