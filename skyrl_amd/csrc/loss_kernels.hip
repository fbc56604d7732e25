// The consumers one step after the LM head: per-token losses on the [B, S] log-probabilities and entropies, each with its
// gradient in the same pass, so that the upstream gradient of the LM-head backward is ready without a chain of elementwise
// kernels and without a host synchronisation.  All of it is a few hundred KiB of fp32 per micro-batch: HBM-bound,
// latency-dominated work; the kernels use fixed reduction orders so that every sum is bit-reproducible.
//
// Reference (paths under skyrl/backends/skyrl_train/utils/):
//   ppo_policy_loss            ppo_utils.py:555-588      (policy loss types "regular", "dual_clip")
//   cross_entropy_loss         ppo_utils.py:1056-1092
//   importance_sampling_loss   ppo_utils.py:1095-1142
//   reduce_loss                ppo_utils.py:1145-1149
//   compute_approx_kl          ppo_utils.py:88-126
//   masked_mean, safe_exp_delta   torch_utils.py:180-192
#include <hip/hip_runtime.h>
#include <math.h>
#include <stdint.h>

#include <cmath>

#include "../../include/skyrl_lmhead.h"

namespace {

// ------------------------------------------------------------------------------------------------------------
// Policy loss and its gradient in one pass.
//   regular / dual clip (ppo_utils.py:555-588):
//     ratio = exp(clamp(lp - old, -20, 20));  surr1 = ratio * A;  surr2 = clamp(ratio, 1 - lo, 1 + hi) * A
//     loss  = -min(surr1, surr2);   dual clip: loss = A < 0 ? min(-A * c, loss) : loss
//     out   = { sum loss * mask * weight,  sum [surr2 < surr1] * mask,  sum mask }
//   cross entropy (:1056-1092):        loss = -lp;                         out[1] = 0
//   importance sampling (:1095-1142):  loss = -exp(lp - old) * A (no clamp);   out[1] = sum exp(lp - old) * mask
//     g     = d(sum loss * mask * weight) / d lp      (min and clamp differentiate as torch does: ties of min split
//             evenly, clamp passes the gradient on its closed interval)
// `weight` carries whatever multiplies the loss without depending on lp (the off-policy importance ratio).
// One workgroup: the data is a few hundred KiB, and a fixed reduction order keeps the sums bit-reproducible.
// ------------------------------------------------------------------------------------------------------------
// One token of the policy loss: value, derivative with respect to lp, and the statistic summed for the metric.
// (lo, hi, c) are the type's three parameters as the header lists them; row_lr is the masked row mean of lp - old, used by
// the sequence-level type only.
__device__ __forceinline__ void policy_term(int type, float lp, float old, float A, float lo, float hi, float c, float row_lr,
                                            float& loss, float& dloss, float& stat) {
  if (type == SKYRL_POLICY_LOSS_CROSS_ENTROPY) {
    loss = -lp;
    dloss = -1.f;
    stat = 0.f;
    return;
  }
  if (type == SKYRL_POLICY_LOSS_IMPORTANCE_SAMPLING) {
    const float ratio = expf(lp - old);
    loss = -(ratio * A);
    dloss = loss;
    stat = ratio;
    return;
  }
  if (type == SKYRL_POLICY_LOSS_KL_COV) {  // c = ppo_kl_coef, row_lr = this token's selector (1: the |log-ratio| penalty applies)
    const float delta = lp - old, ratio = expf(delta);
    loss = -(ratio * A) + c * row_lr * fabsf(delta);
    dloss = -(ratio * A) + c * row_lr * (delta > 0.f ? 1.f : (delta < 0.f ? -1.f : 0.f));
    stat = row_lr;
    return;
  }
  if (type == SKYRL_POLICY_LOSS_CLIP_COV) {  // the clipped surrogate on the unclamped ratio; the selection comes in as the weight
    const float ratio = expf(lp - old);
    const float pg1 = -A * ratio, pg2 = -A * fminf(fmaxf(ratio, lo), hi);
    const float d1 = pg1, d2 = (ratio >= lo && ratio <= hi) ? pg1 : 0.f;
    loss = fmaxf(pg1, pg2);
    dloss = pg1 > pg2 ? d1 : (pg1 < pg2 ? d2 : 0.5f * (d1 + d2));
    stat = pg2 > pg1 ? 1.f : 0.f;
    return;
  }
  // safe_exp_delta: the log-ratio clamped to +-20; the clamp passes the gradient on its closed interval
  const float delta = lp - old;
  float ratio = expf(fminf(fmaxf(delta, -20.f), 20.f));
  float d_ratio = (delta >= -20.f && delta <= 20.f) ? ratio : 0.f;  // d ratio / d lp
  if (type == SKYRL_POLICY_LOSS_GSPO) {  // the sequence's ratio for every token, clamp(max = 10) on the log
    ratio = expf(fminf(row_lr, 10.f));
    d_ratio = row_lr <= 10.f ? ratio : 0.f;
  }
  if (type == SKYRL_POLICY_LOSS_SAPO) {  // lo = tau_pos, hi = tau_neg
    const float tau = A > 0.f ? lo : hi;
    const float sg = 1.f / (1.f + expf(-tau * (ratio - 1.f)));
    loss = -(sg * (4.f / tau)) * A;
    dloss = -4.f * A * sg * (1.f - sg) * d_ratio;
    stat = 0.f;
    return;
  }
  if (type == SKYRL_POLICY_LOSS_CISPO) {  // lo, hi: bounds of the stop-gradient weight; the gradient flows through lp only
    const float w = fminf(fmaxf(ratio, lo), hi);
    loss = -A * w * lp;
    dloss = -A * w;
    stat = (ratio < lo || ratio > hi) ? 1.f : 0.f;
    return;
  }
  if (type == SKYRL_POLICY_LOSS_ROLLOUT_IS) {  // old = rollout log-probabilities; weight zeroed outside the open interval
    const bool in_range = ratio > lo && ratio < hi;
    const float w = in_range ? ratio : 0.f;
    loss = -(w * A * lp);
    dloss = -(w * A);
    stat = in_range ? 0.f : 1.f;
    return;
  }
  if (type == SKYRL_POLICY_LOSS_DPPO_TV || type == SKYRL_POLICY_LOSS_DPPO_KL) {  // lo = delta_low, hi = delta_high
    const float p = expf(lp), pm = expf(old), diff = p - pm;
    bool keep = true;
    if (type == SKYRL_POLICY_LOSS_DPPO_TV) {
      if ((A > 0.f && diff > hi) || (A < 0.f && -diff > lo)) keep = false;
    } else {
      const float eps = 1e-8f;
      const float bkl = pm * (old - lp) + (1.f - pm) * logf((1.f - pm + eps) / (1.f - p + eps));
      if ((A > 0.f && diff > 0.f && bkl > hi) || (A < 0.f && diff < 0.f && bkl > lo)) keep = false;
    }
    loss = keep ? -(ratio * A) : 0.f;
    dloss = keep ? -(d_ratio * A) : 0.f;
    stat = keep ? 0.f : 1.f;
    return;
  }
  // REGULAR, DUAL_CLIP, GSPO: the clipped surrogate
  const float surr1 = ratio * A;
  const float rc = fminf(fmaxf(ratio, lo), hi);
  const float surr2 = rc * A;
  const float d1 = d_ratio * A;
  const float d2 = (ratio >= lo && ratio <= hi) ? d_ratio * A : 0.f;
  loss = -fminf(surr1, surr2);
  dloss = surr1 < surr2 ? -d1 : (surr1 > surr2 ? -d2 : -0.5f * (d1 + d2));
  stat = surr2 < surr1 ? 1.f : 0.f;
  if (type == SKYRL_POLICY_LOSS_DUAL_CLIP && A < 0.f) {
    const float pg3 = -A * c;
    if (pg3 < loss) {
      loss = pg3;
      dloss = 0.f;
    } else if (pg3 == loss) {
      dloss *= 0.5f;
    }
  }
}

// The interval parameters of a type: clip types take (1 - eps_low, 1 + eps_high), the others their two values as given.
__device__ __forceinline__ bool is_interval_type(int type) {
  return type == SKYRL_POLICY_LOSS_REGULAR || type == SKYRL_POLICY_LOSS_DUAL_CLIP || type == SKYRL_POLICY_LOSS_GSPO ||
         type == SKYRL_POLICY_LOSS_CISPO || type == SKYRL_POLICY_LOSS_ROLLOUT_IS || type == SKYRL_POLICY_LOSS_CLIP_COV;
}

// Workgroup b sums tokens [b * slice, (b + 1) * slice) in a fixed order and writes its three sums to out[k * out_stride + b]:
// with one workgroup that is the result itself, with several the partial sums policy_loss_finish_kernel adds up.
__global__ __launch_bounds__(1024) void policy_loss_kernel(const float* __restrict__ lp, const float* __restrict__ old,
                                                           const float* __restrict__ adv, const float* __restrict__ mask,
                                                           const float* __restrict__ weight, int64_t T, int64_t slice,
                                                           float eps_low, float eps_high, float clip_c, int type,
                                                           float* __restrict__ out, int out_stride, float* __restrict__ g) {
  __shared__ float red[3][16];
  float s_loss = 0.f, s_clip = 0.f, s_mask = 0.f;
  const float lo = is_interval_type(type) ? 1.f - eps_low : eps_low, hi = is_interval_type(type) ? 1.f + eps_high : eps_high;
  const int64_t t0 = (int64_t)blockIdx.x * slice, t1 = t0 + slice < T ? t0 + slice : T;
  for (int64_t t = t0 + threadIdx.x; t < t1; t += blockDim.x) {
    float loss, dloss, stat;
    const bool ce = type == SKYRL_POLICY_LOSS_CROSS_ENTROPY;  // reads neither old nor adv
    const bool selector = type == SKYRL_POLICY_LOSS_KL_COV;  // the weight array selects tokens instead of scaling the loss
    policy_term(type, lp[t], ce ? 0.f : old[t], ce ? 0.f : adv[t], lo, hi, clip_c, (selector && weight) ? weight[t] : 0.f, loss,
                dloss, stat);
    const float m = mask ? mask[t] : 1.f;
    const float w = (weight && !selector) ? m * weight[t] : m;
    s_loss += loss * w;
    s_clip += stat * m;
    s_mask += m;
    if (g) g[t] = dloss * w;
  }
  // wave reduction, then across the 16 waves
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) {
    s_loss += __shfl_xor(s_loss, off, 64);
    s_clip += __shfl_xor(s_clip, off, 64);
    s_mask += __shfl_xor(s_mask, off, 64);
  }
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  if (lane == 0) red[0][wave] = s_loss, red[1][wave] = s_clip, red[2][wave] = s_mask;
  __syncthreads();
  if (threadIdx.x < 3) {
    float v = 0.f;
    for (int k = 0; k < (int)(blockDim.x >> 6); ++k) v += red[threadIdx.x][k];
    out[threadIdx.x * out_stride + blockIdx.x] = v;
  }
}

constexpr int kMaxLossSlices = SKYRL_POLICY_LOSS_PARTIALS;
constexpr int64_t kLossSliceTokens = 8192;  // at least this many tokens per workgroup

// One wave: lane l adds the partial sums of slices l, l + 64, ..., then the lanes meet in a fixed tree -- the same order on
// every run, and no chain of dependent loads through one thread.
__global__ __launch_bounds__(64) void policy_loss_finish_kernel(const float* __restrict__ partials, int slices,
                                                                float* __restrict__ out) {
  float v[3] = {0.f, 0.f, 0.f};
  for (int b = threadIdx.x; b < slices; b += 64)
#pragma unroll
    for (int k = 0; k < 3; ++k) v[k] += partials[k * kMaxLossSlices + b];
#pragma unroll
  for (int off = 32; off > 0; off >>= 1)
#pragma unroll
    for (int k = 0; k < 3; ++k) v[k] += __shfl_xor(v[k], off, 64);
  if (threadIdx.x == 0) out[0] = v[0], out[1] = v[1], out[2] = v[2];
}

// ------------------------------------------------------------------------------------------------------------
// Statistics of |logprobs - rollout_logprobs| over the loss tokens of a micro-batch (workers/worker_utils.py:34-58):
//     mean = sum |d| m / max(sum m, 1),  sq_mean = sum d^2 m / max(sum m, 1),  max / min of |d| m      (m = 1 without a mask:
//     plain means).  Workgroup b sweeps tokens [b * slice, (b + 1) * slice) and writes its five partial results to
// part[k * kMaxLossSlices + b]; logprob_diff_finish_kernel merges them in a fixed order.  Maximum and minimum hand a NaN on,
// as Tensor.max() does.
// ------------------------------------------------------------------------------------------------------------
__device__ __forceinline__ float max_nan(float a, float b) { return (a > b || a != a) ? a : b; }
__device__ __forceinline__ float min_nan(float a, float b) { return (a < b || a != a) ? a : b; }

__global__ __launch_bounds__(1024) void logprob_diff_kernel(const float* __restrict__ lp, const float* __restrict__ rollout,
                                                            const float* __restrict__ mask, int64_t n, int64_t slice,
                                                            float* __restrict__ part) {
  __shared__ float red[5][16];
  float s_abs = 0.f, s_sq = 0.f, s_m = 0.f, mx = -INFINITY, mn = INFINITY;
  const int64_t t0 = (int64_t)blockIdx.x * slice, t1 = t0 + slice < n ? t0 + slice : n;
  auto token = [&](float a, float b, float m) {
    const float d = fabsf(a - b);
    const float dm = mask ? d * m : d;
    s_abs += dm;
    s_sq += mask ? d * d * m : d * d;
    s_m += m;
    mx = max_nan(dm, mx), mn = min_nan(dm, mn);
  };
  // 16-byte loads where the slice allows them (slices start at multiples of four tokens when vec is set)
  const bool vec = (slice & 3) == 0 && (((uintptr_t)lp | (uintptr_t)rollout | (uintptr_t)mask) & 15) == 0;
  int64_t t = t0;
  if (vec) {
    const int64_t quads = (t1 - t0) >> 2;
    const float4* __restrict__ lp4 = (const float4*)(lp + t0);
    const float4* __restrict__ ro4 = (const float4*)(rollout + t0);
    const float4* __restrict__ m4 = mask ? (const float4*)(mask + t0) : nullptr;
    // four pieces per array in flight per thread: a slice of 16384 tokens is one batch of loads for the 1024 threads
    for (int64_t i0 = threadIdx.x; i0 < quads; i0 += 4 * (int64_t)blockDim.x) {
      float4 a[4], b[4], m[4];
#pragma unroll
      for (int u = 0; u < 4; ++u) {
        const int64_t i = i0 + u * (int64_t)blockDim.x;
        if (i < quads) {
          a[u] = lp4[i], b[u] = ro4[i];
          m[u] = m4 ? m4[i] : make_float4(1.f, 1.f, 1.f, 1.f);
        }
      }
#pragma unroll
      for (int u = 0; u < 4; ++u)
        if (i0 + u * (int64_t)blockDim.x < quads)
          token(a[u].x, b[u].x, m[u].x), token(a[u].y, b[u].y, m[u].y), token(a[u].z, b[u].z, m[u].z), token(a[u].w, b[u].w, m[u].w);
    }
    t = t0 + (quads << 2);
  }
  for (t += threadIdx.x; t < t1; t += blockDim.x) token(lp[t], rollout[t], mask ? mask[t] : 1.f);
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) {
    s_abs += __shfl_xor(s_abs, off, 64);
    s_sq += __shfl_xor(s_sq, off, 64);
    s_m += __shfl_xor(s_m, off, 64);
    mx = max_nan(__shfl_xor(mx, off, 64), mx);
    mn = min_nan(__shfl_xor(mn, off, 64), mn);
  }
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  if (lane == 0) red[0][wave] = s_abs, red[1][wave] = s_sq, red[2][wave] = s_m, red[3][wave] = mx, red[4][wave] = mn;
  __syncthreads();
  if (threadIdx.x < 5) {
    const int k = threadIdx.x;
    float v = red[k][0];
    for (int w = 1; w < 16; ++w) v = k < 3 ? v + red[k][w] : (k == 3 ? max_nan(red[k][w], v) : min_nan(red[k][w], v));
    part[k * kMaxLossSlices + blockIdx.x] = v;
  }
}

__global__ __launch_bounds__(64) void logprob_diff_finish_kernel(const float* __restrict__ part, int slices,
                                                                 float* __restrict__ out4) {
  double s_abs = 0.0, s_sq = 0.0, s_m = 0.0;
  float mx = -INFINITY, mn = INFINITY;
  for (int b = threadIdx.x; b < slices; b += 64) {  // lane l: slices l, l + 64, ...; then a fixed tree over the lanes
    s_abs += part[b], s_sq += part[kMaxLossSlices + b], s_m += part[2 * kMaxLossSlices + b];
    mx = max_nan(part[3 * kMaxLossSlices + b], mx), mn = min_nan(part[4 * kMaxLossSlices + b], mn);
  }
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) {
    s_abs += __shfl_xor(s_abs, off, 64), s_sq += __shfl_xor(s_sq, off, 64), s_m += __shfl_xor(s_m, off, 64);
    mx = max_nan(__shfl_xor(mx, off, 64), mx), mn = min_nan(__shfl_xor(mn, off, 64), mn);
  }
  if (threadIdx.x != 0) return;
  const double den = s_m > 1.0 ? s_m : 1.0;
  out4[0] = (float)(s_abs / den), out4[1] = (float)(s_sq / den), out4[2] = mx, out4[3] = mn;
}

constexpr int kRowThreads = 1024;  // one workgroup per row of [B, S]: rows are few and long

// Sum of one value per thread over the workgroup, in a fixed order; every thread receives it.
__device__ __forceinline__ float block_sum(float v, float* red) {
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) v += __shfl_xor(v, off, 64);
  __syncthreads();  // red may still be read from an earlier call
  if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = v;
  __syncthreads();
  float s = 0.f;
  for (int k = 0; k < kRowThreads / 64; ++k) s += red[k];
  return s;
}

// ------------------------------------------------------------------------------------------------------------
// Approximate KL between the policy and a base policy, per token (ppo_utils.py:88-126), reduced the way the trainer
// reduces it (workers/worker.py:1071-1077): masked mean over each row, then the mean over rows.
//   k1: d;  abs: |d|;  k2: d^2 / 2   with d = lp - base
//   k3: k = clamp(base - lp, -20, 20);  kld = clamp(exp(k) - k - 1, -10, 10)
//   kld_masked = mask != 0 ? kld * mask : 0            (the value compute_approx_kl returns)
//   row_mean_b = sum_s kld_masked * mask / max(sum_s mask, 1)      (masked_mean multiplies by the mask once more)
// One workgroup per row: mask sum, then values, row sum and gradient in a second sweep.  GRAD: 0 none, 1 the elementwise
// derivative d kld_masked / d lp, 2 the derivative of mean_b row_mean_b.
// ------------------------------------------------------------------------------------------------------------
// One token of the KL estimate: value and derivative with respect to lp (clamp passes the gradient on its closed interval,
// |.| has derivative 0 at 0, as torch differentiates them).
__device__ __forceinline__ void kl_term(int estimator, float lp, float base, float& kld, float& dk) {
  const float d = lp - base;
  if (estimator == SKYRL_KL_K1) {
    kld = d;
    dk = 1.f;
  } else if (estimator == SKYRL_KL_ABS) {
    kld = fabsf(d);
    dk = d > 0.f ? 1.f : (d < 0.f ? -1.f : 0.f);
  } else if (estimator == SKYRL_KL_K2) {
    kld = 0.5f * d * d;
    dk = d;
  } else {
    const float kraw = base - lp;
    const float k = fminf(fmaxf(kraw, -20.f), 20.f);
    const float ratio = expf(k);
    const float v = ratio - k - 1.f;
    kld = fminf(fmaxf(v, -10.f), 10.f);
    const bool open = kraw >= -20.f && kraw <= 20.f && v >= -10.f && v <= 10.f;
    dk = open ? 1.f - ratio : 0.f;  // d/d lp of exp(k) - k - 1 with k = base - lp
  }
}

__global__ __launch_bounds__(kRowThreads) void approx_kl_rows_kernel(const float* __restrict__ lp, const float* __restrict__ base,
                                                                     const float* __restrict__ mask, int64_t rows, int64_t cols,
                                                                     int estimator, int grad_mode, float* __restrict__ kld_out,
                                                                     float* __restrict__ row_mean, float* __restrict__ g) {
  __shared__ float red[kRowThreads / 64];
  const int64_t row0 = (int64_t)blockIdx.x * cols;
  float denom = (float)cols;
  if (mask) {
    float ms = 0.f;
    for (int64_t c = threadIdx.x; c < cols; c += kRowThreads) ms += mask[row0 + c];
    denom = fmaxf(block_sum(ms, red), 1.f);
  }
  const float gscale = 1.f / (denom * (float)rows);
  float acc = 0.f;
  for (int64_t c = threadIdx.x; c < cols; c += kRowThreads) {
    float kld, dk;
    kl_term(estimator, lp[row0 + c], base[row0 + c], kld, dk);
    float m = 1.f;
    if (mask) {
      m = mask[row0 + c];
      if (m != 0.f) {
        kld *= m;
        dk *= m;
      } else {
        kld = 0.f;
        dk = 0.f;
      }
    }
    if (kld_out) kld_out[row0 + c] = kld;
    acc += mask ? kld * m : kld;
    if (grad_mode == 1) g[row0 + c] = dk;
    if (grad_mode == 2) g[row0 + c] = (mask ? dk * m : dk) * gscale;
  }
  const float total = block_sum(acc, red);
  if (threadIdx.x == 0) row_mean[blockIdx.x] = total / denom;
}

// out[0] = sum_i v[i] * scale, one workgroup, fixed order.
__global__ __launch_bounds__(kRowThreads) void scaled_sum_kernel(const float* __restrict__ v, int64_t n, float scale,
                                                                 float* __restrict__ out) {
  __shared__ float red[kRowThreads / 64];
  float acc = 0.f;
  for (int64_t i = threadIdx.x; i < n; i += kRowThreads) acc += v[i];
  const float total = block_sum(acc, red);
  if (threadIdx.x == 0) out[0] = total * scale;
}

// ------------------------------------------------------------------------------------------------------------
// masked_mean (torch_utils.py:180-184).  Per row: means[b] = sum_s v * mask / max(sum_s mask, 1) (mask NULL: plain mean),
// dvalues = d means[b] / d v = mask / max(sum mask, 1).  The global form is the same kernel on one row of rows * cols.
// ------------------------------------------------------------------------------------------------------------
__global__ __launch_bounds__(kRowThreads) void masked_mean_rows_kernel(const float* __restrict__ v, const float* __restrict__ mask,
                                                                       int64_t cols, float* __restrict__ means,
                                                                       float* __restrict__ dv) {
  __shared__ float red[kRowThreads / 64];
  const int64_t row0 = (int64_t)blockIdx.x * cols;
  float sv = 0.f, sm = 0.f;
  for (int64_t c = threadIdx.x; c < cols; c += kRowThreads) {
    const float m = mask ? mask[row0 + c] : 1.f;
    sv += v[row0 + c] * m;
    sm += m;
  }
  const float total = block_sum(sv, red);
  const float denom = mask ? fmaxf(block_sum(sm, red), 1.f) : (float)cols;
  if (threadIdx.x == 0) means[blockIdx.x] = total / denom;
  if (dv) {
    const float r = 1.f / denom;
    for (int64_t c = threadIdx.x; c < cols; c += kRowThreads) dv[row0 + c] = mask ? mask[row0 + c] * r : r;
  }
}

// ------------------------------------------------------------------------------------------------------------
// The whole per-micro-batch actor loss in two launches (workers/worker.py:989-1089, megatron_model_wrapper.py:902-941):
//     loss = policy_scale * policy_loss  +  term_scale * ( kl_coef * kl  -  entropy_coef * entropy_mean )
//     policy_loss  = sum loss_token * mask * weight                                   (policy_term above, reduce_loss)
//     kl           = mean_b [ sum_s kld * mask / max(sum_s mask, 1) ]                  (kl_term above, masked_mean(dim=-1).mean())
//     entropy_mean = sum entropy * mask / max(sum mask, 1)                            (masked_mean over everything)
// and both upstream gradients of the LM-head backward:
//     dlogprobs = policy_scale * d policy_loss / d lp  +  term_scale * kl_coef * d kl / d lp
//     dentropy  = -term_scale * entropy_coef * mask / max(sum mask, 1)
// First launch, one workgroup per row: the row's sums and dlogprobs (the KL gradient needs only the row's own mask count).
// Second launch, one workgroup: the sums over rows in a fixed order, the six results, and dentropy, which needs the
// global mask count.
// ------------------------------------------------------------------------------------------------------------
struct ActorLossArgs {
  const float *lp, *old, *adv, *mask, *weight, *base, *entropy;
  int64_t rows, cols;
  int loss_type, kl_estimator;
  float lo, hi, clip_c, policy_scale, term_scale, kl_coef, entropy_coef;
  float* row_sums;  // [rows, 6]: policy loss, statistic, mask, kl row mean, entropy * mask, (unused)
  float* out;       // [6]: loss, policy_loss, statistic, mask count, kl, entropy_mean
  float *dlp, *dent;
};

__global__ __launch_bounds__(kRowThreads) void actor_loss_rows_kernel(const ActorLossArgs a) {
  __shared__ float red[kRowThreads / 64];
  const int64_t row0 = (int64_t)blockIdx.x * a.cols;
  float msum = 0.f;
  if (a.mask)
    for (int64_t c = threadIdx.x; c < a.cols; c += kRowThreads) msum += a.mask[row0 + c];
  const float row_mask = a.mask ? block_sum(msum, red) : (float)a.cols;
  float row_lr = 0.f;  // masked mean of lp - old over the row: the sequence-level log-ratio
  if (a.loss_type == SKYRL_POLICY_LOSS_GSPO) {
    float lr = 0.f;
    for (int64_t c = threadIdx.x; c < a.cols; c += kRowThreads)
      lr += (a.lp[row0 + c] - a.old[row0 + c]) * (a.mask ? a.mask[row0 + c] : 1.f);
    row_lr = block_sum(lr, red) / (a.mask ? fmaxf(row_mask, 1.f) : (float)a.cols);
  }
  const float kl_denom = fmaxf(row_mask, 1.f);
  const float kl_gscale = a.term_scale * a.kl_coef / (kl_denom * (float)a.rows);
  const bool ce = a.loss_type == SKYRL_POLICY_LOSS_CROSS_ENTROPY;
  float s_loss = 0.f, s_stat = 0.f, s_kl = 0.f, s_ent = 0.f;
  for (int64_t c = threadIdx.x; c < a.cols; c += kRowThreads) {
    const int64_t i = row0 + c;
    const float lp = a.lp[i];
    const float m = a.mask ? a.mask[i] : 1.f;
    float loss, dloss, stat;
    policy_term(a.loss_type, lp, ce ? 0.f : a.old[i], ce ? 0.f : a.adv[i], a.lo, a.hi, a.clip_c, row_lr, loss, dloss, stat);
    const float w = a.weight ? m * a.weight[i] : m;
    s_loss += loss * w;
    s_stat += stat * m;
    float g = a.policy_scale * dloss * w;
    if (a.base) {
      float kld, dk;
      kl_term(a.kl_estimator, lp, a.base[i], kld, dk);
      // compute_approx_kl zeroes masked positions with where(); masked_mean multiplies by the mask once more
      const float km = a.mask ? (m != 0.f ? m * m : 0.f) : 1.f;
      s_kl += kld * km;
      g += dk * km * kl_gscale;
    }
    if (a.entropy) s_ent += a.entropy[i] * m;
    if (a.dlp) a.dlp[i] = g;
  }
  const float t_loss = block_sum(s_loss, red), t_stat = block_sum(s_stat, red);
  const float t_kl = a.base ? block_sum(s_kl, red) : 0.f;
  const float t_ent = a.entropy ? block_sum(s_ent, red) : 0.f;
  if (threadIdx.x == 0) {
    float* r = a.row_sums + (int64_t)blockIdx.x * 6;
    r[0] = t_loss, r[1] = t_stat, r[2] = row_mask, r[3] = t_kl / kl_denom, r[4] = t_ent, r[5] = 0.f;
  }
}

__global__ __launch_bounds__(kRowThreads) void actor_loss_finish_kernel(const ActorLossArgs a) {
  __shared__ float red[kRowThreads / 64];
  float v[5] = {0.f, 0.f, 0.f, 0.f, 0.f};
  for (int64_t r = threadIdx.x; r < a.rows; r += kRowThreads)
    for (int k = 0; k < 5; ++k) v[k] += a.row_sums[r * 6 + k];
  float t[5];
  for (int k = 0; k < 5; ++k) t[k] = block_sum(v[k], red);
  const float mask_denom = fmaxf(t[2], 1.f);
  const float kl = t[3] / (float)a.rows, ent = t[4] / mask_denom;
  if (threadIdx.x == 0) {
    a.out[0] = a.policy_scale * t[0] + a.term_scale * (a.kl_coef * kl - a.entropy_coef * ent);
    a.out[1] = t[0], a.out[2] = t[1], a.out[3] = t[2], a.out[4] = kl, a.out[5] = ent;
  }
}

// d loss / d entropy = -term_scale * entropy_coef * mask / max(sum mask, 1): elementwise once the finish kernel has the count.
__global__ __launch_bounds__(256) void actor_loss_dentropy_kernel(const ActorLossArgs a) {
  const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (i >= a.rows * a.cols) return;
  const float c = -a.term_scale * a.entropy_coef / fmaxf(a.out[3], 1.f);
  a.dent[i] = a.mask ? c * a.mask[i] : c;
}


// ------------------------------------------------------------------------------------------------------------
// Off-policy correction from the rollout engine's log-probabilities (utils/off_policy_correction_utils.py:257-348, the
// steps in the reference's order), one workgroup per row of [B, S]:
//   r = exp(clamp(old - rollout, -20, 20)) per token
//   1. outlier rows (:75-134):  a row with any unmasked token whose r > high or r < low loses its whole mask
//   2. token mask (:137-188):   unmasked tokens with r outside [low, high] lose their mask
//   3. TIS weight (:24-72):     "token": min(r, cap);  "sequence": min(exp(clamp(sum (old - rollout) * mask)), cap) of the row
//   4. sequence mask (:191-254): "geometric": exp(clamp(sum (old - rollout) * mask / max(sum mask, 1))) outside [low, high],
//                                "product": the row's product ratio outside [low, high] -> the row loses its mask
// Steps 3 and 4 see the mask that steps 1 and 2 left.  Outputs: keep [B, S] in {0, 1} (mask_out = mask * keep is what the
// reference returns), tis [B, S] (the row's value repeated for "sequence"), weight = tis * keep (what multiplies a
// per-token loss next to the ORIGINAL mask: the reference's losses count their clip statistic with the original mask and
// sum the loss with the new one, ppo_utils.py:570-587), and SKYRL_OFF_POLICY_ROW_STATS floats per row from which a one-workgroup kernel forms the
// reference's metrics in a fixed order.
// ------------------------------------------------------------------------------------------------------------
struct OffPolicyArgs {
  const float *old, *rollout, *mask;  // mask may be NULL (all ones)
  int64_t rows, cols;
  int tis_type, seq_metric;           // 0 = off; tis 1 token, 2 sequence; metric 1 geometric, 2 product
  float tis_cap, seq_low, seq_high;
  int use_outlier_low, use_outlier_high, use_token_mask;
  float outlier_low, outlier_high, token_low, token_high;
  float *keep_out, *tis_out, *weight_out;  // each may be NULL
  float *row_stats, *metrics;              // [rows, SKYRL_OFF_POLICY_ROW_STATS], [SKYRL_OFF_POLICY_METRICS]
};
enum {
  kOpSumRatioMask = 0, kOpSumMask, kOpSumX, kOpSumXX, kOpMaxX, kOpMinX, kOpRowInvalid, kOpRowOver, kOpRowUnder, kOpValidTokens,
  kOpMaskedTokens, kOpTokens2, kOpCapped, kOpSeqCapped, kOpSeqOver, kOpSeqUnder, kOpSeqMasked,
  kOpRowStats = SKYRL_OFF_POLICY_ROW_STATS
};
static_assert(kOpSeqMasked < kOpRowStats, "row statistics do not fit their slots");

__device__ __forceinline__ float block_max(float v, float* red) {
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) v = fmaxf(v, __shfl_xor(v, off, 64));
  __syncthreads();
  if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = v;
  __syncthreads();
  float s = red[0];
  for (int k = 1; k < kRowThreads / 64; ++k) s = fmaxf(s, red[k]);
  return s;
}

// exp of a log-ratio clamped to +-20 (utils/off_policy_correction_utils.py: _safe_exp_delta).  fmaxf / fminf drop a NaN;
// torch.clamp passes it on, and so does this: a NaN log-probability must show in the weights, the metrics and the loss.
__device__ __forceinline__ float safe_exp_delta(float delta) {
  return delta != delta ? delta : expf(fminf(fmaxf(delta, -20.f), 20.f));
}

__global__ __launch_bounds__(kRowThreads) void off_policy_rows_kernel(const OffPolicyArgs a) {
  __shared__ float red[kRowThreads / 64];
  const int64_t row0 = (int64_t)blockIdx.x * a.cols;
  const bool outlier = a.use_outlier_low || a.use_outlier_high;
  float s_rm = 0.f, s_m = 0.f, s_x = 0.f, s_xx = 0.f, mx = -INFINITY, mn = INFINITY;
  float over = 0.f, under = 0.f, pos = 0.f, oob = 0.f, dm2 = 0.f, m2s = 0.f, pos2 = 0.f, capped = 0.f;
  for (int64_t c = threadIdx.x; c < a.cols; c += kRowThreads) {
    const float delta = a.old[row0 + c] - a.rollout[row0 + c];
    const float r = safe_exp_delta(delta);
    const float m = a.mask ? a.mask[row0 + c] : 1.f;
    const float x = r * m;
    // the two sums behind the standard deviation are taken of x - 1 (the variance does not move with the shift): ratios sit
    // near 1, and sums of x and x^2 themselves would cancel to nothing when the spread is far below the mean
    s_rm += x, s_m += m, s_x += x - 1.f, s_xx += (x - 1.f) * (x - 1.f);
    mx = fmaxf(mx, x), mn = fminf(mn, x);
    const bool live = m > 0.f;
    if (a.use_outlier_high && live && r > a.outlier_high) over = 1.f;
    if (a.use_outlier_low && live && r < a.outlier_low) under = 1.f;
    const bool in_bounds = !a.use_token_mask || (r >= a.token_low && r <= a.token_high);
    pos += live ? 1.f : 0.f;
    oob += (live && !in_bounds) ? 1.f : 0.f;
    const float m2 = (in_bounds || m == 0.f) ? m : 0.f;  // the mask after step 2, if the row survives step 1
    dm2 = fmaf(delta, m2, dm2);
    m2s += m2;
    pos2 += m2 > 0.f ? 1.f : 0.f;
    capped += (a.tis_type == 1 && m2 > 0.f && r > a.tis_cap) ? 1.f : 0.f;
  }
  s_rm = block_sum(s_rm, red), s_m = block_sum(s_m, red), s_x = block_sum(s_x, red), s_xx = block_sum(s_xx, red);
  mx = block_max(mx, red), mn = -block_max(-mn, red);
  if (s_x != s_x) mx = mn = s_x;  // a NaN ratio in the row: the extremes are NaN as well (fmaxf had dropped it)
  over = block_max(over, red), under = block_max(under, red);
  pos = block_sum(pos, red), oob = block_sum(oob, red), dm2 = block_sum(dm2, red), m2s = block_sum(m2s, red);
  pos2 = block_sum(pos2, red), capped = block_sum(capped, red);
  const bool valid = !(outlier && (over > 0.f || under > 0.f));
  if (!valid) pos = 0.f, oob = 0.f, dm2 = 0.f, m2s = 0.f, pos2 = 0.f, capped = 0.f;  // the row's mask is gone from step 1 on
  const float seq_ratio = safe_exp_delta(dm2);
  float tis_row = 1.f, seq_capped = 0.f;
  if (a.tis_type == 2) {
    seq_capped = seq_ratio > a.tis_cap ? 1.f : 0.f;
    tis_row = seq_ratio != seq_ratio ? seq_ratio : fminf(seq_ratio, a.tis_cap);
  }
  float seq_over = 0.f, seq_under = 0.f;
  if (a.seq_metric) {
    const float v = a.seq_metric == 1 ? safe_exp_delta(dm2 / fmaxf(m2s, 1.f)) : seq_ratio;
    seq_over = v > a.seq_high ? 1.f : 0.f;
    seq_under = v < a.seq_low ? 1.f : 0.f;
  }
  const bool keep_row = valid && seq_over == 0.f && seq_under == 0.f;
  for (int64_t c = threadIdx.x; c < a.cols; c += kRowThreads) {
    const float delta = a.old[row0 + c] - a.rollout[row0 + c];
    const float r = safe_exp_delta(delta);
    const float m = a.mask ? a.mask[row0 + c] : 1.f;
    const bool in_bounds = !a.use_token_mask || (r >= a.token_low && r <= a.token_high);
    const float keep = (keep_row && (in_bounds || m == 0.f)) ? 1.f : 0.f;
    const float tis = a.tis_type == 1 ? (r != r ? r : fminf(r, a.tis_cap)) : tis_row;  // torch.clamp keeps a NaN
    if (a.keep_out) a.keep_out[row0 + c] = keep;
    if (a.tis_out) a.tis_out[row0 + c] = tis;
    if (a.weight_out) a.weight_out[row0 + c] = tis * keep;
  }
  if (threadIdx.x == 0) {
    float* st = a.row_stats + (int64_t)blockIdx.x * kOpRowStats;
    st[kOpSumRatioMask] = s_rm, st[kOpSumMask] = s_m, st[kOpSumX] = s_x, st[kOpSumXX] = s_xx, st[kOpMaxX] = mx, st[kOpMinX] = mn;
    st[kOpRowInvalid] = valid ? 0.f : 1.f, st[kOpRowOver] = over, st[kOpRowUnder] = under;
    st[kOpValidTokens] = pos, st[kOpMaskedTokens] = oob, st[kOpTokens2] = pos2, st[kOpCapped] = capped;
    st[kOpSeqCapped] = seq_capped, st[kOpSeqOver] = seq_over, st[kOpSeqUnder] = seq_under;
    st[kOpSeqMasked] = (seq_over > 0.f || seq_under > 0.f) ? 1.f : 0.f;
  }
}

// metrics: 0 is_ratio_mean, 1 is_ratio_std, 2 is_ratio_max, 3 is_ratio_min, 4 outlier_seq_masked_ratio, 5 outlier_seq_over_high_ratio,
// 6 outlier_seq_under_low_ratio, 7 token_mask_ratio, 8 tis_token_clip_high_ratio, 9 tis_seq_clip_high_ratio,
// 10 sequence-mask masked ratio, 11 its over-high ratio, 12 its under-low ratio.  Rows are added in order, in fp64.
__global__ __launch_bounds__(64) void off_policy_finish_kernel(const OffPolicyArgs a) {
  // lane l adds rows l, l + 64, ... in order; lane 0 then adds the 64 partial sums in lane order: a fixed order for any rows
  __shared__ double part[64][kOpRowStats];
  __shared__ double part_max[64], part_min[64];
  {
    double s[kOpRowStats];
    for (int k = 0; k < kOpRowStats; ++k) s[k] = 0.0;
    double mx = -INFINITY, mn = INFINITY;
    for (int64_t r = threadIdx.x; r < a.rows; r += 64) {
      const float* st = a.row_stats + r * kOpRowStats;
      for (int k = 0; k < kOpRowStats; ++k) s[k] += (double)st[k];
      const double rx = (double)st[kOpMaxX], rn = (double)st[kOpMinX];
      mx = (rx != rx || mx != mx) ? NAN : fmax(mx, rx), mn = (rn != rn || mn != mn) ? NAN : fmin(mn, rn);
    }
    for (int k = 0; k < kOpRowStats; ++k) part[threadIdx.x][k] = s[k];
    part_max[threadIdx.x] = mx, part_min[threadIdx.x] = mn;
  }
  __syncthreads();
  if (threadIdx.x != 0) return;
  double s[kOpRowStats];
  for (int k = 0; k < kOpRowStats; ++k) s[k] = 0.0;
  double mx = -INFINITY, mn = INFINITY;
  for (int l = 0; l < 64; ++l) {
    for (int k = 0; k < kOpRowStats; ++k) s[k] += part[l][k];
    mx = (part_max[l] != part_max[l] || mx != mx) ? NAN : fmax(mx, part_max[l]);
    mn = (part_min[l] != part_min[l] || mn != mn) ? NAN : fmin(mn, part_min[l]);
  }
  const double n = (double)a.rows * (double)a.cols, rows = (double)a.rows;
  float* o = a.metrics;
  o[0] = (float)(s[kOpSumRatioMask] / fmax(s[kOpSumMask], 1.0));
  // unbiased, as Tensor.std(): NaN for a single element (the two sums are of x - 1, see the row kernel)
  const double var = (s[kOpSumXX] - s[kOpSumX] * s[kOpSumX] / n) / (n - 1.0);
  o[1] = (n > 1.0 && var == var) ? (float)sqrt(fmax(var, 0.0)) : NAN;  // fmax would turn a NaN variance into 0
  o[2] = (float)mx, o[3] = (float)mn;
  o[4] = (float)(s[kOpRowInvalid] / rows), o[5] = (float)(s[kOpRowOver] / rows), o[6] = (float)(s[kOpRowUnder] / rows);
  o[7] = (float)(s[kOpMaskedTokens] / fmax(s[kOpValidTokens], 1.0));
  o[8] = (float)(s[kOpCapped] / fmax(s[kOpTokens2], 1.0));
  o[9] = (float)(s[kOpSeqCapped] / rows);
  o[10] = (float)(s[kOpSeqMasked] / rows), o[11] = (float)(s[kOpSeqOver] / rows), o[12] = (float)(s[kOpSeqUnder] / rows);
  o[13] = o[14] = o[15] = 0.f;
}

bool finite(float x) { return std::isfinite(x); }
bool valid_loss_type(int t) { return t >= SKYRL_POLICY_LOSS_REGULAR && t <= SKYRL_POLICY_LOSS_DPPO_KL; }
bool interval_type(int t) {
  return t == SKYRL_POLICY_LOSS_REGULAR || t == SKYRL_POLICY_LOSS_DUAL_CLIP || t == SKYRL_POLICY_LOSS_GSPO ||
         t == SKYRL_POLICY_LOSS_CISPO || t == SKYRL_POLICY_LOSS_ROLLOUT_IS;
}
// Types that read their two parameters need them finite (SAPO's temperatures also non-zero); the dual clip its third.
bool valid_loss_params(int t, float a, float b, float c) {
  if (t == SKYRL_POLICY_LOSS_CROSS_ENTROPY || t == SKYRL_POLICY_LOSS_IMPORTANCE_SAMPLING) return true;
  if (t == SKYRL_POLICY_LOSS_KL_COV) return finite(c);
  if (!finite(a) || !finite(b)) return false;
  if (t == SKYRL_POLICY_LOSS_SAPO && (a == 0.f || b == 0.f)) return false;
  return t != SKYRL_POLICY_LOSS_DUAL_CLIP || finite(c);
}

}  // namespace

extern "C" {

int skyrl_ppo_policy_loss(const float* logprobs, const float* old_logprobs, const float* advantages, const float* loss_mask,
                          const float* loss_weight, int64_t T, float eps_clip_low, float eps_clip_high, float clip_ratio_c,
                          int loss_type, float* out3, float* dlogprobs, float* partials, void* stream) {
  // the sequence-level type needs rows: it is part of skyrl_actor_loss only
  const bool cov_type = loss_type == SKYRL_POLICY_LOSS_CLIP_COV || loss_type == SKYRL_POLICY_LOSS_KL_COV;  // this entry point only
  if ((!valid_loss_type(loss_type) && !cov_type) || loss_type == SKYRL_POLICY_LOSS_GSPO) return SKYRL_LMHEAD_ERR_ARG;
  const bool needs_old = loss_type != SKYRL_POLICY_LOSS_CROSS_ENTROPY;
  if (!logprobs || !out3 || (needs_old && (!old_logprobs || !advantages))) return SKYRL_LMHEAD_ERR_NULL;
  if (T < 1) return SKYRL_LMHEAD_ERR_SHAPE;
  if (!valid_loss_params(loss_type, eps_clip_low, eps_clip_high, clip_ratio_c)) return SKYRL_LMHEAD_ERR_ARG;
  // One workgroup up to kLossSliceTokens tokens; beyond that the tokens are cut into equal slices (a fixed number for a given
  // T, so the result is reproducible) whose partial sums a second launch adds in order.
  int64_t slices = (T + kLossSliceTokens - 1) / kLossSliceTokens;
  if (slices > kMaxLossSlices) slices = kMaxLossSlices;
  if (slices > 1 && !partials) return SKYRL_LMHEAD_ERR_WORKSPACE;
  const int64_t slice = (T + slices - 1) / slices;
  hipStream_t s = (hipStream_t)stream;
  hipLaunchKernelGGL(policy_loss_kernel, dim3((unsigned)slices), dim3(1024), 0, s, logprobs, old_logprobs, advantages, loss_mask,
                     loss_weight, T, slice, eps_clip_low, eps_clip_high, clip_ratio_c, loss_type, slices > 1 ? partials : out3,
                     slices > 1 ? kMaxLossSlices : 1, dlogprobs);
  if (slices > 1) hipLaunchKernelGGL(policy_loss_finish_kernel, dim3(1), dim3(64), 0, s, partials, (int)slices, out3);
  return (int)hipGetLastError();
}

int skyrl_approx_kl(const float* logprobs, const float* base_logprobs, const float* loss_mask, int64_t rows, int64_t cols,
                    int estimator, float* kld, float* row_mean, float* mean, int grad_mode, float* dlogprobs, void* stream) {
  if (!logprobs || !base_logprobs || !row_mean || !mean) return SKYRL_LMHEAD_ERR_NULL;
  if (grad_mode < 0 || grad_mode > 2 || estimator < SKYRL_KL_K1 || estimator > SKYRL_KL_K3) return SKYRL_LMHEAD_ERR_ARG;
  if (grad_mode != 0 && !dlogprobs) return SKYRL_LMHEAD_ERR_NULL;
  if (rows < 1 || cols < 1 || rows >= (int64_t(1) << 31) || cols >= (int64_t(1) << 31)) return SKYRL_LMHEAD_ERR_SHAPE;
  hipStream_t s = (hipStream_t)stream;
  hipLaunchKernelGGL(approx_kl_rows_kernel, dim3((unsigned)rows), dim3(kRowThreads), 0, s, logprobs, base_logprobs, loss_mask,
                     rows, cols, estimator, grad_mode, kld, row_mean, dlogprobs);
  hipLaunchKernelGGL(scaled_sum_kernel, dim3(1), dim3(kRowThreads), 0, s, row_mean, rows, 1.f / (float)rows, mean);
  return (int)hipGetLastError();
}

int skyrl_actor_loss(const float* logprobs, const float* old_logprobs, const float* advantages, const float* loss_mask,
                     const float* loss_weight, const float* base_logprobs, const float* entropy, int64_t rows, int64_t cols,
                     int loss_type, float eps_clip_low, float eps_clip_high, float clip_ratio_c, int kl_estimator,
                     float policy_scale, float term_scale, float kl_coef, float entropy_coef, float* row_sums, float* out6,
                     float* dlogprobs, float* dentropy, void* stream) {
  if (!valid_loss_type(loss_type)) return SKYRL_LMHEAD_ERR_ARG;
  if (base_logprobs && (kl_estimator < SKYRL_KL_K1 || kl_estimator > SKYRL_KL_K3)) return SKYRL_LMHEAD_ERR_ARG;
  const bool needs_old = loss_type != SKYRL_POLICY_LOSS_CROSS_ENTROPY;
  if (!logprobs || !row_sums || !out6 || (needs_old && (!old_logprobs || !advantages))) return SKYRL_LMHEAD_ERR_NULL;
  if (dentropy && !entropy) return SKYRL_LMHEAD_ERR_NULL;
  if (rows < 1 || cols < 1 || rows >= (int64_t(1) << 31) || cols >= (int64_t(1) << 31)) return SKYRL_LMHEAD_ERR_SHAPE;
  if (!valid_loss_params(loss_type, eps_clip_low, eps_clip_high, clip_ratio_c)) return SKYRL_LMHEAD_ERR_ARG;
  if (!finite(policy_scale) || !finite(term_scale) || !finite(kl_coef) || !finite(entropy_coef)) return SKYRL_LMHEAD_ERR_ARG;
  const ActorLossArgs a{logprobs,   old_logprobs,       advantages,         loss_mask,    loss_weight,  base_logprobs, entropy,
                        rows,       cols,               loss_type,          kl_estimator,
                        interval_type(loss_type) ? 1.f - eps_clip_low : eps_clip_low,
                        interval_type(loss_type) ? 1.f + eps_clip_high : eps_clip_high, clip_ratio_c, policy_scale,    term_scale,   kl_coef,      entropy_coef,
                        row_sums,   out6,               dlogprobs,          dentropy};
  hipStream_t s = (hipStream_t)stream;
  hipLaunchKernelGGL(actor_loss_rows_kernel, dim3((unsigned)rows), dim3(kRowThreads), 0, s, a);
  hipLaunchKernelGGL(actor_loss_finish_kernel, dim3(1), dim3(kRowThreads), 0, s, a);
  if (dentropy) {
    const int64_t n = rows * cols;
    if (n >= (int64_t(1) << 31) * 256) return SKYRL_LMHEAD_ERR_SHAPE;
    hipLaunchKernelGGL(actor_loss_dentropy_kernel, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, s, a);
  }
  return (int)hipGetLastError();
}

int skyrl_masked_mean(const float* values, const float* mask, int64_t rows, int64_t cols, float* means, float* dvalues,
                      void* stream) {
  if (!values || !means) return SKYRL_LMHEAD_ERR_NULL;
  if (rows < 1 || cols < 1 || rows >= (int64_t(1) << 31) || cols >= (int64_t(1) << 31)) return SKYRL_LMHEAD_ERR_SHAPE;
  hipLaunchKernelGGL(masked_mean_rows_kernel, dim3((unsigned)rows), dim3(kRowThreads), 0, (hipStream_t)stream, values, mask, cols,
                     means, dvalues);
  return (int)hipGetLastError();
}

int skyrl_off_policy_correction(const float* old_log_probs, const float* rollout_logprobs, const float* loss_mask, int64_t rows,
                                int64_t cols, int tis_type, float tis_cap, int seq_metric, float seq_low, float seq_high,
                                const float* outlier_low, const float* outlier_high, const float* token_low,
                                const float* token_high, float* keep_out, float* tis_out, float* weight_out, float* metrics,
                                float* row_stats, void* stream) {
  if (!old_log_probs || !rollout_logprobs || !metrics || !row_stats) return SKYRL_LMHEAD_ERR_NULL;
  if (rows < 1 || cols < 1 || rows > ((int64_t)1 << 31) - 1 || cols > ((int64_t)1 << 40)) return SKYRL_LMHEAD_ERR_SHAPE;
  if (tis_type < 0 || tis_type > 2 || seq_metric < 0 || seq_metric > 2) return SKYRL_LMHEAD_ERR_ARG;
  if ((tis_type && !finite(tis_cap)) || (seq_metric && (!finite(seq_low) || !finite(seq_high)))) return SKYRL_LMHEAD_ERR_ARG;
  for (const float* p : {outlier_low, outlier_high, token_low, token_high})
    if (p && !finite(*p)) return SKYRL_LMHEAD_ERR_ARG;
  OffPolicyArgs a{};
  a.old = old_log_probs, a.rollout = rollout_logprobs, a.mask = loss_mask, a.rows = rows, a.cols = cols;
  a.tis_type = tis_type, a.seq_metric = seq_metric, a.tis_cap = tis_cap, a.seq_low = seq_low, a.seq_high = seq_high;
  a.use_outlier_low = outlier_low != nullptr, a.use_outlier_high = outlier_high != nullptr;
  a.use_token_mask = token_low != nullptr && token_high != nullptr;  // the token mask needs both bounds (:18-21)
  a.outlier_low = outlier_low ? *outlier_low : 0.f, a.outlier_high = outlier_high ? *outlier_high : 0.f;
  a.token_low = a.use_token_mask ? *token_low : 0.f, a.token_high = a.use_token_mask ? *token_high : 0.f;
  a.keep_out = keep_out, a.tis_out = tis_out, a.weight_out = weight_out, a.row_stats = row_stats, a.metrics = metrics;
  hipStream_t s = (hipStream_t)stream;
  hipLaunchKernelGGL(off_policy_rows_kernel, dim3((unsigned)rows), dim3(kRowThreads), 0, s, a);
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) return (int)e;
  hipLaunchKernelGGL(off_policy_finish_kernel, dim3(1), dim3(64), 0, s, a);
  e = hipGetLastError();
  return e == hipSuccess ? SKYRL_LMHEAD_OK : (int)e;
}

int skyrl_logprob_diff_metrics(const float* logprobs, const float* rollout_logprobs, const float* loss_mask, int64_t n, float* out4,
                               float* partials, void* stream) {
  if (!logprobs || !rollout_logprobs || !out4 || !partials) return SKYRL_LMHEAD_ERR_NULL;
  if (n < 1) return SKYRL_LMHEAD_ERR_SHAPE;
  int64_t slices = (n + kLossSliceTokens - 1) / kLossSliceTokens;
  if (slices > kMaxLossSlices) slices = kMaxLossSlices;
  const int64_t slice = (n + slices - 1) / slices;
  hipStream_t s = (hipStream_t)stream;
  hipLaunchKernelGGL(logprob_diff_kernel, dim3((unsigned)slices), dim3(1024), 0, s, logprobs, rollout_logprobs, loss_mask, n, slice,
                     partials);
  hipLaunchKernelGGL(logprob_diff_finish_kernel, dim3(1), dim3(64), 0, s, partials, (int)slices, out4);
  return (int)hipGetLastError();
}

}  // extern "C"
