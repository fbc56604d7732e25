// The same per-token statistics for callers that hold materialised logits (the FSDP worker's forward tail and the
// reference's logits-input autograd functions): log-probability of a label, entropy and their backward from a [T, V]
// logits matrix in bf16 or fp32, each in ONE pass over the matrix.  HBM-bound: T*V*es bytes read in the forward (es = 2 or 4
// bytes per logit), read + written in the backward; what bounds the kernels besides HBM is one v_exp_f32 per logit.
//
// Reference (paths under skyrl/backends/skyrl_train/):
//   logprobs_from_logits / _v2 / _flash_attn   utils/torch_utils.py:115-177   (log_softmax + gather, several passes; the
//                                               flash-attn cross-entropy writes its gradient over the logits, "inplace_backward")
//   chunked_entropy_from_logits                utils/torch_utils.py:58-111    (log_softmax, exp, product, sum per chunk)
//   DistributedLogprob, ChunkedDistributedLogprob   distributed/megatron/model_utils.py:66-272 (fp32 copy of the logits,
//                                               softmax saved for backward; targets outside the shard give 0 and keep -p*g)
//   _VocabParallelEntropy                      distributed/megatron/model_utils.py:1316-1345 (the entropy's gradient)
//
//   forward   y = z / temperature;  lse = log sum exp y;  logprob = y[label] - lse;  pz = sum softmax(y) * y;  entropy = lse - pz
//   backward  dz = ( g * (onehot - p) - q * p * (y - pz) ) / temperature,   p = exp(y - lse)
// One workgroup per row; a thread keeps a running (max, sum, sum z*e) in base 2 and rescales only when a wave-wide vote says
// some lane's maximum moved, which after the first few pieces of a row is rare.
#include <hip/hip_runtime.h>
#include <math.h>
#include <stdint.h>

#include <cmath>

#include "../../include/skyrl_lmhead.h"

namespace {

constexpr float kLog2e = 1.4426950408889634f;
constexpr float kLn2 = 0.6931471805599453f;
constexpr float kLowest = -3.0e38f;  // start of a running maximum: finite, so that (-inf) - max is -inf and never NaN
// A logit of -inf (a masked vocabulary entry) has probability exactly 0; in the products z * p it is taken as this finite
// value so that 0 * inf does not turn the row into NaN (the reference's entropy does return NaN there, torch_utils.py:99-100).
constexpr float kMostNegativeFactor = -1.0e30f;
constexpr int kThreads = 512;
constexpr int kWaves = kThreads / 64;
constexpr int kInFlight = 4;  // 16-byte loads a thread has in flight

// Eight bf16 or four fp32 logits of one 16-byte piece, widened to fp32.
template <bool F32>
struct Piece {
  static constexpr int kElems = F32 ? 4 : 8;
  float v[kElems];
  __device__ __forceinline__ void load(const void* p) {
    const uint4 raw = *(const uint4*)p;
    const uint32_t w[4] = {raw.x, raw.y, raw.z, raw.w};
    if (F32) {
#pragma unroll
      for (int i = 0; i < 4; ++i) v[i] = __uint_as_float(w[i]);
    } else {
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        v[2 * i] = __uint_as_float(w[i] << 16);
        v[2 * i + 1] = __uint_as_float(w[i] & 0xffff0000u);
      }
    }
  }
};

__device__ __forceinline__ float load_one(const void* base, size_t i, bool f32) {
  return f32 ? ((const float*)base)[i] : __uint_as_float((uint32_t)((const uint16_t*)base)[i] << 16);
}

__device__ __forceinline__ uint16_t bf16_bits(float x) {
  typedef __attribute__((ext_vector_type(2))) float f32x2;
  typedef __attribute__((ext_vector_type(2))) __bf16 bf16x2;
  const f32x2 pair = {x, 0.f};
  const bf16x2 b = __builtin_convertvector(pair, bf16x2);
  return (uint16_t)(*(const uint32_t*)&b & 0xffffu);
}

// Running statistics of a row in base 2, with y2 = z * log2e / temperature:  m = max y2,  s = sum 2^(y2 - m),
// e = sum (y2 - m) * 2^(y2 - m).  The third sum is kept relative to the maximum, like the other two, so that a large common
// offset of a row's logits costs no accuracy:  entropy = ln s - ln 2 * e / s,  logprob = ln 2 * (y2[label] - m) - ln s.
struct Stats {
  float m, s, e;
};

template <bool ENT>
__device__ __forceinline__ void absorb(Stats& st, float z, float scale2) {
  const float t = fmaf(z, scale2, -st.m);
  const float p = __builtin_amdgcn_exp2f(t);
  st.s += p;
  if (ENT) st.e = fmaf(fmaxf(t, kMostNegativeFactor), p, st.e);
}

// Sums taken relative to maximum `from`, re-expressed relative to `to` >= from.
__device__ __forceinline__ void rebase(float& s, float& e, float from, float to) {
  const float d = fmaxf(from - to, kMostNegativeFactor);  // <= 0; finite, so that d * 0 is 0 for an empty sum
  const float c = __builtin_amdgcn_exp2f(d);
  e = c * fmaf(d, s, e);
  s *= c;
}

// Raise the running maximum to at least `cand` (a value of y2).
__device__ __forceinline__ void raise_max(Stats& st, float cand) {
  if (cand > st.m) {
    rebase(st.s, st.e, st.m, cand);
    st.m = cand;
  }
}

__device__ __forceinline__ void merge(Stats& a, const Stats& b) {
  const float m = fmaxf(a.m, b.m);
  float bs = b.s, be = b.e;
  rebase(a.s, a.e, a.m, m);
  rebase(bs, be, b.m, m);
  a.s += bs;
  a.e += be;
  a.m = m;
}

// The row's statistics in every thread.
__device__ __forceinline__ Stats block_merge(Stats st, Stats* sm) {
#pragma unroll
  for (int o = 32; o >= 1; o >>= 1) {
    Stats other;
    other.m = __shfl_xor(st.m, o, 64);
    other.s = __shfl_xor(st.s, o, 64);
    other.e = __shfl_xor(st.e, o, 64);
    merge(st, other);
  }
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  if (lane == 0) sm[wave] = st;
  __syncthreads();
  Stats all = sm[0];
  for (int w = 1; w < kWaves; ++w) merge(all, sm[w]);
  return all;
}

// Statistics of row `row`: vector pieces where the row start and pitch allow 16-byte loads, single logits otherwise and
// for the ragged end.
template <bool F32, bool ENT>
__device__ __forceinline__ Stats row_stats(const void* logits, int64_t ld, int64_t row, int V, float scale2, bool vector_ok) {
  constexpr int E = Piece<F32>::kElems;
  const char* base = (const char*)logits + (size_t)row * (size_t)ld * (F32 ? 4 : 2);
  Stats st{kLowest, 0.f, 0.f};
  const int pieces = vector_ok ? V / E : 0;
  for (int p0 = threadIdx.x; p0 < pieces; p0 += kThreads * kInFlight) {
    Piece<F32> pc[kInFlight];
#pragma unroll
    for (int u = 0; u < kInFlight; ++u) {
      const int p = p0 + u * kThreads;
      pc[u].load(base + (size_t)(p < pieces ? p : p0) * 16);
    }
#pragma unroll
    for (int u = 0; u < kInFlight; ++u) {
      if (p0 + u * kThreads < pieces) {
        float mx = pc[u].v[0];
#pragma unroll
        for (int i = 1; i < E; ++i) mx = fmaxf(mx, pc[u].v[i]);
        if (__any(mx * scale2 > st.m)) raise_max(st, mx * scale2);
#pragma unroll
        for (int i = 0; i < E; ++i) absorb<ENT>(st, pc[u].v[i], scale2);
      }
    }
  }
  for (int i = pieces * E + threadIdx.x; i < V; i += kThreads) {
    const float z = load_one(base, (size_t)i, F32);
    raise_max(st, z * scale2);
    absorb<ENT>(st, z, scale2);
  }
  return st;
}

// labels may be NULL (no log-probability wanted).  A label outside [0, V) gives log-probability 0 (model_utils.py:89-99).
template <bool F32, bool ENT>
__global__ __launch_bounds__(kThreads) void logits_fwd_rows(const void* __restrict__ logits, int64_t ld, const int64_t* __restrict__ labels,
                                                            int V, float rcp_temp, int vector_ok, float* __restrict__ logprobs,
                                                            float* __restrict__ entropy, float* __restrict__ row_lse,
                                                            float* __restrict__ row_pz) {
  __shared__ Stats sm[kWaves];
  const int64_t row = blockIdx.x;
  const float scale2 = rcp_temp * kLog2e;
  const Stats st = block_merge(row_stats<F32, ENT>(logits, ld, row, V, scale2, vector_ok != 0), sm);
  if (threadIdx.x == 0) {
    const float log_s = logf(st.s);
    const float lse = fmaf(st.m, kLn2, log_s);
    const float pz = (st.e / st.s + st.m) * kLn2;
    if (logprobs) {
      float lp = 0.f;
      if (labels) {
        const int64_t y = labels[row];
        if (y >= 0 && y < (int64_t)V)
          lp = fmaf(load_one((const char*)logits + (size_t)row * (size_t)ld * (F32 ? 4 : 2), (size_t)y, F32), scale2, -st.m) * kLn2 - log_s;
      }
      logprobs[row] = lp;
    }
    if (entropy) entropy[row] = log_s - st.e / st.s * kLn2;
    if (row_lse) row_lse[row] = lse;
    if (row_pz) row_pz[row] = pz;
  }
}

// dlogits may be the logits themselves (every logit is read before its place is written, by the same thread).
template <bool F32, bool ENTGRAD>
__global__ __launch_bounds__(kThreads) void logits_bwd_rows(const void* logits, int64_t ld, const int64_t* __restrict__ labels, int V,
                                                            float rcp_temp, int vector_ok, const float* __restrict__ row_lse,
                                                            const float* __restrict__ row_pz, const float* __restrict__ dlogprobs,
                                                            const float* __restrict__ dentropy, void* dlogits, int64_t ldd) {
  constexpr int E = Piece<F32>::kElems;
  constexpr int ES = F32 ? 4 : 2;
  const int64_t row = blockIdx.x;
  const char* src = (const char*)logits + (size_t)row * (size_t)ld * ES;
  char* dst = (char*)dlogits + (size_t)row * (size_t)ldd * ES;
  const float g = dlogprobs ? dlogprobs[row] : 0.f;
  const float q = dentropy ? dentropy[row] : 0.f;
  const float scale2 = rcp_temp * kLog2e;
  const float lse2 = row_lse[row] * kLog2e;
  // dz = p * (c0 + c1 * z) [+ g / temperature at the label],  c0 = -(g - q * pz) / temperature,  c1 = -q / temperature^2
  const float pz = (dentropy && row_pz) ? row_pz[row] : 0.f;
  const float c0 = -(g - q * pz) * rcp_temp, c1 = -q * rcp_temp * rcp_temp;
  int64_t y = labels ? labels[row] : (int64_t)-1;
  if (y < 0 || y >= (int64_t)V) y = -1;
  const bool zero_row = g == 0.f && q == 0.f;  // no upstream gradient: zeros, and the logits need not be read
  auto dz = [&](float z, int64_t col) {
    const float p = __builtin_amdgcn_exp2f(fmaf(z, scale2, -lse2));
    float d = ENTGRAD ? p * fmaf(c1, fmaxf(z, kMostNegativeFactor), c0) : p * c0;
    if (col == y) d += g * rcp_temp;
    return d;
  };
  const int pieces = vector_ok ? V / E : 0;
  for (int p0 = threadIdx.x; p0 < pieces; p0 += kThreads * kInFlight) {
    Piece<F32> pc[kInFlight];
    if (!zero_row) {
#pragma unroll
      for (int u = 0; u < kInFlight; ++u) {
        const int p = p0 + u * kThreads;
        pc[u].load(src + (size_t)(p < pieces ? p : p0) * 16);
      }
    }
#pragma unroll
    for (int u = 0; u < kInFlight; ++u) {
      const int p = p0 + u * kThreads;
      if (p >= pieces) continue;
      float d[E];
#pragma unroll
      for (int i = 0; i < E; ++i) d[i] = zero_row ? 0.f : dz(pc[u].v[i], (int64_t)p * E + i);
      uint4 out;
      if (F32) {
        out = make_uint4(__float_as_uint(d[0]), __float_as_uint(d[1]), __float_as_uint(d[2]), __float_as_uint(d[3]));
      } else {
        typedef __attribute__((ext_vector_type(4))) float f32x4;
        typedef __attribute__((ext_vector_type(4))) __bf16 bf16x4;
        const f32x4 lo4 = {d[0], d[1], d[2], d[3]}, hi4 = {d[4 % E], d[5 % E], d[6 % E], d[7 % E]};
        const bf16x4 lo = __builtin_convertvector(lo4, bf16x4), hi = __builtin_convertvector(hi4, bf16x4);
        const uint2 a = *(const uint2*)&lo, b = *(const uint2*)&hi;
        out = make_uint4(a.x, a.y, b.x, b.y);
      }
      *(uint4*)(dst + (size_t)p * 16) = out;
    }
  }
  for (int i = pieces * E + threadIdx.x; i < V; i += kThreads) {
    const float d = zero_row ? 0.f : dz(load_one(src, (size_t)i, F32), (int64_t)i);
    if (F32) ((float*)dst)[i] = d;
    else ((uint16_t*)dst)[i] = bf16_bits(d);
  }
}

constexpr int64_t kMaxRows = (int64_t)1 << 31;  // the grid's x extent

bool pieces_aligned(const void* p, int64_t ld, bool f32) {
  return ((uintptr_t)p & 15u) == 0 && (ld * (f32 ? 4 : 2)) % 16 == 0;
}

int check_logits(const void* logits, int dtype, int64_t ld, int64_t T, int64_t V, float rcp_temperature) {
  if (!logits) return SKYRL_LMHEAD_ERR_NULL;
  if (dtype != SKYRL_LOGITS_BF16 && dtype != SKYRL_LOGITS_F32) return SKYRL_LMHEAD_ERR_ARG;
  if (T < 1 || V < 1 || ld < V || T >= kMaxRows || V >= ((int64_t)1 << 31) || ld >= ((int64_t)1 << 40)) return SKYRL_LMHEAD_ERR_SHAPE;
  if ((uintptr_t)logits & (dtype == SKYRL_LOGITS_F32 ? 3u : 1u)) return SKYRL_LMHEAD_ERR_ALIGN;
  if (!(rcp_temperature > 0.f) || !std::isfinite(rcp_temperature)) return SKYRL_LMHEAD_ERR_ARG;
  return SKYRL_LMHEAD_OK;
}

}  // namespace

extern "C" {

int skyrl_logits_fwd(const void* logits, int logits_dtype, int64_t ld_logits, const int64_t* labels, int64_t T, int64_t V,
                     float rcp_temperature, float* logprobs, float* entropy, float* row_lse, float* row_pz, void* stream) {
  const int st = check_logits(logits, logits_dtype, ld_logits, T, V, rcp_temperature);
  if (st) return st;
  if (logprobs && !labels) return SKYRL_LMHEAD_ERR_NULL;
  if (!logprobs && !entropy && !row_lse && !row_pz) return SKYRL_LMHEAD_ERR_NULL;
  if (labels && ((uintptr_t)labels & 7u)) return SKYRL_LMHEAD_ERR_ALIGN;
  const bool f32 = logits_dtype == SKYRL_LOGITS_F32;
  const int vec = pieces_aligned(logits, ld_logits, f32) ? 1 : 0;
  hipStream_t s = (hipStream_t)stream;
  const bool ent = entropy || row_pz;
  auto launch = [&](auto kernel) {
    hipLaunchKernelGGL(kernel, dim3((unsigned)T), dim3(kThreads), 0, s, logits, ld_logits, labels, (int)V, rcp_temperature, vec,
                       logprobs, entropy, row_lse, row_pz);
  };
  if (f32 && ent) launch(logits_fwd_rows<true, true>);
  else if (f32) launch(logits_fwd_rows<true, false>);
  else if (ent) launch(logits_fwd_rows<false, true>);
  else launch(logits_fwd_rows<false, false>);
  const hipError_t e = hipGetLastError();
  return e == hipSuccess ? SKYRL_LMHEAD_OK : (int)e;
}

int skyrl_logits_bwd(const void* logits, int logits_dtype, int64_t ld_logits, const int64_t* labels, const float* row_lse,
                     const float* row_pz, const float* dlogprobs, const float* dentropy, int64_t T, int64_t V,
                     float rcp_temperature, void* dlogits, int64_t ld_dlogits, void* stream) {
  const int st = check_logits(logits, logits_dtype, ld_logits, T, V, rcp_temperature);
  if (st) return st;
  if (!row_lse || !dlogits || (!dlogprobs && !dentropy) || (dlogprobs && !labels) || (dentropy && !row_pz))
    return SKYRL_LMHEAD_ERR_NULL;
  if (ld_dlogits < V || ld_dlogits >= ((int64_t)1 << 40)) return SKYRL_LMHEAD_ERR_SHAPE;
  const bool f32 = logits_dtype == SKYRL_LOGITS_F32;
  if (((uintptr_t)dlogits & (f32 ? 3u : 1u)) || (labels && ((uintptr_t)labels & 7u))) return SKYRL_LMHEAD_ERR_ALIGN;
  // In place, or apart: a gradient buffer that overlaps the logits in any other way would be read after it was written.
  if (dlogits != logits || ld_dlogits != ld_logits) {
    const char *a0 = (const char*)logits, *b0 = (const char*)dlogits;
    const size_t es = f32 ? 4 : 2;
    const char *a1 = a0 + ((size_t)(T - 1) * (size_t)ld_logits + (size_t)V) * es, *b1 = b0 + ((size_t)(T - 1) * (size_t)ld_dlogits + (size_t)V) * es;
    if (a0 < b1 && b0 < a1) return SKYRL_LMHEAD_ERR_ARG;
  }
  const int vec = (pieces_aligned(logits, ld_logits, f32) && pieces_aligned(dlogits, ld_dlogits, f32)) ? 1 : 0;
  hipStream_t s = (hipStream_t)stream;
  const bool entgrad = dentropy != nullptr;
  auto launch = [&](auto kernel) {
    hipLaunchKernelGGL(kernel, dim3((unsigned)T), dim3(kThreads), 0, s, logits, ld_logits, labels, (int)V, rcp_temperature, vec,
                       row_lse, row_pz, dlogprobs, dentropy, dlogits, ld_dlogits);
  };
  if (f32 && entgrad) launch(logits_bwd_rows<true, true>);
  else if (f32) launch(logits_bwd_rows<true, false>);
  else if (entgrad) launch(logits_bwd_rows<false, true>);
  else launch(logits_bwd_rows<false, false>);
  const hipError_t e = hipGetLastError();
  return e == hipSuccess ? SKYRL_LMHEAD_OK : (int)e;
}

}  // extern "C"
