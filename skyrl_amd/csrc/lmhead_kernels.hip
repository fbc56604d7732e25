// HIP kernels (gfx950) and C-ABI entry points of the fused LM-head log-probability path.
//
// Forward  (2*T*V*H flop):
//   lmhead_fwd_tiles   one 256(vocab) x 256(token) logits tile per workgroup: bf16 MFMA GEMM, then in registers
//                      scale by 1/temperature, per-token max / sum-exp / sum (z-max)*exp over the tile's vocab rows;
//                      writes one (max, sum, pz) partial per token per 128-row half tile, in blocks of 64 tokens.  Logits
//                      never leave VGPRs.
//   lmhead_fwd_merge   per block of 64 tokens: merges the partials (online log-sum-exp), gathers the label logit with an
//                      fp32 dot product hidden[t] . weight[label], writes logprob / entropy / lse / pz.
// Backward (6*T*V*H flop), looped over vocab chunks of `vocab_chunk` columns:
//   transpose_bf16     hidden^T once per call (and weight^T only when V is not a multiple of 64).
//   lmhead_bwd_dz      recompute a logits tile, form dz in registers and write it (bf16) into one token-major panel of
//                      the chunk.
//   lmhead_bwd_gemm    dHidden (+)= dz . weight and dW[chunk] = dz^T . hidden with fp32 accumulation, both from that
//                      panel -- dW reads it K-major, dHidden reads the weight K-major in place -- through the transposing
//                      LDS read (gemm_core.hpp).
// Soft cross-entropy of a draft head against the policy (10*T*V*H flop): softce_pack_rows stacks the two hidden rows of every
//   token, softce_fwd_tiles is the forward tile with a paired third statistic, softce_dz_tiles the matching dz producer; merge
//   and dHidden GEMM are the kernels above.
// The per-token loss kernels and the packed-sequence index kernels live in loss_kernels.hip and packed_kernels.hip.
#include <hip/hip_runtime.h>
#include <math.h>
#include <stdint.h>

#include <algorithm>
#include <mutex>
#include <vector>

#include "../../include/skyrl_lmhead.h"
#include "../../include/skyrl_lmhead_bench.h"
#include "gemm_core.hpp"
#include "topk_kernels.hpp"

using namespace lmhead;

namespace {

constexpr float kLog2e = 1.4426950408889634f;
constexpr float kLn2 = 0.6931471805599453f;
#ifndef LMHEAD_GROUP_M
#define LMHEAD_GROUP_M 4  // measured best of 2, 4, 6, 8, 16, 32 on both passes
#endif
constexpr int kGroupM = LMHEAD_GROUP_M;
// Timing-only ablations for skyrl_amd/bench_ablations.py (results are wrong with any of them; 0 in the product build):
//   1  forward tiles skip their statistics epilogue        2  dz tiles skip their epilogue (arithmetic, staging, stores)
//   4  dz tiles do everything but the global stores        8  forward and dz tiles read the operand panels of one 4 x 8 patch
//  16  the same for the gradient-GEMM tiles                   of tiles, so that every operand read hits the XCD's L2
//  32, 64  in gemm_core.hpp: the mainloop without its LDS fragment reads / without its global -> LDS copies
#ifndef LMHEAD_ABLATE
#define LMHEAD_ABLATE 0
#endif
// Scratch matrices get 64 extra elements (128 B) per row: with a power-of-two row pitch (T' = 16384 -> 32 KiB) the 256 rows of
// an operand tile would all start in the same L2 channel and set.
constexpr int kLdPad = 64;

__host__ __device__ inline int64_t round_up(int64_t x, int64_t m) { return (x + m - 1) / m * m; }
// An even number of k-tiles selects the accumulator-stationary mainloop (the EVEN instantiation of a tile kernel).
inline bool even_ktiles(int64_t contraction) { return (contraction / BK) % 2 == 0; }

// Scratch of skyrl_lmhead_fwd_static_scratch, the entry point for callers that cannot allocate: one fixed array in every
// device's memory, held until the process ends.  In host code this name is only a handle for hipGetSymbolAddress (see
// static_scratch_of_current_device); kernels receive the looked-up address as an ordinary argument.
constexpr size_t kStaticScratchBytes = SKYRL_LMHEAD_STATIC_SCRATCH_BYTES;
static __device__ __align__(256) unsigned char static_scratch[kStaticScratchBytes];

// Partial statistics live in blocks of 64 tokens: [token block][part][64 tokens].  A wave of the tile kernel writes 64
// contiguous bytes (16 tokens) of one part; the merge kernel reads a token block's parts as one contiguous stream, 256 bytes
// per wave instruction.  The arrays hold nparts * round_up(T, 64) floats.
constexpr int kPartTokens = 64;
__host__ __device__ inline size_t part_index(int part, int t, int nparts) {
  return ((size_t)(t / kPartTokens) * (size_t)nparts + (size_t)part) * kPartTokens + (size_t)(t % kPartTokens);
}
__host__ __device__ inline size_t part_elems(size_t nparts, int64_t T) {
  return nparts * (size_t)((T + kPartTokens - 1) / kPartTokens * kPartTokens);
}

// ------------------------------------------------------------------------------------------------------------
// Forward tile kernel.  M axis = vocab (A = weight), N axis = tokens (B = hidden).
// Online softmax statistics follow efficient_entropy_kernel_general_mainloop
// (fused_linear_logprob_triton.py:296-385): scale, running max, sum exp, sum z*exp (kept relative to the maximum here); vocab rows past V take no part.
// The label-logit gather of that kernel (:364-385) is done in lmhead_fwd_merge instead.
// ------------------------------------------------------------------------------------------------------------
// PAIRED (the soft cross-entropy, below): token blocks j >= TN / 2 hold teacher rows, and their third statistic weighs the
// *student's* logit -- the same lane's accumulator TN / 2 blocks earlier -- with the teacher's exp: sum z_student e^(z_teacher - m).
template <bool ENTROPY, bool MASKED, bool PAIRED>
__device__ __forceinline__ void fwd_tile_stats(const acc_t& acc, int j, int vbase, int V, float scale2, int kq, float& m_out,
                                               float& s_out, float& e_out) {
  const int jy = (PAIRED && j >= TN / 2) ? j - TN / 2 : j;  // j is a constant of the caller's unrolled loop
  // Two read-only passes over the accumulators (they live in AGPRs; writing scaled values back would cost a move each
  // way).  scale2 > 0, so the maximum commutes with the scaling.  The third statistic of an ordinary row is taken relative
  // to the tile's maximum, sum (z - m) e^(z - m): the exponent is at hand, and the entropy ln s - e / s then comes out of two
  // small numbers when the row is nearly deterministic, where lse - sum p z would cancel two large ones.  (The paired
  // statistic of the soft cross-entropy stays sum z_student e^(z_teacher - m): it is an expectation of another row's logit.)
  float mx = -INFINITY;
#pragma unroll
  for (int i = 0; i < TM; ++i)
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      float x = acc[i][j][r];
      if (MASKED) {
        const int v = vbase + i * MT + kq * 4 + r;
        if (v >= V) x = -INFINITY;
      }
      mx = fmaxf(mx, x);
    }
  mx = col_max(mx);  // finite: the wave has at least one row below V
  const float m2 = mx * scale2;
  float s = 0.f, e = 0.f;
#pragma unroll
  for (int i = 0; i < TM; ++i)
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      const float x = acc[i][j][r];
      const float t2 = fmaf(x, scale2, -m2);
      float p = __builtin_amdgcn_exp2f(t2);
      if (MASKED) {
        const int v = vbase + i * MT + kq * 4 + r;
        if (v >= V) p = 0.f;
      }
      s += p;
      if (ENTROPY) e = fmaf(PAIRED ? acc[i][jy][r] : t2, p, e);
    }
  s = col_sum(s);
  if (ENTROPY) e = col_sum(e);
  m_out = m2 * kLn2;
  s_out = s;
  e_out = PAIRED ? e * scale2 * kLn2 : e * kLn2;
}

// EVEN: H / 64 is even, which selects the accumulator-stationary mainloop (gemm_core.hpp).
template <bool ENTROPY, bool PAIRED, bool EVEN>
__device__ __forceinline__ void fwd_tile(const uint16_t* __restrict__ W, int ldw, const uint16_t* __restrict__ Hd, int ldh, int T,
                                         int H, int V, float rcp_temp, float* __restrict__ part_max,
                                         float* __restrict__ part_sum, float* __restrict__ part_pz, char* lds) {
  const int tiles_m = (V + BM - 1) / BM;
  const int tiles_n = (T + BN - 1) / BN;
  int tm, tn;
  tile_coords(blockIdx.x, tiles_m, tiles_n, kGroupM, tm, tn);

#if LMHEAD_ABLATE & 8
  Operand a{W, ldw, (tm % 4) * BM, V};
  Operand b{Hd, ldh, (tn % 8) * BN, T};
#else
  Operand a{W, ldw, tm * BM, V};
  Operand b{Hd, ldh, tn * BN, T};
#endif
  acc_t acc;
  prefetch_first_tiles(a, b, 0, H / BK, lds);  // the first copies travel while the accumulators are cleared
  zero_acc(acc);
  mainloop<false, EVEN>(a, b, 0, H / BK, lds, acc);
#if LMHEAD_ABLATE & 1
  return;
#endif

  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int wm = wave / WAVES_N, wn = wave % WAVES_N;
  const int lrow = lane & 15, kq = lane >> 4;
  const int vbase = tm * BM + wm * WM;
  const int part = tm * WAVES_M + wm, nparts = tiles_m * WAVES_M;
  const float scale2 = rcp_temp * kLog2e;
  // Whether the wave's 128 vocab rows all exist (0), partly (1: the last vocab tile) or not at all (2) is the same for the
  // whole wave: decided once, outside the unrolled loop over the token blocks.
  const int rows_kind = __builtin_amdgcn_readfirstlane(vbase + WM <= V ? 0 : (vbase < V ? 1 : 2));
  auto token_blocks = [&](auto kind) {
    constexpr int KIND = decltype(kind)::value;
#pragma unroll
    for (int j = 0; j < TN; ++j) {
      const int t = tn * BN + wn * WN + j * MT + lrow;
      float m = -INFINITY, s = 0.f, e = 0.f;
      if (KIND < 2) fwd_tile_stats<ENTROPY, KIND == 1, PAIRED>(acc, j, vbase, V, scale2, kq, m, s, e);
      if (kq == 0 && t < T) {
        const size_t idx = part_index(part, t, nparts);
        part_max[idx] = m;
        part_sum[idx] = s;
        if (ENTROPY) part_pz[idx] = e;
      }
    }
  };
  if (rows_kind == 0) token_blocks(std::integral_constant<int, 0>{});
  else if (rows_kind == 1) token_blocks(std::integral_constant<int, 1>{});
  else token_blocks(std::integral_constant<int, 2>{});
}

template <bool ENTROPY, bool EVEN>
__global__ __launch_bounds__(NTHREADS) void lmhead_fwd_tiles(const uint16_t* __restrict__ W, int ldw,
                                                             const uint16_t* __restrict__ Hd, int ldh, int T, int H, int V,
                                                             float rcp_temp, float* __restrict__ part_max,
                                                             float* __restrict__ part_sum, float* __restrict__ part_pz) {
  __shared__ __attribute__((aligned(1024))) char lds[LDS_BYTES];
  fwd_tile<ENTROPY, false, EVEN>(W, ldw, Hd, ldh, T, H, V, rcp_temp, part_max, part_sum, part_pz, lds);
}

// ------------------------------------------------------------------------------------------------------------
// Forward merge.  One workgroup of 16 waves per block of 64 tokens: lane = token, wave w merges parts w, w + 16, ... of that
// token (every load of a wave is 256 contiguous bytes), the sixteen running triples meet in LDS; then sixteen lanes per
// token gather the label logit.
// Merge algebra as in efficient_entropy_triton_kernel_epilogue (fused_linear_logprob_triton.py:417-467) except that
// the running max starts at -inf (that kernel starts it at 0, which loses rows whose logits are all << 0).
// Out-of-range labels give logprob 0 (model_utils.py:337; fused_linear_logprob_triton.py:1898-1905).
// ------------------------------------------------------------------------------------------------------------
constexpr int kMergeTokens = kPartTokens;
constexpr int kMergeThreads = 1024;
constexpr int kMergeWaves = kMergeThreads / 64;
constexpr int kDotLanes = kMergeThreads / kMergeTokens;  // lanes per token in the label-logit phase

// Two partial triples (maximum, sum e^(z - max), third statistic) of one token become one.  RELATIVE: the third statistic
// is sum (z - max) e^(z - max) and moves with the maximum, e' = c (e + (max - max') s); otherwise it is sum y e^(z - max) of
// some y that does not depend on the maximum and only scales.
template <bool RELATIVE>
__device__ __forceinline__ void merge_partial(float& M, float& S, float& E, float m, float s, float e) {
  if (!(m > -INFINITY)) return;  // a part without a single vocabulary row
  if (!(M > -INFINITY)) {
    M = m, S = s, E = e;
    return;
  }
  const float Mn = fmaxf(M, m);
  const float da = M - Mn, db = m - Mn;
  const float ca = expf(da), cb = expf(db);
  // Explicit fused multiply-adds: which of the two products of a * b + c * d the compiler would contract is its choice, and it
  // need not make the same one in every build.
  E = RELATIVE ? fmaf(ca, fmaf(da, S, E), cb * fmaf(db, s, e)) : fmaf(E, ca, e * cb);
  S = fmaf(S, ca, s * cb);
  M = Mn;
}

template <bool RELATIVE>
__global__ __launch_bounds__(kMergeThreads) void lmhead_fwd_merge(const float* __restrict__ part_max,
                                                                  const float* __restrict__ part_sum,
                                                                  const float* __restrict__ part_pz, int nparts, int T,
                                                                  const uint16_t* __restrict__ Hd, int ldh,
                                                                  const uint16_t* __restrict__ W, int ldw,
                                                                  const int64_t* __restrict__ labels, int H, int V, float rcp_temp,
                                                                  float* __restrict__ logprobs, float* __restrict__ entropy,
                                                                  float* __restrict__ row_lse, float* __restrict__ row_pz) {
  __shared__ float sm_m[kMergeWaves][kMergeTokens], sm_s[kMergeWaves][kMergeTokens], sm_e[kMergeWaves][kMergeTokens];
  __shared__ float sm_lse[kMergeTokens], sm_pz[kMergeTokens];
  const int tid = threadIdx.x;
  {
    const int lane = tid & 63, wave = tid >> 6;
    const int t = blockIdx.x * kMergeTokens + lane;
    const size_t base = (size_t)blockIdx.x * (size_t)nparts * kPartTokens + lane;
    float M = -INFINITY, S = 0.f, E = 0.f;
    if (t < T) {
      constexpr int kBatch = 4;  // loads in flight per array before the dependent merge chain
      for (int p0 = wave; p0 < nparts; p0 += kMergeWaves * kBatch) {
        float m[kBatch], sv[kBatch], ev[kBatch];
#pragma unroll
        for (int u = 0; u < kBatch; ++u) {
          const int p = p0 + u * kMergeWaves;
          const bool in = p < nparts;
          const size_t idx = base + (size_t)(in ? p : p0) * kPartTokens;
          m[u] = in ? part_max[idx] : -INFINITY;
          sv[u] = part_sum[idx];
          ev[u] = part_pz ? part_pz[idx] : 0.f;
        }
#pragma unroll
        for (int u = 0; u < kBatch; ++u) merge_partial<RELATIVE>(M, S, E, m[u], sv[u], ev[u]);
      }
    }
    sm_m[wave][lane] = M;
    sm_s[wave][lane] = S;
    sm_e[wave][lane] = E;
    __syncthreads();
    if (wave == 0) {
      float Mg = -INFINITY, Sg = 0.f, Eg = 0.f;
      for (int g = 0; g < kMergeWaves; ++g) merge_partial<RELATIVE>(Mg, Sg, Eg, sm_m[g][lane], sm_s[g][lane], sm_e[g][lane]);
      const float log_s = logf(Sg);
      sm_lse[lane] = Mg + log_s;
      // RELATIVE: sm_pz holds the entropy itself, ln s - e / s, and sum p z is recovered as lse - entropy (exactly what the
      // absolute form would have subtracted the other way round).
      sm_pz[lane] = RELATIVE ? log_s - Eg / Sg : Eg / Sg;
    }
    __syncthreads();
  }
  // Label logit: 16 lanes per token, 16-byte loads, fp32 accumulation.
  const int tl = tid / kDotLanes, sub = tid % kDotLanes;
  const int t = blockIdx.x * kMergeTokens + tl;
  float dot = 0.f;
  bool has_label = false;
  if (t < T && labels) {
    const int64_t y = labels[t];
    has_label = (y >= 0 && y < (int64_t)V);
    if (has_label) {
      const uint16_t* hp = Hd + (size_t)t * (size_t)ldh;
      const uint16_t* wp = W + (size_t)y * (size_t)ldw;
      for (int c = sub * 8; c < H; c += kDotLanes * 8) {
        const uint4 hv = *(const uint4*)(hp + c);
        const uint4 wv = *(const uint4*)(wp + c);
        const uint32_t hh[4] = {hv.x, hv.y, hv.z, hv.w};
        const uint32_t ww[4] = {wv.x, wv.y, wv.z, wv.w};
#pragma unroll
        for (int k = 0; k < 4; ++k) {
          dot = fmaf(__uint_as_float(hh[k] << 16), __uint_as_float(ww[k] << 16), dot);
          dot = fmaf(__uint_as_float(hh[k] & 0xffff0000u), __uint_as_float(ww[k] & 0xffff0000u), dot);
        }
      }
    }
  }
#pragma unroll
  for (int o = 1; o < kDotLanes; o <<= 1) dot += __shfl_xor(dot, o, 64);
  if (sub == 0 && t < T) {
    const float lse = sm_lse[tl];
    const float ent = RELATIVE ? sm_pz[tl] : lse - sm_pz[tl];
    const float pz = RELATIVE ? lse - sm_pz[tl] : sm_pz[tl];
    if (logprobs) logprobs[t] = has_label ? dot * rcp_temp - lse : 0.f;
    if (entropy) entropy[t] = ent;
    if (row_lse) row_lse[t] = lse;
    if (row_pz) row_pz[t] = pz;
  }
}

// ------------------------------------------------------------------------------------------------------------
// Backward dz producer.  Same tile as the forward; the epilogue is purely element-wise because the row
// statistics come from the forward pass.  Formula of efficient_entropy_backward_kernel_general_d_logits_split_N
// (fused_linear_logprob_triton.py:1402-1538, the arithmetic is at :947-957 of the fused variant):
//     p  = exp(z - lse);   dz = ( g*(onehot - p) - q*p*(z - pz) ) / temperature
// written as  p * (c0 + c1*x) + onehot*g/temperature  with x the raw dot product.
// Out-of-range labels get no one-hot term but keep -p*g (model_utils.py:405-411).
// ------------------------------------------------------------------------------------------------------------
struct DzArgs {
  const uint16_t* W;
  int ldw;
  const uint16_t* Hd;
  int ldh;
  int T, H, V;
  float rcp_temp;
  const int64_t* labels;
  const float* row_lse;
  const float* row_pz;
  const float* dlogprobs;
  const float* dentropy;
  int vc0, tiles_m, tiles_n;  // first vocab row of the chunk; tiles of the chunk panel along vocab and tokens
  uint16_t* D;                // [tiles_n * 256, ldd]  dz, token-major
  int ldd;
  // When not NULL: the number of tokens, <= T, as a value in device memory (what a compaction kernel counted).  T then
  // only sizes the grid: token tiles at or beyond the device-side count return at once.
  const int* T_dev;
  // When not NULL (fp32 weights): for every token whose label lies in the vocabulary, its label's dz value before the
  // rounding to bf16, fp32 [T].  That one value per token, g (1 - p) / temperature, is of order 1 where every other dz value
  // of the row is of order p; the caller adds what the bf16 product dropped of it (label_residual_update) so that the label
  // rows of dW keep fp32 accuracy.
  float* label_resid;
  // 0, or 126 - n: softmax probabilities below 2^-n are treated as zero (SKYRL_BWD_FLUSH_TINY_DZ).
  float p_shift;
};

template <bool ENTGRAD, bool EVEN>
__device__ __forceinline__ void dz_tile(const DzArgs& z, int id, char* lds) {
  const uint16_t* __restrict__ W = z.W;
  const uint16_t* __restrict__ Hd = z.Hd;
  const int ldw = z.ldw, ldh = z.ldh, H = z.H, V = z.V, vc0 = z.vc0, ldd = z.ldd;
  const int T = z.T_dev ? __builtin_amdgcn_readfirstlane(*z.T_dev) : z.T;
  const float rcp_temp = z.rcp_temp;
  const int64_t* __restrict__ labels = z.labels;
  const float* __restrict__ row_lse = z.row_lse;
  const float* __restrict__ row_pz = z.row_pz;
  const float* __restrict__ dlogprobs = z.dlogprobs;
  const float* __restrict__ dentropy = z.dentropy;
  uint16_t* __restrict__ D = z.D;
  // With a device-side count the tiles that hold tokens are numbered 0 .. tiles_m * ceil(T / 256) - 1, so that the hardware's
  // round-robin of workgroup ids over the XCDs spreads exactly those; the other workgroups of the (static) grid return at once.
  const int tiles_n = z.T_dev ? (T + BN - 1) / BN : z.tiles_n;
  if (id >= z.tiles_m * tiles_n) return;
  int tm, tn;
  tile_coords(id, z.tiles_m, tiles_n, kGroupM, tm, tn);

  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int wm = wave / WAVES_N, wn = wave % WAVES_N;
  const int lrow = lane & 15, kq = lane >> 4;
  const int vloc_base = tm * BM + wm * WM;    // first vocab row of this wave inside the chunk panel
  const int vbase = vc0 + vloc_base;          // ... and in the full vocab
  const int tbase = tn * BN + wn * WN;        // first token of this wave (always inside the padded panels)
  const bool full = vbase + WM <= V;
  const float scale2 = rcp_temp * kLog2e;

  // Per-token inputs of the epilogue.  The loads are issued here, before the mainloop, and their values are first touched
  // behind it, so the mainloop hides their latency; they are unconditional loads from a clamped token index (a load under
  // `t < T` becomes a branch with its own wait: one memory round trip per token block before the first copy is issued).  Lane
  // l loads tokens l and 64 + l of the wave's 128 -- twelve registers to carry through the mainloop -- and the values reach
  // the lanes that need them (token j * 16 + lrow for every token block j) through LDS afterwards.
  float g_[2], q_[2], lse_[2], pz_[2];
  int64_t y_[2];
#pragma unroll
  for (int u = 0; u < 2; ++u) {
    const int t = tbase + u * 64 + lane;
    const int tc = t < T ? t : T - 1;  // T >= 1 here: a tile without a token has returned above
    g_[u] = dlogprobs[tc];
    q_[u] = ENTGRAD ? dentropy[tc] : 0.f;
    lse_[u] = row_lse[tc];
    pz_[u] = ENTGRAD ? row_pz[tc] : 0.f;
    y_[u] = labels[tc];
  }

#if LMHEAD_ABLATE & 8
  Operand a{W, ldw, vc0 + (tm % 4) * BM, V};
  Operand b{Hd, ldh, (tn % 8) * BN, T};
#else
  Operand a{W, ldw, vc0 + tm * BM, V};
  Operand b{Hd, ldh, tn * BN, T};
#endif
  acc_t acc;
  prefetch_first_tiles(a, b, 0, H / BK, lds);  // the first copies travel while the accumulators are cleared
  zero_acc(acc);
  mainloop<false, EVEN>(a, b, 0, H / BK, lds, acc);
#if LMHEAD_ABLATE & 2
  return;
#endif

  constexpr int kTokRow = WM * 2 + 16;  // dz staging (below): 128 token rows x (128 vocab x 2 B + pad) per wave
  constexpr int kStage = WN * kTokRow;
  // The wave's per-token values, through a private 3 KiB of LDS behind the four staging regions (LDS operations of one wave
  // execute in order, so no barrier).
  constexpr int kTokBytes = WN * 24;
  static_assert(NWAVES * (kStage + kTokBytes) <= LDS_BYTES, "dz staging and per-token values do not fit LDS");
  char* tokv = lds + NWAVES * kStage + wave * kTokBytes;  // float4 {g, q, lse, pz} [128], then int64 label [128]
#pragma unroll
  for (int u = 0; u < 2; ++u) {
    const f32x4 v = {g_[u], q_[u], lse_[u], pz_[u]};
    *(f32x4*)(tokv + (u * 64 + lane) * 16) = v;
    *(int64_t*)(tokv + WN * 16 + (u * 64 + lane) * 8) = y_[u];
  }
  float gs_[TN], c0_[TN], c1_[TN], lse2_[TN];
  int yrel_[TN];
#pragma unroll
  for (int j = 0; j < TN; ++j) {
    const bool valid = tbase + j * MT + lrow < T;
    const f32x4 v = *(const f32x4*)(tokv + (j * MT + lrow) * 16);
    const float g = valid ? v[0] : 0.f;
    const float q = (ENTGRAD && valid) ? v[1] : 0.f;
    lse2_[j] = valid ? v[2] * kLog2e : INFINITY;
    const float pz = (ENTGRAD && valid) ? v[3] : 0.f;
    const int64_t y = valid ? *(const int64_t*)(tokv + WN * 16 + (j * MT + lrow) * 8) : (int64_t)-1;
    const int64_t yrel64 = y - (int64_t)vbase;
    yrel_[j] = (y >= 0 && y < (int64_t)V && yrel64 >= 0 && yrel64 < WM) ? (int)yrel64 : -1;
    gs_[j] = g * rcp_temp;
    c0_[j] = -(g - q * pz) * rcp_temp;
    c1_[j] = -q * rcp_temp * rcp_temp;
    // Optional (DzArgs::p_shift > 0): probabilities below 2^(p_shift - 126) count as zero.  The exponent is moved down by
    // p_shift so that v_exp_f32 -- which returns 0 where the result would be a denormal, below 2^-126 -- does the flush,
    // and the two coefficients carry the power of two back (exact).  Not for coefficients so large that the scaled ones
    // could overflow.
    if (z.p_shift > 0.f && fabsf(c0_[j]) < 0x1p30f && fabsf(c1_[j]) < 0x1p20f) {
      const float up = __builtin_amdgcn_exp2f(z.p_shift);
      lse2_[j] += z.p_shift;
      c0_[j] *= up;
      c1_[j] *= up;
    }
  }

  // The wave's 128 x 128 dz block leaves through LDS so that the panel is written with 16-byte stores: a lane holds four
  // consecutive vocab rows of one token, an 8-byte piece of a D row.  mainloop() left LDS free and every wave uses a
  // private region, so no barrier is needed (LDS operations of one wave execute in order).  The stores are marked
  // non-temporal: the panel is a gigabyte that is read back only by the next launch, and letting it displace the operand
  // panels from L2 costs the mainloops of the neighbouring tiles more than the stores themselves.
  char* stage = lds + wave * kStage;
  typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
  // Every staging address is one per-lane base plus a compile-time constant (an immediate of the LDS instruction), and the
  // panel rows are walked with one running pointer: written as (j * 16 + row) * pitch the compiler keeps eight row indices
  // alive across the whole epilogue and spills them, and a spill reload waits for vmcnt(0) -- i.e. for every panel store in flight.
  char* const st_w = stage + lrow * kTokRow + kq * 8;                      // + (j * MT) * kTokRow + i * MT * 2
  const char* const st_r = stage + (lane >> 4) * kTokRow + (lane & 15) * 16;  // + (j * MT + it * 4) * kTokRow
  uint16_t* d_row = D + (size_t)(tbase + (lane >> 4)) * (size_t)ldd + vloc_base + (lane & 15) * 8;  // four rows further per store
  const size_t d_step = (size_t)4 * (size_t)ldd;

  // A token block j (16 token rows x 128 vocab, 4 KiB of the staging region) is complete after its eight i-steps; its 256
  // 16-byte pieces (4 per lane; 16 lanes cover one token row of 256 bytes) go out in the middle of block j + 1, so that the
  // read-back and the store issue hide behind that block's arithmetic instead of forming a tail of their own.  Blocks are
  // flushed in order, j = 0 .. TN - 1.
  auto flush_block = [&](int j) {
#pragma unroll
    for (int it = 0; it < 4; ++it) {
      const u32x4 v = *(const u32x4*)(st_r + (j * MT + it * 4) * kTokRow);
#if LMHEAD_ABLATE & 4
      asm volatile("" ::"v"(v));  // staged and read back, not stored
#else
      __builtin_nontemporal_store(v, (u32x4*)d_row);
#endif
      d_row += d_step;
    }
  };
  // One token block: eight i-steps of four values per lane.  What is the same for the whole wave -- rows past the
  // vocabulary's end (RAGGED: only the last vocab tile), a label of some token inside the wave's rows (LABEL, decided per
  // token block by a ballot), the fp32 residual of the label's value (fp32 operands only) -- is decided once outside the
  // unrolled loops: as tests inside them they cost three branches per i-step, a third of the epilogue's time.
  auto token_block = [&](int j, auto ragged, auto label) {
    constexpr bool RAGGED = decltype(ragged)::value, LABEL = decltype(label)::value;
    const float gs = gs_[j], c0 = c0_[j], c1 = c1_[j], lse2 = lse2_[j];
    const int yrel = yrel_[j];
#pragma unroll
    for (int i = 0; i < TM; ++i) {
      float d[4];
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        const float x = acc[i][j][r];
        const float p = __builtin_amdgcn_exp2f(fmaf(x, scale2, -lse2));
        d[r] = ENTGRAD ? p * fmaf(c1, x, c0) : p * c0;
      }
      const int vl = i * MT + kq * 4;  // vocab row inside the wave block; this lane holds vl .. vl+3
      if (LABEL) {
#pragma unroll
        for (int r = 0; r < 4; ++r)
          if (yrel == vl + r) d[r] += gs;
      }
      if (RAGGED) {
#pragma unroll
        for (int r = 0; r < 4; ++r)
          if (vbase + vl + r >= V) d[r] = 0.f;
      }
      f32x4 v4 = {d[0], d[1], d[2], d[3]};
      const bf16x4 b4 = __builtin_convertvector(v4, bf16x4);
      *(uint2*)(st_w + (j * MT) * kTokRow + i * (MT * 2)) = *(const uint2*)&b4;
      if (LABEL && z.label_resid) {
#pragma unroll
        for (int r = 0; r < 4; ++r)
          if (yrel == vl + r) z.label_resid[tbase + j * MT + lrow] = d[r];
      }
      if (i == TM / 2 - 1 && j > 0) flush_block(j - 1);
    }
  };
  std::true_type yes;
  std::false_type no;
  if (__builtin_amdgcn_readfirstlane((int)full)) {
#pragma unroll
    for (int j = 0; j < TN; ++j) {
      if (__any(yrel_[j] >= 0)) token_block(j, no, yes);  // some token of this block has its label inside the wave's rows
      else token_block(j, no, no);
    }
  } else {
#pragma unroll
    for (int j = 0; j < TN; ++j) token_block(j, yes, yes);
  }
  flush_block(TN - 1);
}


// ------------------------------------------------------------------------------------------------------------
// Soft cross-entropy from hidden states (the draft-head loss of multi-token prediction, skyrl/backends/skyrl_train/mtp/
// soft_ce.py:200-240):  loss[t] = -sum_v softmax(z_teacher[t])_v * log_softmax(z_student[t])_v = lse_student - E_teacher[z_student],
// both logits rows being products with the same (detached) output weight.  The reference materialises both [T, V] logits
// tensors and their fp32 softmaxes; here the two hidden rows of a token sit in one "stacked" operand so that one lane
// holds z_student and z_teacher of the same (token, vocab) pair, TN / 2 accumulator blocks apart:
//   stacked row of token t:   student  (t / 64) * 128 + t % 64,   teacher  (t / 64) * 128 + 64 + t % 64
// i.e. each wave's 128 token rows are 64 student rows followed by the 64 teacher rows of the same tokens.  The forward
// is the ordinary tile kernel on the stacked rows with the paired third statistic; the backward recomputes a tile and
// writes  d loss / d z_student = g * (softmax(z_student) - softmax(z_teacher))  (soft_ce.py:146-151) for the student rows
// into the token-major dz panel, from which the ordinary dHidden GEMM runs.  The weight gets no gradient (it is detached
// in the reference, mtp/adapter.py:51-56), neither does the teacher.
// ------------------------------------------------------------------------------------------------------------
constexpr int kPairRows = WN / 2;  // 64 tokens per wave

__host__ __device__ inline int64_t stacked_row(int64_t t, bool teacher) {
  return (t / kPairRows) * WN + (teacher ? kPairRows : 0) + t % kPairRows;
}

// One workgroup per stacked row: copies the student's or the teacher's hidden row, zeros for the padding tokens.
// Teacher row of token t = b * seq_len + s is the teacher's hidden row b * seq_len + (s + shift) mod seq_len: the roll of
// build_teacher_logits (soft_ce.py:22-34) applied to the hidden states instead of the logits.
__global__ __launch_bounds__(256) void softce_pack_rows(const uint16_t* __restrict__ student, int lds_,
                                                        const uint16_t* __restrict__ teacher, int ldt, int T, int seq_len,
                                                        int shift, int H, uint16_t* __restrict__ stacked) {
  const int r = blockIdx.x;
  const bool is_teacher = (r / kPairRows) & 1;
  const int t = (r / WN) * kPairRows + r % kPairRows;
  const uint16_t* src = nullptr;
  if (t < T) {
    if (is_teacher) {
      const int b = t / seq_len, sft = (t % seq_len + shift) % seq_len;
      src = teacher + (size_t)(b * seq_len + sft) * (size_t)ldt;
    } else {
      src = student + (size_t)t * (size_t)lds_;
    }
  }
  uint16_t* dst = stacked + (size_t)r * (size_t)H;
  for (int c = threadIdx.x * 8; c < H; c += 256 * 8)
    *(uint4*)(dst + c) = src ? *(const uint4*)(src + c) : make_uint4(0, 0, 0, 0);
}

template <bool ENTROPY, bool EVEN>
__global__ __launch_bounds__(NTHREADS) void softce_fwd_tiles(const uint16_t* __restrict__ W, int ldw,
                                                             const uint16_t* __restrict__ Hd, int ldh, int T, int H, int V,
                                                             float rcp_temp, float* __restrict__ part_max,
                                                             float* __restrict__ part_sum, float* __restrict__ part_pz) {
  __shared__ __attribute__((aligned(1024))) char lds[LDS_BYTES];
  fwd_tile<ENTROPY, true, EVEN>(W, ldw, Hd, ldh, T, H, V, rcp_temp, part_max, part_sum, part_pz, lds);
}

// Per token: the merged statistics of its two stacked rows -> loss and the two log-sum-exps the backward needs.
__global__ __launch_bounds__(256) void softce_finish(const float* __restrict__ row_lse, const float* __restrict__ row_pz, int T,
                                                     float* __restrict__ loss, float* __restrict__ lse_student,
                                                     float* __restrict__ lse_teacher) {
  const int t = blockIdx.x * 256 + threadIdx.x;
  if (t >= T) return;
  const int64_t rs = stacked_row(t, false), rt = stacked_row(t, true);
  const float ls = row_lse[rs];
  loss[t] = ls - row_pz[rt];  // row_pz of a teacher row is E_teacher[z_student]
  lse_student[t] = ls;
  lse_teacher[t] = row_lse[rt];
}

struct SoftCeDzArgs {
  const uint16_t* W;
  int ldw;
  const uint16_t* S;  // stacked hidden rows [2 * Tp, H], Tp = T rounded up to whole 128-token tiles
  int T, Tp, H, V;
  float rcp_temp;
  const float* lse_student;
  const float* lse_teacher;
  const float* dloss;
  int vc0, tiles_m, tiles_n;  // first vocab row of the chunk; tiles along the chunk's vocab rows and the stacked rows
  uint16_t* D;                // [Tp, ldd]  dz of the student rows, token-major
  int ldd;
};

template <bool EVEN>
__global__ __launch_bounds__(NTHREADS) void softce_dz_tiles(const SoftCeDzArgs z) {
  __shared__ __attribute__((aligned(1024))) char lds[LDS_BYTES];
  const uint16_t* __restrict__ W = z.W;
  const uint16_t* __restrict__ S = z.S;
  const int T = z.T, H = z.H, V = z.V, vc0 = z.vc0, ldd = z.ldd;
  uint16_t* __restrict__ D = z.D;
  int tm, tn;
  tile_coords(blockIdx.x, z.tiles_m, z.tiles_n, kGroupM, tm, tn);

  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int wm = wave / WAVES_N, wn = wave % WAVES_N;
  const int lrow = lane & 15, kq = lane >> 4;
  const int vloc_base = tm * BM + wm * WM;
  const int vbase = vc0 + vloc_base;
  const int tokbase = (tn * WAVES_N + wn) * kPairRows;  // first token of this wave
  const bool full = vbase + WM <= V;
  const float scale2 = z.rcp_temp * kLog2e;

  // Per-token inputs: unconditional loads from a clamped index, issued before the mainloop and first touched behind it (as
  // in dz_tile: a load under `t < T` is a branch with its own wait in front of the first copy).
  float gs_[TN / 2], ls2_[TN / 2], lt2_[TN / 2];
#pragma unroll
  for (int j = 0; j < TN / 2; ++j) {
    const int t = tokbase + j * MT + lrow;
    const int tc = t < T ? t : T - 1;  // T >= 1: the host launches nothing for an empty batch
    gs_[j] = z.dloss[tc];
    ls2_[j] = z.lse_student[tc];
    lt2_[j] = z.lse_teacher[tc];
  }

  Operand a{W, z.ldw, vc0 + tm * BM, V};
  Operand b{S, H, tn * BN, 2 * z.Tp};
  acc_t acc;
  prefetch_first_tiles(a, b, 0, H / BK, lds);  // the first copies travel while the accumulators are cleared
  zero_acc(acc);
  mainloop<false, EVEN>(a, b, 0, H / BK, lds, acc);
#pragma unroll
  for (int j = 0; j < TN / 2; ++j) {
    const bool valid = tokbase + j * MT + lrow < T;
    gs_[j] = valid ? gs_[j] * z.rcp_temp : 0.f;
    ls2_[j] = valid ? ls2_[j] * kLog2e : INFINITY;
    lt2_[j] = valid ? lt2_[j] * kLog2e : INFINITY;
  }

  // Staging as in dz_tile: a private region per wave, 64 token rows of 128 vocab columns, then 16-byte non-temporal stores.
  constexpr int kTokRow = WM * 2 + 16;
  constexpr int kStage = WN * kTokRow;
  char* stage = lds + wave * kStage;
  typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
  auto flush_block = [&](int j) {  // as in dz_tile: a finished token block leaves while the next one is computed
#pragma unroll
    for (int it = 0; it < 4; ++it) {
      const int idx = it * 64 + lane;
      const int n = j * MT + (idx >> 4), c = idx & 15;
      const u32x4 v = *(const u32x4*)(stage + n * kTokRow + c * 16);
      __builtin_nontemporal_store(v, (u32x4*)(D + (size_t)(tokbase + n) * (size_t)ldd + vloc_base + c * 8));
    }
  };
#pragma unroll
  for (int j = 0; j < TN / 2; ++j) {
    const float gs = gs_[j], ls2 = ls2_[j], lt2 = lt2_[j];
#pragma unroll
    for (int i = 0; i < TM; ++i) {
      float d[4];
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        const float q = __builtin_amdgcn_exp2f(fmaf(acc[i][j][r], scale2, -ls2));
        const float p = __builtin_amdgcn_exp2f(fmaf(acc[i][j + TN / 2][r], scale2, -lt2));
        d[r] = gs * (q - p);
      }
      const int vl = i * MT + kq * 4;
      if (!full) {
#pragma unroll
        for (int r = 0; r < 4; ++r)
          if (vbase + vl + r >= V) d[r] = 0.f;
      }
      f32x4 v4 = {d[0], d[1], d[2], d[3]};
      const bf16x4 b4 = __builtin_convertvector(v4, bf16x4);
      *(uint2*)(stage + (j * MT + lrow) * kTokRow + vl * 2) = *(const uint2*)&b4;
      if (i == TM / 2 - 1 && j > 0) flush_block(j - 1);
    }
  }
  flush_block(TN / 2 - 1);
}

// ------------------------------------------------------------------------------------------------------------
// Plain NT GEMM with an fp32 / bf16 store epilogue:  C[N,M] (+)= B[N,K] . A[M,K]^T, i.e. C[n][m] = sum_k A[m][k] B[n][k]:
// the MFMA M axis (rows of A) runs along the contiguous dimension of C, because a lane's four accumulator values are
// consecutive along M -- one 16-byte fp32 (8-byte bf16) store.  M must be a multiple of 4.
//   Cin != 0   add the existing fp32 C before storing (accumulation across micro-batches)
//   Cf  != 0   store fp32;   Cb != 0  store bf16 (round-to-nearest-even)
// One launch carries up to two independent problems (workgroups [0, tiles0) work on p0, the rest on p1): the dHidden
// and dWeight products of a vocab chunk have no dependency on each other, and together they fill the 256 CUs in whole
// rounds where each alone leaves a partial last round.
// ------------------------------------------------------------------------------------------------------------
struct GemmArgs {
  const uint16_t* A;
  int lda, a_rows;
  const uint16_t* B;
  int ldb, b_rows;  // K-major B: b_rows is the number of valid columns (n) of the stored matrix
  int b_kmajor;     // B is stored K-major, B[k * ldb + n]
  int c_rows_m;     // the bf16 output is C[m * ldc + n] (n contiguous) instead of C[n * ldc + m]
  int nk, M, N;
  const float* Cin;
  float* Cf;
  uint16_t* Cb;
  int ldc;
  // Partial sums carried from launch to launch (dHidden across vocab chunks) live in "accumulator order": tile by tile,
  // wave by wave, MFMA block by MFMA block, each lane's 4 registers contiguous.  Reading and writing them is 16 bytes
  // per lane and 1 KiB contiguous per wave instruction, with no address arithmetic beyond a constant offset.
  const float* Pin;
  float* Pout;
  // When not NULL: a token count in device memory that replaces one extent of the problem, chosen by t_role: the rows M
  // (kTokensOnM), the columns N (kTokensOnN) or the contraction length, nk = ceil(count / 64) (kTokensOnK).  The host-side
  // value of that extent is an upper bound that sizes the grid and the scratch; tiles beyond the count return at once.
  const int* T_dev;
  int t_role;
};
enum { kTokensOnM = 1, kTokensOnN = 2, kTokensOnK = 3 };

// BKM: the B operand is K-major.  The two variants are separate instantiations of the whole tile (mainloop and
// epilogue) so that their accumulators never meet at a join, where the register allocator would shuffle all 256 of them.
template <bool BKM>
__device__ __forceinline__ void gemm_tile(const GemmArgs& p, int bid, char* lds) {
  int M = p.M, N = p.N, nk = p.nk;
  if (p.T_dev) {
    const int count = __builtin_amdgcn_readfirstlane(*p.T_dev);
    if (p.t_role == kTokensOnM) M = count;
    else if (p.t_role == kTokensOnN) N = count;
    else nk = (count + 2 * BK - 1) / (2 * BK) * 2;  // whole pairs of k-tiles: the rows up to the next multiple of 256 are zeros
    // Nothing to contract: C += 0 needs no work; a C that is overwritten or converted still goes through the epilogue.
    if (nk == 0 && !p.Cb && p.Cin == p.Cf) return;
  }
  // Tiles of the extents in force: with a device-side count the tiles that hold tokens are numbered from 0, so that the
  // round-robin of workgroup ids over the XCDs spreads exactly those, and the rest of the (static) grid returns at once.  The
  // partial sums that cross vocab chunks are laid out by the same numbering (the count does not change between chunks).
  const int tiles_m = (M + BM - 1) / BM;
  const int tiles_n = (N + BN - 1) / BN;
  if (bid >= tiles_m * tiles_n) return;
  int tm, tn;
  tile_coords(bid, tiles_m, tiles_n, kGroupM, tm, tn);
#if LMHEAD_ABLATE & 16
  Operand a{p.A, p.lda, (tm % 4) * BM, p.a_rows};
  Operand b{p.B, p.ldb, (tn % 8) * BN, p.b_rows};
#else
  Operand a{p.A, p.lda, tm * BM, p.a_rows};
  Operand b{p.B, p.ldb, tn * BN, p.b_rows};
#endif
  acc_t acc;
  if (nk > 0) prefetch_first_tiles<BKM>(a, b, 0, nk, lds);
  zero_acc(acc);
  if (nk > 0) {
    mainloop<BKM, true>(a, b, 0, nk, lds, acc);  // nk is even for every gradient GEMM (make_gemm checks)
  }

  const float* __restrict__ Cin = p.Cin;
  float* __restrict__ Cf = p.Cf;
  uint16_t* __restrict__ Cb = p.Cb;
  const int ldc = p.ldc;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int wm = wave / WAVES_N, wn = wave % WAVES_N;
  const int lrow = lane & 15, kq = lane >> 4;

  if (p.Pin || p.Pout) {
    const size_t base = ((size_t)(tm * tiles_n + tn) * NWAVES + wave) * (TM * TN * 64 * 4) + (size_t)lane * 4;
    if (p.Pin) {  // sixteen loads in flight at a time: one at a time costs a round trip to HBM each (36 us per tile)
#pragma unroll
      for (int i = 0; i < TM; i += 2) {
        f32x4 t[2 * TN];
#pragma unroll
        for (int x = 0; x < 2 * TN; ++x) t[x] = *(const f32x4*)(p.Pin + base + (size_t)(i * TN + x) * (64 * 4));
#pragma unroll
        for (int x = 0; x < 2 * TN; ++x) acc[i + x / TN][x % TN] += t[x];
      }
    }
    if (p.Pout) {
#pragma unroll
      for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j) *(f32x4*)(p.Pout + base + (size_t)(i * TN + j) * (64 * 4)) = acc[i][j];
    }
  }
  if (!Cf && !Cb) return;

  if (BKM && p.c_rows_m) {
    // Output rows run along M: a lane's four values belong to four different rows; sixteen lanes (n = lrow) cover 32
    // contiguous bytes of each.  Only the last vocab chunk's dHidden tiles come through here.
#pragma unroll
    for (int j = 0; j < TN; ++j) {
      const int n = tn * BN + wn * WN + j * MT + lrow;
      if (n >= N) continue;
#pragma unroll
      for (int i = 0; i < TM; ++i) {
        const int m = tm * BM + wm * WM + i * MT + kq * 4;
        const bf16x4 b4 = __builtin_convertvector(acc[i][j], bf16x4);
        const uint16_t* h4 = (const uint16_t*)&b4;
#pragma unroll
        for (int r = 0; r < 4; ++r)
          if (m + r < M) Cb[(size_t)(m + r) * (size_t)ldc + n] = h4[r];
      }
    }
    return;
  }

#pragma unroll
  for (int j = 0; j < TN; ++j) {
    const int n = tn * BN + wn * WN + j * MT + lrow;
    if (n >= N) continue;
#pragma unroll
    for (int i = 0; i < TM; ++i) {
      const int m = tm * BM + wm * WM + i * MT + kq * 4;  // this lane holds m .. m+3
      if (m < M) {
        const size_t idx = (size_t)n * (size_t)ldc + m;
        f32x4 v = acc[i][j];
        if (Cin) v += *(const f32x4*)(Cin + idx);
        if (Cf) *(f32x4*)(Cf + idx) = v;
        if (Cb) {
          const bf16x4 b4 = __builtin_convertvector(v, bf16x4);
          *(uint2*)(Cb + idx) = *(const uint2*)&b4;
        }
      }
    }
  }
}

// The two kinds of backward launch per vocab chunk, as kernels of their own so that a kernel trace tells them apart:
// the dz tiles of the chunk, then its two gradient GEMMs in one launch (workgroups [0, tiles0) work on p0, the rest on p1).
template <bool ENTGRAD, bool EVEN>
__global__ __launch_bounds__(NTHREADS) void lmhead_bwd_dz(const DzArgs z) {
  __shared__ __attribute__((aligned(1024))) char lds[LDS_BYTES];
  dz_tile<ENTGRAD, EVEN>(z, blockIdx.x, lds);
}

__global__ __launch_bounds__(NTHREADS) void lmhead_bwd_gemm(const GemmArgs p0, const GemmArgs p1, int tiles0) {
  __shared__ __attribute__((aligned(1024))) char lds[LDS_BYTES];
  const int id = blockIdx.x;
  // dW always reads the dz panel K-major (K = tokens); dHidden either reads the weight itself K-major (K = vocab) or,
  // when the vocabulary is not a multiple of two k-tiles, a transposed, zero-padded copy of it with K contiguous.
  const bool second = id >= tiles0;
  if (second || p0.b_kmajor) gemm_tile<true>(second ? p1 : p0, second ? id - tiles0 : id, lds);
  else gemm_tile<false>(p0, id, lds);
}

// Measurement aid: the mainloop's MFMA sequence (two 32-k steps of 64 MFMAs, same order, accumulators in AGPRs) with
// register-resident operands and nothing else in the loop -- what the matrix pipe sustains on a given kind of data.
__global__ __launch_bounds__(NTHREADS) void mfma_probe(const bf16x8* __restrict__ operands, int iters, float* __restrict__ sink) {
  bf16x8 af[2][TM], bfr[2][TN];
#pragma unroll
  for (int s = 0; s < 2; ++s)
#pragma unroll
    for (int i = 0; i < TM; ++i) {
      af[s][i] = operands[((s * TM + i) * 2 + 0) * NTHREADS + threadIdx.x];
      bfr[s][i] = operands[((s * TM + i) * 2 + 1) * NTHREADS + threadIdx.x];
    }
  acc_t acc;
  zero_acc(acc);
  for (int it = 0; it < iters; ++it) {
#pragma unroll
    for (int ks = 0; ks < KSTEPS; ++ks)
#pragma unroll
      for (int x = 0; x < TM * TN; ++x) {
        const int i = mfma_row(x), j = mfma_col(x);
        mfma_16x16x32(acc[i][j], af[ks][i], bfr[ks][j]);
      }
  }
  asm volatile("s_nop 15\n\ts_nop 15" ::: "memory");
  float sum = 0.f;
#pragma unroll
  for (int i = 0; i < TM; ++i)
#pragma unroll
    for (int j = 0; j < TN; ++j) {
      asm volatile("" : "+a"(acc[i][j]));
      sum += acc[i][j][0] + acc[i][j][1] + acc[i][j][2] + acc[i][j][3];
    }
  sink[blockIdx.x * NTHREADS + threadIdx.x] = sum;
}

// Measurement aid: the fp32 atomic traffic of a fully fused backward (efficient_entropy_backward_kernel_general_mainloop_MN,
// fused_linear_logprob_triton.py:807-996) and nothing else.  Such a kernel forms the dz tile of 256 vocab rows x 256 tokens and
// has to add its contribution to dW[256, H] and to dHidden[256, H] in memory, because no workgroup can hold a [256, H]
// accumulator.  One workgroup per (vocab tile, token tile) issues exactly those adds -- in the accumulator layout, a lane's
// four values contiguous -- with no logits recompute and no MFMA: a lower bound of what the fused variant costs.
__global__ __launch_bounds__(NTHREADS) void atomic_floor_probe(float* __restrict__ dW, float* __restrict__ dH, int tiles_v, int H) {
  const int tv = blockIdx.x % tiles_v, tt = blockIdx.x / tiles_v;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int wm = wave / WAVES_N, wn = wave % WAVES_N, lrow = lane & 15, kq = lane >> 4;
  for (int c0 = 0; c0 < H; c0 += BN) {
#pragma unroll
    for (int half = 0; half < 2; ++half) {
      float* dst = half ? dH + (size_t)tt * BM * (size_t)H : dW + (size_t)tv * BM * (size_t)H;
#pragma unroll 4
      for (int x = 0; x < TM * TN; ++x) {
        const int i = x / TN, j = x % TN;
        const int n = c0 + wn * WN + j * MT + lrow;          // column of the [256, H] slice
        if (n >= H) continue;
        const int m = wm * WM + i * MT + kq * 4;             // this lane adds rows m .. m+3
#pragma unroll
        for (int r = 0; r < 4; ++r) atomicAdd(dst + (size_t)(m + r) * (size_t)H + n, 1.0f);
      }
    }
  }
}

// dst[c, r] = src[r, c] for r < R, c < C;  dst[c, r] = 0 for R <= r < Rpad.  bf16 bits, 64 x 64 tiles.
// R_dev (may be NULL): the number of valid source rows as a value in device memory, <= R.
__global__ __launch_bounds__(256) void transpose_bf16(const uint16_t* __restrict__ src, int lds_src, int R, int C,
                                                      uint16_t* __restrict__ dst, int ld_dst, int Rpad,
                                                      const int* __restrict__ R_dev) {
  __shared__ uint16_t tile[64][66];
  if (R_dev) R = *R_dev;
  const int r0 = blockIdx.x * 64, c0 = blockIdx.y * 64;
  const int tid = threadIdx.x;
#pragma unroll
  for (int it = 0; it < 2; ++it) {
    const int idx = it * 256 + tid;  // 512 chunks of 8 elements
    const int rr = idx >> 3, cc = (idx & 7) * 8;
    const int r = r0 + rr, c = c0 + cc;
    uint16_t v[8] = {0, 0, 0, 0, 0, 0, 0, 0};
    if (r < R) {
      if (c + 8 <= C) {
        const uint4 q = *(const uint4*)(src + (size_t)r * (size_t)lds_src + c);
        const uint32_t w[4] = {q.x, q.y, q.z, q.w};
#pragma unroll
        for (int k = 0; k < 4; ++k) {
          v[2 * k] = (uint16_t)(w[k] & 0xffffu);
          v[2 * k + 1] = (uint16_t)(w[k] >> 16);
        }
      } else {
        for (int k = 0; k < 8; ++k)
          if (c + k < C) v[k] = src[(size_t)r * (size_t)lds_src + c + k];
      }
    }
#pragma unroll
    for (int k = 0; k < 8; ++k) tile[rr][cc + k] = v[k];
  }
  __syncthreads();
#pragma unroll
  for (int it = 0; it < 2; ++it) {
    const int idx = it * 256 + tid;
    const int cc = idx >> 3, rr = (idx & 7) * 8;  // output row = source column
    const int c = c0 + cc, r = r0 + rr;
    if (c < C && r < Rpad) {
      uint32_t w[4];
#pragma unroll
      for (int k = 0; k < 4; ++k) w[k] = (uint32_t)tile[rr + 2 * k][cc] | ((uint32_t)tile[rr + 2 * k + 1][cc] << 16);
      *(uint4*)(dst + (size_t)c * (size_t)ld_dst + r) = make_uint4(w[0], w[1], w[2], w[3]);
    }
  }
}

// ------------------------------------------------------------------------------------------------------------
// fp32 operands on the bf16 matrix pipe.  An fp32 value is the sum of bf16 terms, x = hi + lo (+ 2^-17 |x|), hi = bf16(x),
// lo = bf16(x - hi), and a product of sums is a sum of products: stacking the terms along the contraction axis,
//     weight fp32, hidden bf16:   [w_hi | w_lo] . [h | h]^T           = h . (w_hi + w_lo)
//     weight fp32, hidden fp32:   [w_hi | w_lo | w_hi] . [h_hi | h_hi | h_lo]^T = h_hi . w_hi + h_hi . w_lo + h_lo . w_hi
// turns the fp32 logits GEMM (model_utils.py:328-333: hidden is cast to the weight's dtype, the product is fp32) into the
// ordinary bf16 GEMM with two or three times the contraction length; the MFMA accumulates all terms in fp32.  What is dropped
// is below 2^-16 of each product.  This kernel writes one stacked operand: segment s of row r holds the hi (code 0) or lo
// (code 1) terms of the row.
// ------------------------------------------------------------------------------------------------------------
__device__ __forceinline__ uint16_t bf16_rne(float x) {
  const uint32_t u = __float_as_uint(x);
  if ((u & 0x7fffffffu) > 0x7f800000u) return (uint16_t)((u >> 16) | 0x40u);  // NaN stays NaN
  return (uint16_t)((u + 0x7fffu + ((u >> 16) & 1u)) >> 16);
}

template <bool SRC_FP32>
__global__ __launch_bounds__(256) void split_operand_rows(const void* __restrict__ src, int64_t ld_src, int H, int terms, int code0,
                                                          int code1, int code2, uint16_t* __restrict__ dst, int64_t ld_dst) {
  const int64_t r = blockIdx.x;
  const int codes[3] = {code0, code1, code2};
  for (int c = threadIdx.x * 4; c < H; c += 256 * 4) {
    uint16_t hi[4], lo[4];
    if (SRC_FP32) {
      const float4 v = *(const float4*)((const float*)src + r * ld_src + c);
      const float x[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
      for (int k = 0; k < 4; ++k) {
        hi[k] = bf16_rne(x[k]);
        lo[k] = bf16_rne(x[k] - __uint_as_float((uint32_t)hi[k] << 16));
      }
    } else {
      const uint2 v = *(const uint2*)((const uint16_t*)src + r * ld_src + c);
      hi[0] = (uint16_t)(v.x & 0xffffu), hi[1] = (uint16_t)(v.x >> 16), hi[2] = (uint16_t)(v.y & 0xffffu), hi[3] = (uint16_t)(v.y >> 16);
      lo[0] = lo[1] = lo[2] = lo[3] = 0;
    }
    for (int s = 0; s < terms; ++s) {
      const uint16_t* t = codes[s] ? lo : hi;
      *(uint2*)(dst + r * ld_dst + (int64_t)s * H + c) =
          make_uint2((uint32_t)t[0] | ((uint32_t)t[1] << 16), (uint32_t)t[2] | ((uint32_t)t[3] << 16));
    }
  }
}

// ------------------------------------------------------------------------------------------------------------
// Row compaction for the backward.  A token whose upstream gradients are both zero has a zero dz row: it adds nothing to
// dW and its dHidden row is zero.  In RL micro-batches those are the prompt and padding tokens the loss mask removes, often
// more than half of the batch.  Three small kernels let the backward run on the remaining rows without the host ever
// learning how many there are (no synchronisation, so the call can be captured in a HIP graph):
//   compact_active_rows   one workgroup: idx[i] = i-th token with g != 0 or q != 0 (ascending), counts[0] = their number n,
//                         counts[1 + b] = how many of them fall into block b of `block` compacted rows
//   gather_active_rows    compacted copies of hidden rows and of the per-token inputs; zero dHidden rows for the inactive
//   scatter_active_rows   dHidden rows of the compacted problem back to their tokens
// The GEMM kernels take the counts from device memory (T_dev) and run on the static upper-bound grid.
// ------------------------------------------------------------------------------------------------------------
constexpr int kCompactThreads = 1024;

__global__ __launch_bounds__(kCompactThreads) void compact_active_rows(const float* __restrict__ g, const float* __restrict__ q,
                                                                       int T, int block, int nblocks, int* __restrict__ idx,
                                                                       int* __restrict__ counts) {
  __shared__ int wave_sum[kCompactThreads / 64];
  __shared__ int carry;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  if (tid == 0) carry = 0;
  __syncthreads();
  for (int t0 = 0; t0 < T; t0 += kCompactThreads) {
    const int t = t0 + tid;
    const bool active = t < T && (g[t] != 0.f || (q && q[t] != 0.f));
    const unsigned long long ballot = __ballot(active);
    const int before = __popcll(ballot & ((1ull << lane) - 1ull));
    if (lane == 0) wave_sum[wave] = __popcll(ballot);
    __syncthreads();
    int base = carry;
    for (int w = 0; w < wave; ++w) base += wave_sum[w];
    if (active) idx[base + before] = t;
    __syncthreads();
    if (tid == 0) {
      int total = 0;
      for (int w = 0; w < kCompactThreads / 64; ++w) total += wave_sum[w];
      carry += total;
    }
    __syncthreads();
  }
  const int n = carry;
  for (int b = tid; b <= nblocks; b += kCompactThreads) {
    if (b == 0) {
      counts[0] = n;
    } else {
      const long long left = (long long)n - (long long)(b - 1) * block;
      counts[b] = left < 0 ? 0 : (left > block ? block : (int)left);
    }
  }
}

// One workgroup per row r < T: as compacted row r (when r < n) it copies the inputs of token idx[r]; as token r it clears
// d_hidden[r] -- active tokens get their row from scatter_active_rows afterwards.
__global__ __launch_bounds__(256) void gather_active_rows(const int* __restrict__ idx, const int* __restrict__ counts,
                                                          const uint16_t* __restrict__ hidden, int ldh, int Hk, int H,
                                                          const int64_t* __restrict__ labels, const float* __restrict__ lse,
                                                          const float* __restrict__ pz, const float* __restrict__ g,
                                                          const float* __restrict__ q, uint16_t* __restrict__ hidden_c,
                                                          int64_t* __restrict__ labels_c, float* __restrict__ lse_c,
                                                          float* __restrict__ pz_c, float* __restrict__ g_c,
                                                          float* __restrict__ q_c, uint16_t* __restrict__ d_hidden) {
  const int r = blockIdx.x;
  uint16_t* zero_row = d_hidden + (size_t)r * (size_t)H;
  for (int c = threadIdx.x * 8; c < H; c += 256 * 8) *(uint4*)(zero_row + c) = make_uint4(0, 0, 0, 0);
  if (r >= counts[0]) return;
  const int t = idx[r];
  const uint16_t* src = hidden + (size_t)t * (size_t)ldh;
  uint16_t* dst = hidden_c + (size_t)r * (size_t)Hk;
  for (int c = threadIdx.x * 8; c < Hk; c += 256 * 8) *(uint4*)(dst + c) = *(const uint4*)(src + c);
  if (threadIdx.x == 0) {
    labels_c[r] = labels[t];
    lse_c[r] = lse[t];
    g_c[r] = g[t];
    if (q) q_c[r] = q[t], pz_c[r] = pz[t];
  }
}

__global__ __launch_bounds__(256) void scatter_active_rows(const int* __restrict__ idx, const int* __restrict__ counts,
                                                           const uint16_t* __restrict__ d_hidden_c, int H,
                                                           uint16_t* __restrict__ d_hidden) {
  const int r = blockIdx.x;
  if (r >= counts[0]) return;
  const uint16_t* src = d_hidden_c + (size_t)r * (size_t)H;
  uint16_t* dst = d_hidden + (size_t)idx[r] * (size_t)H;
  for (int c = threadIdx.x * 8; c < H; c += 256 * 8) *(uint4*)(dst + c) = *(const uint4*)(src + c);
}

// What the bf16 product dropped of the label's dz value d (see DzArgs::label_resid), added to the weight gradient in fp32:
//     dW[label_t, :] += (d - bf16(d)) * h_hi[t, :]  +  d * h_lo[t, :]
// h_lo is the third segment of a stacked fp32 hidden row (lo_offset = 2 * H) and absent (lo_offset = 0) for a bf16 hidden.
// One workgroup per token; fp32 atomic adds, because several tokens may share a label (their order, and with it the last
// bit of those rows, is not fixed).
__global__ __launch_bounds__(256) void label_residual_update(const float* __restrict__ label_dz, const int64_t* __restrict__ labels,
                                                             const uint16_t* __restrict__ hidden, int ldh, int H, int lo_offset,
                                                             int V, const int* __restrict__ T_dev, float* __restrict__ dW) {
  const int t = blockIdx.x;
  if (T_dev && t >= *T_dev) return;
  const float d = label_dz[t];
  const int64_t y = labels[t];
  if (d == 0.f || y < 0 || y >= (int64_t)V) return;
  const float r = d - __uint_as_float((uint32_t)bf16_rne(d) << 16);
  const uint16_t* hp = hidden + (size_t)t * (size_t)ldh;
  float* wp = dW + (size_t)y * (size_t)H;
  for (int c = threadIdx.x; c < H; c += 256) {
    float add = r * __uint_as_float((uint32_t)hp[c] << 16);
    if (lo_offset) add = fmaf(d, __uint_as_float((uint32_t)hp[lo_offset + c] << 16), add);
    atomicAdd(wp + c, add);
  }
}

__global__ __launch_bounds__(256) void zero_f32(float* __restrict__ p, int n) {
  const int i = blockIdx.x * 256 + threadIdx.x;
  if (i < n) p[i] = 0.f;
}

// ------------------------------------------------------------------------------------------------------------
// Host side
// ------------------------------------------------------------------------------------------------------------
// Optional per-kernel timing: while a profile is open on the calling thread every launch below is bracketed by a pair of
// HIP events on the launch stream.  Closed profiles cost one thread-local load per launch.
enum KernelKind {
  kFwdTiles = 0, kFwdMerge, kTranspose, kBwdChunkDz, kBwdChunkGemm, kSoftCePack, kSoftCeFwdTiles, kSoftCeFinish, kSoftCeDz,
  kCompactRows, kSplitOperand, kTopkFilter, kTopkSelect, kTopkRows, kTopkBwdRows,
  kNumKernelKinds
};
const char* const kKernelNames[kNumKernelKinds] = {"lmhead_fwd_tiles", "lmhead_fwd_merge", "transpose_bf16",
                                                   "lmhead_bwd_dz", "lmhead_bwd_gemm", "softce_pack_rows",
                                                   "softce_fwd_tiles", "softce_finish", "softce_dz_tiles",
                                                   "active_rows[compact+gather+scatter]", "split_operand_rows",
                                                   "topk_filter_tiles", "topk_select", "topk_softce_rows",
                                                   "topk_softce_bwd_rows"};
struct Profile {
  struct Rec {
    int kind;
    hipEvent_t a, b;
  };
  std::vector<Rec> recs;
};
thread_local Profile* tl_profile = nullptr;

struct Timed {
  int kind;
  hipStream_t s;
  hipEvent_t a = nullptr, b = nullptr;
  Timed(int k, hipStream_t st) : kind(k), s(st) {
    if (tl_profile && hipEventCreate(&a) == hipSuccess && hipEventCreate(&b) == hipSuccess) (void)hipEventRecord(a, s);
  }
  ~Timed() {
    if (tl_profile && a && b) {
      (void)hipEventRecord(b, s);
      tl_profile->recs.push_back({kind, a, b});
    }
  }
};

struct Carver {
  char* base;
  size_t off = 0;
  explicit Carver(void* p) : base((char*)p) {}
  template <typename T>
  T* take(size_t count) {
    off = (size_t)round_up((int64_t)off, 256);
    T* p = base ? (T*)(base + off) : nullptr;
    off += count * sizeof(T);
    return p;
  }
};

inline bool aligned16(const void* p) { return ((uintptr_t)p & 15u) == 0; }

// Largest T, H or V any entry point accepts (row pitches are limited to kMaxRowPitch, far below it); the workspace queries
// answer 0 beyond it instead of computing with sizes that no call would accept.
constexpr int64_t kMaxExtent = (int64_t)1 << 30;

// The two bf16 operands of every entry point: hidden rows [T, H] and weight rows [V, H].
// Matrices may be of any size: the copy plan addresses a tile with 32-bit offsets from the tile's own first row, so only
// the row pitch is limited (256 rows must span less than 4 GiB: kMaxRowPitch elements).
int check_operands(const void* hidden, int64_t ldh, const void* weight, int64_t ldw, int64_t T, int64_t H, int64_t V,
                   float rcp_temperature, bool hidden_in_blocks = false) {
  if (!hidden || !weight) return SKYRL_LMHEAD_ERR_NULL;
  if (T < 1 || V < 1 || H < BK || H % BK != 0 || ldh < H || ldw < H) return SKYRL_LMHEAD_ERR_SHAPE;
  if (T > kMaxExtent || V > kMaxExtent) return SKYRL_LMHEAD_ERR_SHAPE;
  (void)hidden_in_blocks;
  if (ldh > kMaxRowPitch || ldw > kMaxRowPitch) return SKYRL_LMHEAD_ERR_SHAPE;
  if (!aligned16(hidden) || !aligned16(weight) || ldh % 8 != 0 || ldw % 8 != 0) return SKYRL_LMHEAD_ERR_ALIGN;
  if (!(rcp_temperature > 0.f) || !isfinite(rcp_temperature)) return SKYRL_LMHEAD_ERR_ARG;
  return SKYRL_LMHEAD_OK;
}

int check_common(const void* hidden, int64_t ldh, const void* weight, int64_t ldw, const int64_t* labels, int64_t T,
                 int64_t H, int64_t V, float rcp_temperature, bool hidden_in_blocks = false) {
  if (!hidden || !weight || !labels) return SKYRL_LMHEAD_ERR_NULL;
  const int st = check_operands(hidden, ldh, weight, ldw, T, H, V, rcp_temperature, hidden_in_blocks);
  if (st == SKYRL_LMHEAD_ERR_SHAPE) return st;  // shape errors are reported before alignment errors, labels included
  if ((uintptr_t)labels & 7u) return SKYRL_LMHEAD_ERR_ALIGN;
  return st;
}

// Compute units of the current device (256 on an MI355X); 256 when no device answers, so that the workspace query gives
// the same figure on a machine without a GPU.
int compute_units() {
  int dev = 0, n = 0;
  if (hipGetDevice(&dev) != hipSuccess || hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess ||
      n < 1) {
    (void)hipGetLastError();
    return 256;
  }
  return n;
}

// Estimated duration, in k-tiles of mainloop per CU, of `count_a` tiles of length `len_a` followed by `count_b` tiles of
// length `len_b` handed to `ncu` CUs in order, each CU taking the next tile when it is free (what the dispatcher does with
// one workgroup per CU).  Closed form: the first kind fills whole rounds plus one partial round; the second kind then
// runs back to back on CUs that became free at one of two times, so the end is the smallest time by which those CUs can
// have completed count_b tiles.
int64_t list_schedule(int64_t count_a, int64_t len_a, int64_t count_b, int64_t len_b, int64_t ncu) {
  const int64_t rounds = count_a / ncu, late = count_a % ncu, early = ncu - late;
  const int64_t t_early = rounds * len_a, t_late = late ? (rounds + 1) * len_a : t_early;
  if (count_b == 0) return t_late;
  auto done_by = [&](int64_t t) {
    return early * (t > t_early ? (t - t_early) / len_b : 0) + late * (t > t_late ? (t - t_late) / len_b : 0);
  };
  // the end is t_early + m * len_b or t_late + m * len_b for some m >= 1: take the smallest that suffices
  int64_t best = -1;
  for (const int64_t t0 : {t_early, t_late}) {
    int64_t lo = 1, hi = count_b;  // m = count_b always suffices (one CU alone)
    while (lo < hi) {
      const int64_t mid = (lo + hi) / 2;
      if (done_by(t0 + mid * len_b) >= count_b) hi = mid; else lo = mid + 1;
    }
    const int64_t t = t0 + lo * len_b;
    if (best < 0 || t < best) best = t;
  }
  return best > t_late ? best : t_late;
}

// Width of the dz panel in vocab columns when the caller does not choose one.  Wider chunks mean fewer launches (every
// launch ends with CUs idling for part of a tile), fewer read-modify-write passes over the dHidden partial sums and a
// larger panel; what matters most is whether the tiles of a launch divide evenly over the CUs.  The candidates
// (multiples of 2048 columns whose panel holds at most 1.5 GiB of dz values) are rated with a small model of the two launches per
// chunk -- dz tiles of H/64 k-tiles plus an epilogue, then dHidden tiles of chunk/64 and dW tiles of T'/64 k-tiles,
// list-scheduled over the CUs, plus a fixed cost per launch -- and the cheapest wins.  At the 7B shape (T = 16384, H = 3584)
// that is 49152 columns: 4096 x 3 dz tiles and 896 + 2688 GEMM tiles per launch, both multiples of 256 CUs.
int64_t default_vocab_chunk(int64_t T, int64_t H, int64_t V) {
  const int64_t Tpad = round_up(T, 256), Vpad = round_up(V, 256), Hpad = round_up(H, 256);
  const int ncu = compute_units();
  const int64_t tiles_t = Tpad / 256, tiles_h = Hpad / 256;
  const int64_t kDzEpilogue = 8, kGemmEpilogue = 6, kLaunch = 24;  // in k-tiles (about 1.3 us each)
  const int64_t kMaxPanelBytes = (int64_t)3 << 29;  // of dz values, before the row padding
  int64_t best_vc = 0, best_cost = 0;
  for (int64_t vc = 2048;; vc += 2048) {
    if (vc > Vpad) vc = Vpad;
    const bool fits = Tpad * vc * 2 <= kMaxPanelBytes;
    if (fits || best_vc == 0) {
      auto chunk_cost = [&](int64_t w) {  // the two launches of a chunk of w columns
        return list_schedule(w / 256 * tiles_t, H / BK + kDzEpilogue, 0, 0, ncu) + kLaunch +
               list_schedule(tiles_h * tiles_t, w / BK + kGemmEpilogue, tiles_h * (w / 256), Tpad / BK + kGemmEpilogue, ncu) + kLaunch;
      };
      const int64_t full = Vpad / vc, rest = Vpad % vc;  // all chunks but the last have the same width
      const int64_t cost = full * chunk_cost(vc) + (rest ? chunk_cost(rest) : 0);
      if (best_vc == 0 || cost < best_cost) best_vc = vc, best_cost = cost;
    }
    if (vc >= Vpad || !fits) break;
  }
  return best_vc;
}

// Forward scratch: three arrays of per-part statistics for `tokens` tokens.
size_t fwd_partials_bytes(int64_t tokens, int64_t V) {
  const size_t nparts = (size_t)((V + BM - 1) / BM) * WAVES_M;
  Carver c(nullptr);
  c.take<float>(part_elems(nparts, tokens));
  c.take<float>(part_elems(nparts, tokens));
  c.take<float>(part_elems(nparts, tokens));
  return (size_t)round_up((int64_t)c.off, 256);
}

// The forward walks the tokens in blocks: tokens are independent, so a block is a complete forward problem on a slice of
// hidden / labels / outputs, and the partials of one block are merged before the next block overwrites them (launches on
// one stream run in order).  The scratch is therefore sized by the block, not by T.  Block boundaries are multiples of the
// 256-token tile, so every token sees the same tiles, in the same order, as in an unblocked run: results are bit-identical
// for any block size.
constexpr int64_t kFwdTokenBlock = 32768;

// Tokens per block: what the caller's scratch allows, at least one 256-token tile.
int64_t fwd_block_tokens(int64_t wanted, int64_t ld_hidden) {
  (void)ld_hidden;
  return wanted < BN ? BN : wanted;
}

int fwd_token_blocks(const void* hidden, int64_t ld_hidden, const void* weight, int64_t ld_weight, const int64_t* labels,
                     int64_t T, int64_t H, int64_t V, float rcp_temperature, float* logprobs, float* entropy, float* row_lse,
                     float* row_pz, void* scratch, int64_t block_tokens, hipStream_t s) {
  const int tiles_m = (int)((V + BM - 1) / BM);
  const size_t nparts = (size_t)tiles_m * WAVES_M;
  const bool want_pz = entropy || row_pz;
  const uint16_t* Wp = (const uint16_t*)weight;
  for (int64_t t0 = 0; t0 < T; t0 += block_tokens) {
    const int64_t Tb = (T - t0) < block_tokens ? (T - t0) : block_tokens;
    const int tiles_n = (int)((Tb + BN - 1) / BN);
    Carver c(scratch);
    float* pmax = c.take<float>(part_elems(nparts, Tb));
    float* psum = c.take<float>(part_elems(nparts, Tb));
    float* ppz = c.take<float>(part_elems(nparts, Tb));
    const uint16_t* Hp = (const uint16_t*)hidden + (size_t)t0 * (size_t)ld_hidden;
    const dim3 grid((unsigned)(tiles_m * tiles_n)), block(NTHREADS);
    {
      Timed timed(kFwdTiles, s);
      auto kernel = want_pz ? (even_ktiles(H) ? lmhead_fwd_tiles<true, true> : lmhead_fwd_tiles<true, false>)
                            : (even_ktiles(H) ? lmhead_fwd_tiles<false, true> : lmhead_fwd_tiles<false, false>);
      hipLaunchKernelGGL(kernel, grid, block, 0, s, Wp, (int)ld_weight, Hp, (int)ld_hidden, (int)Tb, (int)H, (int)V,
                         rcp_temperature, pmax, psum, ppz);
    }
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) return (int)e;
    Timed timed(kFwdMerge, s);
    hipLaunchKernelGGL(lmhead_fwd_merge<true>, dim3((unsigned)((Tb + kMergeTokens - 1) / kMergeTokens)), dim3(kMergeThreads), 0, s, pmax,
                       psum, want_pz ? ppz : (float*)nullptr, (int)nparts, (int)Tb, Hp, (int)ld_hidden, Wp, (int)ld_weight,
                       labels + t0, (int)H, (int)V, rcp_temperature, logprobs + t0, entropy ? entropy + t0 : (float*)nullptr,
                       row_lse ? row_lse + t0 : (float*)nullptr, row_pz ? row_pz + t0 : (float*)nullptr);
    if ((e = hipGetLastError()) != hipSuccess) return (int)e;
  }
  return SKYRL_LMHEAD_OK;
}

// Address of this device's copy of the static scratch array.  Every device holds its own copy of a __device__ array at
// its own address, so the address is looked up once per device, with that device current, and kept.
constexpr int kMaxDevices = 64;
void* g_static_scratch_ptr[kMaxDevices];
std::mutex g_static_scratch_mutex;

int static_scratch_of_current_device(void** out) {
  int dev = -1;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess) return (int)e;
  if (dev < 0 || dev >= kMaxDevices) return SKYRL_LMHEAD_ERR_ARG;
  std::lock_guard<std::mutex> lock(g_static_scratch_mutex);
  if (!g_static_scratch_ptr[dev]) {
    void* p = nullptr;
    e = hipGetSymbolAddress(&p, HIP_SYMBOL(static_scratch));
    if (e != hipSuccess) return (int)e;
    if (!p || ((uintptr_t)p & 255u)) return SKYRL_LMHEAD_ERR_ALIGN;
    g_static_scratch_ptr[dev] = p;
  }
  *out = g_static_scratch_ptr[dev];
  return SKYRL_LMHEAD_OK;
}

// The backward, like the forward, walks the tokens in blocks: dHidden rows are complete within their block, dW is summed
// over the blocks (the first block stores or adds as the caller's dw_mode says, the later ones add), and every scratch
// matrix is sized by the block.  One block for T <= 32768, which covers every shape whose step time is quoted anywhere.
constexpr int64_t kBwdTokenBlock = 32768;

struct BwdWorkspace {
  uint16_t *Wt, *Ht, *D;
  float *dHacc, *dWsum, *label_resid;
  // only with row compaction (skyrl_lmhead_bwd_active_rows):
  uint16_t *hidden_c, *d_hidden_c;
  int64_t* labels_c;
  float *lse_c, *pz_c, *g_c, *q_c;
  int *idx, *counts;
  size_t bytes;
};

// The dHidden GEMM contracts over the vocabulary.  When V is a multiple of two k-tiles (the gradient GEMMs run whole pairs
// of k-tiles) it reads the weight rows where they are (K-major B operand); otherwise the last pair would reach past the
// weight's last row, and a transposed copy, zero-padded to whole tiles, is made in the workspace instead.
inline bool reads_weight_in_place(int64_t V) { return V % (2 * BK) == 0; }

inline int64_t bwd_block_tokens(int64_t T) { return T < kBwdTokenBlock ? T : kBwdTokenBlock; }
inline int64_t bwd_num_blocks(int64_t T) { return (T + kBwdTokenBlock - 1) / kBwdTokenBlock; }

// vc: chunk width for a block of bwd_block_tokens(T) tokens.  compact: the buffers of the row-compacting entry point.
// Hk: length of the logits contraction, a multiple of H when the operands are stacked bf16 terms of fp32 values.
BwdWorkspace carve_bwd(void* ws, int64_t T, int64_t H, int64_t Hk, int64_t V, int64_t vc, bool compact) {
  const int64_t Tb = bwd_block_tokens(T), Tpad = round_up(Tb, 256), Vpad = round_up(V, 256);
  Carver c(ws);
  BwdWorkspace w{};
  w.Wt = reads_weight_in_place(V) ? nullptr : c.take<uint16_t>((size_t)H * (Vpad + kLdPad));
  w.Ht = c.take<uint16_t>((size_t)H * (Tpad + kLdPad));
  w.dHacc = c.take<float>((size_t)Tpad * round_up(H, 256));  // accumulator order, whole tiles
  w.D = c.take<uint16_t>((size_t)Tpad * (vc + kLdPad));
  // Several blocks and a bf16 dW: the sum over the blocks is kept in fp32 here and rounded once, by the last block.
  w.dWsum = bwd_num_blocks(T) > 1 ? c.take<float>((size_t)V * (size_t)H) : nullptr;
  w.label_resid = Hk > H ? c.take<float>((size_t)Tpad) : nullptr;  // stacked terms: fp32 operands
  if (compact) {
    w.hidden_c = c.take<uint16_t>((size_t)T * (size_t)Hk);
    w.d_hidden_c = c.take<uint16_t>((size_t)T * (size_t)H);
    w.labels_c = c.take<int64_t>((size_t)T);
    w.lse_c = c.take<float>((size_t)T);
    w.pz_c = c.take<float>((size_t)T);
    w.g_c = c.take<float>((size_t)T);
    w.q_c = c.take<float>((size_t)T);
    w.idx = c.take<int>((size_t)T);
    w.counts = c.take<int>((size_t)bwd_num_blocks(T) + 1);
  }
  w.bytes = (size_t)round_up((int64_t)c.off, 256);
  return w;
}

GemmArgs make_gemm(const uint16_t* A, int64_t lda, int64_t a_rows, const uint16_t* B, int64_t ldb, int64_t b_rows, bool b_kmajor,
                   bool c_rows_m, int64_t nk, int64_t M, int64_t N, const float* Cin, float* Cf, uint16_t* Cb, int64_t ldc,
                   const float* Pin = nullptr, float* Pout = nullptr, const int* T_dev = nullptr, int t_role = 0) {
  return GemmArgs{A,       (int)lda, (int)a_rows, B,  (int)ldb, (int)b_rows, b_kmajor ? 1 : 0, c_rows_m ? 1 : 0, (int)nk,
                  (int)M,  (int)N,   Cin,         Cf, Cb,       (int)ldc,    Pin,              Pout, T_dev, t_role};
}

unsigned gemm_tiles(const GemmArgs& g) { return (unsigned)(((g.M + BM - 1) / BM) * ((g.N + BN - 1) / BN)); }

hipError_t launch_bwd_dz(hipStream_t s, bool entgrad, const DzArgs& z, unsigned dz_tiles) {
  Timed timed(kBwdChunkDz, s);
  const bool even = even_ktiles(z.H);
  const dim3 grid(dz_tiles), block(NTHREADS);
  if (entgrad) {
    if (even) hipLaunchKernelGGL((lmhead_bwd_dz<true, true>), grid, block, 0, s, z);
    else hipLaunchKernelGGL((lmhead_bwd_dz<true, false>), grid, block, 0, s, z);
  } else {
    if (even) hipLaunchKernelGGL((lmhead_bwd_dz<false, true>), grid, block, 0, s, z);
    else hipLaunchKernelGGL((lmhead_bwd_dz<false, false>), grid, block, 0, s, z);
  }
  return hipGetLastError();
}

// Both problems (p1 may be empty) must have an even number of k-tiles: every caller contracts over padded extents that
// are multiples of 256, or over vocabulary rows that reads_weight_in_place() admits.
hipError_t launch_bwd_gemm(hipStream_t s, const GemmArgs& p0, const GemmArgs& p1) {
  if ((p0.nk & 1) || (p1.nk & 1)) return hipErrorInvalidValue;
  const unsigned t0 = gemm_tiles(p0), t1 = gemm_tiles(p1);
  Timed timed(kBwdChunkGemm, s);
  hipLaunchKernelGGL(lmhead_bwd_gemm, dim3(t0 + t1), dim3(NTHREADS), 0, s, p0, p1, (int)t0);
  return hipGetLastError();
}

// Workspaces of the soft cross-entropy: the stacked hidden rows first in both.
constexpr int64_t kPairTile = BN / 2;  // tokens per workgroup tile of stacked rows

struct SoftCeFwdWorkspace {
  uint16_t* S;
  float *pmax, *psum, *ppz, *row_lse, *row_pz;
  size_t nparts, bytes;
};

SoftCeFwdWorkspace carve_softce_fwd(void* ws, int64_t T, int64_t H, int64_t V) {
  const int64_t Tp = round_up(T, kPairTile);
  Carver c(ws);
  SoftCeFwdWorkspace w;
  w.nparts = (size_t)((V + BM - 1) / BM) * WAVES_M;
  w.S = c.take<uint16_t>((size_t)(2 * Tp) * (size_t)H);
  w.pmax = c.take<float>(part_elems(w.nparts, 2 * Tp));
  w.psum = c.take<float>(part_elems(w.nparts, 2 * Tp));
  w.ppz = c.take<float>(part_elems(w.nparts, 2 * Tp));
  w.row_lse = c.take<float>((size_t)(2 * Tp));
  w.row_pz = c.take<float>((size_t)(2 * Tp));
  w.bytes = (size_t)round_up((int64_t)c.off, 256);
  return w;
}

struct SoftCeBwdWorkspace {
  uint16_t *S, *Wt, *D;
  float* dHacc;
  size_t bytes;
};

SoftCeBwdWorkspace carve_softce_bwd(void* ws, int64_t T, int64_t H, int64_t V, int64_t vc) {
  const int64_t Tp = round_up(T, kPairTile), Vpad = round_up(V, 256);
  Carver c(ws);
  SoftCeBwdWorkspace w;
  w.S = c.take<uint16_t>((size_t)(2 * Tp) * (size_t)H);
  w.Wt = reads_weight_in_place(V) ? nullptr : c.take<uint16_t>((size_t)H * (Vpad + kLdPad));
  w.dHacc = c.take<float>((size_t)round_up(T, 256) * round_up(H, 256));
  w.D = c.take<uint16_t>((size_t)Tp * (vc + kLdPad));
  w.bytes = (size_t)round_up((int64_t)c.off, 256);
  return w;
}

int check_softce(const void* student, int64_t lds_, const void* teacher, int64_t ldt, const void* weight, int64_t ldw, int64_t T,
                 int64_t seq_len, int64_t shift, int64_t H, int64_t V, float rcp_temperature) {
  if (!teacher) return SKYRL_LMHEAD_ERR_NULL;
  int st = check_operands(student, lds_, weight, ldw, T, H, V, rcp_temperature);
  if (st) return st;
  if (ldt < H || ldt > kMaxRowPitch) return SKYRL_LMHEAD_ERR_SHAPE;
  if (seq_len < 1 || T % seq_len != 0 || shift < 0) return SKYRL_LMHEAD_ERR_SHAPE;
  if (!aligned16(teacher) || ldt % 8 != 0) return SKYRL_LMHEAD_ERR_ALIGN;
  return SKYRL_LMHEAD_OK;
}

hipError_t launch_softce_pack(hipStream_t s, const void* student, int64_t lds_, const void* teacher, int64_t ldt, int64_t T,
                              int64_t seq_len, int64_t shift, int64_t H, uint16_t* S) {
  Timed timed(kSoftCePack, s);
  hipLaunchKernelGGL(softce_pack_rows, dim3((unsigned)(2 * round_up(T, kPairTile))), dim3(256), 0, s, (const uint16_t*)student,
                     (int)lds_, (const uint16_t*)teacher, (int)ldt, (int)T, (int)seq_len, (int)(shift % seq_len), (int)H, S);
  return hipGetLastError();
}


// Top-k logits from hidden states.  Tokens are walked in blocks of at most 16384 and the vocabulary in chunks of 1024, 2048,
// 4096 and then 8192 columns: the first chunk passes every logit (no threshold yet), and from then on a logit passes with
// probability k / (columns seen so far) on exchangeable columns, so that short early chunks keep the candidate lists short.
// A candidate list holds a whole chunk (cap columns per token), which makes the filter exact for any data: in the worst
// case -- logits ascending with the column -- every logit is a candidate and the select kernel does all the work.
constexpr int64_t kTopkTokenBlock = 16384;
constexpr int64_t kTopkFirstChunk = 1024, kTopkMaxChunk = 8192;

struct TopkWorkspace {
  unsigned *cnt, *have;
  float* thr;
  topk::key_t *best, *cand;
  int64_t block_tokens, cap;
  size_t bytes;
};

TopkWorkspace carve_topk(void* ws, int64_t T, int64_t V, int64_t k) {
  TopkWorkspace w;
  w.block_tokens = T < kTopkTokenBlock ? T : kTopkTokenBlock;
  const int64_t vpad = round_up(V, 256);
  w.cap = vpad < kTopkMaxChunk ? vpad : kTopkMaxChunk;
  Carver c(ws);
  w.cnt = c.take<unsigned>((size_t)w.block_tokens);
  w.have = c.take<unsigned>((size_t)w.block_tokens);
  w.thr = c.take<float>((size_t)w.block_tokens);
  w.best = c.take<topk::key_t>((size_t)w.block_tokens * (size_t)k);
  w.cand = c.take<topk::key_t>((size_t)w.block_tokens * (size_t)w.cap);
  w.bytes = (size_t)round_up((int64_t)c.off, 256);
  return w;
}

size_t bwd_workspace_bytes(int64_t T, int64_t H, int64_t V, int64_t vocab_chunk, bool compact, int64_t terms = 1) {
  if (T < 1 || V < 1 || H < 1 || vocab_chunk < 0 || vocab_chunk % 256 != 0 || terms < 1 || terms > 3) return 0;
  if (T > kMaxExtent || V > kMaxExtent || H > kMaxExtent / 4 || vocab_chunk > kMaxExtent) return 0;
  int64_t vc = vocab_chunk ? vocab_chunk : default_vocab_chunk(bwd_block_tokens(T), H, V);
  if (vc > round_up(V, 256)) vc = round_up(V, 256);
  return carve_bwd(nullptr, T, H, terms * H, V, vc, compact).bytes;
}

// One token block of the backward: the vocab-chunk loop.  Hk is the contraction length of the logits recompute (H, or a
// multiple of it for stacked bf16 terms, in which case the two gradient GEMMs use the leading H columns: the hi terms).  `Tb` tokens (an upper bound when `T_dev` points at the block's
// count in device memory), per-token inputs and d_hidden already offset to the block.  dW of every chunk leaves the GEMM
// epilogue as  (Cin ? Cin : 0) + product  ->  Cf (fp32) and / or Cb (bf16), each a [V, H] matrix or NULL.
int bwd_token_block(const uint16_t* Hp, int64_t ld_hidden, const uint16_t* Wp, int64_t ld_weight, const int64_t* labels,
                    const float* row_lse, const float* row_pz, const float* dlogprobs, const float* dentropy, int64_t Tb,
                    const int* T_dev, int64_t H, int64_t Hk, int64_t V, float rcp_temperature, uint16_t* d_hidden, bool want_dw,
                    const float* dw_in, float* dw_f32, uint16_t* dw_bf16, int64_t vc, const BwdWorkspace& w, float p_shift,
                    hipStream_t s) {
  const int64_t Tpad = round_up(Tb, 256), Vpad = round_up(V, 256);
  const bool w_in_place = reads_weight_in_place(V);
  hipError_t e;
  if (want_dw) {  // only the dW product reads hidden^T [H, Tpad]; zero in the padding columns
    Timed timed(kTranspose, s);
    hipLaunchKernelGGL(transpose_bf16, dim3((unsigned)(Tpad / 64), (unsigned)(H / 64)), dim3(256), 0, s, Hp, (int)ld_hidden,
                       (int)Tb, (int)H, w.Ht, (int)(Tpad + kLdPad), (int)Tpad, T_dev);
    if ((e = hipGetLastError()) != hipSuccess) return (int)e;
  }
  // fp32 operands (stacked terms) with an fp32 dW: the label's dz value keeps fp32 accuracy through a residual (DzArgs).
  float* resid = (Hk > H && want_dw && dw_f32) ? w.label_resid : nullptr;
  if (resid) {
    hipLaunchKernelGGL(zero_f32, dim3((unsigned)(Tpad / 256)), dim3(256), 0, s, resid, (int)Tpad);
    if ((e = hipGetLastError()) != hipSuccess) return (int)e;
  }
  const int tiles_t = (int)(Tpad / 256);
  const int64_t nchunks = (Vpad + vc - 1) / vc;
  auto chunk_width = [&](int64_t ci) { return (Vpad - ci * vc) < vc ? (Vpad - ci * vc) : vc; };  // multiple of 256
  const GemmArgs none{};
  for (int64_t ci = 0; ci < nchunks; ++ci) {
    // dz panel of this chunk, then the two gradient GEMMs that consume it (one launch, they are independent).
    // Carrying the next chunk's dz tiles in the GEMM launch (to fill its tail) was measured: no gain at the default chunk
    // width, and it needs a second panel.
    const int64_t vc0 = ci * vc, vcw = chunk_width(ci);
    const DzArgs z{Wp, (int)ld_weight, Hp, (int)ld_hidden, (int)Tb, (int)Hk, (int)V, rcp_temperature, labels, row_lse, row_pz,
                   dlogprobs, dentropy, (int)vc0, (int)(vcw / 256), tiles_t, w.D, (int)(vcw + kLdPad), T_dev, resid, p_shift};
    e = launch_bwd_dz(s, dentropy != nullptr, z, (unsigned)(vcw / 256 * tiles_t));
    if (e != hipSuccess) return (int)e;
    // dHidden[t, h] (+)= sum_v D[t, v] . weight^T[h, vc0 + v]        (A = weight^T rows at k offset vc0, B = D rows)
    // dW[vc0 + v, h]  (+)= sum_t D[t, v] . hidden^T[h, t]             (A = hidden^T rows, B = D read K-major)
    const bool first = ci == 0, last = ci == nchunks - 1;
    const int64_t rows = (V - vc0) < vcw ? (V - vc0) : vcw;
    // dW rows are complete within their chunk (for this token block), so they can leave the GEMM epilogue in either precision.
    const size_t dw_off = (size_t)vc0 * (size_t)H;
    uint16_t* dh_out = last ? d_hidden : (uint16_t*)nullptr;
    const float* dh_in = first ? (const float*)nullptr : (const float*)w.dHacc;
    float* dh_keep = last ? (float*)nullptr : w.dHacc;
    // In place: C[t, h] with A = D rows (K = vocab, contiguous), B = weight rows vc0.. read K-major; the k extent stops at V.
    // Otherwise: C[h, t] with A = weight^T rows, B = D rows.  The partial sums are in accumulator order either way.
    const int64_t kext = (V - vc0) < vcw ? (V - vc0) : vcw;
    const GemmArgs gh =
        w_in_place ? make_gemm(w.D, vcw + kLdPad, Tpad, Wp + (size_t)vc0 * (size_t)ld_weight, ld_weight, H, true, true, kext / BK, Tb,
                               H, nullptr, nullptr, dh_out, H, dh_in, dh_keep, T_dev, kTokensOnM)
                   : make_gemm(w.Wt + vc0, Vpad + kLdPad, H, w.D, vcw + kLdPad, Tpad, false, false, vcw / BK, H, Tb, nullptr,
                               nullptr, dh_out, H, dh_in, dh_keep, T_dev, kTokensOnN);
    // A frozen LM head needs no dW: the launch then carries the dHidden tiles alone.
    const GemmArgs gw = want_dw ? make_gemm(w.Ht, Tpad + kLdPad, H, w.D, vcw + kLdPad, vcw, true, false, Tpad / BK, H, rows,
                                            dw_in ? dw_in + dw_off : (const float*)nullptr,
                                            dw_f32 ? dw_f32 + dw_off : (float*)nullptr,
                                            dw_bf16 ? dw_bf16 + dw_off : (uint16_t*)nullptr, H, nullptr, nullptr, T_dev,
                                            kTokensOnK)
                                : none;
    e = launch_bwd_gemm(s, gh, gw);
    if (e != hipSuccess) return (int)e;
  }
  if (resid) {
    hipLaunchKernelGGL(label_residual_update, dim3((unsigned)Tb), dim3(256), 0, s, (const float*)resid, labels, Hp, (int)ld_hidden,
                       (int)H, Hk == 3 * H ? (int)(2 * H) : 0, (int)V, T_dev, dw_f32);
    if ((e = hipGetLastError()) != hipSuccess) return (int)e;
  }
  return SKYRL_LMHEAD_OK;
}

int bwd_entry(const void* hidden, int64_t ld_hidden, const void* weight, int64_t ld_weight, const int64_t* labels,
              const float* row_lse, const float* row_pz, const float* dlogprobs, const float* dentropy, int64_t T, int64_t H,
              int64_t V, float rcp_temperature, void* d_hidden, void* d_weight, int dw_mode, int64_t vocab_chunk,
              void* workspace, size_t workspace_bytes, hipStream_t s, bool compact, int64_t terms = 1) {
  if (terms < 1 || terms > 3 || H < 1 || H > kMaxExtent / 4) return SKYRL_LMHEAD_ERR_ARG;
  // dw_mode carries one option bit next to the mode: softmax probabilities below 2^-24 count as zero in dz.
  const float p_shift = (dw_mode & SKYRL_BWD_FLUSH_TINY_DZ) ? 126.f - 24.f : 0.f;
  if (dw_mode >= 0) dw_mode &= ~SKYRL_BWD_FLUSH_TINY_DZ;
  const int64_t Hk = terms * H;
  int st = check_common(hidden, ld_hidden, weight, ld_weight, labels, T, Hk, V, rcp_temperature, true);
  if (st) return st;
  if (H % BK != 0) return SKYRL_LMHEAD_ERR_SHAPE;
  if (!row_lse || !dlogprobs || !d_hidden) return SKYRL_LMHEAD_ERR_NULL;
  if (dentropy && !row_pz) return SKYRL_LMHEAD_ERR_NULL;
  if (!aligned16(d_hidden) || !aligned16(d_weight)) return SKYRL_LMHEAD_ERR_ALIGN;  // d_weight NULL: no dW wanted
  if (dw_mode < SKYRL_DW_FP32 || dw_mode > SKYRL_DW_BF16) return SKYRL_LMHEAD_ERR_ARG;
  if (vocab_chunk < 0 || vocab_chunk % 256 != 0) return SKYRL_LMHEAD_ERR_ARG;
  if (compact && T >= ((int64_t)1 << 31)) return SKYRL_LMHEAD_ERR_SHAPE;  // the row index list is 32-bit
  const int64_t Tb = bwd_block_tokens(T), Tbpad = round_up(Tb, 256), Vpad = round_up(V, 256);
  int64_t vc = vocab_chunk ? vocab_chunk : default_vocab_chunk(Tb, H, V);
  if (vc > Vpad) vc = Vpad;
  // Row pitches of the scratch matrices (weight^T, hidden^T, the dz panel) under the copy plan's limit; Hk <= ld_hidden is.
  if ((!reads_weight_in_place(V) && Vpad + kLdPad > kMaxRowPitch) || Tbpad + kLdPad > kMaxRowPitch || vc + kLdPad > kMaxRowPitch)
    return SKYRL_LMHEAD_ERR_SHAPE;
  if (!workspace || workspace_bytes < bwd_workspace_bytes(T, H, V, vc, compact, terms)) return SKYRL_LMHEAD_ERR_WORKSPACE;
  if ((uintptr_t)workspace & 255u) return SKYRL_LMHEAD_ERR_ALIGN;

  const BwdWorkspace w = carve_bwd(workspace, T, H, Hk, V, vc, compact);
  const uint16_t* Wp = (const uint16_t*)weight;
  const uint16_t* Hp = (const uint16_t*)hidden;
  const int64_t nblocks = bwd_num_blocks(T);
  hipError_t e;

  if (compact) {
    Timed timed(kCompactRows, s);
    hipLaunchKernelGGL(compact_active_rows, dim3(1), dim3(kCompactThreads), 0, s, dlogprobs, dentropy, (int)T, (int)Tb,
                       (int)nblocks, w.idx, w.counts);
    hipLaunchKernelGGL(gather_active_rows, dim3((unsigned)T), dim3(256), 0, s, (const int*)w.idx, (const int*)w.counts, Hp,
                       (int)ld_hidden, (int)Hk, (int)H, labels, row_lse, row_pz, dlogprobs, dentropy, w.hidden_c, w.labels_c,
                       w.lse_c, w.pz_c, w.g_c, w.q_c, (uint16_t*)d_hidden);
    if ((e = hipGetLastError()) != hipSuccess) return (int)e;
  }
  if (!reads_weight_in_place(V)) {  // weight^T [H, Vpad], zero in the padding columns
    Timed timed(kTranspose, s);
    hipLaunchKernelGGL(transpose_bf16, dim3((unsigned)(Vpad / 64), (unsigned)(H / 64)), dim3(256), 0, s, Wp, (int)ld_weight,
                       (int)V, (int)H, w.Wt, (int)(Vpad + kLdPad), (int)Vpad, (const int*)nullptr);
    if ((e = hipGetLastError()) != hipSuccess) return (int)e;
  }

  for (int64_t b = 0; b < nblocks; ++b) {
    const int64_t t0 = b * Tb, Tcur = (T - t0) < Tb ? (T - t0) : Tb;
    // Where dW of this block comes from and goes to.  One block: straight to the caller's matrix as dw_mode says.  Several
    // blocks: fp32 modes add every later block to the caller's matrix; the bf16 mode sums in the fp32 scratch matrix and
    // the last block rounds the sum into the caller's.
    const float* dw_in = nullptr;
    float* dw_f32 = nullptr;
    uint16_t* dw_bf16 = nullptr;
    if (d_weight) {
      const bool first = b == 0, last = b == nblocks - 1;
      if (dw_mode == SKYRL_DW_BF16) {
        if (nblocks == 1) {
          dw_bf16 = (uint16_t*)d_weight;
        } else {
          dw_in = first ? nullptr : w.dWsum;
          if (last) dw_bf16 = (uint16_t*)d_weight; else dw_f32 = w.dWsum;
        }
      } else {
        dw_f32 = (float*)d_weight;
        dw_in = (dw_mode == SKYRL_DW_FP32_ACCUMULATE || !first) ? (const float*)d_weight : nullptr;
      }
    }
    if (compact) {
      st = bwd_token_block(w.hidden_c + (size_t)t0 * (size_t)Hk, Hk, Wp, ld_weight, w.labels_c + t0, w.lse_c + t0,
                           dentropy ? w.pz_c + t0 : nullptr, w.g_c + t0, dentropy ? w.q_c + t0 : nullptr, Tcur,
                           w.counts + 1 + b, H, Hk, V, rcp_temperature, w.d_hidden_c + (size_t)t0 * (size_t)H, d_weight != nullptr,
                           dw_in, dw_f32, dw_bf16, vc, w, p_shift, s);
    } else {
      st = bwd_token_block(Hp + (size_t)t0 * (size_t)ld_hidden, ld_hidden, Wp, ld_weight, labels + t0, row_lse + t0,
                           row_pz ? row_pz + t0 : nullptr, dlogprobs + t0, dentropy ? dentropy + t0 : nullptr, Tcur, nullptr, H,
                           Hk, V, rcp_temperature, (uint16_t*)d_hidden + (size_t)t0 * (size_t)H, d_weight != nullptr, dw_in, dw_f32,
                           dw_bf16, vc, w, p_shift, s);
    }
    if (st) return st;
  }
  if (compact) {
    Timed timed(kCompactRows, s);
    hipLaunchKernelGGL(scatter_active_rows, dim3((unsigned)T), dim3(256), 0, s, (const int*)w.idx, (const int*)w.counts,
                       (const uint16_t*)w.d_hidden_c, (int)H, (uint16_t*)d_hidden);
    if ((e = hipGetLastError()) != hipSuccess) return (int)e;
  }
  return SKYRL_LMHEAD_OK;
}

}  // namespace

extern "C" {

int skyrl_lmhead_version(void) { return 20; }

const char* skyrl_lmhead_strerror(int status) {
  switch (status) {
    case SKYRL_LMHEAD_OK: return "ok";
    case SKYRL_LMHEAD_ERR_NULL: return "a required pointer is NULL (or only some of seg_row, seg_col, seg_len are given)";
    case SKYRL_LMHEAD_ERR_SHAPE:
      return "bad shape: need T >= 1, V >= 1, H a positive multiple of 64, leading dimensions >= H and at most 4194304 elements; "
             "packed-sequence calls: counts >= 0, rows == num_seqs with an attention mask";
    case SKYRL_LMHEAD_ERR_ALIGN: return "bad alignment: pointers must be 16-byte aligned, leading dimensions multiples of 8";
    case SKYRL_LMHEAD_ERR_WORKSPACE: return "workspace is NULL or too small";
    case SKYRL_LMHEAD_ERR_TOO_LARGE:
      return "too large for the entry point that uses the library's fixed scratch array: V exceeds "
             "SKYRL_LMHEAD_STATIC_SCRATCH_MAX_V; use skyrl_lmhead_fwd with a caller-provided workspace";
    case SKYRL_LMHEAD_ERR_ARG:
      return "bad argument: rcp_temperature must be finite and > 0, vocab_chunk a multiple of 256; packed-sequence calls take "
             "sub-sequence arrays or an attention mask, not both";
    default: break;
  }
  if (status > 0) return hipGetErrorString((hipError_t)status);
  return "unknown skyrl_lmhead status";
}

size_t skyrl_lmhead_fwd_workspace_bytes(int64_t T, int64_t H, int64_t V) {
  (void)H;
  if (T < 1 || V < 1 || T > kMaxExtent || V > kMaxExtent) return 0;
  return fwd_partials_bytes(T < kFwdTokenBlock ? T : kFwdTokenBlock, V);
}

size_t skyrl_lmhead_bwd_workspace_bytes(int64_t T, int64_t H, int64_t V, int64_t vocab_chunk) {
  return bwd_workspace_bytes(T, H, V, vocab_chunk, false);
}

size_t skyrl_lmhead_bwd_active_rows_workspace_bytes(int64_t T, int64_t H, int64_t V, int64_t vocab_chunk) {
  return bwd_workspace_bytes(T, H, V, vocab_chunk, true);
}

int skyrl_lmhead_fwd(const void* hidden, int64_t ld_hidden, const void* weight, int64_t ld_weight, const int64_t* labels,
                     int64_t T, int64_t H, int64_t V, float rcp_temperature, float* logprobs, float* entropy,
                     float* row_lse, float* row_pz, void* workspace, size_t workspace_bytes, void* stream) {
  int st = check_common(hidden, ld_hidden, weight, ld_weight, labels, T, H, V, rcp_temperature, true);
  if (st) return st;
  if (!logprobs) return SKYRL_LMHEAD_ERR_NULL;
  if (!workspace || workspace_bytes < skyrl_lmhead_fwd_workspace_bytes(T, H, V)) return SKYRL_LMHEAD_ERR_WORKSPACE;
  if ((uintptr_t)workspace & 255u) return SKYRL_LMHEAD_ERR_ALIGN;
  return fwd_token_blocks(hidden, ld_hidden, weight, ld_weight, labels, T, H, V, rcp_temperature, logprobs, entropy, row_lse,
                          row_pz, workspace, fwd_block_tokens(kFwdTokenBlock, ld_hidden), (hipStream_t)stream);
}

int skyrl_lmhead_fwd_static_scratch(const void* hidden, int64_t ld_hidden, const void* weight, int64_t ld_weight,
                                    const int64_t* labels, int64_t T, int64_t H, int64_t V, float rcp_temperature,
                                    float* logprobs, float* entropy, float* row_lse, float* row_pz, void* stream) {
  int st = check_common(hidden, ld_hidden, weight, ld_weight, labels, T, H, V, rcp_temperature, true);
  if (st) return st;
  if (!logprobs) return SKYRL_LMHEAD_ERR_NULL;
  // Token block: the most 256-token tiles whose partials fit the static array.
  const int64_t block = (int64_t)(kStaticScratchBytes / fwd_partials_bytes(BN, V)) * BN;
  if (V > SKYRL_LMHEAD_STATIC_SCRATCH_MAX_V || block < BN) return SKYRL_LMHEAD_ERR_TOO_LARGE;
  void* scratch_ptr = nullptr;
  if ((st = static_scratch_of_current_device(&scratch_ptr)) != SKYRL_LMHEAD_OK) return st;
  return fwd_token_blocks(hidden, ld_hidden, weight, ld_weight, labels, T, H, V, rcp_temperature, logprobs, entropy, row_lse,
                          row_pz, scratch_ptr, fwd_block_tokens(block, ld_hidden), (hipStream_t)stream);
}

size_t skyrl_lmhead_static_scratch_bytes(void) { return kStaticScratchBytes; }

int skyrl_lmhead_bwd(const void* hidden, int64_t ld_hidden, const void* weight, int64_t ld_weight, const int64_t* labels,
                     const float* row_lse, const float* row_pz, const float* dlogprobs, const float* dentropy, int64_t T,
                     int64_t H, int64_t V, float rcp_temperature, void* d_hidden, void* d_weight, int dw_mode,
                     int64_t vocab_chunk, void* workspace, size_t workspace_bytes, void* stream) {
  return bwd_entry(hidden, ld_hidden, weight, ld_weight, labels, row_lse, row_pz, dlogprobs, dentropy, T, H, V, rcp_temperature,
                   d_hidden, d_weight, dw_mode, vocab_chunk, workspace, workspace_bytes, (hipStream_t)stream, false);
}

int skyrl_lmhead_bwd_active_rows(const void* hidden, int64_t ld_hidden, const void* weight, int64_t ld_weight,
                                 const int64_t* labels, const float* row_lse, const float* row_pz, const float* dlogprobs,
                                 const float* dentropy, int64_t T, int64_t H, int64_t V, float rcp_temperature, void* d_hidden,
                                 void* d_weight, int dw_mode, int64_t vocab_chunk, void* workspace, size_t workspace_bytes,
                                 void* stream) {
  return bwd_entry(hidden, ld_hidden, weight, ld_weight, labels, row_lse, row_pz, dlogprobs, dentropy, T, H, V, rcp_temperature,
                   d_hidden, d_weight, dw_mode, vocab_chunk, workspace, workspace_bytes, (hipStream_t)stream, true);
}

size_t skyrl_lmhead_bwd_split_workspace_bytes(int64_t T, int64_t H, int64_t terms, int64_t V, int64_t vocab_chunk,
                                              int active_rows) {
  return bwd_workspace_bytes(T, H, V, vocab_chunk, active_rows != 0, terms);
}

int skyrl_lmhead_bwd_split(const void* hidden_terms, int64_t ld_hidden, const void* weight_terms, int64_t ld_weight,
                           const int64_t* labels, const float* row_lse, const float* row_pz, const float* dlogprobs,
                           const float* dentropy, int64_t T, int64_t H, int64_t terms, int64_t V, float rcp_temperature,
                           void* d_hidden, void* d_weight, int dw_mode, int64_t vocab_chunk, int active_rows, void* workspace,
                           size_t workspace_bytes, void* stream) {
  return bwd_entry(hidden_terms, ld_hidden, weight_terms, ld_weight, labels, row_lse, row_pz, dlogprobs, dentropy, T, H, V,
                   rcp_temperature, d_hidden, d_weight, dw_mode, vocab_chunk, workspace, workspace_bytes, (hipStream_t)stream,
                   active_rows != 0, terms);
}

int skyrl_lmhead_split_operand(const void* src, int src_is_fp32, int64_t ld_src, int64_t rows, int64_t H, int layout, void* dst,
                               int64_t ld_dst, void* stream) {
  if (!src || !dst) return SKYRL_LMHEAD_ERR_NULL;
  int terms, codes[3] = {0, 0, 0};
  switch (layout) {
    case SKYRL_SPLIT_HI_LO: terms = 2, codes[1] = 1; break;
    case SKYRL_SPLIT_HI_HI: terms = 2; break;
    case SKYRL_SPLIT_HI_LO_HI: terms = 3, codes[1] = 1; break;
    case SKYRL_SPLIT_HI_HI_LO: terms = 3, codes[2] = 1; break;
    default: return SKYRL_LMHEAD_ERR_ARG;
  }
  if (rows < 1 || rows > kMaxExtent || H < 4 || H % 4 != 0 || H > kMaxExtent / 4 || ld_src < H || ld_dst < terms * H ||
      ld_src > kMaxExtent || ld_dst > kMaxExtent)
    return SKYRL_LMHEAD_ERR_SHAPE;
  if (!aligned16(src) || !aligned16(dst) || ld_src % 4 != 0 || ld_dst % 8 != 0) return SKYRL_LMHEAD_ERR_ALIGN;
  hipStream_t s = (hipStream_t)stream;
  Timed timed(kSplitOperand, s);
  if (src_is_fp32)
    hipLaunchKernelGGL(split_operand_rows<true>, dim3((unsigned)rows), dim3(256), 0, s, src, ld_src, (int)H, terms, codes[0],
                       codes[1], codes[2], (uint16_t*)dst, ld_dst);
  else
    hipLaunchKernelGGL(split_operand_rows<false>, dim3((unsigned)rows), dim3(256), 0, s, src, ld_src, (int)H, terms, codes[0],
                       codes[1], codes[2], (uint16_t*)dst, ld_dst);
  const hipError_t e = hipGetLastError();
  return e == hipSuccess ? SKYRL_LMHEAD_OK : (int)e;
}

size_t skyrl_softce_fwd_workspace_bytes(int64_t T, int64_t H, int64_t V) {
  if (T < 1 || V < 1 || H < 1 || T > kMaxExtent || V > kMaxExtent || H > kMaxExtent) return 0;
  return carve_softce_fwd(nullptr, T, H, V).bytes;
}

size_t skyrl_softce_bwd_workspace_bytes(int64_t T, int64_t H, int64_t V, int64_t vocab_chunk) {
  if (T < 1 || V < 1 || H < 1 || vocab_chunk < 0 || vocab_chunk % 256 != 0) return 0;
  if (T > kMaxExtent || V > kMaxExtent || H > kMaxExtent || vocab_chunk > kMaxExtent) return 0;
  int64_t vc = vocab_chunk ? vocab_chunk : default_vocab_chunk(T, H, V);
  if (vc > round_up(V, 256)) vc = round_up(V, 256);
  return carve_softce_bwd(nullptr, T, H, V, vc).bytes;
}

int skyrl_softce_fwd(const void* student_hidden, int64_t ld_student, const void* teacher_hidden, int64_t ld_teacher,
                     const void* weight, int64_t ld_weight, int64_t T, int64_t seq_len, int64_t shift, int64_t H, int64_t V,
                     float rcp_temperature, float* loss, float* lse_student, float* lse_teacher, void* workspace,
                     size_t workspace_bytes, void* stream) {
  int st = check_softce(student_hidden, ld_student, teacher_hidden, ld_teacher, weight, ld_weight, T, seq_len, shift, H, V,
                        rcp_temperature);
  if (st) return st;
  if (!loss || !lse_student || !lse_teacher) return SKYRL_LMHEAD_ERR_NULL;
  if (!workspace || workspace_bytes < skyrl_softce_fwd_workspace_bytes(T, H, V)) return SKYRL_LMHEAD_ERR_WORKSPACE;
  if ((uintptr_t)workspace & 255u) return SKYRL_LMHEAD_ERR_ALIGN;

  hipStream_t s = (hipStream_t)stream;
  const SoftCeFwdWorkspace w = carve_softce_fwd(workspace, T, H, V);
  const int64_t rows = 2 * round_up(T, kPairTile);
  const uint16_t* Wp = (const uint16_t*)weight;
  hipError_t e = launch_softce_pack(s, student_hidden, ld_student, teacher_hidden, ld_teacher, T, seq_len, shift, H, w.S);
  if (e != hipSuccess) return (int)e;
  const int tiles_m = (int)((V + BM - 1) / BM), tiles_n = (int)(rows / BN);
  {
    Timed timed(kSoftCeFwdTiles, s);
    auto kernel = even_ktiles(H) ? softce_fwd_tiles<true, true> : softce_fwd_tiles<true, false>;
    hipLaunchKernelGGL(kernel, dim3((unsigned)(tiles_m * tiles_n)), dim3(NTHREADS), 0, s, Wp, (int)ld_weight, w.S, (int)H,
                       (int)rows, (int)H, (int)V, rcp_temperature, w.pmax, w.psum, w.ppz);
  }
  if ((e = hipGetLastError()) != hipSuccess) return (int)e;
  {
    Timed timed(kFwdMerge, s);
    hipLaunchKernelGGL(lmhead_fwd_merge<false>, dim3((unsigned)((rows + kMergeTokens - 1) / kMergeTokens)), dim3(kMergeThreads), 0, s, w.pmax,
                       w.psum, w.ppz, (int)w.nparts, (int)rows, w.S, (int)H, Wp, (int)ld_weight, (const int64_t*)nullptr, (int)H,
                       (int)V, rcp_temperature, (float*)nullptr, (float*)nullptr, w.row_lse, w.row_pz);
  }
  if ((e = hipGetLastError()) != hipSuccess) return (int)e;
  Timed timed(kSoftCeFinish, s);
  hipLaunchKernelGGL(softce_finish, dim3((unsigned)((T + 255) / 256)), dim3(256), 0, s, w.row_lse, w.row_pz, (int)T, loss,
                     lse_student, lse_teacher);
  e = hipGetLastError();
  return e == hipSuccess ? SKYRL_LMHEAD_OK : (int)e;
}

int skyrl_softce_bwd(const void* student_hidden, int64_t ld_student, const void* teacher_hidden, int64_t ld_teacher,
                     const void* weight, int64_t ld_weight, const float* lse_student, const float* lse_teacher,
                     const float* dloss, int64_t T, int64_t seq_len, int64_t shift, int64_t H, int64_t V, float rcp_temperature,
                     void* d_student_hidden, int64_t vocab_chunk, void* workspace, size_t workspace_bytes, void* stream) {
  int st = check_softce(student_hidden, ld_student, teacher_hidden, ld_teacher, weight, ld_weight, T, seq_len, shift, H, V,
                        rcp_temperature);
  if (st) return st;
  if (!lse_student || !lse_teacher || !dloss || !d_student_hidden) return SKYRL_LMHEAD_ERR_NULL;
  if (!aligned16(d_student_hidden)) return SKYRL_LMHEAD_ERR_ALIGN;
  if (vocab_chunk < 0 || vocab_chunk % 256 != 0) return SKYRL_LMHEAD_ERR_ARG;
  const int64_t Tp = round_up(T, kPairTile), Vpad = round_up(V, 256);
  int64_t vc = vocab_chunk ? vocab_chunk : default_vocab_chunk(T, H, V);
  if (vc > Vpad) vc = Vpad;
  if ((!reads_weight_in_place(V) && Vpad + kLdPad > kMaxRowPitch) || vc + kLdPad > kMaxRowPitch) return SKYRL_LMHEAD_ERR_SHAPE;
  if (!workspace || workspace_bytes < skyrl_softce_bwd_workspace_bytes(T, H, V, vc)) return SKYRL_LMHEAD_ERR_WORKSPACE;
  if ((uintptr_t)workspace & 255u) return SKYRL_LMHEAD_ERR_ALIGN;

  hipStream_t s = (hipStream_t)stream;
  const SoftCeBwdWorkspace w = carve_softce_bwd(workspace, T, H, V, vc);
  const uint16_t* Wp = (const uint16_t*)weight;
  hipError_t e = launch_softce_pack(s, student_hidden, ld_student, teacher_hidden, ld_teacher, T, seq_len, shift, H, w.S);
  if (e != hipSuccess) return (int)e;
  const bool w_in_place = reads_weight_in_place(V);
  if (!w_in_place) {
    Timed timed(kTranspose, s);
    hipLaunchKernelGGL(transpose_bf16, dim3((unsigned)(Vpad / 64), (unsigned)(H / 64)), dim3(256), 0, s, Wp, (int)ld_weight,
                       (int)V, (int)H, w.Wt, (int)(Vpad + kLdPad), (int)Vpad, (const int*)nullptr);
    if ((e = hipGetLastError()) != hipSuccess) return (int)e;
  }
  const int64_t nchunks = (Vpad + vc - 1) / vc;
  const GemmArgs none{};
  for (int64_t ci = 0; ci < nchunks; ++ci) {
    const int64_t vc0 = ci * vc, vcw = (Vpad - vc0) < vc ? (Vpad - vc0) : vc;
    const SoftCeDzArgs z{Wp, (int)ld_weight, w.S, (int)T, (int)Tp, (int)H, (int)V, rcp_temperature, lse_student, lse_teacher,
                         dloss, (int)vc0, (int)(vcw / 256), (int)(2 * Tp / BN), w.D, (int)(vcw + kLdPad)};
    {
      Timed timed(kSoftCeDz, s);
      auto kernel = even_ktiles(H) ? softce_dz_tiles<true> : softce_dz_tiles<false>;
      hipLaunchKernelGGL(kernel, dim3((unsigned)(z.tiles_m * z.tiles_n)), dim3(NTHREADS), 0, s, z);
    }
    if ((e = hipGetLastError()) != hipSuccess) return (int)e;
    // d student hidden [t, h] (+)= sum_v D[t, v] . weight[vc0 + v, h]: the dHidden GEMM of the log-probability backward,
    // partial sums carried from chunk to chunk in accumulator order, bf16 rows written by the last chunk.
    const bool first = ci == 0, last = ci == nchunks - 1;
    uint16_t* dh_out = last ? (uint16_t*)d_student_hidden : (uint16_t*)nullptr;
    const float* dh_in = first ? (const float*)nullptr : (const float*)w.dHacc;
    float* dh_keep = last ? (float*)nullptr : w.dHacc;
    const int64_t kext = (V - vc0) < vcw ? (V - vc0) : vcw;
    const GemmArgs gh =
        w_in_place ? make_gemm(w.D, vcw + kLdPad, Tp, Wp + (size_t)vc0 * (size_t)ld_weight, ld_weight, H, true, true, kext / BK, T,
                               H, nullptr, nullptr, dh_out, H, dh_in, dh_keep)
                   : make_gemm(w.Wt + vc0, Vpad + kLdPad, H, w.D, vcw + kLdPad, Tp, false, false, vcw / BK, H, T, nullptr,
                               nullptr, dh_out, H, dh_in, dh_keep);
    e = launch_bwd_gemm(s, gh, none);
    if (e != hipSuccess) return (int)e;
  }
  return SKYRL_LMHEAD_OK;
}


size_t skyrl_lmhead_topk_workspace_bytes(int64_t T, int64_t H, int64_t V, int64_t k) {
  if (T < 1 || V < 1 || H < 1 || k < 1 || k > V || k > topk::kMaxK) return 0;
  if (T > kMaxExtent || V > kMaxExtent || H > kMaxExtent) return 0;
  return carve_topk(nullptr, T, V, k).bytes;
}

int skyrl_lmhead_topk_logits(const void* hidden, int64_t ld_hidden, const void* weight, int64_t ld_weight, int64_t T, int64_t H,
                             int64_t V, int64_t k, float rcp_temperature, float* values, int32_t* columns, void* workspace,
                             size_t workspace_bytes, void* stream) {
  int st = check_operands(hidden, ld_hidden, weight, ld_weight, T, H, V, rcp_temperature, true);
  if (st) return st;
  if (!values || !columns) return SKYRL_LMHEAD_ERR_NULL;
  if (k < 1 || k > V || k > topk::kMaxK) return SKYRL_LMHEAD_ERR_ARG;
  if (!workspace || workspace_bytes < skyrl_lmhead_topk_workspace_bytes(T, H, V, k)) return SKYRL_LMHEAD_ERR_WORKSPACE;
  if ((uintptr_t)workspace & 255u) return SKYRL_LMHEAD_ERR_ALIGN;

  hipStream_t s = (hipStream_t)stream;
  const TopkWorkspace w = carve_topk(workspace, T, V, k);
  const int64_t block_tokens = fwd_block_tokens(w.block_tokens, ld_hidden);
  const uint16_t* Wp = (const uint16_t*)weight;
  const size_t select_lds = (size_t)topk::kSelectWaves * (size_t)(k + topk::kSelectStage) * sizeof(topk::key_t);
  hipError_t e;
  for (int64_t t0 = 0; t0 < T; t0 += block_tokens) {
    const int64_t Tb = (T - t0) < block_tokens ? (T - t0) : block_tokens;
    const int tiles_n = (int)((Tb + BN - 1) / BN);
    const uint16_t* Hp = (const uint16_t*)hidden + (size_t)t0 * (size_t)ld_hidden;
    hipLaunchKernelGGL(topk::topk_reset, dim3((unsigned)((Tb + 255) / 256)), dim3(256), 0, s, (int)Tb, w.have, w.thr, w.cnt);
    if ((e = hipGetLastError()) != hipSuccess) return (int)e;
    int64_t width = kTopkFirstChunk;
    for (int64_t v0 = 0; v0 < V;) {
      const int64_t chunk = width < w.cap ? width : w.cap;
      const int64_t vrows = (V - v0) < chunk ? (V - v0) : chunk;
      const bool last = v0 + vrows >= V;
      topk::FilterArgs a{Wp + (size_t)v0 * (size_t)ld_weight, (int)ld_weight, Hp, (int)ld_hidden, (int)Tb, (int)H, (int)vrows,
                         (int)v0, rcp_temperature, (int)((vrows + BM - 1) / BM), tiles_n, kGroupM, w.thr, w.cnt, w.cand,
                         (int)w.cap};
      {
        Timed timed(kTopkFilter, s);
        auto kernel = even_ktiles(H) ? topk::topk_filter_tiles<true> : topk::topk_filter_tiles<false>;
        hipLaunchKernelGGL(kernel, dim3((unsigned)(a.tiles_m * a.tiles_n)), dim3(NTHREADS), 0, s, a);
      }
      if ((e = hipGetLastError()) != hipSuccess) return (int)e;
      {
        Timed timed(kTopkSelect, s);
        hipLaunchKernelGGL(topk::topk_select, dim3((unsigned)((Tb + topk::kSelectWaves - 1) / topk::kSelectWaves)),
                           dim3(64 * topk::kSelectWaves), select_lds, s, (int)Tb, (int)k, w.best, w.have, w.thr, w.cnt, w.cand,
                           (int)w.cap, last ? values + (size_t)t0 * (size_t)k : (float*)nullptr,
                           last ? columns + (size_t)t0 * (size_t)k : (int32_t*)nullptr);
      }
      if ((e = hipGetLastError()) != hipSuccess) return (int)e;
      v0 += vrows;
      width *= 2;
    }
  }
  return SKYRL_LMHEAD_OK;
}

namespace {
int check_topk_rows(const void* weight, int64_t ld_weight, int64_t T, int64_t H, int64_t V, int64_t k, float rcp_temperature) {
  if (!weight) return SKYRL_LMHEAD_ERR_NULL;
  if (T < 1 || V < 1 || H < 8 || H % 8 != 0 || ld_weight < H || k < 1 || k > V || k > topk::kMaxK) return SKYRL_LMHEAD_ERR_SHAPE;
  if (T > kMaxExtent || V > kMaxExtent || H > kMaxExtent || ld_weight > kMaxExtent) return SKYRL_LMHEAD_ERR_SHAPE;
  if (!aligned16(weight) || ld_weight % 8 != 0) return SKYRL_LMHEAD_ERR_ALIGN;
  if (!(rcp_temperature > 0.f) || !isfinite(rcp_temperature)) return SKYRL_LMHEAD_ERR_ARG;
  return SKYRL_LMHEAD_OK;
}
}  // namespace

int skyrl_softce_topk_fwd(const void* student_hidden, int64_t ld_student, const void* weight, int64_t ld_weight,
                          const float* teacher_values, const int32_t* teacher_columns, int64_t T, int64_t seq_len, int64_t shift,
                          int64_t H, int64_t V, int64_t k, float rcp_temperature, float* loss, float* coef, int32_t* columns,
                          void* stream) {
  int st = check_topk_rows(weight, ld_weight, T, H, V, k, rcp_temperature);
  if (st) return st;
  if (!student_hidden || !teacher_values || !teacher_columns || !loss || !coef || !columns) return SKYRL_LMHEAD_ERR_NULL;
  if (ld_student < H || ld_student > kMaxExtent || seq_len < 1 || T % seq_len != 0 || shift < 0) return SKYRL_LMHEAD_ERR_SHAPE;
  if (!aligned16(student_hidden) || ld_student % 8 != 0) return SKYRL_LMHEAD_ERR_ALIGN;
  hipStream_t s = (hipStream_t)stream;
  Timed timed(kTopkRows, s);
  hipLaunchKernelGGL(topk::topk_softce_rows, dim3((unsigned)T), dim3(topk::kRowThreads), (size_t)(2 * k + 4) * sizeof(float), s,
                     (const uint16_t*)student_hidden, (int)ld_student, (const uint16_t*)weight, (int)ld_weight, teacher_values,
                     teacher_columns, (int)T, (int)seq_len, (int)(shift % seq_len), (int)H, (int)V, (int)k, rcp_temperature, loss,
                     coef, columns);
  const hipError_t e = hipGetLastError();
  return e == hipSuccess ? SKYRL_LMHEAD_OK : (int)e;
}

int skyrl_softce_topk_bwd(const void* weight, int64_t ld_weight, const float* coef, const int32_t* columns, const float* dloss,
                          int64_t T, int64_t H, int64_t V, int64_t k, float rcp_temperature, void* d_student_hidden,
                          int64_t ld_d_student, void* stream) {
  int st = check_topk_rows(weight, ld_weight, T, H, V, k, rcp_temperature);
  if (st) return st;
  if (!coef || !columns || !dloss || !d_student_hidden) return SKYRL_LMHEAD_ERR_NULL;
  if (ld_d_student < H || ld_d_student > kMaxExtent) return SKYRL_LMHEAD_ERR_SHAPE;
  if (!aligned16(d_student_hidden) || ld_d_student % 8 != 0) return SKYRL_LMHEAD_ERR_ALIGN;
  hipStream_t s = (hipStream_t)stream;
  Timed timed(kTopkBwdRows, s);
  hipLaunchKernelGGL(topk::topk_softce_bwd_rows, dim3((unsigned)T), dim3(topk::kRowThreads), (size_t)(2 * k) * sizeof(float), s,
                     (const uint16_t*)weight, (int)ld_weight, coef, columns, dloss, (int)H, (int)V, (int)k, rcp_temperature,
                     (uint16_t*)d_student_hidden, (int)ld_d_student);
  const hipError_t e = hipGetLastError();
  return e == hipSuccess ? SKYRL_LMHEAD_OK : (int)e;
}

int skyrl_lmhead_mfma_probe(const void* operands, int workgroups, int iters, float* sink, void* stream) {
  if (!operands || !sink) return SKYRL_LMHEAD_ERR_NULL;
  if (workgroups < 1 || workgroups > 65536 || iters < 1) return SKYRL_LMHEAD_ERR_ARG;
  if (!aligned16(operands)) return SKYRL_LMHEAD_ERR_ALIGN;
  hipLaunchKernelGGL(mfma_probe, dim3((unsigned)workgroups), dim3(NTHREADS), 0, (hipStream_t)stream, (const bf16x8*)operands, iters,
                     sink);
  return (int)hipGetLastError();
}

int skyrl_lmhead_atomic_floor_probe(float* d_weight, float* d_hidden, int64_t T, int64_t H, int64_t V, void* stream) {
  if (!d_weight || !d_hidden) return SKYRL_LMHEAD_ERR_NULL;
  if (T < BN || V < BM || T % BN != 0 || V % BM != 0 || H < 1 || T > kMaxExtent || V > kMaxExtent) return SKYRL_LMHEAD_ERR_SHAPE;
  const int64_t tiles = (T / BN) * (V / BM);
  if (tiles > ((int64_t)1 << 30)) return SKYRL_LMHEAD_ERR_SHAPE;
  hipLaunchKernelGGL(atomic_floor_probe, dim3((unsigned)tiles), dim3(NTHREADS), 0, (hipStream_t)stream, d_weight, d_hidden,
                     (int)(V / BM), (int)H);
  return (int)hipGetLastError();
}

int skyrl_lmhead_device_info(int* compute_units_out, int* max_clock_khz) {
  if (!compute_units_out || !max_clock_khz) return SKYRL_LMHEAD_ERR_NULL;
  int dev = 0;
  hipError_t e = hipGetDevice(&dev);
  if (e == hipSuccess) e = hipDeviceGetAttribute(compute_units_out, hipDeviceAttributeMultiprocessorCount, dev);
  if (e == hipSuccess) e = hipDeviceGetAttribute(max_clock_khz, hipDeviceAttributeClockRate, dev);
  return e == hipSuccess ? SKYRL_LMHEAD_OK : (int)e;
}

int skyrl_lmhead_num_kernel_kinds(void) { return kNumKernelKinds; }

const char* skyrl_lmhead_kernel_name(int kind) {
  return (kind >= 0 && kind < kNumKernelKinds) ? kKernelNames[kind] : "";
}

void* skyrl_lmhead_profile_begin(void) {
  if (tl_profile) return nullptr;
  tl_profile = new Profile();
  return tl_profile;
}

int skyrl_lmhead_profile_end(void* handle, double* total_ms, int64_t* launches) {
  if (!handle || handle != (void*)tl_profile || !total_ms || !launches) return SKYRL_LMHEAD_ERR_NULL;
  Profile* p = tl_profile;
  tl_profile = nullptr;
  for (int k = 0; k < kNumKernelKinds; ++k) total_ms[k] = 0.0, launches[k] = 0;
  int status = SKYRL_LMHEAD_OK;
  for (auto& r : p->recs) {
    hipError_t e = hipEventSynchronize(r.b);
    float ms = 0.f;
    if (e == hipSuccess) e = hipEventElapsedTime(&ms, r.a, r.b);
    if (e == hipSuccess) {
      total_ms[r.kind] += ms;
      launches[r.kind] += 1;
    } else if (status == SKYRL_LMHEAD_OK) {
      status = (int)e;
    }
    (void)hipEventDestroy(r.a);
    (void)hipEventDestroy(r.b);
  }
  delete p;
  return status;
}

}  // extern "C"
