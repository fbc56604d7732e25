// Device code of the top-k draft loss of multi-token prediction (skyrl/backends/skyrl_train/mtp/soft_ce.py:243-341,
// _VocabParallelTopkSoftCE on one vocabulary shard): the k largest teacher logits of every token straight from the teacher's
// hidden states -- no [T, V] logits tensor -- and the soft cross-entropy of the student over those k columns.
//
//   topk_filter_tiles   one 256(vocab) x 256(token) logits tile of a vocabulary chunk, the forward's GEMM; the epilogue compares
//                       every logit with the token's threshold (the k-th largest logit among the columns of earlier chunks, a
//                       lower bound of the final one) and appends the few that pass to the token's candidate list.
//   topk_select         one wave per token: merges the chunk's candidates into the token's running k best, raises its
//                       threshold, empties the candidate list.  After the last chunk it also writes the k logits and their
//                       columns, best first.
//   topk_softce_rows    one workgroup per token: the student's logits at the (rolled) teacher's k columns, k dot products with
//                       gathered weight rows; softmax of both over the k columns; loss and d loss / d student logits.
//   topk_softce_bwd_rows  one workgroup per token: d student hidden = upstream * sum_j coef[j] * weight[column j] / temperature.
//
// Order of logits: higher value first, lower column first among equal values; -0.0 sorts below +0.0.  That order is total,
// so the k best of a row are a unique set whatever order the candidates arrive in, and the results are reproducible although
// the candidate lists are filled with atomic counters.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "gemm_core.hpp"

namespace topk {
using namespace lmhead;

typedef unsigned long long key_t;

// Bits of a float such that unsigned comparison orders them as the floats order (negative values below positive ones).
__device__ __forceinline__ uint32_t ordered_bits(float z) {
  const uint32_t b = __float_as_uint(z);
  return b ^ ((b >> 31) ? 0xffffffffu : 0x80000000u);
}
__device__ __forceinline__ float value_of_bits(uint32_t o) {
  return __uint_as_float(o ^ ((o >> 31) ? 0x80000000u : 0xffffffffu));
}
// A logit and its column as one key: a larger key is a better candidate.
__device__ __forceinline__ key_t make_key(float z, int column) { return ((key_t)ordered_bits(z) << 32) | (key_t)(uint32_t)(~column); }
__device__ __forceinline__ float key_value(key_t k) { return value_of_bits((uint32_t)(k >> 32)); }
__device__ __forceinline__ int key_column(key_t k) { return (int)(~(uint32_t)k); }

struct FilterArgs {
  const uint16_t* W;   // first weight row of the chunk
  int ldw;
  const uint16_t* Hd;  // hidden rows of the token block
  int ldh;
  int T, H;
  int vrows;           // weight rows of the chunk that exist (the last tile may overhang them)
  int v0;              // column number of the chunk's first row
  float rcp_temp;
  int tiles_m, tiles_n, group_m;
  const float* thr;    // [T] threshold per token, -inf while fewer than k columns have been seen
  unsigned* cnt;       // [T] candidates appended in this launch
  key_t* cand;         // [T, cap]
  int cap;             // >= columns of a chunk, so that a list cannot overflow
};

template <bool EVEN>
__global__ __launch_bounds__(NTHREADS) void topk_filter_tiles(const FilterArgs a) {
  __shared__ __attribute__((aligned(1024))) char lds[LDS_BYTES];
  int tm, tn;
  tile_coords(blockIdx.x, a.tiles_m, a.tiles_n, a.group_m, tm, tn);

  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int wm = wave / WAVES_N, wn = wave % WAVES_N;
  const int lrow = lane & 15, kq = lane >> 4;
  // The tokens' thresholds (fixed for the launch): unconditional loads from a clamped index, issued before the mainloop and
  // first touched behind it -- a load under `t < T` is a branch with its own wait, eight memory round trips in a row.
  float th[TN];
#pragma unroll
  for (int j = 0; j < TN; ++j) {
    const int t = tn * BN + wn * WN + j * MT + lrow;
    th[j] = a.thr[t < a.T ? t : a.T - 1];
  }

  Operand oa{a.W, a.ldw, tm * BM, a.vrows};
  Operand ob{a.Hd, a.ldh, tn * BN, a.T};
  acc_t acc;
  prefetch_first_tiles(oa, ob, 0, a.H / BK, lds);
  zero_acc(acc);
  mainloop<false, EVEN>(oa, ob, 0, a.H / BK, lds, acc);

  const int vbase = tm * BM + wm * WM;  // first row of this wave inside the chunk
  if (vbase >= a.vrows) return;
  const float s = a.rcp_temp;
#pragma unroll
  for (int j = 0; j < TN; ++j) {
    const int t = tn * BN + wn * WN + j * MT + lrow;
    if (t >= a.T) th[j] = NAN;  // rows past the last token never pass: every comparison with NaN is false
  }
  // A lane holds 32 logits of each of its eight tokens.  First sweep: how many of them pass (a wave-wide vote on the largest
  // of four skips the blocks in which nothing does -- nearly all of them once a threshold exists; rounding is monotone and
  // s > 0, so the scaled maximum is the maximum of the scaled values).  Then one atomic add per lane and token reserves that
  // many slots of the token's list -- eight independent atomics in flight, one round trip per tile -- and a second sweep
  // stores the keys.  The accumulators are only read, so both sweeps see the same values.
  const bool ragged = vbase + WM > a.vrows;
  int hits[TN];
  unsigned long long voted[TN];  // bit i: block i of token column j has a passing logit somewhere in the wave
#pragma unroll
  for (int j = 0; j < TN; ++j) {
    hits[j] = 0;
    voted[j] = 0;
#pragma unroll
    for (int i = 0; i < TM; ++i) {
      const float m4 = fmaxf(fmaxf(acc[i][j][0], acc[i][j][1]), fmaxf(acc[i][j][2], acc[i][j][3])) * s;
      if (__any(m4 >= th[j])) {
        voted[j] |= 1ull << i;
#pragma unroll
        for (int r = 0; r < 4; ++r) {
          const int vr = vbase + i * MT + kq * 4 + r;
          hits[j] += (acc[i][j][r] * s >= th[j] && (!ragged || vr < a.vrows)) ? 1 : 0;
        }
      }
    }
  }
  unsigned base[TN];
#pragma unroll
  for (int j = 0; j < TN; ++j) {
    const int t = tn * BN + wn * WN + j * MT + lrow;
    base[j] = hits[j] > 0 ? atomicAdd(a.cnt + t, (unsigned)hits[j]) : 0u;
  }
#pragma unroll
  for (int j = 0; j < TN; ++j) {
    if (voted[j] == 0) continue;  // wave-uniform
    const int t = tn * BN + wn * WN + j * MT + lrow;
    key_t* list = a.cand + (size_t)t * (size_t)a.cap;
    unsigned slot = base[j];
#pragma unroll
    for (int i = 0; i < TM; ++i) {
      if (!((voted[j] >> i) & 1)) continue;  // wave-uniform
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        const float z = acc[i][j][r] * s;
        const int vr = vbase + i * MT + kq * 4 + r;
        if (z >= th[j] && (!ragged || vr < a.vrows)) {
          if (slot < (unsigned)a.cap) list[slot] = make_key(z, a.v0 + vr);
          ++slot;
        }
      }
    }
  }
}

// Smallest key of the wave's values, in every lane.
__device__ __forceinline__ key_t wave_min_key(key_t v) {
#pragma unroll
  for (int o = 32; o >= 1; o >>= 1) {
    const key_t w = __shfl_xor(v, o, 64);
    v = w < v ? w : v;
  }
  return v;
}

constexpr int kSelectWaves = 4;
constexpr int kMaxK = 1024;
constexpr int kSelectStage = 1024;   // candidates one bulk round takes into LDS, behind the list
constexpr int kSelectBulkMin = 96;   // fewer candidates than this are inserted one by one

// best: [T, k] running lists (unordered), have: [T] entries of the list that are filled.  One wave per token; the list lives
// in LDS while the wave works on it.  Many candidates (the first chunks, a large k, adversarial data) are merged in bulk: up to
// kSelectStage of them are put behind the list, a bisection over the key bits finds a threshold that exactly k keys reach
// (keys are unique, so one exists; a pass over the keys per bit, usually 20 to 30 bits until the count is exact), and the keys
// that reach it are compacted to the front in place.  A few candidates are inserted one by one, each replacing the worst
// entry.  With `final_vals` the finished list is written out best first.
__global__ __launch_bounds__(64 * kSelectWaves) void topk_select(int T, int k, key_t* __restrict__ best, unsigned* __restrict__ have,
                                                                 float* __restrict__ thr, unsigned* __restrict__ cnt,
                                                                 const key_t* __restrict__ cand, int cap,
                                                                 float* __restrict__ final_vals, int* __restrict__ final_idx) {
  extern __shared__ key_t sm_list[];  // kSelectWaves * (k + kSelectStage) keys
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int t = blockIdx.x * kSelectWaves + wave;
  if (t >= T) return;  // whole waves leave; no barrier below
  key_t* list = sm_list + (size_t)wave * (size_t)(k + kSelectStage);
  key_t* gl = best + (size_t)t * (size_t)k;
  int n_have = (int)have[t];
  for (int e = lane; e < n_have; e += 64) list[e] = gl[e];
  // LDS operations of one wave execute in order; the fences below only keep the compiler from caching list entries that
  // another lane has rewritten.
  auto lds_fence = []() { __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront"); };
  lds_fence();
  const unsigned n_raw = cnt[t];
  const int n = (int)(n_raw < (unsigned)cap ? n_raw : (unsigned)cap);

  // the worst entry of a full list: its key and position
  key_t worst = 0;
  int worst_pos = 0;
  auto find_worst = [&]() {
    key_t mine = ~(key_t)0;
    for (int e = lane; e < k; e += 64) mine = list[e] < mine ? list[e] : mine;
    worst = wave_min_key(mine);
    int pos = -1;
    for (int e = lane; e < k; e += 64)
      if (list[e] == worst) pos = e;  // keys are unique (columns are)
    const unsigned long long owner = __ballot(pos >= 0);
    worst_pos = __shfl(pos, (int)__ffsll((long long)owner) - 1, 64);
  };
  const key_t* cl = cand + (size_t)t * (size_t)cap;
  int done = 0;
  while (n - done >= kSelectBulkMin) {
    const int take = (n - done) < kSelectStage ? (n - done) : kSelectStage;
    for (int e = lane; e < take; e += 64) list[n_have + e] = cl[done + e];
    lds_fence();
    const int M = n_have + take;
    done += take;
    if (M <= k) {
      n_have = M;
      continue;
    }
    key_t reach = 0;  // grows bit by bit while at least k keys reach it; done when exactly k do
    for (int b = 63; b >= 0; --b) {
      const key_t trial = reach | ((key_t)1 << b);
      int c = 0;
      for (int e = lane; e < M; e += 64) c += list[e] >= trial ? 1 : 0;
#pragma unroll
      for (int o = 32; o >= 1; o >>= 1) c += __shfl_xor(c, o, 64);
      if (c >= k) {
        reach = trial;
        if (c == k) break;
      }
    }
    int w = 0;  // in-place compaction: a step reads 64 entries and writes at or below where it read
    for (int base = 0; base < M; base += 64) {
      const int e = base + lane;
      const key_t x = e < M ? list[e] : 0;
      const bool keep = e < M && x >= reach;
      const unsigned long long mask = __ballot(keep);
      lds_fence();
      if (keep) list[w + __popcll(mask & (((key_t)1 << lane) - 1))] = x;
      w += (int)__popcll(mask);
      lds_fence();
    }
    n_have = k;
  }
  if (n_have == k) find_worst();

  for (int c0 = done; c0 < n; c0 += 64) {
    const bool in = c0 + lane < n;
    const key_t c = in ? cl[c0 + lane] : 0;
    unsigned long long pending = __ballot(in && (n_have < k || c > worst));
    while (pending) {
      const int src = (int)__ffsll((long long)pending) - 1;
      pending &= pending - 1;
      const key_t x = __shfl(c, src, 64);
      if (n_have < k) {
        if (lane == 0) list[n_have] = x;
        lds_fence();
        ++n_have;
        if (n_have == k) {
          find_worst();
          pending &= __ballot(c > worst);
        }
      } else if (x > worst) {
        if (lane == 0) list[worst_pos] = x;
        lds_fence();
        find_worst();
        pending &= __ballot(c > worst);
      }
    }
  }

  if (!final_vals) {
    for (int e = lane; e < n_have; e += 64) gl[e] = list[e];
    if (lane == 0) {
      have[t] = (unsigned)n_have;
      thr[t] = n_have == k ? key_value(worst) : -INFINITY;
      cnt[t] = 0u;
    }
    return;
  }
  // Final pass: rank every entry among the k (number of better keys) and write value and column at that rank.
  for (int e = lane; e < k; e += 64) {
    if (e < n_have) {
      const key_t mine = list[e];
      int rank = 0;
      for (int o = 0; o < n_have; ++o) rank += list[o] > mine ? 1 : 0;
      final_vals[(size_t)t * (size_t)k + rank] = key_value(mine);
      final_idx[(size_t)t * (size_t)k + rank] = key_column(mine);
    } else {
      // Fewer than k comparable logits: the row holds NaNs (a NaN never passes the filter's comparison).  torch.topk ranks
      // NaN first and the loss built on it is NaN (mtp/soft_ce.py:258-305); the ranks nobody filled say the same.
      final_vals[(size_t)t * (size_t)k + e] = NAN;
      final_idx[(size_t)t * (size_t)k + e] = 0;
    }
  }
  if (lane == 0) cnt[t] = 0u;
}

__global__ __launch_bounds__(256) void topk_reset(int T, unsigned* __restrict__ have, float* __restrict__ thr,
                                                  unsigned* __restrict__ cnt) {
  const int t = blockIdx.x * 256 + threadIdx.x;
  if (t < T) have[t] = 0u, thr[t] = -INFINITY, cnt[t] = 0u;
}

// fp32 dot product of two bf16 rows, the wave's lanes taking 16-byte pieces; the sum in every lane.
__device__ __forceinline__ float wave_dot_bf16(const uint16_t* __restrict__ x, const uint16_t* __restrict__ y, int H, int lane) {
  float dot = 0.f;
  for (int c = lane * 8; c < H; c += 64 * 8) {
    const uint4 xv = *(const uint4*)(x + c);
    const uint4 yv = *(const uint4*)(y + c);
    const uint32_t xx[4] = {xv.x, xv.y, xv.z, xv.w};
    const uint32_t yy[4] = {yv.x, yv.y, yv.z, yv.w};
#pragma unroll
    for (int q = 0; q < 4; ++q) {
      dot = fmaf(__uint_as_float(xx[q] << 16), __uint_as_float(yy[q] << 16), dot);
      dot = fmaf(__uint_as_float(xx[q] & 0xffff0000u), __uint_as_float(yy[q] & 0xffff0000u), dot);
    }
  }
#pragma unroll
  for (int o = 32; o >= 1; o >>= 1) dot += __shfl_xor(dot, o, 64);
  return dot;
}

constexpr int kRowThreads = 256;

__device__ __forceinline__ float block_reduce(float v, bool take_max, float* sm) {
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
#pragma unroll
  for (int o = 32; o >= 1; o >>= 1) {
    const float w = __shfl_xor(v, o, 64);
    v = take_max ? fmaxf(v, w) : v + w;
  }
  __syncthreads();  // sm may still be read from the previous reduction
  if (lane == 0) sm[wave] = v;
  __syncthreads();
  float r = sm[0];
  for (int w = 1; w < kRowThreads / 64; ++w) r = take_max ? fmaxf(r, sm[w]) : r + sm[w];
  return r;
}

// Token b * seq_len + s is scored against the teacher's list of token b * seq_len + (s + shift) mod seq_len
// (torch.roll of the [B, S, k] top-k result by -shift, soft_ce.py:277-279).
//   t_p = softmax(teacher values), q_s = softmax(student values) over the k columns,
//   loss = -sum_j t_p[j] log q_s[j]   (soft_ce.py:282-300),   coef[j] = q_s[j] - t_p[j]   (:309)
__global__ __launch_bounds__(kRowThreads) void topk_softce_rows(const uint16_t* __restrict__ student, int lds_,
                                                                const uint16_t* __restrict__ W, int ldw,
                                                                const float* __restrict__ t_vals, const int* __restrict__ t_idx,
                                                                int T, int seq_len, int shift, int H, int V, int k, float rcp_temp,
                                                                float* __restrict__ loss, float* __restrict__ coef,
                                                                int* __restrict__ columns) {
  extern __shared__ float sm_rows[];  // k student values, k teacher values, 4 reduction slots
  float* sv = sm_rows;
  float* tv = sm_rows + k;
  float* red = sm_rows + 2 * k;
  const int t = blockIdx.x;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int row = t / seq_len, pos = t - row * seq_len;
  const size_t tt = (size_t)row * (size_t)seq_len + (size_t)((pos + shift) % seq_len);
  const uint16_t* hs = student + (size_t)t * (size_t)lds_;
  for (int j = wave; j < k; j += kRowThreads / 64) {
    int col = t_idx[tt * (size_t)k + j];
    col = col < 0 ? 0 : (col >= V ? V - 1 : col);  // a caller's own column list cannot make the gather leave the weight
    const float dot = wave_dot_bf16(hs, W + (size_t)col * (size_t)ldw, H, lane);
    if (lane == 0) {
      sv[j] = dot * rcp_temp;
      tv[j] = t_vals[tt * (size_t)k + j];
      columns[(size_t)t * (size_t)k + j] = col;
    }
  }
  __syncthreads();
  float ms = -INFINITY, mt = -INFINITY;
  for (int j = threadIdx.x; j < k; j += kRowThreads) ms = fmaxf(ms, sv[j]), mt = fmaxf(mt, tv[j]);
  ms = block_reduce(ms, true, red);
  mt = block_reduce(mt, true, red);
  float ss = 0.f, st = 0.f;
  for (int j = threadIdx.x; j < k; j += kRowThreads) ss += expf(sv[j] - ms), st += expf(tv[j] - mt);
  ss = block_reduce(ss, false, red);
  st = block_reduce(st, false, red);
  const float log_ss = logf(ss);
  float l = 0.f;
  for (int j = threadIdx.x; j < k; j += kRowThreads) {
    const float tp = expf(tv[j] - mt) / st;
    const float qs = expf(sv[j] - ms) / ss;
    l -= tp * ((sv[j] - ms) - log_ss);
    coef[(size_t)t * (size_t)k + j] = qs - tp;
  }
  l = block_reduce(l, false, red);
  if (threadIdx.x == 0) loss[t] = l;
}

// d student hidden[t, :] = dloss[t] / temperature * sum_j coef[t, j] * weight[columns[t, j], :]   (the scatter of
// soft_ce.py:309-312 followed by the output layer's backward), fp32 sums, bf16 result.
__global__ __launch_bounds__(kRowThreads) void topk_softce_bwd_rows(const uint16_t* __restrict__ W, int ldw,
                                                                    const float* __restrict__ coef, const int* __restrict__ columns,
                                                                    const float* __restrict__ dloss, int H, int V, int k, float rcp_temp,
                                                                    uint16_t* __restrict__ d_student, int ldd) {
  extern __shared__ float sm_bwd[];  // k coefficients, then k columns
  float* cf = sm_bwd;
  int* cl = (int*)(sm_bwd + k);
  const int t = blockIdx.x;
  const float g = dloss[t] * rcp_temp;
  for (int j = threadIdx.x; j < k; j += kRowThreads) {
    cf[j] = coef[(size_t)t * (size_t)k + j] * g;
    const int col = columns[(size_t)t * (size_t)k + j];
    cl[j] = col < 0 ? 0 : (col >= V ? V - 1 : col);
  }
  __syncthreads();
  for (int c = threadIdx.x * 8; c < H; c += kRowThreads * 8) {
    float acc[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
    for (int j = 0; j < k; ++j) {
      const uint4 wv = *(const uint4*)(W + (size_t)cl[j] * (size_t)ldw + c);
      const uint32_t ww[4] = {wv.x, wv.y, wv.z, wv.w};
      const float f = cf[j];
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        acc[2 * q] = fmaf(f, __uint_as_float(ww[q] << 16), acc[2 * q]);
        acc[2 * q + 1] = fmaf(f, __uint_as_float(ww[q] & 0xffff0000u), acc[2 * q + 1]);
      }
    }
    const f32x4 lo4 = {acc[0], acc[1], acc[2], acc[3]}, hi4 = {acc[4], acc[5], acc[6], acc[7]};
    const bf16x4 lo = __builtin_convertvector(lo4, bf16x4), hi = __builtin_convertvector(hi4, bf16x4);
    const uint2 a2 = *(const uint2*)&lo, b2 = *(const uint2*)&hi;
    *(uint4*)(d_student + (size_t)t * (size_t)ldd + c) = make_uint4(a2.x, a2.y, b2.x, b2.y);
  }
}

}  // namespace topk
