// Packed-sequence front and back end of the fused LM-head path: integer index work either side of the GEMM kernels.
//
// The trainer packs the sequences of a micro-batch into one [T] token stream described by cu_seqlens [n+1] (sequence s owns
// tokens cu[s] .. cu[s+1]-1).  Before the LM head, every token needs the id of its successor *inside its own sequence* as
// the label; after it, the [T] log-probabilities go back to a [rows, cols] batch layout.  The reference does both with about
// twenty torch index kernels and boolean-mask indexing, which synchronises with the host
// (skyrl/backends/skyrl_train/distributed/megatron/model_utils.py:810-815, 851-883, 920-928).  Here each direction is one
// launch, and the scatter has its adjoint (the gradient of the log-probabilities) as a kernel of its own.
//
// All of it is HBM-bound at a few bytes per token; the kernels are one thread per token (or per output column) with
// coalesced 4- and 8-byte accesses, and a binary search over cu_seqlens that stays in L1/L2.
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "../../include/skyrl_lmhead.h"

namespace {

constexpr int kThreads = 256;
constexpr int kMaskThreads = 1024;  // workgroup of the attention-mask scatter: one per row, rows are few and long
constexpr int64_t kNotInVocab = INT64_MAX;

// Sequence that holds packed token t: the smallest s with cu[s+1] > t (what searchsorted(cu[1:], t, right=True) returns,
// model_utils.py:925).  Returns n when t lies at or beyond cu[n].  Empty sequences are skipped.
__device__ __forceinline__ int64_t sequence_of(const int64_t* __restrict__ cu, int64_t n, int64_t t) {
  int64_t lo = 0, hi = n;
  while (lo < hi) {
    const int64_t mid = (lo + hi) >> 1;
    if (cu[mid + 1] > t) hi = mid; else lo = mid + 1;
  }
  return lo;
}

__global__ void __launch_bounds__(kThreads) next_token_labels_kernel(const int64_t* __restrict__ tokens,
                                                                     const int64_t* __restrict__ cu, int64_t n, int64_t T,
                                                                     int64_t* __restrict__ labels) {
  const int64_t t = (int64_t)blockIdx.x * kThreads + threadIdx.x;
  if (t >= T) return;
  const int64_t s = sequence_of(cu, n, t);
  int64_t label = kNotInVocab;
  if (s < n) {
    const int64_t begin = cu[s], len = cu[s + 1] - begin;
    int64_t next = t - begin + 1;
    if (next == len) next = 0;  // (offset + 1) mod len, model_utils.py:814
    const int64_t src = begin + next;
    if (src < T) label = tokens[src];
  }
  labels[t] = label;
}

__global__ void __launch_bounds__(kThreads) fill_f32_kernel(float* __restrict__ p, int64_t n, float v) {
  const int64_t i = (int64_t)blockIdx.x * kThreads + threadIdx.x;
  if (i < n) p[i] = v;
}

// Destination of packed token t in the [rows, cols] output, or -1.  Plain branch (model_utils.py:880-883): row = sequence,
// column = offset, for offset < len - 1.  Sub-sequence branch (:859-871): row / first column / true length per packed
// segment; offset < true length - 1.  Both: the column must lie inside the output.
__device__ __forceinline__ int64_t destination(const int64_t* __restrict__ cu, int64_t n, int64_t t,
                                               const int64_t* __restrict__ seg_row, const int64_t* __restrict__ seg_col,
                                               const int64_t* __restrict__ seg_len, int64_t rows, int64_t cols) {
  const int64_t s = sequence_of(cu, n, t);
  if (s >= n) return -1;
  const int64_t off = t - cu[s];
  int64_t row, col, valid;
  if (seg_row) {
    row = seg_row[s];
    col = seg_col[s] + off;
    valid = seg_len[s] - 1;
  } else {
    row = s;
    col = off;
    valid = cu[s + 1] - cu[s] - 1;
  }
  if (off >= valid || col >= cols || col < 0 || row < 0 || row >= rows) return -1;
  return row * cols + col;
}

template <bool ADJOINT>
__global__ void __launch_bounds__(kThreads) scatter_kernel(float* __restrict__ packed, const int64_t* __restrict__ cu,
                                                           int64_t n, int64_t T, const int64_t* __restrict__ seg_row,
                                                           const int64_t* __restrict__ seg_col,
                                                           const int64_t* __restrict__ seg_len, int64_t rows, int64_t cols,
                                                           float* __restrict__ out) {
  const int64_t t = (int64_t)blockIdx.x * kThreads + threadIdx.x;
  if (t >= T) return;
  const int64_t d = destination(cu, n, t, seg_row, seg_col, seg_len, rows, cols);
  if (ADJOINT) {
    packed[t] = d >= 0 ? out[d] : 0.f;
  } else if (d >= 0) {
    out[d] = packed[t];
  }
}

// Attention-mask branch (model_utils.py:873-878): row b of the [rows, cols + 1] mask marks the real tokens of sequence b;
// its j-th real token (j = 0 ..) takes packed token cu[b] + j, for every real token but the last one.  One workgroup per
// row walks the row in pieces of 1024 columns, numbering the real tokens with wave ballots.
template <bool ADJOINT>
__global__ void __launch_bounds__(kMaskThreads) scatter_masked_kernel(float* __restrict__ packed, const int64_t* __restrict__ cu,
                                                                  int64_t T, const uint8_t* __restrict__ mask, int64_t cols,
                                                                  float* __restrict__ out) {
  __shared__ int wave_count[kMaskThreads / 64];
  const int64_t b = blockIdx.x;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const uint8_t* mrow = mask + b * (cols + 1);
  const int64_t begin = cu[b], padded = cu[b + 1] - begin;

  // Number of real tokens in the row.
  int mine = 0;
  for (int64_t c = threadIdx.x; c <= cols; c += kMaskThreads) mine += mrow[c] != 0;
  for (int o = 32; o > 0; o >>= 1) mine += __shfl_xor(mine, o);
  if (lane == 0) wave_count[wave] = mine;
  __syncthreads();
  int64_t seq_len = 0;
  for (int w = 0; w < kMaskThreads / 64; ++w) seq_len += wave_count[w];
  __syncthreads();

  int64_t seen = 0;  // real tokens in the columns before this piece
  for (int64_t c0 = 0; c0 < cols; c0 += kMaskThreads) {
    const int64_t c = c0 + threadIdx.x;
    const bool real = c < cols && mrow[c] != 0;
    const unsigned long long ballot = __ballot(real);
    if (lane == 0) wave_count[wave] = __popcll(ballot);
    __syncthreads();
    int64_t before = seen, piece = 0;
    for (int w = 0; w < kMaskThreads / 64; ++w) {
      if (w < wave) before += wave_count[w];
      piece += wave_count[w];
    }
    __syncthreads();
    const int64_t j = before + __popcll(ballot & ((1ull << lane) - 1ull));  // index of this real token in its row
    if (c < cols) {
      // ordinal j + 1 < seq_len (:875): every real token but the last; the source must lie in the packed segment.
      const bool use = real && j + 1 < seq_len && j < padded && begin + j < T;
      if (ADJOINT) {
        if (use) packed[begin + j] = out[b * cols + c];
      } else {
        out[b * cols + c] = use ? packed[begin + j] : 0.f;
      }
    }
    seen += piece;
  }
}

inline unsigned blocks_for(int64_t n) { return (unsigned)((n + kThreads - 1) / kThreads); }

int check_scatter(const void* packed, const int64_t* cu, int64_t n, int64_t T, const int64_t* seg_row, const int64_t* seg_col,
                  const int64_t* seg_len, const uint8_t* mask, int64_t rows, int64_t cols, const void* out) {
  if (!cu || (!packed && T > 0) || (!out && rows > 0 && cols > 0)) return SKYRL_LMHEAD_ERR_NULL;
  const int given = (seg_row != nullptr) + (seg_col != nullptr) + (seg_len != nullptr);
  if (given != 0 && given != 3) return SKYRL_LMHEAD_ERR_NULL;
  if (given == 3 && mask) return SKYRL_LMHEAD_ERR_ARG;
  if (n < 0 || T < 0 || rows < 0 || cols < 0) return SKYRL_LMHEAD_ERR_SHAPE;
  if (mask && rows != n) return SKYRL_LMHEAD_ERR_SHAPE;
  // one thread per token or output element, at most 2^31 workgroups; rows and columns are bounded first so that their
  // product cannot overflow
  const int64_t kMaxDim = int64_t(1) << 31, kMaxElems = kMaxDim * kThreads;
  if (T >= kMaxElems || rows >= kMaxDim || cols >= kMaxDim || rows * cols >= kMaxElems) return SKYRL_LMHEAD_ERR_SHAPE;
  return SKYRL_LMHEAD_OK;
}

}  // namespace

extern "C" {

int skyrl_packed_next_token_labels(const int64_t* tokens, const int64_t* cu_seqlens, int64_t num_seqs, int64_t T,
                                   int64_t* labels, void* stream) {
  if (!tokens || !cu_seqlens || !labels) return SKYRL_LMHEAD_ERR_NULL;
  if (num_seqs < 0 || T < 0 || T >= (int64_t(1) << 31) * kThreads) return SKYRL_LMHEAD_ERR_SHAPE;
  if (T == 0) return SKYRL_LMHEAD_OK;
  hipLaunchKernelGGL(next_token_labels_kernel, dim3(blocks_for(T)), dim3(kThreads), 0, (hipStream_t)stream, tokens, cu_seqlens,
                     num_seqs, T, labels);
  return (int)hipGetLastError();
}

int skyrl_packed_scatter_logprobs(const float* packed, const int64_t* cu_seqlens, int64_t num_seqs, int64_t T,
                                  const int64_t* seg_row, const int64_t* seg_col, const int64_t* seg_len,
                                  const uint8_t* attention_mask, int64_t rows, int64_t cols, float* out, void* stream) {
  const int st = check_scatter(packed, cu_seqlens, num_seqs, T, seg_row, seg_col, seg_len, attention_mask, rows, cols, out);
  if (st != SKYRL_LMHEAD_OK) return st;
  if (rows * cols == 0) return SKYRL_LMHEAD_OK;
  hipStream_t s = (hipStream_t)stream;
  if (attention_mask) {
    hipLaunchKernelGGL(scatter_masked_kernel<false>, dim3((unsigned)rows), dim3(kMaskThreads), 0, s, const_cast<float*>(packed),
                       cu_seqlens, T, attention_mask, cols, out);
    return (int)hipGetLastError();
  }
  hipLaunchKernelGGL(fill_f32_kernel, dim3(blocks_for(rows * cols)), dim3(kThreads), 0, s, out, rows * cols, 0.f);
  if (T > 0)
    hipLaunchKernelGGL(scatter_kernel<false>, dim3(blocks_for(T)), dim3(kThreads), 0, s, const_cast<float*>(packed), cu_seqlens,
                       num_seqs, T, seg_row, seg_col, seg_len, rows, cols, out);
  return (int)hipGetLastError();
}

int skyrl_packed_gather_grad(const float* d_out, const int64_t* cu_seqlens, int64_t num_seqs, int64_t T,
                             const int64_t* seg_row, const int64_t* seg_col, const int64_t* seg_len,
                             const uint8_t* attention_mask, int64_t rows, int64_t cols, float* d_packed, void* stream) {
  const int st = check_scatter(d_packed, cu_seqlens, num_seqs, T, seg_row, seg_col, seg_len, attention_mask, rows, cols, d_out);
  if (st != SKYRL_LMHEAD_OK) return st;
  if (T == 0) return SKYRL_LMHEAD_OK;
  hipStream_t s = (hipStream_t)stream;
  float* src = const_cast<float*>(d_out);
  if (attention_mask) {
    hipLaunchKernelGGL(fill_f32_kernel, dim3(blocks_for(T)), dim3(kThreads), 0, s, d_packed, T, 0.f);
    if (rows * cols > 0)
      hipLaunchKernelGGL(scatter_masked_kernel<true>, dim3((unsigned)rows), dim3(kMaskThreads), 0, s, d_packed, cu_seqlens, T,
                         attention_mask, cols, src);
    return (int)hipGetLastError();
  }
  hipLaunchKernelGGL(scatter_kernel<true>, dim3(blocks_for(T)), dim3(kThreads), 0, s, d_packed, cu_seqlens, num_seqs, T, seg_row,
                     seg_col, seg_len, rows, cols, src);
  return (int)hipGetLastError();
}

}  // extern "C"
