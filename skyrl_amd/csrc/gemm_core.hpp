// bf16 MFMA mainloop shared by every GEMM-shaped kernel of the fused LM-head path (gfx950 / CDNA4 only).
//
// All contractions on the path are brought into one form, C[M,N] = A[M,K] * B[N,K]^T with A and B bf16,
// row-major and K-contiguous, so one software-pipelined mainloop serves the forward logits GEMM, the
// backward logits recompute, dHidden and dW.  A workgroup of 8 wavefronts (2 along M x 4 along N) owns a
// 256x256 tile of C; each wavefront owns 128x64 of it as 4x2 accumulators of v_mfma_f32_32x32x16_bf16.
//
// Data path: 16-byte global_load_lds (global -> LDS without a VGPR round trip) into a double-buffered,
// XOR-swizzled LDS tile; ds_read_b128 fragments; MFMA with fp32 accumulation.
//
// LDS tile layout (one operand, one stage): 256 rows x 64 k bf16 = 256 x 128 B.  The 16-byte chunk
// (row, kc) lives at byte  row*128 + ((kc ^ (row & 7)) << 4).  Eight consecutive rows at the same kc then
// fall into eight different 16-byte slots of a 128-byte line, so the fragment reads (lane -> row) sweep all
// 32 banks instead of hammering four of them.
//
// Accumulator layout of v_mfma_f32_32x32x16 (lane l, register r in 0..15):
//     m = (r >> 2) * 8 + (l >> 5) * 4 + (r & 3),   n = l & 31
// i.e. a lane holds one column n and 16 rows m.  The kernels put the *vocab* index on M and the *token*
// index on N, so every per-token quantity (running max, sum-exp, upstream grads) is a per-lane scalar and
// the vocab reduction is an in-register loop plus one lane^32 exchange.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace lmhead {

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(4))) __bf16 bf16x4;
typedef __attribute__((ext_vector_type(2))) __bf16 bf16x2;
typedef __attribute__((ext_vector_type(16))) float f32x16;
typedef __attribute__((ext_vector_type(4))) float f32x4;
typedef __attribute__((ext_vector_type(2))) float f32x2;

constexpr int BM = 256;            // tile rows (A rows)
constexpr int BN = 256;            // tile cols (B rows)
constexpr int BK = 64;             // k per pipeline stage
constexpr int NTHREADS = 512;      // 8 wavefronts
constexpr int WAVES_M = 2, WAVES_N = 4;
constexpr int WM = BM / WAVES_M;   // 128
constexpr int WN = BN / WAVES_N;   // 64
constexpr int TM = WM / 32;        // 4 MFMA tiles along M per wave
constexpr int TN = WN / 32;        // 2 MFMA tiles along N per wave
constexpr int OPERAND_BYTES = BM * BK * 2;         // 32 KiB
constexpr int STAGE_BYTES = 2 * OPERAND_BYTES;     // 64 KiB (A then B)
constexpr int NSTAGES = 2;
constexpr int LDS_BYTES = NSTAGES * STAGE_BYTES;   // 128 KiB of the CU's 160 KiB

typedef f32x16 acc_t[TM][TN];

struct Operand {
  const uint16_t* ptr;  // bf16 bits, row-major, K contiguous
  int ld;               // elements between rows (multiple of 8)
  int row0;             // first row of this tile
  int rows;             // total valid rows; rows past the end are clamped (their results are masked later)
};

// Issue the global->LDS copies of one 256 x 64 operand tile (4 x 16 B per lane).
// One instruction of one wave fills 64 consecutive 16-byte chunks = 8 LDS rows; the lane picks the global
// chunk whose swizzled home is its LDS slot.
__device__ __forceinline__ void issue_operand_loads(const Operand& op, int k0, char* lds_operand, int wave, int lane) {
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    const int grp = j * 8 + wave;          // 32 groups of 64 chunks
    const int p = grp * 64 + lane;         // chunk slot in LDS
    const int row = p >> 3;
    const int kc = (p & 7) ^ (row & 7);    // global chunk that lives in this slot
    int grow = op.row0 + row;
    grow = grow < op.rows ? grow : op.rows - 1;
    const uint16_t* src = op.ptr + (size_t)grow * (size_t)op.ld + (size_t)(k0 + kc * 8);
    __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)src,
                                     (__attribute__((address_space(3))) void*)(lds_operand + grp * 1024), 16, 0, 0);
  }
}

__device__ __forceinline__ void zero_acc(acc_t& acc) {
#pragma unroll
  for (int i = 0; i < TM; ++i)
#pragma unroll
    for (int j = 0; j < TN; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.f;
}

// acc += A[a.row0 : +256, k_begin : k_begin + nk*64] * B[b.row0 : +256, same k]^T
// Every thread of the workgroup must call this with identical arguments (it contains barriers).
__device__ __forceinline__ void mainloop(const Operand& a, const Operand& b, int k_begin, int nk, char* lds, acc_t& acc) {
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = tid >> 6;
  const int wm = wave / WAVES_N;
  const int wn = wave % WAVES_N;

  // Per-lane fragment addresses inside an operand tile (k-step 0); k-step s XORs in (2*s) << 4 ... the
  // swizzle is (kc ^ (row & 7)) << 4 with kc = 2*s + (lane >> 5), and row & 7 == lane & 7 for every tile.
  const int lrow = lane & 31;
  const int sw = lane & 7;
  const int khalf = lane >> 5;
  int a_off[TM], b_off[TN];
#pragma unroll
  for (int i = 0; i < TM; ++i) a_off[i] = (wm * WM + i * 32 + lrow) * 128;
#pragma unroll
  for (int j = 0; j < TN; ++j) b_off[j] = OPERAND_BYTES + (wn * WN + j * 32 + lrow) * 128;

  issue_operand_loads(a, k_begin, lds, wave, lane);
  issue_operand_loads(b, k_begin, lds + OPERAND_BYTES, wave, lane);

  for (int kt = 0; kt < nk; ++kt) {
    char* cur = lds + (kt & 1) * STAGE_BYTES;
    char* nxt = lds + ((kt + 1) & 1) * STAGE_BYTES;
    // Tile kt has landed in every wave's share of LDS, and every wave has finished reading the other stage.
    __syncthreads();
    if (kt + 1 < nk) {
      const int k0 = k_begin + (kt + 1) * BK;
      issue_operand_loads(a, k0, nxt, wave, lane);
      issue_operand_loads(b, k0, nxt + OPERAND_BYTES, wave, lane);
    }
#pragma unroll
    for (int ks = 0; ks < BK / 16; ++ks) {
      const int kc_sw = ((ks * 2 + khalf) ^ sw) << 4;
      bf16x8 af[TM], bfr[TN];
#pragma unroll
      for (int i = 0; i < TM; ++i) af[i] = *(const bf16x8*)(cur + a_off[i] + kc_sw);
#pragma unroll
      for (int j = 0; j < TN; ++j) bfr[j] = *(const bf16x8*)(cur + b_off[j] + kc_sw);
#pragma unroll
      for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j) acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(af[i], bfr[j], acc[i][j], 0, 0, 0);
    }
  }
  // The caller may reuse LDS (or start another mainloop) only after all waves are done reading.
  __syncthreads();
}

// Workgroup id -> tile coordinates.
//  1. Hardware hands consecutive workgroup ids to the 8 XCDs round-robin; undo that so each XCD (own L2)
//     owns a contiguous range of the logical order.
//  2. Walk the logical order in bands of `group_m` tiles along M, N-major inside a band, so the ~32
//     workgroups concurrently resident on one XCD cover a compact group_m x (32/group_m) patch and share
//     operand panels in that XCD's L2.
__device__ __forceinline__ void tile_coords(int bid, int tiles_m, int tiles_n, int group_m, int& tm, int& tn) {
  const int total = tiles_m * tiles_n;
  const int per_xcd = total >> 3;
  int logical = bid;
  if (bid < (per_xcd << 3)) logical = (bid & 7) * per_xcd + (bid >> 3);
  const int band_sz = group_m * tiles_n;
  const int band = logical / band_sz;
  const int in_band = logical - band * band_sz;
  const int m_first = band * group_m;
  int gm = tiles_m - m_first;
  gm = gm < group_m ? gm : group_m;
  tn = in_band / gm;
  tm = m_first + (in_band - tn * gm);
}

__device__ __forceinline__ float shfl_xor32(float v) { return __shfl_xor(v, 32, 64); }

}  // namespace lmhead
