// bf16 MFMA mainloop shared by every GEMM-shaped kernel of the fused LM-head path (gfx950 / CDNA4 only).
//
// All contractions on the path are brought into one form, C[M,N] = A[M,K] * B[N,K]^T with A and B bf16,
// row-major and K-contiguous, so one software-pipelined mainloop serves the forward logits GEMM, the
// backward logits recompute, dHidden and dW.  A workgroup of 8 wavefronts (2 along M x 4 along N) owns a
// 256x256 tile of C; each wavefront owns 128x64 of it as 4x2 accumulators of v_mfma_f32_32x32x16_bf16.
//
// Data path: 16-byte global_load_lds (global -> LDS without a VGPR round trip) into two XOR-swizzled LDS
// stages; ds_read_b128 fragments; MFMA with fp32 accumulation.
//
// LDS tile layout (one operand, one stage): 256 rows x BK k bf16.  The 16-byte chunk (row, kc) lives at byte
// row*ROW_BYTES + ((kc ^ swz(row)) << 4), see swz() below.
//
// Accumulator layout of v_mfma_f32_32x32x16 (lane l, register r in 0..15):
//     m = (r >> 2) * 8 + (l >> 5) * 4 + (r & 3),   n = l & 31
// i.e. a lane holds one column n and 16 rows m.  The kernels put the *vocab* index on M and the *token*
// index on N, so every per-token quantity (running max, sum-exp, upstream grads) is a per-lane scalar and
// the vocab reduction is an in-register loop plus one lane^32 exchange.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#include <type_traits>

namespace lmhead {

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(4))) __bf16 bf16x4;
typedef __attribute__((ext_vector_type(2))) __bf16 bf16x2;
typedef __attribute__((ext_vector_type(16))) float f32x16;
typedef __attribute__((ext_vector_type(4))) float f32x4;
typedef __attribute__((ext_vector_type(2))) float f32x2;

constexpr int BM = 256;            // tile rows (A rows)
constexpr int BN = 256;            // tile cols (B rows)
constexpr int BK = 64;             // k per pipeline stage: 128-byte rows keep the direct-to-LDS copies at full rate
constexpr int NSTAGES = 2;         // two 64 KiB stages; a third does not fit the CU's 160 KiB
#ifndef LMHEAD_WAVES_N
#define LMHEAD_WAVES_N 4
#endif
constexpr int WAVES_M = 2, WAVES_N = LMHEAD_WAVES_N;
constexpr int NWAVES = WAVES_M * WAVES_N;
constexpr int NTHREADS = 64 * NWAVES;
constexpr int WM = BM / WAVES_M;   // 128
constexpr int WN = BN / WAVES_N;   // 64
constexpr int TM = WM / 32;        // 4 MFMA tiles along M per wave
constexpr int TN = WN / 32;        // 2 MFMA tiles along N per wave
constexpr int KSTEPS = BK / 16;                    // MFMA k-steps per stage
constexpr int ROW_BYTES = BK * 2;                  // one operand row inside a stage
constexpr int CHUNKS_PER_ROW = ROW_BYTES / 16;     // 16-byte chunks per row
constexpr int OPERAND_BYTES = BM * ROW_BYTES;      // 16 or 32 KiB
constexpr int STAGE_BYTES = 2 * OPERAND_BYTES;     // A then B
constexpr int GROUPS = OPERAND_BYTES / 1024;       // global_load_lds instructions (one wave each) per operand tile
constexpr int LOADS_PER_TILE = 2 * GROUPS / NWAVES;  // per lane, both operands
constexpr int LDS_BYTES = NSTAGES * STAGE_BYTES;   // 128 KiB of the CU's 160 KiB
static_assert(LDS_BYTES <= 160 * 1024, "stages do not fit LDS");
#ifndef LMHEAD_SCHED
#define LMHEAD_SCHED 1
#endif
#ifndef LMHEAD_ABL
#define LMHEAD_ABL 0  // timing-only ablations (wrong results): 1 no global loads, 2 no fragment reads, 8 wait one tile late
#endif

// LDS on gfx950 has 64 banks of 4 bytes and serves a ds_read_b128 sixteen lanes (256 B) at a time.  Lanes 0..15 of a
// fragment read touch 16 consecutive rows at one k-chunk.  XOR-ing the chunk index with a few row bits spreads those
// sixteen reads over all sixteen 16-byte slots of a 256-byte window: with 128-byte rows (BK = 64) a window holds
// 2 rows x 8 chunks and the key is (row >> 1) & 7; with 64-byte rows (BK = 32) it holds 4 rows x 4 chunks and the key
// is (row >> 2) & 3.
__device__ __forceinline__ int swz(int row) { return BK == 64 ? ((row >> 1) & 7) : ((row >> 2) & 3); }

typedef f32x16 acc_t[TM][TN];

struct Operand {
  const uint16_t* ptr;  // bf16 bits, row-major, K contiguous
  int ld;               // elements between rows (multiple of 8)
  int row0;             // first row of this tile
  int rows;             // total valid rows; rows past the end are clamped (their results are masked later)
};

// Issue the global->LDS copies of one 256 x BK operand tile (16 B per lane and instruction).
// One instruction of one wave fills 64 consecutive 16-byte chunks of LDS; the lane picks the global chunk whose
// swizzled home is its LDS slot.
__device__ __forceinline__ void issue_operand_loads(const Operand& op, int k0, char* lds_operand, int wave, int lane) {
#pragma unroll
  for (int j = 0; j < GROUPS / NWAVES; ++j) {
    const int grp = j * NWAVES + wave;
    const int p = grp * 64 + lane;         // chunk slot in LDS
    const int row = p / CHUNKS_PER_ROW;
    const int kc = (p % CHUNKS_PER_ROW) ^ swz(row);  // global chunk that lives in this slot
    int grow = op.row0 + row;
    grow = grow < op.rows ? grow : op.rows - 1;
    const uint16_t* src = op.ptr + (size_t)grow * (size_t)op.ld + (size_t)(k0 + kc * 8);
    __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)src,
                                     (__attribute__((address_space(3))) void*)(lds_operand + grp * 1024), 16, 0, 0);
  }
}

// Wait until at most N of this lane's global->LDS copies are still in flight and all of its LDS reads have returned,
// then meet the rest of the workgroup.  The "memory" clobber keeps the compiler from moving LDS accesses across it.
template <int N>
__device__ __forceinline__ void wait_copies_and_barrier() {
  static_assert(N >= 0 && N < 64, "vmcnt is a 6-bit counter");
  asm volatile("s_waitcnt vmcnt(%0) lgkmcnt(0)\n\ts_barrier" ::"n"(N) : "memory");
}
__device__ __forceinline__ void zero_acc(acc_t& acc) {
#pragma unroll
  for (int i = 0; i < TM; ++i)
#pragma unroll
    for (int j = 0; j < TN; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.f;
}

__device__ __forceinline__ void read_frags(const char* stage, const int (&a_off)[TM], const int (&b_off)[TN], int kc_sw,
                                           bf16x8 (&af)[TM], bf16x8 (&bfr)[TN]) {
#pragma unroll
  for (int i = 0; i < TM; ++i) af[i] = *(const bf16x8*)(stage + a_off[i] + kc_sw);
#pragma unroll
  for (int j = 0; j < TN; ++j) bfr[j] = *(const bf16x8*)(stage + b_off[j] + kc_sw);
}

__device__ __forceinline__ void mfma_step(const bf16x8 (&af)[TM], const bf16x8 (&bfr)[TN], acc_t& acc) {
#pragma unroll
  for (int i = 0; i < TM; ++i)
#pragma unroll
    for (int j = 0; j < TN; ++j) acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(af[i], bfr[j], acc[i][j], 0, 0, 0);
}

// acc += A[a.row0 : +256, k_begin : k_begin + nk*BK] * B[b.row0 : +256, same k]^T
// Every thread of the workgroup must call this with identical arguments (it contains barriers).
//
// Pipeline: global->LDS copies run one k-tile ahead (two LDS stages); LDS->register fragment reads run one 16-k step
// ahead (two fragment sets).  The one barrier per k-tile sits between the last fragment read of a tile and the MFMAs
// that consume it, so the matrix pipe has a full step of work queued while the copies of tile kt+2 are issued and the
// first fragments of tile kt+1 come back from LDS.
__device__ __forceinline__ void mainloop(const Operand& a, const Operand& b, int k_begin, int nk, char* lds, acc_t& acc) {
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = tid >> 6;
  const int wm = wave / WAVES_N;
  const int wn = wave % WAVES_N;

  // Per-lane fragment addresses inside a stage; k-step s XORs in the swizzled chunk (2*s + lane/32).
  const int lrow = lane & 31;
  const int sw = swz(lrow);  // every fragment row is lrow plus a multiple of 32, so the swizzle depends on the lane only
  const int khalf = lane >> 5;
  int a_off[TM], b_off[TN];
#pragma unroll
  for (int i = 0; i < TM; ++i) a_off[i] = (wm * WM + i * 32 + lrow) * ROW_BYTES;
#pragma unroll
  for (int j = 0; j < TN; ++j) b_off[j] = OPERAND_BYTES + (wn * WN + j * 32 + lrow) * ROW_BYTES;
  int kc_sw[KSTEPS];
#pragma unroll
  for (int ks = 0; ks < KSTEPS; ++ks) kc_sw[ks] = ((ks * 2 + khalf) ^ sw) << 4;

  bf16x8 af[2][TM], bfr[2][TN];

  // Prologue: tiles 0 and 1 in flight, wait for tile 0.
  issue_operand_loads(a, k_begin, lds, wave, lane);
  issue_operand_loads(b, k_begin, lds + OPERAND_BYTES, wave, lane);
  if (nk > 1) {
    issue_operand_loads(a, k_begin + BK, lds + STAGE_BYTES, wave, lane);
    issue_operand_loads(b, k_begin + BK, lds + STAGE_BYTES + OPERAND_BYTES, wave, lane);
    wait_copies_and_barrier<LOADS_PER_TILE>();
  } else {
    wait_copies_and_barrier<0>();
  }
  read_frags(lds, a_off, b_off, kc_sw[0], af[0], bfr[0]);

  // Three copies of the tile step (steady state, second-to-last, last) instead of conditions inside one loop body: a
  // branch that joins a path with outstanding LDS reads makes the compiler wait for all of them.
  auto tile_step = [&](int kt, auto has_next, auto load_next2) {
    char* cur = lds + (kt & 1) * STAGE_BYTES;
    char* nxt = lds + ((kt + 1) & 1) * STAGE_BYTES;
#pragma unroll
    for (int ks = 0; ks < KSTEPS; ++ks) {
      if (LMHEAD_ABL & 2) {
      } else if (ks + 1 < KSTEPS) {
        read_frags(cur, a_off, b_off, kc_sw[ks + 1], af[(ks + 1) & 1], bfr[(ks + 1) & 1]);
      } else if (has_next) {
        // All of this wave's reads of `cur` are complete and its copies into `nxt` have landed; after the barrier that
        // holds for every wave, so `cur` may be overwritten (tile kt+2) and `nxt` may be read.
        if (LMHEAD_ABL & 8) wait_copies_and_barrier<LOADS_PER_TILE>(); else wait_copies_and_barrier<0>();
        if (load_next2 && !(LMHEAD_ABL & 1)) {
          const int k0 = k_begin + (kt + 2) * BK;
          issue_operand_loads(a, k0, cur, wave, lane);
          issue_operand_loads(b, k0, cur + OPERAND_BYTES, wave, lane);
        }
        read_frags(nxt, a_off, b_off, kc_sw[0], af[(ks + 1) & 1], bfr[(ks + 1) & 1]);
      }
      mfma_step(af[ks & 1], bfr[ks & 1], acc);
#if LMHEAD_SCHED == 1
      // one LDS read behind each of the first MFMAs of the step
      if (ks + 1 < KSTEPS || has_next) {
#pragma unroll
        for (int x = 0; x < TM + TN; ++x) {
          __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
          __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
        }
        __builtin_amdgcn_sched_group_barrier(0x008, TM * TN - TM - TN, 0);
      }
#endif
    }
  };
  int kt = 0;
  for (; kt + 2 < nk; ++kt) tile_step(kt, std::true_type{}, std::true_type{});
  if (kt + 1 < nk) {
    tile_step(kt, std::true_type{}, std::false_type{});
    ++kt;
  }
  tile_step(kt, std::false_type{}, std::false_type{});
  // The caller may reuse LDS (or start another mainloop) only after all waves are done reading.
  wait_copies_and_barrier<0>();
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
