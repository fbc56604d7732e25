// bf16 MFMA mainloop shared by every GEMM-shaped kernel of the fused LM-head path (gfx950 / CDNA4 only).
//
// All contractions on the path are brought into one form, C[M,N] = A[M,K] * B[N,K]^T with A and B bf16, row-major and
// K-contiguous, so one software-pipelined mainloop serves the forward logits GEMM, the backward logits recompute,
// dHidden and dW.  A workgroup of 4 wavefronts (2 x 2, one per SIMD) owns a 256 x 256 tile of C; each wavefront owns
// 128 x 128 of it as 8 x 8 accumulators of v_mfma_f32_16x16x32_bf16 (256 accumulator registers, in AGPRs).
//
// What bounds the loop (measured on the MI355X):
//   * with random operands the matrix pipe is power-limited, not issue-limited: a loop of nothing but MFMAs on
//     N(0,1) data sustains 1.69-1.84 PFLOP/s with v_mfma_f32_32x32x16_bf16 and 2.00-2.10 PFLOP/s with
//     v_mfma_f32_16x16x32_bf16 (both 2.46-2.49 on zeros), so the 16 x 16 x 32 shape is used although it needs twice
//     the MFMA instructions;
//   * a CU takes at most ~32 B/clk from L2, through global_load_lds as well as through ordinary loads; a 64 KiB k-tile
//     (256 + 256 rows x 64 k) therefore needs >= 2048 clk, exactly the MFMA time of a 256 x 256 x 64 tile: the copy
//     path, not the matrix pipe, is the resource that must never idle;
//   * LDS reads and direct-to-LDS copies share the LDS port, so LDS is read as little as possible: 128 x 128 wave
//     tiles need 16 fragment reads per 32-k step (128 x 64 tiles need 24); the 8 extra reads of a K-major B operand
//     (two 64-bit transposing reads per fragment) measured free;
//   * the copy unit takes one 1 KiB copy about every 34 clk for the whole CU and a wave that issues into a full queue
//     stalls -- with one wave per SIMD that stalls the matrix pipe -- so a lane's 16 copies per k-tile are spread
//     evenly over its 128 MFMAs.
//
// Data path: 16-byte global_load_lds (global -> LDS without a VGPR round trip) into a ring of five 32 KiB operand
// slots (2.5 k-tiles, all of the CU's 160 KiB); ds_read_b128 fragments one 32-k step ahead; MFMA, fp32 accumulation.
// The B operand may also be given K-major (see Operand); its fragments then come through ds_read_b64_tr_b16, the
// transposing LDS read, so that a producer's output can be contracted along either of its axes without a second copy.
//
// LDS operand slot: 256 rows x 64 k bf16 = 256 x 128 B.  The 16-byte chunk (row, kc) lives at byte
// row*128 + ((kc ^ swz(row)) << 4), see swz() below.
//
// Operand layout of v_mfma_f32_16x16x32 (lane l): row (A) or column (B) l & 15, the eight k values (l >> 4) * 8 .. + 7,
// i.e. one 16-byte LDS chunk per lane.  Accumulator layout (lane l, register r in 0..3):
//     m = (l >> 4) * 4 + r,   n = l & 15
// i.e. a lane holds one column n and four consecutive rows m.  The kernels put the *vocab* index on M and the *token*
// index on N, so every per-token quantity (running max, sum-exp, upstream grads) is a per-lane scalar and the vocab
// reduction is an in-register loop plus the lane^16 and lane^32 exchanges; a lane's four values are an 8-byte piece
// of a bf16 row (16 bytes of an fp32 row) along M.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#include <type_traits>

// Timing-only ablations (skyrl_amd/bench_ablations.py): 32 = mainloop_pairs() without its fragment reads from LDS (the MFMAs
// run on the fragments read before the loop), 64 = without its global -> LDS copies behind the first two k-tiles.  Results
// are wrong with either; 0 in the product.
#ifndef LMHEAD_ABLATE
#define LMHEAD_ABLATE 0
#endif

namespace lmhead {

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(4))) __bf16 bf16x4;
typedef __attribute__((ext_vector_type(4))) short i16x4;
typedef __attribute__((ext_vector_type(16))) float f32x16;
typedef __attribute__((ext_vector_type(4))) float f32x4;

constexpr int BM = 256;            // tile rows (A rows)
constexpr int BN = 256;            // tile cols (B rows)
constexpr int BK = 64;             // k per tile: 128-byte rows keep the direct-to-LDS copies at full rate (64-byte rows lose 10 %)
constexpr int WAVES_M = 2, WAVES_N = 2;
constexpr int NWAVES = WAVES_M * WAVES_N;
constexpr int NTHREADS = 64 * NWAVES;
constexpr int WM = BM / WAVES_M;   // 128
constexpr int WN = BN / WAVES_N;   // 128
constexpr int MT = 16;             // MFMA tile edge
constexpr int TM = WM / MT;        // 8 MFMA tiles along M per wave
constexpr int TN = WN / MT;        // 8 MFMA tiles along N per wave
constexpr int KSTEPS = BK / 32;                    // MFMA k-steps per k-tile
constexpr int ROW_BYTES = BK * 2;                  // one operand row inside a slot
constexpr int OPERAND_BYTES = BM * ROW_BYTES;      // 32 KiB
constexpr int RING_SLOTS = 5;
constexpr int LDS_BYTES = RING_SLOTS * OPERAND_BYTES;  // 160 KiB: the whole LDS of a CU
constexpr int COPIES_PER_OPERAND = OPERAND_BYTES / 1024 / NWAVES;  // 8 global_load_lds per lane per operand tile
static_assert(KSTEPS == 2 && TM == 8 && TN == 8 && COPIES_PER_OPERAND == 8, "the schedule below is written for these");

// LDS on gfx950 has 64 banks of 4 bytes and serves a ds_read_b128 sixteen lanes (256 B) at a time.  Sixteen consecutive
// lanes of a fragment read touch 16 consecutive rows at one k-chunk.  XOR-ing the chunk index with (row >> 1) & 7 spreads those
// sixteen reads over all sixteen 16-byte slots of a 256-byte window (2 rows x 8 chunks): conflict-free, 256 B/clk
// measured; the obvious key row & 7 reaches 159 B/clk.
__device__ __forceinline__ int swz(int row) { return (row >> 1) & 7; }

typedef f32x4 acc_t[TM][TN];

// Order in which the 64 MFMAs of a 32-k step visit the 8 x 8 accumulators: a zigzag inside strips of two rows,
// (0,0) (1,0) (1,1) (0,1) (0,2) (1,2) ..., the next strip walked back.  Consecutive MFMAs share one operand and the
// operand that changes alternates A, B, A, B.  With random data the matrix pipe is power-limited and the order is
// measurable: a loop of nothing but MFMAs runs 2 % faster in this order than in a row-by-row serpentine (the A fragment
// kept for eight MFMAs), 6 % faster than in an order that changes both operands every time; on zeros all orders tie.
__host__ __device__ constexpr int mfma_row(int x) { return (x / 16) * 2 + ((x % 16 + 1) / 2) % 2; }
__host__ __device__ constexpr int mfma_col(int x) { return (x / 16) % 2 ? TN - 1 - (x % 16) / 2 : (x % 16) / 2; }
static_assert(TM == 8 && TN == 8, "mfma_row / mfma_col walk an 8 x 8 grid");

// The n-th (n = 0, 1, ...) MFMA gap of a 64-MFMA step at or behind x that is odd (the even ones carry fragment reads)
// and is not a copy gap (x % 8 == 5).
constexpr int free_gap(int x, int n) {
  for (int g = x | 1;; g += 2)
    if (g % 8 != 5 && n-- == 0) return g;
}

struct Operand {
  const uint16_t* ptr;  // bf16 bits, row-major, K contiguous
  int ld;               // elements between rows (multiple of 8)
  int row0;             // first row of this tile
  int rows;             // total valid rows (> row0); rows past the end are clamped (their results are masked later)
};
// A B operand may instead be "K-major": the same matrix stored transposed, ptr[k * ld + n], so that a 16-byte chunk
// holds eight consecutive n of one k (what a producer writes when n is its contiguous axis).  Then row0 is the first
// column n of the tile and `rows` the number of valid columns (a multiple of 8): a tile may overhang them, the overhanging
// lanes re-read the last valid chunk (their results belong to output columns that the epilogue drops).  The caller
// guarantees that every k row of the loop exists.
//
// K-major slot layout: 64 k-rows x 256 n = 32 blocks of 1 KiB, block b = rows 2b and 2b+1 (what one wave-wide copy
// fills).  A block is 16 windows of 64 bytes, a window = 32 bytes (16 n) of the even row, then of the odd row.  The 16 n
// of pair q sit in window q ^ sigma(b), sigma(b) = (b & 1) + 2 * ((b >> 2) & 1): the transposing fragment read below
// takes, per 16 lanes, four consecutive rows at one pair, and with this key the eight row pieces of lanes 0-31 (and of
// lanes 32-63) fall into the eight different 32-byte bank groups.
__device__ __forceinline__ int kmajor_sigma(int block) { return (block & 1) + 2 * ((block >> 2) & 1); }

// Wait until at most N of this lane's global->LDS copies are still in flight and all of its LDS reads have returned,
// then meet the rest of the workgroup.  The "memory" clobber keeps the compiler from moving LDS accesses across it.
// Memory operations complete in issue order, so N counts the youngest ones; any other load or store the compiler has
// in flight only makes the wait longer, never shorter.
template <int N>
__device__ __forceinline__ void wait_copies_and_barrier() {
  static_assert(N >= 0 && N < 64, "vmcnt is a 6-bit counter");
  asm volatile("s_waitcnt vmcnt(%0) lgkmcnt(0)\n\ts_barrier" ::"n"(N) : "memory");
}

// One MFMA, accumulating in place in AGPRs.  Written as inline assembly because the register allocator, given 64
// separate four-register accumulators through the builtin, rotates them through the loop (MFMA destination != source)
// and repairs the permutation with hundreds of v_accvgpr moves per iteration.  The compiler does not know this is an
// MFMA, so the hazards it would otherwise pad are handled by construction: an MFMA that reads as its C operand exactly the
// registers the previous MFMA wrote is interlocked by the hardware (that is what mainloop_pairs() issues back to back), and
// every mainloop ends with explicit wait states before anything else reads the accumulators.
__device__ __forceinline__ void mfma_16x16x32(f32x4& c, const bf16x8& a, const bf16x8& b) {
  asm volatile("v_mfma_f32_16x16x32_bf16 %0, %1, %2, %0" : "+a"(c) : "v"(a), "v"(b));
}

__device__ __forceinline__ void zero_acc(acc_t& acc) {
#pragma unroll
  for (int i = 0; i < TM; ++i)
#pragma unroll
    for (int j = 0; j < TN; ++j)
#pragma unroll
      for (int r = 0; r < 4; ++r) acc[i][j][r] = 0.f;
  // The other hazard the compiler cannot see: an MFMA must not read an accumulator within a few cycles of the
  // v_accvgpr_write that set it.  Wait states here, and every accumulator passes through an empty volatile asm so that
  // the writes are placed before them.
  asm volatile("s_nop 7" ::: "memory");
#pragma unroll
  for (int i = 0; i < TM; ++i)
#pragma unroll
    for (int j = 0; j < TN; ++j) asm volatile("" : "+a"(acc[i][j]));
}

// Per-lane plan of the global->LDS copies of one output tile: which global 16-byte chunk lands in which LDS chunk.
// One copy instruction of one wave fills 64 consecutive 16-byte chunks of a slot (8 rows); the lane picks the global
// chunk whose swizzled home is its LDS chunk.  Offsets are 32-bit byte offsets from the tile's first row (K-contiguous
// operand) or first column (K-major operand), which the 64-bit uniform base pointer carries together with the k offset:
// an operand may be of any size as long as 256 of its rows (64 for a K-major one) span less than 4 GiB, i.e. its row
// pitch stays below kMaxRowPitch elements (checked on the host).
constexpr int64_t kMaxRowPitch = (int64_t)1 << 22;  // elements: 256 rows of 8 MiB are 2 GiB of 32-bit offsets
struct CopyPlan {
  const char* a_bytes;
  const char* b_bytes;
  uint32_t a_src[COPIES_PER_OPERAND], b_src[COPIES_PER_OPERAND];
};

template <bool BKM>
__device__ __forceinline__ void make_plan(CopyPlan& p, const Operand& a, const Operand& b, int k_begin) {
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
#pragma unroll
  for (int j = 0; j < COPIES_PER_OPERAND; ++j) {
    const int c = (j * NWAVES + wave) * 64 + lane;  // chunk index inside the slot
    const int row = c >> 3;
    const int kc = (c & 7) ^ swz(row);
    int ra = a.row0 + row < a.rows ? row : a.rows - 1 - a.row0;  // row inside the tile; rows past the end re-read the last one
    p.a_src[j] = (uint32_t)ra * (uint32_t)a.ld * 2u + (uint32_t)(kc * 16);
    if (BKM) {
      const int block = j * NWAVES + wave;             // rows 2 * block, 2 * block + 1 of the k-tile
      const int q = (lane >> 2) ^ kmajor_sigma(block);  // the pair whose home is this lane's window
      const int krow = 2 * block + ((lane >> 1) & 1);
      int n = q * 16 + (lane & 1) * 8;  // column inside the tile
      n = b.row0 + n < b.rows - 8 ? n : b.rows - 8 - b.row0;
      p.b_src[j] = (uint32_t)krow * (uint32_t)b.ld * 2u + (uint32_t)(n * 2);
    } else {
      int rb = b.row0 + row < b.rows ? row : b.rows - 1 - b.row0;
      p.b_src[j] = (uint32_t)rb * (uint32_t)b.ld * 2u + (uint32_t)(kc * 16);
    }
  }
  // The tile origins are wave-uniform, but they come out of integer divisions that the compiler runs on the vector unit:
  // readfirstlane puts them (and with them the two base pointers) back into scalar registers.
  const size_t a_row0 = (size_t)__builtin_amdgcn_readfirstlane(a.row0), b_row0 = (size_t)__builtin_amdgcn_readfirstlane(b.row0);
  p.a_bytes = (const char*)a.ptr + (a_row0 * (size_t)a.ld + (size_t)k_begin) * 2;
  p.b_bytes = (const char*)b.ptr +
              (BKM ? ((size_t)k_begin * (size_t)b.ld + b_row0) * 2 : (b_row0 * (size_t)b.ld + (size_t)k_begin) * 2);
}

// Bytes between consecutive k-tiles of the B operand.
template <bool BKM>
__device__ __forceinline__ uint32_t b_tile_stride(const Operand& b) {
  return BKM ? (uint32_t)BK * (uint32_t)b.ld * 2u : (uint32_t)(BK * 2);
}

// Copies j0 .. j0+n-1 (of COPIES_PER_OPERAND) of one k-tile of one operand into a ring slot.  `g` is the wave-uniform
// address of the operand at that k-tile (base + k offset); `slot_wave_addr` is the LDS address of the slot plus this wave's
// share of a 4 KiB copy group (wave_copy_base() + slot offset).
// Written as assembly to get the "SGPR base + 32-bit VGPR offset" address form: through the builtin the compiler keeps
// sixteen 64-bit per-lane addresses and spends a 64-bit VALU add per copy, and with one wave per SIMD an MFMA leaves
// room for only three other instructions before the matrix pipe runs dry.  M0 (the LDS destination of the copy) is
// written immediately before every use and nothing else in these kernels reads it.
__device__ __forceinline__ void copy_part(const char* g, const uint32_t (&src)[COPIES_PER_OPERAND],
                                          uint32_t slot_wave_addr, int j0, int n) {
#pragma unroll
  for (int j = j0; j < j0 + n; ++j)
    asm volatile("s_add_u32 m0, %0, %1\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %2, %3"
                 :
                 : "s"(slot_wave_addr), "n"(j * NWAVES * 1024), "v"(src[j]), "s"(g)
                 : "memory", "m0", "scc");
}

// LDS address of this wave's first 1 KiB copy destination inside ring slot 0 (wave-uniform, kept in an SGPR); slot k
// is k * OPERAND_BYTES further.
__device__ __forceinline__ uint32_t wave_copy_base(char* lds) {
  const uint32_t wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  return (uint32_t)(uintptr_t)(__attribute__((address_space(3))) char*)lds + wave * 1024u;
}

// Put the first k-tiles of an output tile in flight: A(0) B(0) A(1) B(1) into slots 0..3.  All five slots must be free
// (true at kernel start and after mainloop() returns).  Called before the epilogue of the previous output tile so that
// the copy path keeps working while the VALU does the epilogue.
template <bool BKM = false>
__device__ __forceinline__ void prefetch_first_tiles(const Operand& a, const Operand& b, int k_begin, int nk, char* lds) {
  CopyPlan p;  // rebuilt by mainloop(): keeping it in registers across an epilogue costs more than recomputing it
  make_plan<BKM>(p, a, b, k_begin);
  const uint32_t w0 = wave_copy_base(lds);
  copy_part(p.a_bytes, p.a_src, w0 + 0 * OPERAND_BYTES, 0, COPIES_PER_OPERAND);
  copy_part(p.b_bytes, p.b_src, w0 + 1 * OPERAND_BYTES, 0, COPIES_PER_OPERAND);
  if (nk > 1) {
    copy_part(p.a_bytes + BK * 2, p.a_src, w0 + 2 * OPERAND_BYTES, 0, COPIES_PER_OPERAND);
    copy_part(p.b_bytes + b_tile_stride<BKM>(b), p.b_src, w0 + 3 * OPERAND_BYTES, 0, COPIES_PER_OPERAND);
  }
}

// acc += A[a.row0 : +256, k_begin : k_begin + nk*64] * B[b.row0 : +256, same k]^T.
// prefetch_first_tiles() with the same arguments must have been issued by every wave before.  Every thread of the workgroup must call
// this with identical arguments (it contains barriers).  On return no copy is in flight, every wave has finished
// reading LDS, and all ring slots are free.
//
// Ring: A(t) sits in slot 2t mod 5, B(t) in slot (2t+1) mod 5.  While k-tile kt is consumed, A(kt+1) and B(kt+1) are
// ready or landing and A(kt+2) is being issued.  Per k-tile (two 32-k steps of 64 MFMAs):
//   step 0:      copies of A(kt+2) into the slot that held B(kt-1)          (freed by the barrier of iteration kt-1);
//                fragment reads of step 1
//   step 1:      barrier -- all fragment reads of tile kt have returned, this wave's copies of tile kt+1 have landed --
//                then B(kt+2) into the slot that held A(kt); fragment reads of step 0 of tile kt+1
//   every step:  the sixteen fragment reads of the next step ride behind every second MFMA of its first half (two
//                register sets), one copy behind every eighth MFMA, in a gap without a read; sched_barrier pins that order.
// MFMA order inside a step: mfma_row() / mfma_col() above (every fragment of the step is in registers before the step
// starts, so the order is free to serve the power budget).
template <bool BKM = false>
__device__ __forceinline__ void mainloop_ksteps(const Operand& a, const Operand& b, int k_begin, int nk, char* lds, acc_t& acc) {
  CopyPlan p;
  make_plan<BKM>(p, a, b, k_begin);
  const uint32_t b_stride = b_tile_stride<BKM>(b);
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int wm = wave / WAVES_N, wn = wave % WAVES_N;
  const int lrow = lane & 15;
  const int xsw = ((lane >> 4) ^ swz(lrow)) << 4;  // chunk offset of k-step 0; k-step 1 is xsw ^ 64
  // Per-lane fragment addresses inside a slot, for k-step 0 and 1 of the A and of the B operand.
  // The ring state below carries LDS addresses that already include this wave's copy offset (what the copies need, with
  // no further arithmetic); the per-lane fragment offsets are taken relative to it.
  const uint32_t w0 = wave_copy_base(lds);
  const int rel = -(wave * 1024);
  const int a_off0 = (wm * WM + lrow) * ROW_BYTES + xsw + rel, a_off1 = (wm * WM + lrow) * ROW_BYTES + (xsw ^ 64) + rel;
  const int b_off0 = (wn * WN + lrow) * ROW_BYTES + xsw + rel, b_off1 = (wn * WN + lrow) * ROW_BYTES + (xsw ^ 64) + rel;
  typedef const __attribute__((address_space(3))) bf16x8* frag_ptr;
  typedef __attribute__((address_space(3))) i16x4* half_ptr;

  // K-major B: a fragment (16 n x 32 k -> per lane one n, eight k) is two ds_read_b64_tr_b16, each of which takes four
  // consecutive k-rows at one pair of 16 n from sixteen lanes and hands lane l column l of each.  Lane l = (kq, s)
  // supplies the address of row kq*8 + half*4 + (s >> 2), n quarter s & 3.  The window key of those rows,
  // sigma = ((s >> 3) & 1) + 2 * (kq & 1), is a per-lane constant, so pair j of the wave is found at one of four
  // per-lane offsets (j & 3) ^ sigma plus immediates for j >> 2, the half and the k-step.
  constexpr int NB = BKM ? 4 : 1;  // B fragment address registers per k-step
  int kb_off[4];
  {
    const int kq = lane >> 4, s = lane & 15, r = s >> 2;
    const int sigma = ((r >> 1) & 1) + 2 * (kq & 1);
    const int base = (kq * 4 + (r >> 1)) * 1024 + wn * (WN / 16) * 64 + (r & 1) * 32 + (s & 3) * 8 + rel;
#pragma unroll
    for (int e = 0; e < 4; ++e) kb_off[e] = base + ((e ^ sigma) * 64);
  }
  constexpr int kKStepBytes = 16 * 1024;  // 32 k-rows of a K-major slot
  constexpr int kHalfBytes = 2 * 1024;    // 4 k-rows

  // Fragment registers.  A K-major B fragment arrives as two 64-bit halves (k 0-3 and k 4-7 of the lane's eight).
  bf16x8 af[2][TM], bfr[2][BKM ? 1 : TN];
  i16x4 bh[2][BKM ? TN : 1][2];
  auto b_frag = [&](int set, int j) -> bf16x8 {
    if constexpr (BKM) {
      typedef __attribute__((ext_vector_type(8))) short i16x8;
      const i16x8 v = __builtin_shufflevector(bh[set][j][0], bh[set][j][1], 0, 1, 2, 3, 4, 5, 6, 7);
      return __builtin_bit_cast(bf16x8, v);
    } else {
      return bfr[set][j];
    }
  };
  // Read instruction y of a 32-k step: y < TM is the A fragment of MFMA row y; then the B fragments, one instruction each
  // (K-contiguous B) or two (K-major B).  pa: LDS address of A fragment 0; pb: NB LDS addresses for B.
  constexpr int READS_PER_STEP = TM + (BKM ? 2 * TN : TN);
  auto read_one = [&](uint32_t pa, const uint32_t (&pb)[NB], int set, int y) {
    if (y < TM) {
      af[set][y] = *(frag_ptr)(uintptr_t)(pa + y * MT * ROW_BYTES);
    } else if constexpr (BKM) {
      const int j = (y - TM) >> 1, half = (y - TM) & 1;
      const uint32_t addr = pb[j & 3] + (j >> 2) * 256 + half * kHalfBytes + (set == 1 ? kKStepBytes : 0);
      bh[set][j][half] = __builtin_amdgcn_ds_read_tr16_b64_v4i16((half_ptr)(uintptr_t)addr);
    } else {
      bfr[set][y - TM] = *(frag_ptr)(uintptr_t)(pb[0] + (y - TM) * MT * ROW_BYTES);
    }
  };
  // Lane offsets of the B fragment addresses for k-step 0 / k-step 1 of a slot (the k-step of a K-major slot is an
  // immediate in read_one, so both are the same four offsets there).
  int boff0[NB], boff1[NB];
#pragma unroll
  for (int e = 0; e < NB; ++e) {
    boff0[e] = BKM ? kb_off[e] : b_off0;
    boff1[e] = BKM ? kb_off[e] : b_off1;
  }

  if (nk > 1) wait_copies_and_barrier<2 * COPIES_PER_OPERAND>(); else wait_copies_and_barrier<0>();  // tile 0 has landed
  {
    uint32_t pb[NB];
#pragma unroll
    for (int e = 0; e < NB; ++e) pb[e] = w0 + OPERAND_BYTES + boff0[e];
#pragma unroll
    for (int y = 0; y < READS_PER_STEP; ++y) read_one(w0 + a_off0, pb, 0, y);
  }

  // Ring state, as byte offsets of the slots in the order A(kt), B(kt), A(kt+1), B(kt+1), free.  Advancing one k-tile
  // rotates the five values by two places, so no arithmetic is needed; the fragment addresses of the next k-tile are
  // formed in the shadow of MFMAs in the middle of a step, not at the top of the loop where nothing would hide them.
  uint32_t o0 = w0, o1 = w0 + OPERAND_BYTES, o2 = w0 + 2 * OPERAND_BYTES, o3 = w0 + 3 * OPERAND_BYTES, o4 = w0 + 4 * OPERAND_BYTES;
  uint32_t ra1 = o0 + a_off1, ra0 = o2 + a_off0;  // step-0 reads: k-step 1 of this k-tile; step-1 reads: k-step 0 of the next
  uint32_t rb1[NB], rb0[NB];
#pragma unroll
  for (int e = 0; e < NB; ++e) rb1[e] = o1 + boff1[e], rb0[e] = o3 + boff0[e];
  // An add the compiler cannot move: it would otherwise collect these at the top of the loop body.
  auto pinned_add = [](uint32_t slot_off, int lane_off) {
    uint32_t r;
    asm volatile("v_add_u32_e32 %0, %1, %2" : "=v"(r) : "s"(slot_off), "v"(lane_off));
    return r;
  };
  // Source addresses of the k-tile being copied (two ahead of the one being consumed).  They advance in an MFMA shadow
  // right behind the last copy that uses them -- the empty asm keeps the compiler from gathering the increments at the
  // end of the loop body, where every instruction is a bubble.
  const char* ga = p.a_bytes + 2 * (BK * 2);
  const char* gb = p.b_bytes + 2 * (size_t)b_stride;
  // Three copies of the tile step (steady state, second-to-last, last) instead of conditions inside one loop body: a
  // branch that joins a path with outstanding LDS reads makes the compiler wait for all of them.
  auto tile_step = [&](auto has_next, auto load2) {
    // The fragment addresses of the next k-tile are formed in place, one add per MFMA shadow, in gaps behind the last
    // read of the step (which still uses the old value) that carry neither a read nor a copy.
    constexpr int kAddX0 = BKM ? 2 * READS_PER_STEP - 1 : 41;
    constexpr int kGapA = free_gap(kAddX0, 0);
    constexpr int kGapB[4] = {free_gap(kAddX0, 1), free_gap(kAddX0, 2), free_gap(kAddX0, 3), free_gap(kAddX0, 4)};
    static_assert(kGapB[3] < TM * TN, "address adds must fit the step");
#pragma unroll
    for (int ks = 0; ks < KSTEPS; ++ks) {
      if (ks == 1 && has_next) {
        if (load2) wait_copies_and_barrier<COPIES_PER_OPERAND>();  // A(kt+2) may still be in flight
        else wait_copies_and_barrier<0>();
      }
#pragma unroll
      for (int x = 0; x < TM * TN; ++x) {
        const int i = mfma_row(x), j = mfma_col(x);
        mfma_16x16x32(acc[i][j], af[ks][i], b_frag(ks, j));
        __builtin_amdgcn_sched_barrier(0);
        if (x % 2 == 0 && x < 2 * READS_PER_STEP) {
          if (ks == 0) read_one(ra1, rb1, 1, x / 2);
          else if (has_next) read_one(ra0, rb0, 0, x / 2);
        }
        if (load2 && x % 8 == 5) {  // an MFMA gap that carries no fragment read
          if (ks == 0) copy_part(ga, p.a_src, o4, x / 8, 1);
          else copy_part(gb, p.b_src, o0, x / 8, 1);
        }
        if (load2 && x == 62) {
          if (ks == 0) {
            ga += BK * 2;
            asm volatile("" : "+s"(ga));
          } else {
            gb += b_stride;
            asm volatile("" : "+s"(gb));
          }
        }
        if (has_next) {  // next k-tile's fragment addresses, one per MFMA shadow, after this step's reads are issued
          if (ks == 0 && x == kGapA) ra1 = pinned_add(o2, a_off1);
          if (ks == 1 && x == kGapA) ra0 = pinned_add(o4, a_off0);
#pragma unroll
          for (int e = 0; e < NB; ++e) {
            if (ks == 0 && x == kGapB[e]) rb1[e] = pinned_add(o3, boff1[e]);
            if (ks == 1 && x == kGapB[e]) rb0[e] = pinned_add(o0, boff0[e]);
          }
        }
        __builtin_amdgcn_sched_barrier(0);
      }
    }
    const uint32_t t0 = o0, t1 = o1;
    o0 = o2, o1 = o3, o2 = o4, o3 = t0, o4 = t1;
  };
  std::true_type yes;
  std::false_type no;
  int kt = 0;
  for (; kt + 2 < nk; ++kt) tile_step(yes, yes);
  if (kt + 1 < nk) tile_step(yes, no);
  tile_step(no, no);
  wait_copies_and_barrier<0>();
  // The hardware does not interlock an accumulator read (v_accvgpr_read) against an MFMA still in flight, and the
  // compiler does not know that the inline assembly is one: left alone it copies an accumulator to a VGPR right
  // behind the MFMA that wrote it last and gets the old value.  So: 32 wait states behind the last MFMA, then every
  // accumulator passes through an empty volatile asm -- a new value as far as the compiler can tell, so whatever
  // reads it is placed after this point.
  asm volatile("s_nop 15\n\ts_nop 15" ::: "memory");
#pragma unroll
  for (int i = 0; i < TM; ++i)
#pragma unroll
    for (int j = 0; j < TN; ++j) asm volatile("" : "+a"(acc[i][j]));
}

// ---- accumulator-stationary pairs -------------------------------------------------------------------------------------
// The same contraction with the MFMAs of a k-tile reordered so that the two k-steps of an accumulator are issued back to
// back.  With random operands the matrix pipe is power-limited, and an MFMA that accumulates into the register the previous
// one wrote costs less than one that switches accumulators: a loop of nothing but MFMAs runs 4 % faster in this order, the
// kernels 2-2.5 %.  Every accumulator still receives its products in the same order (k-tile by k-tile, k-step 0 then 1), so
// results are bit-identical to mainloop_ksteps().
//
// Both k-steps of an accumulator's operands must then be in registers at once.  With the same 128 fragment registers this
// works quadrant by quadrant: the wave's 8 x 8 accumulators are four 4 x 4 quadrants; a quadrant needs one "half-set" of A
// (4 row blocks x 2 k-steps = 8 fragments) and one of B.  There are two A slots and two B slots of 8 fragments each.  A
// k-tile walks its quadrants in a U -- (A0,B0) (A0,B1) (A1,B1) (A1,B0) -- changing one operand per step, and each quadrant
// loads the one half-set the next step needs into the slot that just died: 8 fragment reads per 32 MFMAs, 32 per k-tile, as
// before.  The last quadrant of a tile still holds one A and one B slot, so the next tile starts from the other two and
// walks the U backwards -- (A1,B0) (A1,B1) (A0,B1) (A0,B0) -- after which the first pattern fits again: tiles alternate
// between two schedules ("even" / "odd"), fixed at compile time in kQuadPlan.  The ring of LDS slots, the copies (one
// behind every eighth MFMA) and the single barrier per k-tile (now between the second and third quadrant: the first half of
// a tile reads the rest of its own LDS slots, the second half the first half-sets of the next tile's) are those of
// mainloop_ksteps().
//
// nk must be even and >= 2: with one fixed sequence of tile bodies (steady-state pair, then even, then odd) the
// accumulators pass through no join of different bodies; any remainder handling by branches made the register allocator
// move accumulators between AGPRs and VGPRs right behind the MFMAs that wrote them.  Callers pick mainloop_ksteps() for an
// odd number of k-tiles.
// Order of the 16 accumulators of a 4 x 4 quadrant: a zigzag inside strips of two rows.
__host__ __device__ constexpr int quad_row(int p) { return (p / 8) * 2 + ((p % 8 + 1) / 2) % 2; }
__host__ __device__ constexpr int quad_col(int p) { return (p / 8) % 2 ? 3 - (p % 8) / 2 : (p % 8) / 2; }

// One quadrant of a k-tile: which halves of the wave's A rows / B columns it multiplies, the fragment slots that hold them,
// and the half-set it loads meanwhile (operand, half, of this k-tile or the next, destination slot).
struct QuadPlan {
  int a_half, b_half, a_slot, b_slot;
  int ld_is_b, ld_half, ld_next, ld_slot;
};
constexpr QuadPlan kQuadPlan[2][4] = {
    {{0, 0, 0, 0, 1, 1, 0, 1}, {0, 1, 0, 1, 0, 1, 0, 1}, {1, 1, 1, 1, 0, 1, 1, 0}, {1, 0, 1, 0, 1, 0, 1, 1}},
    {{1, 0, 0, 1, 1, 1, 0, 0}, {1, 1, 0, 0, 0, 0, 0, 1}, {0, 1, 1, 0, 0, 0, 1, 0}, {0, 0, 1, 1, 1, 0, 1, 0}}};

template <bool BKM = false>
__device__ __forceinline__ void mainloop_pairs(const Operand& a, const Operand& b, int k_begin, int nk, char* lds, acc_t& acc) {
  CopyPlan p;
  make_plan<BKM>(p, a, b, k_begin);
  const uint32_t b_stride = b_tile_stride<BKM>(b);
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int wm = wave / WAVES_N, wn = wave % WAVES_N;
  const int lrow = lane & 15;
  const int xsw = ((lane >> 4) ^ swz(lrow)) << 4;
  const uint32_t w0 = wave_copy_base(lds);
  const int rel = -(wave * 1024);
  typedef const __attribute__((address_space(3))) bf16x8* frag_ptr;
  typedef __attribute__((address_space(3))) i16x4* half_ptr;
  constexpr int NB = BKM ? 4 : 2;  // B address registers per k-tile
  // Lane offsets inside a slot: A (and K-contiguous B) per k-step; K-major B per column of a half (see mainloop_ksteps).
  int a_off[2], b_off[NB];
  a_off[0] = (wm * WM + lrow) * ROW_BYTES + xsw + rel;
  a_off[1] = (wm * WM + lrow) * ROW_BYTES + (xsw ^ 64) + rel;
  if constexpr (BKM) {
    const int kq = lane >> 4, s = lane & 15, r = s >> 2;
    const int sigma = ((r >> 1) & 1) + 2 * (kq & 1);
    const int base = (kq * 4 + (r >> 1)) * 1024 + wn * (WN / 16) * 64 + (r & 1) * 32 + (s & 3) * 8 + rel;
#pragma unroll
    for (int e = 0; e < 4; ++e) b_off[e] = base + ((e ^ sigma) * 64);
  } else {
    b_off[0] = (wn * WN + lrow) * ROW_BYTES + xsw + rel;
    b_off[1] = (wn * WN + lrow) * ROW_BYTES + (xsw ^ 64) + rel;
  }
  constexpr int kKStepBytes = 16 * 1024;
  constexpr int kHalfBytes = 2 * 1024;

  // Fragment slots: two for A half-sets, two for B half-sets; a half-set is 4 row blocks x 2 k-steps, index r * 2 + ks.
  bf16x8 sa[2][8], sb[2][BKM ? 1 : 8];
  i16x4 sbh[2][BKM ? 8 : 1][2];
  auto b_frag = [&](int slot, int f) -> bf16x8 {
    if constexpr (BKM) {
      typedef __attribute__((ext_vector_type(8))) short i16x8;
      const i16x8 v = __builtin_shufflevector(sbh[slot][f][0], sbh[slot][f][1], 0, 1, 2, 3, 4, 5, 6, 7);
      return __builtin_bit_cast(bf16x8, v);
    } else {
      return sb[slot][f];
    }
  };
  struct Addr {
    uint32_t a[2], b[NB];
  };
  constexpr int A_READS = 8, B_READS = BKM ? 16 : 8;
  // Read instruction y of a half-set load.
  auto read_a = [&](const Addr& ad, int half, int slot, int y) {
    const int r = y / 2, ks = y % 2;
    sa[slot][y] = *(frag_ptr)(uintptr_t)(ad.a[ks] + (half * 4 + r) * MT * ROW_BYTES);
  };
  auto read_b = [&](const Addr& ad, int half, int slot, int y) {
    if constexpr (BKM) {
      const int c = y / 4, ks = (y / 2) % 2, hf = y % 2;
      const uint32_t addr = ad.b[c] + half * 256 + hf * kHalfBytes + ks * kKStepBytes;
      sbh[slot][c * 2 + ks][hf] = __builtin_amdgcn_ds_read_tr16_b64_v4i16((half_ptr)(uintptr_t)addr);
    } else {
      const int r = y / 2, ks = y % 2;
      sb[slot][y] = *(frag_ptr)(uintptr_t)(ad.b[ks] + (half * 4 + r) * MT * ROW_BYTES);
    }
  };

  if (nk > 1) wait_copies_and_barrier<2 * COPIES_PER_OPERAND>(); else wait_copies_and_barrier<0>();  // tile 0 has landed
  uint32_t o0 = w0, o1 = w0 + OPERAND_BYTES, o2 = w0 + 2 * OPERAND_BYTES, o3 = w0 + 3 * OPERAND_BYTES, o4 = w0 + 4 * OPERAND_BYTES;
  Addr X, Y;
#pragma unroll
  for (int e = 0; e < 2; ++e) X.a[e] = Y.a[e] = o0 + a_off[e];
#pragma unroll
  for (int e = 0; e < NB; ++e) X.b[e] = Y.b[e] = o1 + b_off[e];
#pragma unroll
  for (int y = 0; y < A_READS; ++y) read_a(X, 0, 0, y);
#pragma unroll
  for (int y = 0; y < B_READS; ++y) read_b(X, 0, 0, y);

  auto pinned_add = [](uint32_t slot_off, int lane_off) {
    uint32_t r;
    asm volatile("v_add_u32_e32 %0, %1, %2" : "=v"(r) : "s"(slot_off), "v"(lane_off));
    return r;
  };
  const char* ga = p.a_bytes + 2 * (BK * 2);
  const char* gb = p.b_bytes + 2 * (size_t)b_stride;

  // One k-tile = four quadrants of 32 MFMAs.  cur: fragment addresses of this k-tile's slots, nxt: of the next k-tile's
  // (formed here, in MFMA shadows of the first half; they are this tile's second-half addresses and the next tile's cur).
  auto tile_step = [&](auto par, auto has_next, auto load2, Addr& cur, Addr& nxt) {
    constexpr int PAR = decltype(par)::value;
#pragma unroll
    for (int q = 0; q < 4; ++q) {
      constexpr QuadPlan const* plans = kQuadPlan[PAR];
      const QuadPlan pl = plans[q];
      if (q == 2 && has_next) {
        if (load2) wait_copies_and_barrier<COPIES_PER_OPERAND>();  // A(kt+2) may still be in flight
        else wait_copies_and_barrier<0>();
      }
      const bool do_load = q < 2 || has_next;
      const int nreads = pl.ld_is_b ? B_READS : A_READS;
#pragma unroll
      for (int pos = 0; pos < 32; ++pos) {
        const int pr = pos / 2, ks = pos % 2;
        const int r = quad_row(pr), c = quad_col(pr);
        mfma_16x16x32(acc[pl.a_half * 4 + r][pl.b_half * 4 + c], sa[pl.a_slot][r * 2 + ks], b_frag(pl.b_slot, c * 2 + ks));
        __builtin_amdgcn_sched_barrier(0);
        if (!(LMHEAD_ABLATE & 32) && do_load && pos % 2 == 0 && pos / 2 < nreads) {
          if (pl.ld_is_b) read_b(pl.ld_next ? nxt : cur, pl.ld_half, pl.ld_slot, pos / 2);
          else read_a(pl.ld_next ? nxt : cur, pl.ld_half, pl.ld_slot, pos / 2);
        }
        if (!(LMHEAD_ABLATE & 64) && load2 && pos % 8 == 5) {
          if (q < 2) copy_part(ga, p.a_src, o4, q * 4 + pos / 8, 1);
          else copy_part(gb, p.b_src, o0, (q - 2) * 4 + pos / 8, 1);
        }
        if (load2 && pos == 31 && q == 1) {
          ga += BK * 2;
          asm volatile("" : "+s"(ga));
        }
        if (load2 && pos == 31 && q == 3) {
          gb += b_stride;
          asm volatile("" : "+s"(gb));
        }
        if (has_next && q == 0) {  // next k-tile's fragment addresses, one add per MFMA shadow, in gaps without a read or a copy
          if (pos == 1) nxt.a[0] = pinned_add(o2, a_off[0]);
          if (pos == 3) nxt.a[1] = pinned_add(o2, a_off[1]);
          if (pos == 7) nxt.b[0] = pinned_add(o3, b_off[0]);
          if (pos == 9) nxt.b[1] = pinned_add(o3, b_off[1]);
          if (NB == 4 && pos == 11) nxt.b[NB - 2] = pinned_add(o3, b_off[NB - 2]);
          if (NB == 4 && pos == 15) nxt.b[NB - 1] = pinned_add(o3, b_off[NB - 1]);
        }
        __builtin_amdgcn_sched_barrier(0);
      }
    }
    const uint32_t t0 = o0, t1 = o1;
    o0 = o2, o1 = o3, o2 = o4, o3 = t0, o4 = t1;
  };
  std::integral_constant<int, 0> even;
  std::integral_constant<int, 1> odd;
  std::true_type yes;
  std::false_type no;
  // nk is even: tiles alternate even, odd and the sequence is a straight line.
  for (int kt = 0; kt + 3 < nk; kt += 2) {
    tile_step(even, yes, yes, X, Y);
    tile_step(odd, yes, yes, Y, X);
  }
  tile_step(even, yes, no, X, Y);
  tile_step(odd, no, no, Y, X);
  wait_copies_and_barrier<0>();
  asm volatile("s_nop 15\n\ts_nop 15" ::: "memory");
#pragma unroll
  for (int i = 0; i < TM; ++i)
#pragma unroll
    for (int j = 0; j < TN; ++j) asm volatile("" : "+a"(acc[i][j]));
}

// The mainloop of a tile: EVEN_NK (the caller guarantees an even number of k-tiles, at least two) takes the
// accumulator-stationary order, anything else the k-step order.  Both leave identical accumulators.
template <bool BKM = false, bool EVEN_NK = false>
__device__ __forceinline__ void mainloop(const Operand& a, const Operand& b, int k_begin, int nk, char* lds, acc_t& acc) {
  if constexpr (EVEN_NK) mainloop_pairs<BKM>(a, b, k_begin, nk, lds, acc);
  else mainloop_ksteps<BKM>(a, b, k_begin, nk, lds, acc);
}

// Work item id -> tile coordinates.
//  1. Hardware hands consecutive workgroup ids to the 8 XCDs round-robin; undo that so each XCD (own L2) owns a
//     contiguous range of the logical order.  (Persistent workgroups walk ids bid, bid + grid, ...: with a grid that is
//     a multiple of 8 a workgroup's ids keep the XCD of its first one.)
//  2. Walk the logical order in bands of `group_m` tiles along M, N-major inside a band, so the ~32 workgroups
//     concurrently resident on one XCD cover a compact group_m x (32/group_m) patch and share operand panels in that
//     XCD's L2.
__device__ __forceinline__ void tile_coords(int id, int tiles_m, int tiles_n, int group_m, int& tm, int& tn) {
  const int total = tiles_m * tiles_n;
  const int per_xcd = total >> 3;
  int logical = id;
  if (id < (per_xcd << 3)) logical = (id & 7) * per_xcd + (id >> 3);
  const int band_sz = group_m * tiles_n;
  const int band = logical / band_sz;
  const int in_band = logical - band * band_sz;
  const int m_first = band * group_m;
  int gm = tiles_m - m_first;
  gm = gm < group_m ? gm : group_m;
  tn = in_band / gm;
  tm = m_first + (in_band - tn * gm);
}

// Sum / maximum over the four lanes (l, l^16, l^32, l^48) that hold the same accumulator column, result in all four.
// v_permlane16_swap exchanges the odd 16-lane rows of its first operand with the even rows of its second, and
// v_permlane32_swap the upper half of the first with the lower half of the second: fed the same value twice, the two
// results hold the two partners' values side by side in every lane.  Plain VALU operations -- the ds_bpermute form costs
// an LDS round trip per step, and the statistics epilogue has six of these chains per 16 tokens.
__device__ __forceinline__ void swap16(float v, float& a, float& b) {
  const auto r = __builtin_amdgcn_permlane16_swap(__float_as_uint(v), __float_as_uint(v), false, false);
  a = __uint_as_float(r[0]), b = __uint_as_float(r[1]);
}
__device__ __forceinline__ void swap32(float v, float& a, float& b) {
  const auto r = __builtin_amdgcn_permlane32_swap(__float_as_uint(v), __float_as_uint(v), false, false);
  a = __uint_as_float(r[0]), b = __uint_as_float(r[1]);
}
__device__ __forceinline__ float col_sum(float v) {
  float a, b;
  swap16(v, a, b);
  swap32(a + b, a, b);
  return a + b;
}
__device__ __forceinline__ float col_max(float v) {
  float a, b;
  swap16(v, a, b);
  swap32(fmaxf(a, b), a, b);
  return fmaxf(a, b);
}

}  // namespace lmhead
