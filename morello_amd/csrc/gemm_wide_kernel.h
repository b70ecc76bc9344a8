// The 256 x 256 Matmul tile on four waves, one per SIMD, each holding a 128 x 128 block of C in
// 256 accumulation registers: u8|i8 x i8 -> i32 and bf16 x bf16 -> f32 on whole tiles with a long
// K.  k loop and epilogue are written in assembly (gemm_wide_gfx950.inc, generated and
// documented by gen_gemm_wide.py, which also says why this shape -- the fewest instructions per
// MFMA cycle -- and why MFMAs of 16 x 16 x 64 bytes: the least energy per multiply-add on a
// power-limited board).
//
// Same arithmetic as k_gemm (gemm_mfma_kernel.h; semantics: morello/src/spec.rs:480-485,
// morello/src/codegen/cpu.rs:2114-2124).  For an accumulating Spec the old value of an element
// joins its sum during the first k steps instead of after the last; integers are exact either
// way, floats differ from k_gemm's order by one rounding.
//   move_param(A, L1)  -> global_load_dwordx4 -> (xor 0x80 for u8) -> ds_write_b128, two stages
//   move_param(B, L1)  -> global_load_lds_dwordx4 into a ring of three 32 KiB slots
// The A tile is stored as k_gemm stores it (rows of 128 bytes, 16-byte chunks XOR-ed with
// (row / 2) & 7).  The B tile is stored [k][n] without row padding.  One half of a transposing
// read (32 lanes) touches 8 (i8) / 4 (bf16) k rows of two lane groups, 16 k (8 k) apart, at the
// same 16 (32) bytes of the row: the pieces of a row (32 bytes for i8, 64 for bf16) are XOR-ed
// with the low bits of the row number and the halves of a piece with the row bit that tells the
// two lane groups apart, so that these rows fall on different banks.  A direct-to-LDS instruction
// writes 1 KiB of consecutive LDS bytes, 16 per lane, so the swizzle is applied on the source side.
#pragma once
#include "gemm_mfma_kernel.h"
#include "gemm_wide_gfx950.inc"

namespace mrl {
namespace gemm {

template <class T> struct WideTraits;
// PIECE, RMASK: see above; GROUP_SHIFT: log2 of the k rows one lane group of an MFMA operand holds.
template <> struct WideTraits<I8> { static constexpr int PIECE = 32, RMASK = 7, GROUP_SHIFT = 4; };
template <> struct WideTraits<BF16> { static constexpr int PIECE = 64, RMASK = 3, GROUP_SHIFT = 3; };

// Byte position within a k row of the B tile in LDS <-> within the row in memory (an involution).
template <class T>
__device__ inline int wide_b_swizzle(int byte, int k) {
  constexpr int PIECE = WideTraits<T>::PIECE, HALF = PIECE / 2;
  const int piece = (byte / PIECE) ^ (k & WideTraits<T>::RMASK);
  const int half = ((byte % PIECE) / HALF) ^ ((k >> WideTraits<T>::GROUP_SHIFT) & 1);
  return piece * PIECE + half * HALF + byte % HALF;
}

constexpr int WIDE_B_BASE = 2 * 32768;       // LDS: [A stage 0][A stage 1][B slot 0][B slot 1][B slot 2]
constexpr int WIDE_LDS_BYTES = 5 * 32768;
constexpr int WIDE_MIN_STEPS = GEMM_WIDE_MIN_STEPS;

#define MRL_WIDE_10(p, b) p #b "0", p #b "1", p #b "2", p #b "3", p #b "4", p #b "5", p #b "6", p #b "7", p #b "8", p #b "9"
#define MRL_WIDE_100(p, h)                                                                                   \
  MRL_WIDE_10(p, h##0), MRL_WIDE_10(p, h##1), MRL_WIDE_10(p, h##2), MRL_WIDE_10(p, h##3), MRL_WIDE_10(p, h##4), \
      MRL_WIDE_10(p, h##5), MRL_WIDE_10(p, h##6), MRL_WIDE_10(p, h##7), MRL_WIDE_10(p, h##8), MRL_WIDE_10(p, h##9)
#define MRL_WIDE_FIRST_100(p)                                                                              \
  p "0", p "1", p "2", p "3", p "4", p "5", p "6", p "7", p "8", p "9", MRL_WIDE_10(p, 1), MRL_WIDE_10(p, 2), \
      MRL_WIDE_10(p, 3), MRL_WIDE_10(p, 4), MRL_WIDE_10(p, 5), MRL_WIDE_10(p, 6), MRL_WIDE_10(p, 7),        \
      MRL_WIDE_10(p, 8), MRL_WIDE_10(p, 9)
#define MRL_WIDE_CLOBBERS                                                                                   \
  MRL_WIDE_FIRST_100("v"), MRL_WIDE_100("v", 1), MRL_WIDE_10("v", 20), "v210", "v211",                      \
      MRL_WIDE_FIRST_100("a"), MRL_WIDE_100("a", 1), MRL_WIDE_10("a", 20), MRL_WIDE_10("a", 21),            \
      MRL_WIDE_10("a", 22), MRL_WIDE_10("a", 23), MRL_WIDE_10("a", 24), "a250", "a251", "a252", "a253",     \
      "a254", "a255", "s60", "s61", "s62", "s63", "s64", "s65", "s66", "s67", "s68", "s69", "s70", "s71",   \
      "s72", "s73", "s74", "s75", "s78", "s79", "s80", "s81", "s82", "s83", "s84", "s85", "s86", "s87", "s88", "s89", "s90",     \
      "s91", "s92", "s93", "s94", "s95", "scc", "memory"

#define MRL_WIDE_RUN(TEXT)                                                                                         \
  asm volatile(TEXT                                                                                                \
               :                                                                                                   \
               : [a_off0] "v"(a_off[0]), [a_off1] "v"(a_off[1]), [a_off2] "v"(a_off[2]), [a_off3] "v"(a_off[3]),   \
                 [a_off4] "v"(a_off[4]), [a_off5] "v"(a_off[5]), [a_off6] "v"(a_off[6]), [a_off7] "v"(a_off[7]),   \
                 [b_off0] "v"(b_off[0]), [b_off1] "v"(b_off[1]), [b_off2] "v"(b_off[2]), [b_off3] "v"(b_off[3]),   \
                 [b_off4] "v"(b_off[4]), [b_off5] "v"(b_off[5]), [b_off6] "v"(b_off[6]), [b_off7] "v"(b_off[7]),   \
                 [a_wr] "v"(a_wr), [a_rd0] "v"(a_rd[0]), [a_rd1] "v"(a_rd[1]), [b_rd0] "v"(b_rd[0]),               \
                 [b_rd1] "v"(b_rd[1]), [b_rd2] "v"(b_rd[2]), [b_rd3] "v"(b_rd[3]), [b_rd4] "v"(b_rd[4]),           \
                 [b_rd5] "v"(b_rd[5]), [b_rd6] "v"(b_rd[6]), [b_rd7] "v"(b_rd[7]), [c_lo0] "v"(c_lo[0]),           \
                 [c_lo1] "v"(c_lo[1]), [c_lo2] "v"(c_lo[2]), [c_lo3] "v"(c_lo[3]), [c_hi0] "v"(c_hi[0]),           \
                 [c_hi1] "v"(c_hi[1]), [c_hi2] "v"(c_hi[2]), [c_hi3] "v"(c_hi[3]), [part_wr] "v"(part_wr),         \
                 [part_rd_lo] "v"(part_rd_lo), [part_rd_hi] "v"(part_rd_hi), [abase] "s"(A), [bbase] "s"(B),       \
                 [bstep] "s"(b_step), [nk] "s"(nk), [dma_base] "s"(dma_base), [cbase] "s"(c_base),                 \
                 [ldc16] "s"(ldc16), [k32] "s"(k32)                                                                \
               : MRL_WIDE_CLOBBERS)

// M, N multiples of 256; K an even number of k steps: GEMM_WIDE_MIN_STEPS at least for an accumulating
// Spec (whose first eight steps carry the loads of C's old values), four otherwise; see wide_applicable().
template <class T, bool A_UNSIGNED>
__global__ __launch_bounds__(256) void k_gemm_wide(MRL_WALK_PARAMS, GemmArgs g) {
  extern __shared__ __attribute__((aligned(16))) uint8_t lds[];
  constexpr int BM = 256, BN = 256, BKB = 128, WM = 128, WN = 128, TN = 8;
  constexpr int ES = T::ES, BK = BKB / ES;
  constexpr int B_ROWB = BN * ES;              // bytes per k row of the B tile
  constexpr int ROWS_PER_DMA = 1024 / B_ROWB;  // k rows one direct-to-LDS instruction fills: 4 (i8), 2 (bf16)
  constexpr int GROUP_K = 16 / ES;             // k rows a lane group of an MFMA operand holds: 16 (i8), 8 (bf16)
  typedef typename T::Out Out;

  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wm = wave >> 1, wn = wave & 1;
  // The four waves run one instruction stream (a second one costs instruction-cache misses all
  // through the unrolled steps: 340 cycles a step measured).  What differs between the wave rows
  // is in registers: for a u8 operand the lower wave row numbers its eight block columns from the
  // fifth on (rot = 4), so that "add up the column sums of block columns 0 .. 3" covers columns
  // 64 .. 127 of the wave's 128 there and columns 0 .. 63 in the upper wave row.
  const int rot = (A_UNSIGNED && wm == 1) ? TN / 2 : 0;

  // Workgroups go to the 8 XCDs round-robin; each XCD gets a contiguous run of tiles which, taken
  // group_m tile rows at a time, covers a compact block of C (its A rows and B columns stay in
  // that XCD's L2).
  MRL_WALK_TILE(tile_m, tile_n)
  const int64_t m0 = int64_t(tile_m) * BM, n0 = int64_t(tile_n) * BN;

#ifdef MRL_WIDE_SAME_PANELS  // energy experiment: every workgroup fetches the first tile's operands (L2 hits)
  const uint8_t *A = (const uint8_t *)g.a + (int64_t(blockIdx.y) * g.sa) * ES;
  const uint8_t *B = (const uint8_t *)g.b + (int64_t(blockIdx.y) * g.sb) * ES;
#else
  const uint8_t *A = (const uint8_t *)g.a + (int64_t(blockIdx.y) * g.sa + m0 * g.lda) * ES;
  const uint8_t *B = (const uint8_t *)g.b + (int64_t(blockIdx.y) * g.sb + n0) * ES;
#endif
  Out *C = (Out *)g.c + int64_t(blockIdx.y) * g.sc + m0 * g.ldc + n0;
  const uint32_t lda_b = uint32_t(g.lda) * ES, ldb_b = uint32_t(g.ldb) * ES, ldc_b = uint32_t(g.ldc) * 4;
  const uint32_t lds0 = uint32_t(uintptr_t(lds));

  // A staging: thread `tid` moves 16-byte chunk tid + i * 256 of a tile (rows 32 apart); chunks of
  // a row are XOR-ed with (row / 2) & 7 in LDS, as in k_gemm.
  uint32_t a_off[8], a_wr;
  {
    const int row = tid / 8, ch = tid % 8;
#pragma unroll
    for (int i = 0; i < 8; i++) a_off[i] = uint32_t(row + i * 32) * lda_b + ch * 16;
    a_wr = lds0 + row * BKB + ((ch ^ ((row / 2) & 7)) << 4);
  }
  // B staging: instruction j of this wave fills LDS bytes [(8 * wave + j) * 1024, +1024) of the slot,
  // lane L the 16 bytes at 16 * L of them.  The instruction's immediate offset j * 1024 - 4096 is
  // added to the LDS address and to the global one alike, so it is taken off the latter here.
  uint32_t b_off[8];
#pragma unroll
  for (int j = 0; j < 8; j++) {
    const int r = (wave * 8 + j) * ROWS_PER_DMA + (lane * 16) / B_ROWB;
    b_off[j] = uint32_t(r) * ldb_b + wide_b_swizzle<T>((lane * 16) % B_ROWB, r) + 4096 - j * 1024;
  }
  const uint32_t dma_base = lds0 + WIDE_B_BASE + wave * 8192;
  // Operand reads.  A: lane (l % 16, l / 16) of block row tm reads 16 bytes of row
  // wm * 128 + tm * 16 + l % 16 at chunk 4 * s + l / 16 of the 64-byte slab s.
  uint32_t a_rd[2];
  {
    const int sw = ((lane & 15) / 2) & 7, group = lane >> 4;
#pragma unroll
    for (int s = 0; s < 2; s++) a_rd[s] = lds0 + (wm * WM + (lane & 15)) * BKB + (((4 * s + group) ^ sw) << 4);
  }
  // B: a 16-lane group of a transposing read fetches 8 (i8) / 4 (bf16) k rows x 16 columns; lane p
  // of the group addresses 8 bytes of one k row and receives the column it indexes.  Group g reads
  // the k rows GROUP_K * g on of the slab (a second read takes the other half of them) for the
  // 16 columns of block column tn.
  uint32_t b_rd[TN];
  {
    constexpr int LANES_PER_ROW = 16 / (8 / ES);
    const int p = lane & 15;
    const int k = GROUP_K * (lane >> 4) + p / LANES_PER_ROW;
#pragma unroll
    for (int t = 0; t < TN; t++) {
      const int tn = (t + rot) % TN;
      const int byte = (wn * WN + tn * 16 + (8 / ES) * (p % LANES_PER_ROW)) * ES;
      b_rd[t] = lds0 + WIDE_B_BASE + k * B_ROWB + wide_b_swizzle<T>(byte, k);
    }
  }
  // C: register i of a 16 x 16 block holds row 4 * (l / 16) + i, column l % 16.  The loop addresses
  // block column t as c_lo (t < 4) or c_hi (t >= 4) plus t * 64 bytes: with the columns rotated by
  // four blocks the base pointer sits four blocks to the left and c_lo makes up for eight.
  uint32_t c_lo[4], c_hi[4];
#pragma unroll
  for (int i = 0; i < 4; i++) {
    c_hi[i] = uint32_t((lane >> 4) * 4 + i) * ldc_b + (lane & 15) * 4;
    c_lo[i] = c_hi[i] + (rot ? 512 : 0);
  }
  const uint8_t *c_base = (const uint8_t *)(C + int64_t(wm * WM) * g.ldc + wn * WN) - (rot ? 256 : 0);
  const uint32_t ldc16 = 16 * ldc_b;
  // Column-sum partials [lane group][256 columns] of 4 bytes, 1 KiB into LDS once the loop is over:
  // a wave writes those of its block columns 0 .. 3 and reads all eight (rotated like C's).
  const uint32_t part = lds0 + 1024 + (wn * WN + (lane & 15)) * 4;
  const uint32_t part_wr = part + (lane >> 4) * (BN * 4) + (rot ? 256 : 0);
  const uint32_t part_rd_lo = part + (rot ? 256 : 0), part_rd_hi = part - (rot ? 256 : 0);

  const uint32_t b_step = uint32_t(BK) * ldb_b;
  const uint32_t nk = g.k / BK, k32 = 32 * g.k;

  // An accumulating Spec loads C's old values in nine of its first steps and adds them to the
  // accumulators a step later: one step after the other when K is short, with two or eleven steps
  // of the loop between them when K has room.  Those loads sit in the same in-order queue as the
  // operands', which wait behind them for HBM's latency: a step that carries them takes 2200
  // cycles longer (bf16 8192^3, cycle stamps), and close together they also ask HBM for all it
  // delivers (int8 4096^3: 64 MiB of C in the first quarter of the launch).
  const int spacing = !g.accum ? -1 : nk >= GEMM_WIDE_G11_MIN_STEPS ? 11 : nk >= GEMM_WIDE_G2_MIN_STEPS ? 2 : 0;
#define MRL_WIDE_PICK(KIND)                                           \
  do {                                                                \
    if (spacing < 0) MRL_WIDE_RUN(GEMM_WIDE_##KIND);                  \
    else if (spacing == 11) MRL_WIDE_RUN(GEMM_WIDE_##KIND##_ACC_G11); \
    else if (spacing == 2) MRL_WIDE_RUN(GEMM_WIDE_##KIND##_ACC_G2);   \
    else MRL_WIDE_RUN(GEMM_WIDE_##KIND##_ACC);                        \
  } while (0)
  if constexpr (std::is_same<T, BF16>::value) MRL_WIDE_PICK(BF16);
  else if constexpr (!A_UNSIGNED) MRL_WIDE_PICK(I8);
  else MRL_WIDE_PICK(U8);
#undef MRL_WIDE_PICK
}

// Whole tiles, an even number of k steps, offsets the loop's 32-bit arithmetic can hold.  An
// accumulating Spec needs the steps that carry C's old values (GEMM_WIDE_MIN_STEPS); another one
// may be as short as four steps.  Below twenty steps the kernel is taken when its tiles run in one
// round (measured against the eight-wave tile, non-accumulating: int8 4096 x 512 x 4096 19.5 against
// 21.3 us, 3072 x 2048 x 3072 27.3 / 31.0, bf16 4096 x 1024 x 4096 34.6 / 38.4; but 8192 x 768 x 8192,
// four rounds of tiles bound by the write of C, 99.0 / 94.3: this kernel's stores are 64-byte row
// segments).
constexpr int WIDE_LONG_K_STEPS = 20;
inline bool wide_applicable(const GemmArgs &g, int elem_size) {
  const int64_t bk = 128 / elem_size;
  const bool long_k = g.k >= WIDE_LONG_K_STEPS * bk;
  const bool one_round = uint64_t(g.m / 256) * (g.n / 256) * g.batch <= g_compute_units;
  return !g.b_kmajor && g.m % 256 == 0 && g.n % 256 == 0 && g.k % (2 * bk) == 0 &&
         (long_k || (one_round && g.k >= (g.accum ? WIDE_MIN_STEPS : 4) * bk)) &&
         g.lda * elem_size * 256 < (int64_t(1) << 32) && g.ldb * elem_size * (bk + 1) < (int64_t(1) << 31) &&
         g.ldc * 4 * 32 < (int64_t(1) << 31);
}

template <class T, bool A_UNSIGNED>
hipError_t launch_wide(const GemmArgs &g, hipStream_t stream) {
  constexpr auto kern = k_gemm_wide<T, A_UNSIGNED>;
  static std::atomic<uint64_t> lds_limit_set{0};
  if (!plan::recording()) {
    hipError_t e = raise_lds_limit(lds_limit_set, (const void *)kern, WIDE_LDS_BYTES);
    if (e != hipSuccess) return e;
  }
  const int tiles_m = int(g.m / 256), tiles_n = int(g.n / 256);
  const double mn = double(g.m) * g.n * g.batch;
  plan::work(T::ES == 1 ? plan::UNIT_MFMA_I8 : plan::UNIT_MFMA_BF16, 2.0 * mn * g.k,
             (double(g.m) * g.k + double(g.k) * g.n) * g.batch * T::ES + mn * 4 * (g.accum ? 2 : 1),
             2.0 * 256 * 256 * double(g.k), 500.0 + 1200.0 * double(g.k * T::ES / 128),
             T::ES == 1 ? 1.62 : 1.18);  // measured: 2230-2330 TOPS int8 at 4096^3, 1360 TFLOPS bf16 at 8192^3
  const TileWalk walk = tile_walk(tiles_m, tiles_n);
  MRL_LAUNCH((k_gemm_wide<T, A_UNSIGNED>), dim3(tiles_m * tiles_n, g.batch), dim3(256), WIDE_LDS_BYTES, stream,
             MRL_WALK_ARGS(walk), g);
  return mrl::plan::last_error();
}

}  // namespace gemm
}  // namespace mrl
