// The 256 x 256 Matmul tile with its k loop written in assembly (gemm_loop_gfx950.inc, generated
// and documented by gen_gemm_loop.py): u8|i8 x i8 -> i32 and bf16 x bf16 -> f32 on whole tiles.
//
// Same arithmetic, tile shape, LDS operand layouts and epilogue as k_gemm (gemm_mfma_kernel.h;
// semantics: morello/src/spec.rs:480-485, morello/src/codegen/cpu.rs:2114-2124).  What differs is
// how operands travel: B goes from global memory straight into one of three LDS slots
// (direct-to-LDS loads, two k steps ahead), A through two register sets into two LDS stages
// (also two k steps ahead), and the instruction order of the k loop is fixed by hand.
//   move_param(B, L1)  -> global_load_lds_dwordx4 into a ring of three 32 KiB slots
//   move_param(A, L1)  -> global_load_dwordx4 -> (xor 0x80 for u8) -> ds_write_b128, two stages
// The B tile is stored [k][n] without row padding; the pieces of a row (32 bytes for i8, 64 for
// bf16) are XOR-ed with the low bits of the row number so that the rows one transposing read
// touches fall on different banks.  A direct-to-LDS instruction writes 1 KiB of consecutive LDS
// bytes, 16 per lane, so the swizzle is applied on the source side: a lane fetches the piece
// that belongs at its place.
#pragma once
#include "gemm_loop_gfx950.inc"
#include "gemm_mfma_kernel.h"

namespace mrl {
namespace gemm {

template <class T> struct BigTraits;
template <> struct BigTraits<I8> { static constexpr int SLOT = 32, RMASK = 7; };
template <> struct BigTraits<BF16> { static constexpr int SLOT = 64, RMASK = 3; };

constexpr int BIG_LDS_BYTES = 5 * 32768;  // two A stages and three B slots

#define MRL_GEMM_LOOP_CLOBBERS                                                                             \
  "v128", "v129", "v130", "v131", "v132", "v133", "v134", "v135", "v136", "v137", "v138", "v139", "v140", \
      "v141", "v142", "v143", "v144", "v145", "v146", "v147", "v148", "v149", "v150", "v151", "v152",     \
      "v153", "v154", "v155", "v156", "v157", "v158", "v159", "v160", "v161", "v162", "v163", "v164",     \
      "v165", "v166", "v167", "v168", "v169", "v170", "v171", "v172", "v173", "v174", "v175", "v176",     \
      "v177", "v178", "v179", "v180", "v181", "v182", "v183", "v184", "v185", "v186", "v187", "v188",     \
      "v189", "v190", "v191", "v192", "v193", "v194", "v195", "v196", "v197", "v198", "v199", "v200",     \
      "v201", "v202", "v203", "v204", "v205", "v206", "v207", "v208", "v209", "s60", "s61", "s62", "s63", \
      "s64", "s65", "s66", "s67", "s68", "s69", "s70", "s71", "scc", "memory"

#define MRL_GEMM_LOOP(TEXT)                                                                                   \
  asm volatile(TEXT                                                                                           \
               : "=&{v[0:15]}"(c0), "=&{v[16:31]}"(c1), "=&{v[32:47]}"(c2), "=&{v[48:63]}"(c3),               \
                 "=&{v[64:79]}"(c4), "=&{v[80:95]}"(c5), "=&{v[96:111]}"(c6), "=&{v[112:127]}"(c7),           \
                 "=&{v[210:211]}"(sums)                                                                       \
               : [a_off0] "v"(a_off[0]), [a_off1] "v"(a_off[1]), [a_off2] "v"(a_off[2]), [a_off3] "v"(a_off[3]), \
                 [b_off0] "v"(b_off[0]), [b_off1] "v"(b_off[1]), [b_off2] "v"(b_off[2]), [b_off3] "v"(b_off[3]), \
                 [a_wr] "v"(a_wr), [a_rd0] "v"(a_rd[0]), [a_rd1] "v"(a_rd[1]), [a_rd2] "v"(a_rd[2]),          \
                 [a_rd3] "v"(a_rd[3]), [b_rd0] "v"(b_rd[0]), [b_rd1] "v"(b_rd[1]), [abase] "s"(A),            \
                 [bbase] "s"(B), [bstep] "s"(b_step), [nk] "s"(nk), [dma_base] "s"(dma_base)                  \
               : MRL_GEMM_LOOP_CLOBBERS)

// M, N multiples of 256; K a multiple of two k steps (256 bytes); see big_applicable().
template <class T, bool A_UNSIGNED>
__global__ __launch_bounds__(512) void k_gemm_big(MRL_WALK_PARAMS, GemmArgs g) {
  extern __shared__ __attribute__((aligned(16))) uint8_t lds[];
  constexpr int BM = 256, BN = 256, BKB = 128, WAVES_M = 2, WAVES_N = 4, NT = 512;
  constexpr int WM = BM / WAVES_M, WN = BN / WAVES_N, TM = WM / 32, TN = WN / 32;
  constexpr int ES = T::ES, BK = BKB / ES;
  constexpr int B_ROWB = BN * ES;              // bytes per k row of the B tile
  constexpr int B_BASE = 2 * BM * BKB;         // LDS: [A stage 0][A stage 1][B slot 0][B slot 1][B slot 2]
  constexpr int SLOT = BigTraits<T>::SLOT, RMASK = BigTraits<T>::RMASK;
  constexpr int A_ROW_CH = BKB / 16, A_ROWS_PER_LINE = 256 / BKB, A_ROWS_PER_I = NT / A_ROW_CH;
  constexpr int ROWS_PER_DMA = 1024 / B_ROWB;  // k rows one direct-to-LDS instruction fills: 4 (i8), 2 (bf16)
  constexpr int K_SLAB = 32 / ES;
  static_assert(TM == 4 && TN == 2, "the assembly loop is written for 4 x 2 MFMA blocks per wave");
  typedef typename T::Acc Acc;
  typedef typename T::Out Out;

  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wm = wave / WAVES_N, wn = wave % WAVES_N;

  // Workgroups go to the 8 XCDs round-robin; each XCD gets a contiguous run of tiles which, taken
  // group_m tile rows at a time, covers a compact block of C (its A rows and B columns stay in
  // that XCD's L2).
  MRL_WALK_TILE(tile_m, tile_n)
  const int64_t m0 = int64_t(tile_m) * BM, n0 = int64_t(tile_n) * BN;

  const uint8_t *A = (const uint8_t *)g.a + (int64_t(blockIdx.y) * g.sa + m0 * g.lda) * ES;
  const uint8_t *B = (const uint8_t *)g.b + (int64_t(blockIdx.y) * g.sb + n0) * ES;
  Out *C = (Out *)g.c + int64_t(blockIdx.y) * g.sc + m0 * g.ldc + n0;
  const uint32_t lda_b = uint32_t(g.lda) * ES, ldb_b = uint32_t(g.ldb) * ES;
  const uint32_t lds0 = uint32_t(uintptr_t(lds));  // LDS byte address of the dynamic allocation

  // A staging: thread `tid` moves 16-byte chunk tid + i * NT of a tile (rows 64 apart); chunks of
  // a row are XOR-ed with (row / 2) & 7 in LDS, as in k_gemm.
  uint32_t a_off[4], a_wr;
  {
    const int row = tid / A_ROW_CH, ch = tid % A_ROW_CH;
#pragma unroll
    for (int i = 0; i < 4; i++) a_off[i] = uint32_t(row + i * A_ROWS_PER_I) * lda_b + ch * 16;
    a_wr = lds0 + row * BKB + ((ch ^ ((row / A_ROWS_PER_LINE) & (A_ROW_CH - 1))) << 4);
  }
  // B staging: instruction i of this wave fills LDS bytes [(4 * wave + i) * 1024, +1024) of the slot,
  // lane L the 16 bytes at 16 * L of them.
  uint32_t b_off[4];
#pragma unroll
  for (int i = 0; i < 4; i++) {
    const int r = (wave * 4 + i) * ROWS_PER_DMA + (lane * 16) / B_ROWB;
    const int inrow = (lane * 16) % B_ROWB;
    const int piece = (inrow / SLOT) ^ (r & RMASK);
    b_off[i] = uint32_t(r) * ldb_b + piece * SLOT + inrow % SLOT;
  }
  const uint32_t dma_base = lds0 + B_BASE + wave * 4096;
  // Operand reads.  A: lane (l % 32, l / 32) of MFMA block tm reads 16 bytes of row
  // wm * 128 + tm * 32 + l % 32 at chunk 2 * s + l / 32 of slab s.
  uint32_t a_rd[4];
  {
    const int swz = ((lane & 31) / A_ROWS_PER_LINE) & (A_ROW_CH - 1), half = lane >> 5;
#pragma unroll
    for (int s = 0; s < 4; s++) a_rd[s] = lds0 + (wm * WM + (lane & 31)) * BKB + (((2 * s + half) ^ swz) << 4);
  }
  // B: a 16-lane group of a transposing read fetches K_PER_READ k rows x 16 columns; lane p of
  // the group addresses 8 bytes of one k row and receives the column it indexes.
  uint32_t b_rd[2];
  {
    constexpr int LANES_PER_ROW = 16 / (8 / ES);
    const int p = lane & 15;
    const int k = (K_SLAB / 2) * (lane >> 5) + p / LANES_PER_ROW;
#pragma unroll
    for (int tn = 0; tn < TN; tn++) {
      const int byte = (wn * WN + tn * 32 + 16 * ((lane >> 4) & 1) + (8 / ES) * (p % LANES_PER_ROW)) * ES;
      b_rd[tn] = lds0 + k * B_ROWB + (((byte / SLOT) ^ (k & RMASK)) * SLOT) + byte % SLOT;
    }
  }
  const uint32_t b_step = uint32_t(BK) * ldb_b;
  const uint32_t nk = g.k / BK;

  v16i c0, c1, c2, c3, c4, c5, c6, c7;
  v2i sums;
  if constexpr (std::is_same<T, BF16>::value) {
    MRL_GEMM_LOOP(GEMM_LOOP_BF16);
  } else if constexpr (!A_UNSIGNED) {
    MRL_GEMM_LOOP(GEMM_LOOP_I8);
  } else {
    // The two wave rows share B's columns and each adds up the column sums of every other slab.
    if (wm == 0) MRL_GEMM_LOOP(GEMM_LOOP_U8_0);
    else MRL_GEMM_LOOP(GEMM_LOOP_U8_1);
  }
  Acc acc[TM][TN];
  acc[0][0] = __builtin_bit_cast(Acc, c0), acc[0][1] = __builtin_bit_cast(Acc, c1);
  acc[1][0] = __builtin_bit_cast(Acc, c2), acc[1][1] = __builtin_bit_cast(Acc, c3);
  acc[2][0] = __builtin_bit_cast(Acc, c4), acc[2][1] = __builtin_bit_cast(Acc, c5);
  acc[3][0] = __builtin_bit_cast(Acc, c6), acc[3][1] = __builtin_bit_cast(Acc, c7);
  int colsum[TN] = {sums[0], sums[1]};
  epilogue<T, A_UNSIGNED, false, BN, WAVES_M, TM, TN>(g, C, lds, acc, colsum, lane, wm, wm * WM, wn * WN,
                                                      int(g.m - m0), int(g.n - n0));
}

// Whole tiles, an even number of k steps, and offsets the loop's 32-bit arithmetic can hold.
inline bool big_applicable(const GemmArgs &g, int elem_size) {
  const int64_t bk = 128 / elem_size;
  return !g.b_kmajor && g.m % 256 == 0 && g.n % 256 == 0 && g.k % (2 * bk) == 0 && g.k >= 2 * bk &&
         g.lda * elem_size * 256 < (int64_t(1) << 32) && g.ldb * elem_size * (bk + 1) < (int64_t(1) << 31) &&
         g.ldc * 4 < EDGE_MAX_ROW_BYTES;
}

template <class T, bool A_UNSIGNED>
hipError_t launch_big(const GemmArgs &g, hipStream_t stream) {
  constexpr auto kern = k_gemm_big<T, A_UNSIGNED>;
  static std::atomic<uint64_t> lds_limit_set{0};
  if (!plan::recording()) {
    hipError_t e = raise_lds_limit(lds_limit_set, (const void *)kern, BIG_LDS_BYTES);
    if (e != hipSuccess) return e;
  }
  const int tiles_m = int(g.m / 256), tiles_n = int(g.n / 256);
  const double mn = double(g.m) * g.n * g.batch;
  plan::work(T::ES == 1 ? plan::UNIT_MFMA_I8 : plan::UNIT_MFMA_BF16, 2.0 * mn * g.k,
             (double(g.m) * g.k + double(g.k) * g.n) * g.batch * T::ES + mn * 4 * (g.accum ? 2 : 1),
             2.0 * 256 * 256 * double(g.k), 500.0 + 1200.0 * double(g.k * T::ES / 128),
             T::ES == 1 ? 1.25 : 1.08);  // measured: 1800 TOPS int8 at 4096^3
  const TileWalk walk = tile_walk(tiles_m, tiles_n);
  MRL_LAUNCH((k_gemm_big<T, A_UNSIGNED>), dim3(tiles_m * tiles_n, g.batch), dim3(512), BIG_LDS_BYTES, stream,
             MRL_WALK_ARGS(walk), g);
  return mrl::plan::last_error();
}

}  // namespace gemm
}  // namespace mrl
