// Dispatch of the Matmul Spec onto the matrix-core kernel of gemm_mfma_kernel.h.  Without a
// manual schedule the workgroup tile is chosen from the problem size (the reference prices
// schedules with a cost model before it emits one, morello/src/cost.rs; here the table is
// three entries long and comes from measurement).
#include <algorithm>

#include "gemm_big_kernel.h"
#include "gemm_wide_kernel.h"
#include "gemm_mfma_kernel.h"

namespace mrl {
namespace {
using namespace gemm;

// Whole tiles only (the fast instantiation) or any shape whose rows are whole 16-byte chunks.
bool whole_tiles(const GemmArgs &g, int es) {
  return g.m % TileBig::BM == 0 && g.n % TileBig::BN == 0 && g.k % (TileBig::BKB / es) == 0;
}

bool applicable(const GemmArgs &g, int es) {
  auto al16 = [](const void *p) { return (reinterpret_cast<uintptr_t>(p) & 15) == 0; };
  const int64_t per16 = 16 / es;
  constexpr int BM = TileBig::BM, BN = TileBig::BN;
  // K and N themselves may be anything: a row's bytes from its end to its leading dimension are
  // read along with it, and are zeros wherever the caller padded the row.
  return g.m >= 1 && g.n >= 1 && g.k >= 1 &&
         g.lda % per16 == 0 && g.ldb % per16 == 0 && g.sa % per16 == 0 && g.sb % per16 == 0 &&
         al16(g.a) && al16(g.b) && (reinterpret_cast<uintptr_t>(g.c) & 3) == 0 &&
         g.batch <= 65535 && uint64_t((g.m + BM - 1) / BM) * ((g.n + BN - 1) / BN) < (1u << 30);
}

// Side of the square workgroup tile for a problem size, from launch timings on an MI355X of
// every built tile over cubes from 64^3 to 4096^3.  The 256 x 256 tile is the fastest per CU
// but fills the chip in rounds of 256 tiles, one per CU; smaller tiles run several to a CU.
// All three step through K 128 bytes at a time (a 64-byte step costs the small tiles 10-30 %).
//   int8, bf16: 256 once a round is at least half full (3072^3, 144 tiles: int8 47 us against
//     49 us for 128 and 62 us for 64); below that 64 while the 128 tile would leave well over a
//     third of the compute units without one (1024^3: 6.5 us against 10.0 and 17.7; up to 512
//     tiles of 64: int8 6272 x 2304 x 256, 392 of them, 15.4 us against 16.2, 2048 x 2048 x 1024, 512,
//     14.8 against 15.6, at 576 13.6 against 14.4 the other way; bf16 392 tiles 22.9 against 23.5,
//     8 x 512^3, 512 tiles, 7.7 against 8.8, 1536^3, 576, 21.3 against 17.6 the other way), then 128
//     (2048^3: 17.3 us against 20.6 and 29.9; 1792^3, 784 tiles: 16.5 against 19.4).
//   f32: its MFMA has a sixteenth of the int8 rate, so operand traffic never limits a small
//     tile: 64 (1024^3: 27 us against 70 and 239; 3072^3: 460 against 559 and 711) until the
//     256 tile fills its rounds (4096^3: 948 us against 1066).
// A tile wider than the matrix is mostly padding: at most 64 (128) rows or columns cap the side
// at 64 (128) whatever the counts say.
uint32_t tile_side(const GemmArgs &g, int es) {
  const uint32_t narrow = std::min(g.m, g.n), cap = narrow <= 64 ? 64 : narrow <= 128 ? 128 : 256;
  const uint64_t big = uint64_t((g.m + 255) / 256) * ((g.n + 255) / 256) * g.batch;
  const double round_fill = double(big) / double((big + 255) / 256 * 256);
  if (cap == 256 && round_fill >= (es == 4 ? 0.85 : 0.5)) return 256;
  if (es == 4 || cap == 64) return 64;
  const uint64_t small = uint64_t((g.m + 63) / 64) * ((g.n + 63) / 64) * g.batch;
  if (small <= 512) return 64;
  // A side that the 128 tile pads by much more than the 64 tile does (192 rows: 256 against 192)
  // costs it more than its larger tile gains (bf16 192 x 192 x 16384: 5.8 us against 6.3).
  const double area64 = double((g.m + 63) / 64 * 64) * double((g.n + 63) / 64 * 64);
  const double area128 = double((g.m + 127) / 128 * 128) * double((g.n + 127) / 128 * 128);
  return area128 > 1.25 * area64 ? 64 : 128;
}

constexpr int elem_size_of(int kind) { return kind == 3 ? 4 : kind == 2 ? 2 : 1; }

}  // namespace

// Ragged shapes also need leading dimensions the EDGE kernels' 32-bit offsets can span.
bool gemm_possible(const GemmArgs &g, int kind) {
  const int es = elem_size_of(kind);
  return applicable(g, es) && (edge_addressable(g, es) || whole_tiles(g, es));
}
// The 64 x 64 tile beats the generic kernel on anything but the tiniest problems, skinny ones
// included (int8 32 x 4096 x 4096: 23 us against 237 us; f32 16 x 64 x 16: 4.1 us against 3.6 us).
bool gemm_pays(const GemmArgs &g, int) { return double(g.m) * g.n * g.k * g.batch >= 100e3; }

uint32_t gemm_tile_side(const GemmArgs &g, int kind) { return tile_side(g, elem_size_of(kind)); }

// Fewer than three quarters of the compute units would get a 64 x 64 tile and every tile walks at
// least sixteen k steps: share K out so that up to 512 workgroups run, eight steps each at least
// (int8 512 x 8192 x 512: 64 tiles of 64 steps, 36 us; as 8 x 64 tiles of 8 steps plus the sum, 10 us).
uint32_t gemm_k_splits(const GemmArgs &g, int kind, uint32_t *remainder) {
  // remainder: where the caller can run one more, shorter slice behind the equal ones (a K that
  // is not a whole number of 128-byte steps, or whose steps have no divisor near the wanted
  // count: 300 x 30000 x 300 int8 is 234 steps and 48 bytes); without it only equal slices.
  if (remainder) *remainder = 0;
  const uint64_t es = elem_size_of(kind);
  const uint64_t k_bytes = uint64_t(g.k) * es;
  if (g.batch != 1 || gemv_applicable(g, kind) || (k_bytes % 128 != 0 && !remainder)) return 1;
  const uint64_t steps = k_bytes / 128;
  const uint64_t tiles = uint64_t((g.m + 63) / 64) * ((g.n + 63) / 64);
  if (tiles >= 384 || steps < 16) return 1;
  const uint64_t wanted = std::min<uint64_t>({32, 768 / tiles, steps / 8});
  uint64_t want = wanted;
  while (want > 1 && (steps % want != 0 || k_bytes % 128 != 0)) want--;
  uint64_t left = 0;   // elements of K behind the equal slices
  if (remainder && wanted > 1 && want * 2 <= wanted) {
    want = wanted;
    left = g.k - want * (steps / want) * (128 / es);
  }
  if (want <= 1) return 1;
  // What the slices save: a workgroup's chain of k steps (~0.48 us each on the 64 x 64 tile)
  // shortens by the factor by which they add workgroups the chip has room for (about 384
  // overlap well); what they cost: the summing launch and its traffic.  bf16 1024^3 (256 tiles
  // of 16 steps) ran 15 us in two slices against 8.8 us whole.
  const double spread = std::min<double>(double(want), 384.0 / double(tiles));
  const double saved_us = double(steps) * (1.0 - 1.0 / spread) * 0.48;
  const double cost_us = 2.5 + (left ? 3.0 : 0.0) + (double(want) + (left ? 2.0 : 1.0)) * double(g.m) * double(g.n) * 4.0 / 5.5e6;
  if (spread <= 1.0 || saved_us < 1.2 * cost_us) return 1;
  if (remainder) *remainder = uint32_t(left);
  return uint32_t(want);
}

hipError_t launch_gemm_big(const GemmArgs &g, int kind, hipStream_t stream, uint32_t staging) {
  if (g.b_kmajor) return launch_gemm_nt(g, kind, 256, stream);
  const bool whole = whole_tiles(g, elem_size_of(kind));
  // Whole tiles and an even number of k steps: the tiles with hand-scheduled k loops.  With a K
  // long enough for its first steps to carry C's old values, four waves with 128 x 128 outputs each
  // (int8 4096^3 accumulating: 69 us; eight waves of 128 x 64: 76 us; the compiler-scheduled loop: 87 us).
  if ((staging == 0 || staging == 3) && whole && kind <= 2 && wide_applicable(g, elem_size_of(kind))) {
    switch (kind) {
      case 0: return launch_wide<I8, false>(g, stream);
      case 1: return launch_wide<I8, true>(g, stream);
      case 2: return launch_wide<BF16, false>(g, stream);
    }
  }
  if (staging == 3) return hipErrorInvalidValue;
  if ((staging == 0 || staging == 2) && whole && kind <= 2 && big_applicable(g, elem_size_of(kind))) {
    switch (kind) {
      case 0: return launch_big<I8, false>(g, stream);
      case 1: return launch_big<I8, true>(g, stream);
      case 2: return launch_big<BF16, false>(g, stream);
    }
  }
  if (staging == 2) return hipErrorInvalidValue;
  switch (kind) {
    case 0: return whole ? launch<I8, false, TileBig, false>(g, stream) : launch<I8, false, TileBig, true>(g, stream);
    case 1: return whole ? launch<I8, true, TileBig, false>(g, stream) : launch<I8, true, TileBig, true>(g, stream);
    case 2: return whole ? launch<BF16, false, TileBig, false>(g, stream) : launch<BF16, false, TileBig, true>(g, stream);
    case 3: return whole ? launch<F32, false, TileBig, false>(g, stream) : launch<F32, false, TileBig, true>(g, stream);
  }
  return hipErrorInvalidValue;
}

hipError_t launch_gemm(const GemmArgs &g, int kind, hipStream_t stream) {
  if (gemv_applicable(g, kind)) return launch_gemv(g, kind, stream);
  const int es = elem_size_of(kind);
  // Only the 256 tile has a build without the EDGE kernels' limit on leading dimensions.
  const uint32_t side = edge_addressable(g, es) ? tile_side(g, es) : 256;
  if (side == 256) return launch_gemm_big(g, kind, stream);
  if (g.b_kmajor) return launch_gemm_nt(g, kind, side, stream);
  return launch_gemm_scheduled(g, kind, side, side, 128 / es, stream);
}

}  // namespace mrl
