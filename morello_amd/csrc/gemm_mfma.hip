// Dispatch of the Matmul Spec onto the matrix-core kernel of gemm_mfma_kernel.h with the
// default tile (256 x 256 outputs, 128 bytes of K per step).
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
  // Below a tile's worth of work in either direction the generic kernel is the better fit.
  return g.m >= 64 && g.n >= 64 && g.k >= 64 && (g.b_kmajor || g.n % per16 == 0) && g.k % per16 == 0 &&
         g.lda % per16 == 0 && g.ldb % per16 == 0 && g.sa % per16 == 0 && g.sb % per16 == 0 &&
         al16(g.a) && al16(g.b) && (reinterpret_cast<uintptr_t>(g.c) & 3) == 0 &&
         g.batch <= 65535 && uint64_t((g.m + BM - 1) / BM) * ((g.n + BN - 1) / BN) < (1u << 30);
}

}  // namespace

bool gemm_i8_applicable(const GemmArgs &g) { return applicable(g, 1); }
hipError_t launch_gemm_i8(const GemmArgs &g, bool a_unsigned, hipStream_t stream) {
  if (g.b_kmajor) return launch_gemm_nt(g, a_unsigned ? 1 : 0, stream);
  if (whole_tiles(g, 1))
    return a_unsigned ? launch<I8, true, TileBig, false>(g, stream) : launch<I8, false, TileBig, false>(g, stream);
  return a_unsigned ? launch<I8, true, TileBig, true>(g, stream) : launch<I8, false, TileBig, true>(g, stream);
}
bool gemm_f32_applicable(const GemmArgs &g) { return applicable(g, 4); }
hipError_t launch_gemm_f32(const GemmArgs &g, hipStream_t stream) {
  if (g.b_kmajor) return launch_gemm_nt(g, 3, stream);
  return whole_tiles(g, 4) ? launch<F32, false, TileBig, false>(g, stream)
                           : launch<F32, false, TileBig, true>(g, stream);
}
bool gemm_bf16_applicable(const GemmArgs &g) { return applicable(g, 2); }
hipError_t launch_gemm_bf16(const GemmArgs &g, hipStream_t stream) {
  if (g.b_kmajor) return launch_gemm_nt(g, 2, stream);
  return whole_tiles(g, 2) ? launch<BF16, false, TileBig, false>(g, stream)
                           : launch<BF16, false, TileBig, true>(g, stream);
}

}  // namespace mrl
