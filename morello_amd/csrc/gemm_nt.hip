// Matmul whose B operand is stored with k fastest (Morello's col_major / batched_col_major
// layouts, layout![0,2,1]): the matrix-core kernel of gemm_mfma_kernel.h with B staged and read
// like A.  Kept in its own translation unit so the instantiations compile in parallel.
#include "gemm_mfma_kernel.h"

namespace mrl {
namespace {
using namespace gemm;

typedef Tile<64, 64, 128, 2, 2> T64;

template <class T, bool A_UNSIGNED>
hipError_t launch_for(const GemmArgs &g, uint32_t tile, hipStream_t stream) {
  if (tile == 64) return launch<T, A_UNSIGNED, T64, true, true>(g, stream);
  if (tile == 128) return launch<T, A_UNSIGNED, Tile128<T, true>, true, true>(g, stream);
  const bool whole = g.m % TileBig::BM == 0 && g.n % TileBig::BN == 0 && g.k % (TileBig::BKB / T::ES) == 0;
  return whole ? launch<T, A_UNSIGNED, TileBig, false, true>(g, stream)
               : launch<T, A_UNSIGNED, TileBig, true, true>(g, stream);
}

}  // namespace

hipError_t launch_gemm_nt(const GemmArgs &g, int kind, uint32_t tile, hipStream_t stream) {
  switch (kind) {
    case 0: return launch_for<I8, false>(g, tile, stream);
    case 1: return launch_for<I8, true>(g, tile, stream);
    case 2: return launch_for<BF16, false>(g, tile, stream);
    case 3: return launch_for<F32, false>(g, tile, stream);
    default: return hipErrorInvalidValue;
  }
}

}  // namespace mrl
