// Conv as an implicit Matmul on the matrix cores: the kernel of gemm_mfma_kernel.h with its left
// operand addressed as the windows of a channels-last image (the CONV build) and the KRSC
// filters as a B operand stored k-fastest.  Takes any Conv whose channel vectors are whole
// 16-byte chunks (morello/src/spec.rs:486-494: no stride, no padding); nothing is unfolded in
// memory.  Its own translation unit so that the instantiations compile beside the others.
#include "gemm_mfma_kernel.h"

namespace mrl {
namespace {
using namespace gemm;

typedef Tile<64, 64, 128, 2, 2> T64;

template <class T, bool A_UNSIGNED>
hipError_t launch_for(const GemmArgs &g, uint32_t tile, hipStream_t stream) {
  if (tile == 64) return launch<T, A_UNSIGNED, T64, true, true, true>(g, stream);
  if (tile == 128) return launch<T, A_UNSIGNED, Tile128<T, true>, true, true, true>(g, stream);
  return launch<T, A_UNSIGNED, TileBig, true, true, true>(g, stream);
}

}  // namespace

bool conv_gemm_applicable(const GemmArgs &g, int kind) {
  const int es = kind == 3 ? 4 : kind == 2 ? 2 : 1;
  auto al16 = [](const void *p) { return (reinterpret_cast<uintptr_t>(p) & 15) == 0; };
  return g.b_kmajor && (g.batch == 1 || (g.conv.slice_bytes != 0 && g.conv.slice_bytes % 16 == 0)) && g.conv.c_bytes != 0 && g.conv.c_bytes % 16 == 0 &&
         g.conv.image_bytes < (1ull << 31) && g.m >= 1 && g.n >= 1 && g.k >= 1 && g.ldb % (16 / es) == 0 &&
         al16(g.a) && al16(g.b) && (reinterpret_cast<uintptr_t>(g.c) & 3) == 0 && edge_addressable(g, es) &&
         uint64_t((g.m + 63) / 64) * ((g.n + 63) / 64) < (1u << 30);
}

hipError_t launch_conv_gemm(const GemmArgs &args, int kind, hipStream_t stream, uint32_t tile) {
  if (!conv_gemm_applicable(args, kind) || (tile != 0 && tile != 64 && tile != 128 && tile != 256)) return hipErrorInvalidValue;
  if (tile == 0) tile = gemm_tile_side(args, kind);
  // Pixel numbers and window bytes stay below 2^31 (conv_gemm_applicable), as FastDiv asks.
  GemmArgs g = args;
  g.conv.by_ow = FastDiv(g.conv.ow), g.conv.by_oh = FastDiv(g.conv.oh);
  g.conv.by_c_bytes = FastDiv(g.conv.c_bytes), g.conv.by_fw = FastDiv(g.conv.fw);
  switch (kind) {
    case 0: return launch_for<I8, false>(g, tile, stream);
    case 1: return launch_for<I8, true>(g, tile, stream);
    case 2: return launch_for<BF16, false>(g, tile, stream);
    case 3: return launch_for<F32, false>(g, tile, stream);
    default: return hipErrorInvalidValue;
  }
}

}  // namespace mrl
