// Schedule-driven Matmul: a Morello manual schedule
//     spec.tile_out([1, m, n]) ... .split(k)
// (morello/src/scheduling_sugar.rs:37-132; the worked examples are
// morello/examples/simple_matmul_x86.rs:60-100 and matmul_x86.rs:27-70) picks the workgroup
// tile and the k step of the matrix-core kernel instead of the library's default.  Only the
// shapes listed in kSchedules are built.  The move_param steps of a CPU schedule (which operand is
// staged in which memory, how many buffers deep) have one counterpart: `staging` chooses among the
// three 256 x 256 kernels, which differ in exactly that (mrl_staging in the public header).
#include "gemm_mfma_kernel.h"

namespace mrl {
namespace {
using namespace gemm;

typedef Tile<256, 256, 64, 2, 4> T256x256k64;
typedef Tile<256, 128, 64, 2, 2> T256x128k64;
typedef Tile<128, 256, 64, 2, 2> T128x256k64;
typedef Tile<128, 128, 64, 2, 2> T128x128k64;
typedef Tile<64, 64, 64, 2, 2> T64x64k64;
typedef Tile<64, 64, 128, 2, 2> T64x64k128;

struct Entry {
  uint32_t tile_m, tile_n, k_bytes, staging;
};
// k_bytes is the k step in bytes of an operand row: 128 = 128 i8, 64 bf16 or 32 f32 elements.
const Entry kSchedules[] = {{256, 256, 128, 0}, {256, 256, 64, 0}, {256, 128, 64, 0}, {128, 256, 64, 0}, {128, 128, 64, 0}, {64, 64, 64, 0},
                            {128, 128, 128, 0}, {64, 64, 128, 0}, {256, 256, 128, 1}, {256, 256, 128, 2}, {256, 256, 128, 3}};

template <class TL>
hipError_t launch_kind(const GemmArgs &g, int kind, hipStream_t stream) {
  switch (kind) {
    case 0: return launch<I8, false, TL, true>(g, stream);
    case 1: return launch<I8, true, TL, true>(g, stream);
    case 2: return launch<BF16, false, TL, true>(g, stream);
    default: return launch<F32, false, TL, true>(g, stream);
  }
}

// The 128 x 128 tile with a 128-byte step is laid out over its waves per element type (Tile128).
hipError_t launch_128(const GemmArgs &g, int kind, hipStream_t stream) {
  switch (kind) {
    case 0: return launch<I8, false, Tile128<I8, false>, true>(g, stream);
    case 1: return launch<I8, true, Tile128<I8, false>, true>(g, stream);
    case 2: return launch<BF16, false, Tile128<BF16, false>, true>(g, stream);
    default: return launch<F32, false, Tile128<F32, false>, true>(g, stream);
  }
}

}  // namespace

uint32_t gemm_schedule_count() { return sizeof(kSchedules) / sizeof(kSchedules[0]); }

void gemm_schedule_at(uint32_t i, int elem_size, uint32_t *tile_m, uint32_t *tile_n, uint32_t *split_k, uint32_t *staging) {
  *tile_m = kSchedules[i].tile_m, *tile_n = kSchedules[i].tile_n, *split_k = kSchedules[i].k_bytes / elem_size;
  *staging = kSchedules[i].staging;
}

// kind: 0 = i8 x i8, 1 = u8 x i8, 2 = bf16 x bf16, 3 = f32 x f32.  Returns hipErrorInvalidValue for a
// schedule that is not built.
hipError_t launch_gemm_scheduled(const GemmArgs &g, int kind, uint32_t tile_m, uint32_t tile_n,
                                 uint32_t split_k, hipStream_t stream, uint32_t staging) {
  const uint32_t k_bytes = split_k * (kind == 2 ? 2 : kind == 3 ? 4 : 1);
  if (staging > 3) return hipErrorInvalidValue;
  if (tile_m == 256 && tile_n == 256 && k_bytes == 128)
    return launch_gemm_big(g, kind, stream, staging);
  if (staging > 1) return hipErrorInvalidValue;  // the other tiles exist with register staging only
  if (tile_m == 256 && tile_n == 256 && k_bytes == 64) return launch_kind<T256x256k64>(g, kind, stream);
  if (tile_m == 256 && tile_n == 128 && k_bytes == 64) return launch_kind<T256x128k64>(g, kind, stream);
  if (tile_m == 128 && tile_n == 256 && k_bytes == 64) return launch_kind<T128x256k64>(g, kind, stream);
  if (tile_m == 128 && tile_n == 128 && k_bytes == 64) return launch_kind<T128x128k64>(g, kind, stream);
  if (tile_m == 64 && tile_n == 64 && k_bytes == 64) return launch_kind<T64x64k64>(g, kind, stream);
  if (tile_m == 128 && tile_n == 128 && k_bytes == 128) return launch_128(g, kind, stream);
  if (tile_m == 64 && tile_n == 64 && k_bytes == 128) return launch_kind<T64x64k128>(g, kind, stream);
  return hipErrorInvalidValue;
}

}  // namespace mrl
