// Matmul with very few rows of A against a B stored k-fastest: the matrix-vector shape of
// morello/examples/matvec_gemma_x86_bf16f32.rs:24-37 (bf16[1 x 2048] . bf16[2048 x 16384] with B
// as layout![0,2,1] -> f32).  Such a problem streams B once and does next to no arithmetic, so it
// is run as dot products instead of on the matrix cores: a wavefront owns COLS rows of B (=
// output columns), its 64 lanes stride along K in 16-byte chunks with non-temporal loads, the
// few rows of A come through the cache, and a butterfly over the lanes finishes each dot product.
// Same results as the MFMA kernel: exact for integers (u8 through the a xor 0x80 form and the
// 128 * sum_k B[k,j] correction), f32 accumulation for bf16 and f32.
#include "gemm_mfma_kernel.h"

namespace mrl {
namespace {
using gemm::v4i;

// Rows of B per wavefront (up to four rows of A) and steps of K in flight: two and four measured
// fastest (bf16 1 x 2048 x 16384: 10.5 us; four rows and two steps 12.4, eight rows 13.3, one row
// 11.2); the switches are for such measurements.
#ifndef MRL_GEMV_MAX_M
#define MRL_GEMV_MAX_M 8
#endif
#ifndef MRL_GEMV_UNROLL
#define MRL_GEMV_UNROLL 4
#endif
#ifndef MRL_GEMV_COLS
#define MRL_GEMV_COLS 2
#endif
constexpr int WAVES = 4;         // wavefronts per workgroup
constexpr int MAX_ROWS = 8;      // rows of A the kernel is built for

template <int KIND>
struct Acc {
  typedef int type;
};
template <>
struct Acc<2> {
  typedef float type;
};
template <>
struct Acc<3> {
  typedef float type;
};

// acc += a . b over one 16-byte chunk.  KIND as in launch_gemm: 0 i8, 1 u8 (a already xor 0x80),
// 2 bf16, 3 f32.
template <int KIND>
__device__ inline typename Acc<KIND>::type dot16(v4i a, v4i b, typename Acc<KIND>::type acc) {
  if constexpr (KIND <= 1) {
#pragma unroll
    for (int w = 0; w < 4; w++) acc = __builtin_amdgcn_sdot4(a[w], b[w], acc, false);
  } else if constexpr (KIND == 2) {
#pragma unroll
    for (int w = 0; w < 4; w++) {
      acc = __builtin_fmaf(__uint_as_float(uint32_t(a[w]) << 16), __uint_as_float(uint32_t(b[w]) << 16), acc);
      acc = __builtin_fmaf(__uint_as_float(uint32_t(a[w]) & 0xffff0000u), __uint_as_float(uint32_t(b[w]) & 0xffff0000u), acc);
    }
  } else {
#pragma unroll
    for (int w = 0; w < 4; w++) acc = __builtin_fmaf(__int_as_float(a[w]), __int_as_float(b[w]), acc);
  }
  return acc;
}

// COLS: output columns (rows of B) per wavefront, all in flight together.
template <int KIND, int ROWS, int COLS>
__global__ __launch_bounds__(64 * WAVES) void k_gemv(GemmArgs g) {
  typedef typename Acc<KIND>::type acc_t;
  constexpr int ES = KIND == 3 ? 4 : KIND == 2 ? 2 : 1;
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int64_t col0 = (int64_t(blockIdx.x) * WAVES + wave) * COLS;
  if (col0 >= int64_t(g.n)) return;
  const uint8_t *A = (const uint8_t *)g.a + int64_t(blockIdx.y) * g.sa * ES;
  const uint8_t *B = (const uint8_t *)g.b + int64_t(blockIdx.y) * g.sb * ES;
  const int64_t lda_b = g.lda * ES, ldb_b = g.ldb * ES;
  const int k_bytes = int(g.k) * ES;
  // Rows past M and columns past N are computed on the last valid one and not stored.
  const uint8_t *a_row[ROWS], *b_row[COLS];
#pragma unroll
  for (int r = 0; r < ROWS; r++) a_row[r] = A + int64_t(min(r, int(g.m) - 1)) * lda_b;
#pragma unroll
  for (int c = 0; c < COLS; c++) b_row[c] = B + min(col0 + c, int64_t(g.n) - 1) * ldb_b;

  acc_t acc[ROWS][COLS];
  int colsum[COLS];
#pragma unroll
  for (int c = 0; c < COLS; c++) {
    colsum[c] = 0;
#pragma unroll
    for (int r = 0; r < ROWS; r++) acc[r][c] = 0;
  }
#pragma unroll MRL_GEMV_UNROLL
  for (int kb = lane * 16; kb < k_bytes; kb += 64 * 16) {
    v4i bv[COLS], av[ROWS];
#pragma unroll
    for (int c = 0; c < COLS; c++) bv[c] = __builtin_nontemporal_load((const v4i *)(b_row[c] + kb));
#pragma unroll
    for (int r = 0; r < ROWS; r++) {
      av[r] = *(const v4i *)(a_row[r] + kb);
      if (KIND == 1) av[r] ^= v4i{int(0x80808080), int(0x80808080), int(0x80808080), int(0x80808080)};
    }
#pragma unroll
    for (int c = 0; c < COLS; c++) {
      if (KIND == 1) {
#pragma unroll
        for (int w = 0; w < 4; w++) colsum[c] = __builtin_amdgcn_sdot4(bv[c][w], 0x01010101, colsum[c], false);
      }
#pragma unroll
      for (int r = 0; r < ROWS; r++) acc[r][c] = dot16<KIND>(av[r], bv[c], acc[r][c]);
    }
  }
  // Butterfly over the 64 lanes; afterwards every lane holds every total.
#pragma unroll
  for (int c = 0; c < COLS; c++) {
#pragma unroll
    for (int off = 32; off >= 1; off >>= 1) {
      if (KIND == 1) colsum[c] += __shfl_xor(colsum[c], off);
#pragma unroll
      for (int r = 0; r < ROWS; r++) acc[r][c] += __shfl_xor(acc[r][c], off);
    }
  }
  // Lane r * COLS + c stores C[r][col0 + c].
  acc_t *C = (acc_t *)g.c + int64_t(blockIdx.y) * g.sc;
#pragma unroll
  for (int r = 0; r < ROWS; r++)
#pragma unroll
    for (int c = 0; c < COLS; c++)
      if (lane == r * COLS + c && r < int(g.m) && col0 + c < int64_t(g.n)) {
        acc_t v = acc[r][c];
        if (KIND == 1) v += acc_t(colsum[c] * 128);
        acc_t *out = C + int64_t(r) * g.ldc + col0 + c;
        if (g.accum) v += *out;
        *out = v;
      }
}

template <int KIND, int ROWS, int COLS>
hipError_t launch_as(const GemmArgs &g, hipStream_t stream) {
  const dim3 grid(uint32_t((uint64_t(g.n) + COLS * WAVES - 1) / (COLS * WAVES)), g.batch), block(64 * WAVES);
  constexpr int ES = KIND == 3 ? 4 : KIND == 2 ? 2 : 1;
  plan::work(plan::UNIT_STREAM, 2.0 * g.m * g.n * g.k * g.batch,
             double(g.batch) * ((double(g.m) + g.n) * g.k * ES + 4.0 * g.m * g.n));
  MRL_LAUNCH((k_gemv<KIND, ROWS, COLS>), grid, block, 0, stream, g);
  return mrl::plan::last_error();
}

template <int KIND>
hipError_t launch_rows(const GemmArgs &g, hipStream_t stream) {
  // One row of B per wavefront once B is some 200 MB (bf16 1 x 4096 x 32768: 39.6 us against 42.3
  // with two; at 134 MB the same, at 67 MB 11.2 against 10.6).
  constexpr int ES = KIND == 3 ? 4 : KIND == 2 ? 2 : 1;
  if (g.m == 1 && double(g.n) * g.k * ES * g.batch >= 200e6) return launch_as<KIND, 1, 1>(g, stream);
  if (g.m == 1) return launch_as<KIND, 1, MRL_GEMV_COLS>(g, stream);
  if (g.m == 2) return launch_as<KIND, 2, MRL_GEMV_COLS>(g, stream);
  if (g.m <= 4) return launch_as<KIND, 4, MRL_GEMV_COLS>(g, stream);
  return launch_as<KIND, MAX_ROWS, 2>(g, stream);
}

}  // namespace

// Few rows, long k-fastest rows of B: the problem is a stream over B.  The dot products' VALU work
// grows with the rows of A, while the matrix-core kernel with K shared out over workgroups takes the
// same time for any row count up to its tile's 64, about what streaming B at 5.8 TB/s takes plus
// the summing launch; so beyond two rows (f32, whose MFMA is slow: four) only the smaller problems
// (8 MiB of B, 4 MiB from five rows on) stay here, and rows of B too long for their number (16 KiB and more, at most 2048 of them: too few
// wavefronts with too long a walk each) go to the other kernel at any row count.  Measured, this
// kernel / the other (us): bf16 4 x 4096 x 16384 28.2 / 22.8, 8 rows 42.0 / 23.0, u8 8 x 4096 x 16384
// 29.8 / 15.2, bf16 4 x 2048 x 2048 4.6 / 7.2, 8 rows 6.5 / 7.2, bf16 2 x 8192 x 1024 11.1 / 8.1,
// f32 4 x 4096 x 16384 52.6 / 72.8.
bool gemv_applicable(const GemmArgs &g, int kind) {
  const int es = kind == 3 ? 4 : kind == 2 ? 2 : 1;
  const int64_t per16 = 16 / es;
  auto al16 = [](const void *p) { return (reinterpret_cast<uintptr_t>(p) & 15) == 0; };
  // (all batch entries count: the slices of a K shared out are batch entries, and follow what was decided for the whole)
  const uint64_t k_bytes = uint64_t(g.k) * es, b_bytes = k_bytes * g.n * g.batch;
  const uint32_t few = kind == 3 ? 4 : 2;   // rows of A up to which the stream, not the arithmetic, sets the time
  if (k_bytes >= 16384 && g.n <= 2048) return false;   // (its slices, once K is shared out, may come back here: 2 x 8192 x 1024 bf16 7.6 us that way)
  if (g.m > few && b_bytes > (g.m <= 2 * few ? (8ull << 20) : (4ull << 20))) return false;
  return g.b_kmajor && g.m >= 1 && g.m <= uint32_t(MRL_GEMV_MAX_M) && g.n >= 64 && int64_t(g.k) * es >= 1024 &&
         g.k % per16 == 0 && g.lda % per16 == 0 && g.ldb % per16 == 0 && g.sa % per16 == 0 && g.sb % per16 == 0 &&
         al16(g.a) && al16(g.b) && (reinterpret_cast<uintptr_t>(g.c) & 3) == 0 && g.batch <= 65535 &&
         uint64_t(g.n) < (1ull << 31);
}

hipError_t launch_gemv(const GemmArgs &g, int kind, hipStream_t stream) {
  if (!gemv_applicable(g, kind)) return hipErrorInvalidValue;
  switch (kind) {
    case 0: return launch_rows<0>(g, stream);
    case 1: return launch_rows<1>(g, stream);
    case 2: return launch_rows<2>(g, stream);
    default: return launch_rows<3>(g, stream);
  }
}

}  // namespace mrl
