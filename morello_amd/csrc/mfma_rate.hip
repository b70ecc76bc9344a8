// Measures what the matrix cores of this board sustain, as opposed to the datasheet peak:
// every SIMD issues back-to-back MFMAs on register operands (no memory traffic at all) for
// long enough that the clock settles at the board's power limit.  With all-zero operands
// the datapath barely toggles and the rate sits near the nominal figure; with operands
// drawn like a benchmark's (uniform bytes, or bf16 values of N(0,1) shape) the clock drops
// and so does the rate.  The second number is the ceiling any Matmul kernel on such data
// can approach here; bench.py reports it beside the nominal peak.  The MFMAs are the 16 x 16 forms
// (v_mfma_i32_16x16x64_i8, v_mfma_f32_16x16x32_bf16): on random operands they sustain more than
// the 32 x 32 forms of the same nominal rate (4000 against 3360 TOPS int8, 2070 against 1840
// TFLOPS bf16 on an MI355X), one accumulator update per 64 multiply-adds instead of per 32, so
// theirs is the ceiling.
#include <vector>

#include "kernels.h"

namespace mrl {
namespace {

typedef int v4i __attribute__((ext_vector_type(4)));
typedef float v4f __attribute__((ext_vector_type(4)));
typedef __bf16 v8bf __attribute__((ext_vector_type(8)));

constexpr int OPERANDS = 8;  // distinct A and B register quads per lane
constexpr int CHAINS = 8;    // independent accumulators
constexpr int PER_ITER = 64; // MFMAs per loop iteration and wave

template <bool BF16>
__global__ __launch_bounds__(512) void k_mfma_rate(const v4i *src, float *sink, uint32_t iters) {
  v4i a[OPERANDS], b[OPERANDS];
#pragma unroll
  for (int i = 0; i < OPERANDS; i++) {
    a[i] = src[i * 512 + threadIdx.x];
    b[i] = src[(OPERANDS + i) * 512 + threadIdx.x];
  }
  v4f accf[CHAINS];
  v4i acci[CHAINS];
#pragma unroll
  for (int c = 0; c < CHAINS; c++)
#pragma unroll
    for (int r = 0; r < 4; r++) accf[c][r] = 0.0f, acci[c][r] = 0;
  for (uint32_t it = 0; it < iters; it++) {
#pragma unroll
    for (int u = 0; u < PER_ITER; u++) {
      const int c = u % CHAINS, ia = u % OPERANDS, ib = (u / CHAINS) % OPERANDS;
      if (BF16)
        accf[c] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(v8bf, a[ia]),
                                                          __builtin_bit_cast(v8bf, b[ib]), accf[c], 0, 0, 0);
      else
        acci[c] = __builtin_amdgcn_mfma_i32_16x16x64_i8(a[ia], b[ib], acci[c], 0, 0, 0);
    }
  }
  float s = 0.0f;
#pragma unroll
  for (int c = 0; c < CHAINS; c++)
#pragma unroll
    for (int r = 0; r < 4; r++) s += accf[c][r] + float(acci[c][r]);
  sink[blockIdx.x * 512 + threadIdx.x] = s;
}

}  // namespace

// kind 0: int8 (v_mfma_i32_16x16x64_i8), 1: bf16 (v_mfma_f32_16x16x32_bf16).
// Returns operations (2 per multiply-add) per second over `iters` iterations per wave.
hipError_t measure_mfma_rate(int kind, bool random_operands, uint32_t iters, hipStream_t stream,
                             double *ops_per_second) {
  int cus = 0;
  hipError_t e = hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, 0);
  if (e != hipSuccess) return e;
  const size_t quads = size_t(2 * OPERANDS) * 512;
  std::vector<v4i> host(quads);
  uint64_t x = 0x9E3779B97F4A7C15ull;
  for (size_t i = 0; i < quads; i++)
    for (int c = 0; c < 4; c++) {
      x ^= x << 13, x ^= x >> 7, x ^= x << 17;  // xorshift64
      uint32_t v = uint32_t(x >> 16);
      if (kind == 1) {
        // Two bf16 values of magnitude [0.25, 2) with random sign and mantissa.
        const uint32_t lo = ((v & 0x8000u) | 0x3e80u | (v & 0xffu)) + ((v >> 8) & 0x100u);
        const uint32_t hi = (((v >> 16) & 0x8000u) | 0x3e80u | ((v >> 16) & 0xffu)) + ((v >> 24) & 0x100u);
        v = (lo & 0xffffu) | (hi << 16);
      }
      host[i][c] = random_operands ? int(v) : 0;
    }
  v4i *src = nullptr;
  float *sink = nullptr;
  hipEvent_t e0 = nullptr, e1 = nullptr;
  auto cleanup = [&]() {
    if (src) (void)hipFree(src);
    if (sink) (void)hipFree(sink);
    if (e0) (void)hipEventDestroy(e0);
    if (e1) (void)hipEventDestroy(e1);
  };
#define TRY(x)              \
  if ((e = (x)) != hipSuccess) { \
    cleanup();              \
    return e;               \
  }
  TRY(hipMalloc(&src, quads * sizeof(v4i)));
  TRY(hipMalloc(&sink, size_t(cus) * 512 * sizeof(float)));
  TRY(hipMemcpyAsync(src, host.data(), quads * sizeof(v4i), hipMemcpyHostToDevice, stream));
  TRY(hipEventCreate(&e0));
  TRY(hipEventCreate(&e1));
  auto launch = [&](uint32_t n) {
    if (kind == 1) hipLaunchKernelGGL(k_mfma_rate<true>, dim3(cus), dim3(512), 0, stream, src, sink, n);
    else hipLaunchKernelGGL(k_mfma_rate<false>, dim3(cus), dim3(512), 0, stream, src, sink, n);
    return hipGetLastError();
  };
  TRY(launch(iters / 8 + 1));  // warm-up, also brings the clock down to its loaded level
  TRY(hipEventRecord(e0, stream));
  TRY(launch(iters));
  TRY(hipEventRecord(e1, stream));
  TRY(hipEventSynchronize(e1));
  float ms = 0.0f;
  TRY(hipEventElapsedTime(&ms, e0, e1));
#undef TRY
  const double ops_per_mfma = 2.0 * 16 * 16 * (kind == 1 ? 32 : 64);
  *ops_per_second = double(iters) * PER_ITER * 8 * cus * ops_per_mfma / (double(ms) * 1e-3);
  cleanup();
  return hipSuccess;
}

}  // namespace mrl
