// f32 Softmax over a contiguous innermost dim: y = exp(x - max) / sum(exp(x - max))
// (morello/src/spec.rs:86-90; oracle morello/src/verification.rs:166-184).
//
// Morello decomposes Softmax into max / denominator / normalise passes over the row
// (morello/src/scheduling/to_softmax_parts.rs:33-181, examples/softmax2.rs:47-113: three
// trips through memory).  Here one wavefront owns a row, keeps it in registers between the
// passes (one HBM read, one HBM write per element) and reduces with cross-lane shuffles;
// rows too long for the register budget fall back to re-reading, and the per-lane partial
// (max, denom) pairs are merged with the reference's online formula
// new = max(a,b); d = d_a*exp(a-new) + d_b*exp(b-new) (morello/src/spec.rs:116-123).
#include "kernels.h"

namespace mrl {
namespace {

__device__ inline float wave_max(float v) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) v = fmaxf(v, __shfl_xor(v, o));
  return v;
}
__device__ inline float wave_sum(float v) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o);
  return v;
}

typedef float f4 __attribute__((ext_vector_type(4)));
constexpr float F32_MIN = -3.40282347e+38f;  // f32::MIN, the oracle's max identity

// f32 -> bf16, round to nearest even (softmax values are finite and in [0, 1]).
__device__ inline uint32_t bf16_bits(float f) {
  const uint32_t bits = __float_as_uint(f);
  return (bits + 0x7fffu + ((bits >> 16) & 1u)) >> 16;
}

// NV float4 vectors per lane; cols is a multiple of 4 and <= NV * 256.  OUT_BF16: the result is
// written as bf16 (the left operand of the product that follows a Softmax in a Compose whose
// inputs are bf16).
template <int NV, bool OUT_BF16>
__global__ __launch_bounds__(256) void k_softmax_regs(const float *__restrict__ in,
                                                      void *__restrict__ out_any, uint64_t rows,
                                                      uint32_t cols) {
  float *out = static_cast<float *>(out_any);
  const uint64_t row = uint64_t(blockIdx.x) * 4 + (threadIdx.x >> 6);
  if (row >= rows) return;
  const uint32_t lane = threadIdx.x & 63;
  const float4 *src = (const float4 *)(in + row * cols);
  float4 *dst = (float4 *)(out + row * cols);
  const uint32_t nvec = cols / 4;
  float4 v[NV];
  float mx = F32_MIN;
  bool nan = false;
#pragma unroll
  for (int i = 0; i < NV; i++) {
    const uint32_t idx = i * 64 + lane;
    if (idx < nvec) {
      // Streamed once: keep it out of the caches' way.
      const f4 t = __builtin_nontemporal_load((const f4 *)src + idx);
      v[i] = float4{t[0], t[1], t[2], t[3]};
      nan |= (v[i].x != v[i].x) | (v[i].y != v[i].y) | (v[i].z != v[i].z) | (v[i].w != v[i].w);
      mx = fmaxf(fmaxf(mx, fmaxf(v[i].x, v[i].y)), fmaxf(v[i].z, v[i].w));
    }
  }
  mx = wave_max(mx);
  if (__any(nan)) mx = __uint_as_float(0x7fc00000u);
  float sum = 0.0f;
#pragma unroll
  for (int i = 0; i < NV; i++) {
    const uint32_t idx = i * 64 + lane;
    if (idx < nvec) {
      v[i].x = expf(v[i].x - mx);
      v[i].y = expf(v[i].y - mx);
      v[i].z = expf(v[i].z - mx);
      v[i].w = expf(v[i].w - mx);
      sum += (v[i].x + v[i].y) + (v[i].z + v[i].w);
    }
  }
  sum = wave_sum(sum);
#pragma unroll
  for (int i = 0; i < NV; i++) {
    const uint32_t idx = i * 64 + lane;
    if (idx < nvec) {
      v[i].x /= sum, v[i].y /= sum, v[i].z /= sum, v[i].w /= sum;
      if constexpr (OUT_BF16) {
        typedef unsigned u2 __attribute__((ext_vector_type(2)));
        u2 *dst16 = reinterpret_cast<u2 *>(static_cast<uint16_t *>(out_any) + row * cols);
        __builtin_nontemporal_store(u2{bf16_bits(v[i].x) | (bf16_bits(v[i].y) << 16), bf16_bits(v[i].z) | (bf16_bits(v[i].w) << 16)},
                                    dst16 + idx);
      } else {
        __builtin_nontemporal_store(f4{v[i].x, v[i].y, v[i].z, v[i].w}, (f4 *)dst + idx);
      }
    }
  }
}

// Any cols: each lane runs the online (max, denom) update over its elements, the lanes'
// pairs are merged, then the row is read again to write exp(x - max) / denom.
template <bool OUT_BF16>
__global__ __launch_bounds__(256) void k_softmax_stream(const float *__restrict__ in,
                                                        void *__restrict__ out_any, uint64_t rows,
                                                        uint32_t cols) {
  float *out = static_cast<float *>(out_any);
  const uint64_t row = uint64_t(blockIdx.x) * 4 + (threadIdx.x >> 6);
  if (row >= rows) return;
  const uint32_t lane = threadIdx.x & 63;
  const float *src = in + row * cols;
  float *dst = out + row * cols;
  float mx = F32_MIN, den = 0.0f;
  bool nan = false;
  for (uint32_t i = lane; i < cols; i += 64) {
    const float x = src[i];
    nan |= x != x;
    const float nm = fmaxf(mx, x);
    den = den * expf(mx - nm) + expf(x - nm);
    mx = nm;
  }
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) {
    const float om = __shfl_xor(mx, o), od = __shfl_xor(den, o);
    const float nm = fmaxf(mx, om);
    den = den * expf(mx - nm) + od * expf(om - nm);
    mx = nm;
  }
  if (__any(nan)) mx = __uint_as_float(0x7fc00000u);
  for (uint32_t i = lane; i < cols; i += 64) {
    const float y = expf(src[i] - mx) / den;
    if constexpr (OUT_BF16) (static_cast<uint16_t *>(out_any) + row * cols)[i] = uint16_t(bf16_bits(y));
    else dst[i] = y;
  }
}

}  // namespace

namespace {
template <bool OUT_BF16>
hipError_t launch_rows(const float *in, void *out, uint64_t rows, uint32_t cols, hipStream_t stream) {
  if (rows == 0 || cols == 0) return hipSuccess;
  const uint64_t blocks64 = (rows + 3) / 4;
  if (blocks64 > 0x7fffffffull) return hipErrorInvalidValue;
  const dim3 grid{uint32_t(blocks64)}, block{256};
  if (cols % 4 == 0 && cols <= 16 * 256) {
    const uint32_t nv = (cols / 4 + 63) / 64;
    if (nv <= 1) hipLaunchKernelGGL((k_softmax_regs<1, OUT_BF16>), grid, block, 0, stream, in, out, rows, cols);
    else if (nv <= 2) hipLaunchKernelGGL((k_softmax_regs<2, OUT_BF16>), grid, block, 0, stream, in, out, rows, cols);
    else if (nv <= 4) hipLaunchKernelGGL((k_softmax_regs<4, OUT_BF16>), grid, block, 0, stream, in, out, rows, cols);
    else if (nv <= 8) hipLaunchKernelGGL((k_softmax_regs<8, OUT_BF16>), grid, block, 0, stream, in, out, rows, cols);
    else hipLaunchKernelGGL((k_softmax_regs<16, OUT_BF16>), grid, block, 0, stream, in, out, rows, cols);
  } else {
    hipLaunchKernelGGL(k_softmax_stream<OUT_BF16>, grid, block, 0, stream, in, out, rows, cols);
  }
  return hipGetLastError();
}
}  // namespace

hipError_t launch_softmax_rows(const float *in, float *out, uint64_t rows, uint32_t cols,
                               hipStream_t stream) {
  return launch_rows<false>(in, out, rows, cols, stream);
}

hipError_t launch_softmax_rows_bf16(const float *in, void *out, uint64_t rows, uint32_t cols,
                                    hipStream_t stream) {
  return launch_rows<true>(in, out, rows, cols, stream);
}

}  // namespace mrl
