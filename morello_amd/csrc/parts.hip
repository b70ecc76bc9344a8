// The remaining primitive Specs of Morello's Softmax decomposition as stand-alone GPU ops
// (morello/src/spec.rs:57-162): Max, SoftmaxDenominator, SoftmaxDenominatorAndMax,
// SoftmaxDenominatorAndMaxFromParts, SoftmaxDenominatorAndUnscaled,
// SoftmaxDenominatorAndUnscaledFromMax, SoftmaxComplete, DivideVec, DivideVecScalar, plus
// Broadcast and Fill.  Their arithmetic is what the emitter's scalar kernels print
// (morello/src/codegen/cpu.rs:1350-1433, 1968-2113, 3103-3227) applied along the scan dim:
//   Max                       out = max(out?, x_i)
//   SoftmaxDenominator        d (+)= sum exp(x_i - max)
//   SoftmaxDenominatorAndMax  new = max(old, x); d = d*exp(old-new) + exp(x-new)   (online)
//   ...FromParts              new = max(m, tm_t); d = d*exp(m-new) + td_t*exp(tm_t-new)
//   ...AndUnscaled            e_i = exp(x_i - max_k x_k); d = sum e_i
//   ...AndUnscaledFromMax     e_i = exp(x_i - max); d (+)= sum e_i
//   SoftmaxComplete           y_i = exp(x_i - max) / d
//   DivideVec / DivideVecScalar   a_i /= b_i  /  a_i /= b        (true division)
// One wavefront owns one line along the scan dim of strided f32 tensors; these are the
// building blocks a caller composes when it schedules Softmax by hand, not throughput
// kernels (the fused forms live in softmax.hip and attention.hip).
#include "kernels.h"

namespace mrl {
namespace {

constexpr float NEG_INF = -__builtin_inff();

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

__global__ __launch_bounds__(256) void k_parts(PartsArgs p) {
  const uint64_t line = uint64_t(blockIdx.x) * 4 + (threadIdx.x >> 6);
  if (line >= p.lines) return;
  const uint32_t lane = threadIdx.x & 63;
  // Coordinates of the line in every dim but the scan dim -> base offset per parameter.
  int64_t base[4] = {0, 0, 0, 0};
  uint64_t r = line;
  for (int d = int(p.rank) - 1; d >= 0; d--) {
    if (uint32_t(d) == p.scan_dim) continue;
    const uint32_t c = uint32_t(r % p.shape[d]);
    r /= p.shape[d];
    for (uint32_t t = 0; t < p.n_params; t++) base[t] += int64_t(c) * p.stride[t][d];
  }
  const uint32_t n = p.shape[p.scan_dim];
  int64_t step[4];
  for (uint32_t t = 0; t < 4; t++) step[t] = t < p.n_params ? p.stride[t][p.scan_dim] : 0;
  float *const *q = p.ptr;
#define AT(t, i) q[t][base[t] + int64_t(i) * step[t]]
#define RED(t) q[t][base[t]]  // a parameter whose scan dim has size one

  switch (p.kind) {
    case MRL_SPEC_MAX: {  // [in, out]
      float m = p.accum ? RED(1) : NEG_INF;
      for (uint32_t i = lane; i < n; i += 64) m = fmaxf(m, AT(0, i));
      m = wave_max(m);
      if (lane == 0) RED(1) = m;
      break;
    }
    case MRL_SPEC_SOFTMAX_DENOMINATOR: {  // [in, max, denom]
      const float m = RED(1);
      float d = 0.0f;
      for (uint32_t i = lane; i < n; i += 64) d += expf(AT(0, i) - m);
      d = wave_sum(d);
      if (lane == 0) RED(2) = (p.accum ? RED(2) : 0.0f) + d;
      break;
    }
    case MRL_SPEC_SOFTMAX_DENOMINATOR_AND_MAX: {  // [in, max, denom]
      const float m0 = p.accum ? RED(1) : NEG_INF, d0 = p.accum ? RED(2) : 0.0f;
      float m = m0;
      for (uint32_t i = lane; i < n; i += 64) m = fmaxf(m, AT(0, i));
      m = wave_max(m);
      float d = 0.0f;
      for (uint32_t i = lane; i < n; i += 64) d += expf(AT(0, i) - m);
      d = wave_sum(d);
      if (lane == 0) {
        RED(2) = (p.accum ? d0 * expf(m0 - m) : 0.0f) + d;
        RED(1) = m;
      }
      break;
    }
    case MRL_SPEC_SOFTMAX_DENOMINATOR_AND_MAX_FROM_PARTS: {  // [tile_max, tile_denom, out_max, out_denom]
      const float m0 = p.accum ? RED(2) : NEG_INF, d0 = p.accum ? RED(3) : 0.0f;
      float m = m0;
      for (uint32_t i = lane; i < n; i += 64) m = fmaxf(m, AT(0, i));
      m = wave_max(m);
      float d = 0.0f;
      for (uint32_t i = lane; i < n; i += 64) d += AT(1, i) * expf(AT(0, i) - m);
      d = wave_sum(d);
      if (lane == 0) {
        RED(3) = (p.accum ? d0 * expf(m0 - m) : 0.0f) + d;
        RED(2) = m;
      }
      break;
    }
    case MRL_SPEC_SOFTMAX_DENOMINATOR_AND_UNSCALED: {  // [in, denom, unscaled]
      float m = NEG_INF;
      for (uint32_t i = lane; i < n; i += 64) m = fmaxf(m, AT(0, i));
      m = wave_max(m);
      float d = 0.0f;
      for (uint32_t i = lane; i < n; i += 64) {
        const float e = expf(AT(0, i) - m);
        AT(2, i) = e;
        d += e;
      }
      d = wave_sum(d);
      if (lane == 0) RED(1) = d;
      break;
    }
    case MRL_SPEC_SOFTMAX_DENOMINATOR_AND_UNSCALED_FROM_MAX: {  // [in, max, denom, unscaled]
      const float m = RED(1);
      float d = 0.0f;
      for (uint32_t i = lane; i < n; i += 64) {
        const float e = expf(AT(0, i) - m);
        AT(3, i) = e;
        d += e;
      }
      d = wave_sum(d);
      if (lane == 0) RED(2) = (p.accum ? RED(2) : 0.0f) + d;
      break;
    }
    case MRL_SPEC_SOFTMAX_COMPLETE: {  // [in, max, denom, out]
      const float m = RED(1), d = RED(2);
      for (uint32_t i = lane; i < n; i += 64) AT(3, i) = expf(AT(0, i) - m) / d;
      break;
    }
    case MRL_SPEC_DIVIDE_VEC: {  // [numer, denom], same shape
      for (uint32_t i = lane; i < n; i += 64) AT(0, i) = AT(0, i) / AT(1, i);
      break;
    }
    case MRL_SPEC_DIVIDE_VEC_SCALAR: {  // [numer, denom (scan dim of size one)]
      const float d = RED(1);
      for (uint32_t i = lane; i < n; i += 64) AT(0, i) = AT(0, i) / d;
      break;
    }
    default:
      break;
  }
#undef AT
#undef RED
}

// Broadcast along `dim`: out[pt] = in[pt with pt[dim] = 0], any element size.
__global__ void k_broadcast(const uint8_t *in, uint8_t *out, LayoutEval il, LayoutEval ol, uint32_t dim,
                            uint32_t es, uint64_t count) {
  const uint64_t i = uint64_t(blockIdx.x) * blockDim.x + threadIdx.x;
  if (i >= count) return;
  uint32_t pt[MRL_MAX_RANK];
  uint64_t rem = i;
  for (int d = int(ol.rank) - 1; d >= 0; d--) {
    pt[d] = uint32_t(rem % ol.shape[d]);
    rem /= ol.shape[d];
  }
  const int64_t d_o = layout_offset(ol, pt);
  pt[dim] = 0;
  const int64_t so = layout_offset(il, pt);
  if (es == 1) out[d_o] = in[so];
  else if (es == 2) ((uint16_t *)out)[d_o] = ((const uint16_t *)in)[so];
  else ((uint32_t *)out)[d_o] = ((const uint32_t *)in)[so];
}

__global__ void k_fill(uint8_t *out, uint32_t pattern, uint32_t es, uint64_t count) {
  const uint64_t i = uint64_t(blockIdx.x) * blockDim.x + threadIdx.x;
  if (i >= count) return;
  if (es == 1) out[i] = uint8_t(pattern);
  else if (es == 2) ((uint16_t *)out)[i] = uint16_t(pattern);
  else ((uint32_t *)out)[i] = pattern;
}

}  // namespace

hipError_t launch_parts(const PartsArgs &p, hipStream_t stream) {
  if (p.lines == 0) return hipSuccess;
  const uint64_t blocks = (p.lines + 3) / 4;
  if (blocks > 0x7fffffffull) return hipErrorInvalidValue;
  plan::work(plan::UNIT_STREAM, 0, 8.0 * p.lines * p.shape[p.scan_dim]);  // the full-size tensors, read and written
  MRL_LAUNCH(k_parts, dim3(uint32_t(blocks)), dim3(256), 0, stream, p);
  return mrl::plan::last_error();
}

hipError_t launch_broadcast(const void *in, void *out, const LayoutEval &il, const LayoutEval &ol,
                            uint32_t dim, uint32_t elem_size, uint64_t count, hipStream_t stream) {
  if (count == 0) return hipSuccess;
  plan::work(plan::UNIT_VALU, 30.0 * count, 2.0 * count * elem_size);
  MRL_LAUNCH(k_broadcast, dim3(uint32_t((count + 255) / 256)), dim3(256), 0, stream,
                     (const uint8_t *)in, (uint8_t *)out, il, ol, dim, elem_size, count);
  return mrl::plan::last_error();
}

// FillValue (spec.rs:165-170): 0 Zero, 1 NegInf (floats), 2 Min (the dtype's minimum;
// f32::MIN / bf16::MIN for floats, as verification.rs:534-545 fills).
hipError_t launch_fill(void *out, int dtype, int fill_value, uint64_t count, hipStream_t stream) {
  if (count == 0) return hipSuccess;
  uint32_t pattern = 0;
  if (fill_value == 1) pattern = dtype == MRL_F32 ? 0xff800000u : 0xff80u;
  if (fill_value == 2) {
    switch (dtype) {
      case MRL_I8: pattern = 0x80u; break;
      case MRL_I16: pattern = 0x8000u; break;
      case MRL_I32: pattern = 0x80000000u; break;
      case MRL_F32: pattern = 0xff7fffffu; break;
      case MRL_BF16: pattern = 0xff7fu; break;
      default: pattern = 0; break;
    }
  }
  const uint32_t es = dtype == MRL_U8 || dtype == MRL_I8 ? 1 : (dtype == MRL_U16 || dtype == MRL_I16 || dtype == MRL_BF16 ? 2 : 4);
  plan::work(plan::UNIT_STREAM, 0, double(count) * es);
  MRL_LAUNCH(k_fill, dim3(uint32_t((count + 255) / 256)), dim3(256), 0, stream, (uint8_t *)out,
                     pattern, es, count);
  return mrl::plan::last_error();
}

}  // namespace mrl
