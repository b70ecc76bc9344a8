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
// The tensors are strided f32; a line is the scan dim at fixed coordinates in the others.  Three
// ways of sharing the lines out, chosen by shape and strides (launch_parts):
//   k_parts        a wavefront per line, lane i takes elements i, i + 64, ..; any strides, any length;
//   k_parts_rows   the same for contiguous lines of up to 4096 elements in whole 16-byte vectors: the
//                  line stays in the wavefront's registers between the passes over it, so a Spec
//                  that needs the maximum before the exponentials still reads its input once;
//   k_parts_cols   the scan dim is not the innermost one: C adjacent lines side by side in a
//                  workgroup (adjacent in memory when the innermost dim is contiguous, so a
//                  wavefront's loads are whole cache lines), each shared by 256 / C threads that
//                  walk the scan dim in steps of 256 / C and combine through LDS; with C = 256, a
//                  thread per line, also the form for lines of a handful of elements.
// The arithmetic is written once (parts_line) over a Share: how the threads of a line divide
// it and combine their partial results.
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

// Offsets of a line's first element per parameter and the parameters' steps along the scan dim.
struct Line {
  int64_t base[4], step[4];
};
__device__ inline Line line_of(const PartsArgs &p, uint64_t line) {
  // Constant loop bounds throughout: with indices known at compile time the eight offsets live in
  // registers (arrays indexed at run time are placed in LDS or scratch).
  Line l;
#pragma unroll
  for (int t = 0; t < 4; t++) l.base[t] = 0;
  if (p.lines < (1ull << 31)) {
    // multiply-and-shift (FastDiv: exact below 2^31) where a 64-bit division by a run-time value is
    // a hundred instructions and more, per dim, in front of the line's first load
    uint32_t r = uint32_t(line);
#pragma unroll
    for (int d = MRL_MAX_RANK - 1; d >= 0; d--) {
      if (uint32_t(d) >= p.rank || uint32_t(d) == p.scan_dim) continue;
      const uint32_t q = p.by_shape[d].div(r), c = r - q * p.shape[d];
      r = q;
#pragma unroll
      for (int t = 0; t < 4; t++) l.base[t] += int64_t(c) * p.stride[t][d];   // 0 for a parameter the Spec does not have
    }
  } else {
    uint64_t r = line;
#pragma unroll
    for (int d = MRL_MAX_RANK - 1; d >= 0; d--) {
      if (uint32_t(d) >= p.rank || uint32_t(d) == p.scan_dim) continue;
      const uint32_t c = uint32_t(r % p.shape[d]);
      r /= p.shape[d];
#pragma unroll
      for (int t = 0; t < 4; t++) l.base[t] += int64_t(c) * p.stride[t][d];
    }
  }
#pragma unroll
  for (int t = 0; t < 4; t++) {
    int64_t step = 0;
#pragma unroll
    for (int d = 0; d < MRL_MAX_RANK; d++) step = uint32_t(d) == p.scan_dim ? p.stride[t][d] : step;
    l.step[t] = step;
  }
  return l;
}

// A wavefront per line.
struct WaveShare {
  uint32_t first, stride;
  bool lead;
  __device__ float max(float v) const { return wave_max(v); }
  __device__ float sum(float v) const { return wave_sum(v); }
};
// A workgroup of four wavefronts per line: a wavefront's partial result first, then the four meet in LDS.
struct BlockShare {
  uint32_t first, stride;
  bool lead;
  float *lds;  // [4]
  template <bool MAX>
  __device__ float combine(float v) const {
    v = MAX ? wave_max(v) : wave_sum(v);
    __syncthreads();  // the previous round's readers are done
    if ((threadIdx.x & 63) == 0) lds[threadIdx.x >> 6] = v;
    __syncthreads();
    const float a = lds[0], b = lds[1], c = lds[2], d = lds[3];
    return MAX ? fmaxf(fmaxf(a, b), fmaxf(c, d)) : (a + b) + (c + d);
  }
  __device__ float max(float v) const { return combine<true>(v); }
  __device__ float sum(float v) const { return combine<false>(v); }
};
// 256 / C threads of a workgroup per line, C lines side by side: partial results meet in LDS.
template <int C>
struct GroupShare {
  static constexpr int G = 256 / C;
  uint32_t first, stride;
  bool lead;
  float *lds;  // [G][C]
  uint32_t col;
  template <bool MAX>
  __device__ float combine(float v) const {
    if constexpr (G == 1) return v;   // a thread per line: nothing to combine
    __syncthreads();  // the previous round's readers are done
    lds[first * C + col] = v;
    __syncthreads();
    float r = lds[col];
#pragma unroll
    for (int g = 1; g < G; g++) r = MAX ? fmaxf(r, lds[g * C + col]) : r + lds[g * C + col];
    return r;
  }
  __device__ float max(float v) const { return combine<true>(v); }
  __device__ float sum(float v) const { return combine<false>(v); }
};

// One line of one of the Specs.  n: the line's length for this thread (0 for a thread whose
// line lies past the end: it takes part in the combining steps and touches no memory).  A
// thread takes its elements eight at a time, the eight loads issued before the first is used.
template <class S>
__device__ inline void parts_line(const PartsArgs &p, const Line &l, const S &sh, uint32_t n, bool live) {
  float *const *q = p.ptr;
#define AT(t, i) q[t][l.base[t] + int64_t(i) * l.step[t]]
#define RED(t) q[t][l.base[t]]  // a parameter whose scan dim has size one
#define EACH8(i) for (uint32_t i = sh.first; i < n; i += 8 * sh.stride)
#define LOAD8(x, t, i, pad)                                   \
  float x[8];                                                 \
  _Pragma("unroll") for (uint32_t k = 0; k < 8; k++) {        \
    const uint32_t at = i + k * sh.stride;                    \
    x[k] = at < n ? AT(t, at) : pad;                          \
  }
#define STORE8(t, i, x)                                       \
  _Pragma("unroll") for (uint32_t k = 0; k < 8; k++) {        \
    const uint32_t at = i + k * sh.stride;                    \
    if (at < n) MRL_STORE_ONCE(x[k], &AT(t, at));             \
  }
  auto line_max = [&](uint32_t t) {
    float m = NEG_INF;
    EACH8(i) {
      LOAD8(x, t, i, NEG_INF)
      m = fmaxf(fmaxf(fmaxf(m, fmaxf(x[0], x[1])), fmaxf(x[2], x[3])), fmaxf(fmaxf(x[4], x[5]), fmaxf(x[6], x[7])));
    }
    return sh.max(m);
  };
  // sum of exp(x - m) over the line; the exponentials go to parameter `to` if there is one
  auto line_exp = [&](float m, int to) {
    float d = 0.0f;
    EACH8(i) {
      LOAD8(x, 0, i, NEG_INF)   // exp(-inf - m) = 0 for the positions past the end
#pragma unroll
      for (int k = 0; k < 8; k++) x[k] = expf(x[k] - m);
      if (to >= 0) { STORE8(to, i, x) }
      d += ((x[0] + x[1]) + (x[2] + x[3])) + ((x[4] + x[5]) + (x[6] + x[7]));
    }
    return sh.sum(d);
  };
  switch (p.kind) {
    case MRL_SPEC_MAX: {  // [in, out]
      const float m = line_max(0);
      if (live && sh.lead) RED(1) = p.accum ? fmaxf(RED(1), m) : m;
      break;
    }
    case MRL_SPEC_SOFTMAX_DENOMINATOR: {  // [in, max, denom]
      const float d = line_exp(live ? RED(1) : 0.0f, -1);
      if (live && sh.lead) RED(2) = (p.accum ? RED(2) : 0.0f) + d;
      break;
    }
    case MRL_SPEC_SOFTMAX_DENOMINATOR_AND_MAX:               // [in, max, denom]
    case MRL_SPEC_SOFTMAX_DENOMINATOR_AND_MAX_FROM_PARTS: {  // [tile_max, tile_denom, out_max, out_denom]
      // The online recurrence, eight elements (or tiles) a step: one pass over the line.
      const bool parts = p.kind == MRL_SPEC_SOFTMAX_DENOMINATOR_AND_MAX_FROM_PARTS;
      const int om = parts ? 2 : 1, od = parts ? 3 : 2;
      const float m0 = p.accum && live ? RED(om) : NEG_INF, d0 = p.accum && live ? RED(od) : 0.0f;
      float m = NEG_INF, d = 0.0f;
      EACH8(i) {
        LOAD8(x, 0, i, NEG_INF)
        float w[8];
        if (parts) {
          LOAD8(y, 1, i, 0.0f)
#pragma unroll
          for (int k = 0; k < 8; k++) w[k] = y[k];
        }
        const float bm = fmaxf(fmaxf(fmaxf(x[0], x[1]), fmaxf(x[2], x[3])), fmaxf(fmaxf(x[4], x[5]), fmaxf(x[6], x[7])));
        if (bm > m) {
          d *= expf(m - bm);
          m = bm;
        }
#pragma unroll
        for (int k = 0; k < 8; k++) {
          // An element of -inf (and a position past the end) is exp(-inf - max) = 0 against any
          // maximum the line ends up with but -inf itself, which is settled below.
          const float e = x[k] == NEG_INF ? 0.0f : expf(x[k] - m);
          d += parts ? w[k] * e : e;
        }
      }
      const float mm = fmaxf(m0, sh.max(m));
      // a share that saw nothing but -inf (m = -inf, d = 0) adds nothing
      d = sh.sum(d == 0.0f ? 0.0f : d * expf(m - mm));
      if (mm == NEG_INF) d = __builtin_nanf("");   // every term was exp(-inf - -inf)
      if (live && sh.lead) {
        RED(od) = (p.accum ? d0 * expf(m0 - mm) : 0.0f) + d;
        RED(om) = mm;
      }
      break;
    }
    case MRL_SPEC_SOFTMAX_DENOMINATOR_AND_UNSCALED: {  // [in, denom, unscaled]
      const float d = line_exp(line_max(0), 2);
      if (live && sh.lead) RED(1) = d;
      break;
    }
    case MRL_SPEC_SOFTMAX_DENOMINATOR_AND_UNSCALED_FROM_MAX: {  // [in, max, denom, unscaled]
      const float d = line_exp(live ? RED(1) : 0.0f, 3);
      if (live && sh.lead) RED(2) = (p.accum ? RED(2) : 0.0f) + d;
      break;
    }
    case MRL_SPEC_SOFTMAX_COMPLETE: {  // [in, max, denom, out]
      const float m = live ? RED(1) : 0.0f, d = live ? RED(2) : 1.0f;
      EACH8(i) {
        LOAD8(x, 0, i, 0.0f)
#pragma unroll
        for (int k = 0; k < 8; k++) x[k] = expf(x[k] - m) / d;
        STORE8(3, i, x)
      }
      break;
    }
    case MRL_SPEC_DIVIDE_VEC: {  // [numer, denom], same shape
      EACH8(i) {
        LOAD8(x, 0, i, 0.0f)
        LOAD8(y, 1, i, 1.0f)
#pragma unroll
        for (int k = 0; k < 8; k++) x[k] = x[k] / y[k];
        STORE8(0, i, x)
      }
      break;
    }
    case MRL_SPEC_DIVIDE_VEC_SCALAR: {  // [numer, denom (scan dim of size one)]
      const float d = live ? RED(1) : 1.0f;
      EACH8(i) {
        LOAD8(x, 0, i, 0.0f)
#pragma unroll
        for (int k = 0; k < 8; k++) x[k] = x[k] / d;
        STORE8(0, i, x)
      }
      break;
    }
    default:
      break;
  }
#undef STORE8
#undef LOAD8
#undef EACH8
#undef AT
#undef RED
}

__global__ __launch_bounds__(256) void k_parts(PartsArgs p) {
  const uint64_t line = uint64_t(blockIdx.x) * 4 + (threadIdx.x >> 6);
  if (line >= p.lines) return;
  const uint32_t lane = threadIdx.x & 63;
  const WaveShare sh{lane, 64, lane == 0};
  parts_line(p, line_of(p, line), sh, p.shape[p.scan_dim], true);
}

// Few long lines: a workgroup per line (a wavefront per line would leave most of the chip's load
// queues empty: 1000 lines of 65536, denominator and max 138 -> 62 us).
__global__ __launch_bounds__(256) void k_parts_block(PartsArgs p) {
  __shared__ float lds[4];
  const BlockShare sh{threadIdx.x, 256, threadIdx.x == 0, lds};
  parts_line(p, line_of(p, blockIdx.x), sh, p.shape[p.scan_dim], true);
}

template <int C>
__global__ __launch_bounds__(256) void k_parts_cols(PartsArgs p) {
  __shared__ float lds[256];
  const uint32_t col = threadIdx.x % C, group = threadIdx.x / C;
  const uint64_t line = uint64_t(blockIdx.x) * C + col;
  const bool live = line < p.lines;
  const GroupShare<C> sh{group, 256 / C, group == 0, lds, col};
  parts_line(p, line_of(p, live ? line : 0), sh, live ? p.shape[p.scan_dim] : 0, live);
}

// Contiguous lines of n <= NV * 256 elements, n a multiple of 4, every line of every full-size
// parameter starting on 16 bytes: the line in registers, one read of it whatever the Spec.
template <int NV>
__global__ __launch_bounds__(256) void k_parts_rows(PartsArgs p) {
  typedef float f4 __attribute__((ext_vector_type(4)));
  const uint64_t line = uint64_t(blockIdx.x) * 4 + (threadIdx.x >> 6);
  if (line >= p.lines) return;
  const uint32_t lane = threadIdx.x & 63;
  const Line l = line_of(p, line);
  const uint32_t nvec = p.shape[p.scan_dim] / 4;
  float *const *q = p.ptr;
#define RED(t) q[t][l.base[t]]
#define VEC(t) ((f4 *)(q[t] + l.base[t]))
#define EACH(i, idx) for (uint32_t i = 0, idx = lane; i < NV; i++, idx += 64) if (idx < nvec)
  f4 v[NV];
  {
    const f4 *x = VEC(0);
#pragma unroll
    EACH(i, idx) v[i] = x[idx];
  }
  auto line_max = [&]() {
    float m = NEG_INF;
#pragma unroll
    EACH(i, idx) m = fmaxf(fmaxf(m, fmaxf(v[i][0], v[i][1])), fmaxf(v[i][2], v[i][3]));
    return wave_max(m);
  };
  // v <- exp(v - m); returns the line's sum of them
  auto exponentials = [&](float m) {
    float d = 0.0f;
#pragma unroll
    EACH(i, idx) {
#pragma unroll
      for (int r = 0; r < 4; r++) v[i][r] = expf(v[i][r] - m);
      d += (v[i][0] + v[i][1]) + (v[i][2] + v[i][3]);
    }
    return wave_sum(d);
  };
  auto store = [&](f4 *dst) {
#pragma unroll
    EACH(i, idx) MRL_STORE_ONCE(v[i], dst + idx);
  };
  switch (p.kind) {
    case MRL_SPEC_MAX: {
      const float m = line_max();
      if (lane == 0) RED(1) = p.accum ? fmaxf(RED(1), m) : m;
      break;
    }
    case MRL_SPEC_SOFTMAX_DENOMINATOR: {
      const float d = exponentials(RED(1));
      if (lane == 0) RED(2) = (p.accum ? RED(2) : 0.0f) + d;
      break;
    }
    case MRL_SPEC_SOFTMAX_DENOMINATOR_AND_MAX: {
      const float m0 = p.accum ? RED(1) : NEG_INF, d0 = p.accum ? RED(2) : 0.0f;
      const float m = fmaxf(m0, line_max());
      const float d = exponentials(m);
      if (lane == 0) {
        RED(2) = (p.accum ? d0 * expf(m0 - m) : 0.0f) + d;
        RED(1) = m;
      }
      break;
    }
    case MRL_SPEC_SOFTMAX_DENOMINATOR_AND_UNSCALED: {
      const float d = exponentials(line_max());
      store(VEC(2));
      if (lane == 0) RED(1) = d;
      break;
    }
    case MRL_SPEC_SOFTMAX_DENOMINATOR_AND_UNSCALED_FROM_MAX: {
      const float d = exponentials(RED(1));
      store(VEC(3));
      if (lane == 0) RED(2) = (p.accum ? RED(2) : 0.0f) + d;
      break;
    }
    case MRL_SPEC_SOFTMAX_COMPLETE: {
      const float m = RED(1), d = RED(2);
#pragma unroll
      EACH(i, idx) {
#pragma unroll
        for (int r = 0; r < 4; r++) v[i][r] = expf(v[i][r] - m) / d;
      }
      store(VEC(3));
      break;
    }
    case MRL_SPEC_DIVIDE_VEC_SCALAR: {
      const float d = RED(1);
#pragma unroll
      EACH(i, idx) {
#pragma unroll
        for (int r = 0; r < 4; r++) v[i][r] = v[i][r] / d;
      }
      store(VEC(0));
      break;
    }
    case MRL_SPEC_DIVIDE_VEC: {   // the denominators' line vector by vector beside the numerators'
      const f4 *den = VEC(1);
#pragma unroll
      EACH(i, idx) v[i] = v[i] / den[idx];
      store(VEC(0));
      break;
    }
    default:
      break;
  }
#undef EACH
#undef VEC
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

// Broadcast between row-major tensors, seen as out[before][n][after] <- in[before][after] in 16-byte
// units of `after`: a thread loads its unit once and stores it to its share of the n positions
// (blockIdx.y shares n out when before * after alone would not fill the chip).
typedef uint32_t u4 __attribute__((ext_vector_type(4)));
__global__ __launch_bounds__(256) void k_broadcast_rows(const u4 *__restrict__ in, u4 *__restrict__ out, uint64_t units,
                                                        uint32_t after, uint32_t n, uint32_t chunk) {
  const uint64_t t = uint64_t(blockIdx.x) * 256 + threadIdx.x;
  if (t >= units) return;
  const uint64_t b = units <= 0xffffffffull ? uint32_t(t) / after : t / after;
  const uint32_t a = uint32_t(t - b * after);
  const u4 v = in[t];
  const uint32_t i0 = blockIdx.y * chunk, i1 = min(n, i0 + chunk);
  u4 *dst = out + (b * n + i0) * after + a;
  for (uint32_t i = i0; i < i1; i++, dst += after) __builtin_nontemporal_store(v, dst);
}

// The innermost dim broadcast: out[row][0 .. n) <- in[row], n elements of ES bytes filling whole
// 16-byte units; a thread writes one unit.
template <int ES>
__global__ __launch_bounds__(256) void k_broadcast_fill_rows(const uint8_t *__restrict__ in, u4 *__restrict__ out,
                                                             uint64_t units, uint32_t per_row) {
  const uint64_t t = uint64_t(blockIdx.x) * 256 + threadIdx.x;
  if (t >= units) return;
  const uint64_t row = units <= 0xffffffffull ? uint32_t(t) / per_row : t / per_row;
  uint32_t w;
  if (ES == 1) w = in[row] * 0x01010101u;
  else if (ES == 2) w = ((const uint16_t *)in)[row] * 0x00010001u;
  else w = ((const uint32_t *)in)[row];
  __builtin_nontemporal_store(u4{w, w, w, w}, out + t);
}

__global__ void k_fill(uint8_t *out, uint32_t pattern, uint32_t es, uint64_t count) {
  const uint64_t i = uint64_t(blockIdx.x) * blockDim.x + threadIdx.x;
  if (i >= count) return;
  if (es == 1) out[i] = uint8_t(pattern);
  else if (es == 2) ((uint16_t *)out)[i] = uint16_t(pattern);
  else ((uint32_t *)out)[i] = pattern;
}

}  // namespace

// A parameter that has the scan dim in full (the others hold one value per line).
inline bool full_size(const PartsArgs &p, uint32_t t) { return p.stride[t][p.scan_dim] != 0; }

hipError_t launch_parts(const PartsArgs &args, hipStream_t stream) {
  if (args.lines == 0) return hipSuccess;
  PartsArgs p = args;
  for (uint32_t d = 0; d < p.rank && d < MRL_MAX_RANK; d++) p.by_shape[d] = FastDiv(std::max(1u, p.shape[d]));
  const uint32_t n = p.shape[p.scan_dim];
  // Contiguous lines in whole, aligned 16-byte vectors: the register-resident form.
  bool rows = n % 4 == 0 && n > 1 && n <= 4096 && p.kind != MRL_SPEC_SOFTMAX_DENOMINATOR_AND_MAX_FROM_PARTS && full_size(p, 0);
  // Lines side by side: the dim along which consecutive lines differ (the last one that is not
  // the scan dim) is contiguous in the full-size parameters, as the innermost dim of a row-major
  // tensor scanned along another dim is, or dim 0 of a column-major matrix scanned along dim 1.
  uint32_t last = p.rank - 1;
  if (last == p.scan_dim && last > 0) last--;
  bool cols = p.rank >= 2 && p.scan_dim != last && p.shape[last] >= 16;
  for (uint32_t t = 0; t < p.n_params; t++) {
    if (!full_size(p, t)) continue;
    rows = rows && p.stride[t][p.scan_dim] == 1 && (reinterpret_cast<uintptr_t>(p.ptr[t]) & 15) == 0;
    for (uint32_t d = 0; d < p.rank; d++)
      if (d != p.scan_dim && p.shape[d] > 1) rows = rows && p.stride[t][d] % 4 == 0;
    cols = cols && p.stride[t][last] == 1;
  }
  const uint64_t blocks = (p.lines + 3) / 4;
  if (blocks > 0x7fffffffull) return hipErrorInvalidValue;
  // Full-size tensors read and written; the register-resident form alone reads its input once
  // where the maximum must be known before the exponentials are written.
  double passes = 1;
  switch (p.kind) {
    case MRL_SPEC_SOFTMAX_DENOMINATOR_AND_MAX_FROM_PARTS:
    case MRL_SPEC_SOFTMAX_DENOMINATOR_AND_UNSCALED_FROM_MAX:
    case MRL_SPEC_SOFTMAX_COMPLETE:
    case MRL_SPEC_DIVIDE_VEC_SCALAR: passes = 2; break;
    case MRL_SPEC_SOFTMAX_DENOMINATOR_AND_UNSCALED: passes = rows ? 2 : 3; break;
    case MRL_SPEC_DIVIDE_VEC: passes = 3; break;
    default: break;
  }
  plan::work(plan::UNIT_STREAM, 0, 4.0 * passes * p.lines * n);
  if (n <= 16 && p.lines >= 1024) {
    // Lines of a handful of elements (the merge of a few tiles' pairs): a thread per line; a
    // wavefront per line would leave all but a few lanes idle (65536 lines of 2: 25 us).
    MRL_LAUNCH(k_parts_cols<256>, dim3(uint32_t((p.lines + 255) / 256)), dim3(256), 0, stream, p);
  } else if (rows) {
    if (n <= 1024) MRL_LAUNCH(k_parts_rows<4>, dim3(uint32_t(blocks)), dim3(256), 0, stream, p);
    else if (n <= 2048) MRL_LAUNCH(k_parts_rows<8>, dim3(uint32_t(blocks)), dim3(256), 0, stream, p);
    else MRL_LAUNCH(k_parts_rows<16>, dim3(uint32_t(blocks)), dim3(256), 0, stream, p);
  } else if (cols) {
    // Narrower tiles while that takes the workgroups towards two per compute unit; 16 lines are
    // still whole 64-byte pieces of the rows.
    const uint64_t want = 2ull * g_compute_units;
    if (p.lines / 64 >= want)
      MRL_LAUNCH(k_parts_cols<64>, dim3(uint32_t((p.lines + 63) / 64)), dim3(256), 0, stream, p);
    else if (p.lines / 32 >= want)
      MRL_LAUNCH(k_parts_cols<32>, dim3(uint32_t((p.lines + 31) / 32)), dim3(256), 0, stream, p);
    else
      MRL_LAUNCH(k_parts_cols<16>, dim3(uint32_t((p.lines + 15) / 16)), dim3(256), 0, stream, p);
  } else if (n >= 4096 && p.lines <= 8ull * g_compute_units) {
    MRL_LAUNCH(k_parts_block, dim3(uint32_t(p.lines)), dim3(256), 0, stream, p);
  } else {
    MRL_LAUNCH(k_parts, dim3(uint32_t(blocks)), dim3(256), 0, stream, p);
  }
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
// Fill in 16-byte stores of the replicated pattern; the elements past the last whole 16 bytes are
// written one each by the first threads.
__global__ __launch_bounds__(256) void k_fill16(u4 *out, uint32_t word, uint64_t units, uint8_t *tail, uint32_t tail_elems,
                                                uint32_t es) {
  const uint64_t t = uint64_t(blockIdx.x) * 256 + threadIdx.x;
  if (t < units) __builtin_nontemporal_store(u4{word, word, word, word}, out + t);
  if (t < tail_elems) {
    if (es == 1) tail[t] = uint8_t(word);
    else if (es == 2) ((uint16_t *)tail)[t] = uint16_t(word);
    else ((uint32_t *)tail)[t] = word;
  }
}

bool launch_broadcast_rows(const void *in, void *out, uint64_t before, uint32_t n, uint64_t after, uint32_t es,
                           hipStream_t stream, hipError_t *err) {
  if (before == 0 || n == 0 || after == 0) return false;
  if ((reinterpret_cast<uintptr_t>(in) | reinterpret_cast<uintptr_t>(out)) & 15) return false;
  const double bytes = double(before) * n * after * es;
  if (after * es % 16 == 0 && after * es / 16 <= 0xffffffffull) {
    const uint32_t after_units = uint32_t(after * es / 16);
    const uint64_t units = before * after_units;
    const uint64_t blocks = (units + 255) / 256;
    if (blocks > 0x7fffffffull) return false;
    // enough workgroups for every compute unit to hold a few
    const uint32_t share = uint32_t(std::min<uint64_t>(std::min<uint32_t>(n, 65535u), std::max<uint64_t>(1, 8ull * g_compute_units / blocks)));
    const uint32_t chunk = (n + share - 1) / share;
    plan::work(plan::UNIT_STREAM, 0, bytes);
    MRL_LAUNCH(k_broadcast_rows, dim3(uint32_t(blocks), (n + chunk - 1) / chunk), dim3(256), 0, stream, (const u4 *)in,
               (u4 *)out, units, after_units, n, chunk);
    *err = mrl::plan::last_error();
    return true;
  }
  if (after == 1 && uint64_t(n) * es % 16 == 0) {
    const uint32_t per_row = uint32_t(uint64_t(n) * es / 16);
    const uint64_t units = before * per_row;
    const uint64_t blocks = (units + 255) / 256;
    if (blocks > 0x7fffffffull) return false;
    plan::work(plan::UNIT_STREAM, 0, bytes);
    if (es == 1) MRL_LAUNCH(k_broadcast_fill_rows<1>, dim3(uint32_t(blocks)), dim3(256), 0, stream, (const uint8_t *)in, (u4 *)out, units, per_row);
    else if (es == 2) MRL_LAUNCH(k_broadcast_fill_rows<2>, dim3(uint32_t(blocks)), dim3(256), 0, stream, (const uint8_t *)in, (u4 *)out, units, per_row);
    else MRL_LAUNCH(k_broadcast_fill_rows<4>, dim3(uint32_t(blocks)), dim3(256), 0, stream, (const uint8_t *)in, (u4 *)out, units, per_row);
    *err = mrl::plan::last_error();
    return true;
  }
  return false;
}

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
  const uint64_t units = count * es / 16;
  if ((reinterpret_cast<uintptr_t>(out) & 15) == 0 && units > 0 && (units + 255) / 256 <= 0x7fffffffull) {
    const uint32_t word = es == 1 ? pattern * 0x01010101u : es == 2 ? pattern * 0x00010001u : pattern;
    MRL_LAUNCH(k_fill16, dim3(uint32_t((units + 255) / 256)), dim3(256), 0, stream, (u4 *)out, word, units,
               (uint8_t *)out + units * 16, uint32_t((count * es - units * 16) / es), es);
    return mrl::plan::last_error();
  }
  MRL_LAUNCH(k_fill, dim3(uint32_t((count + 255) / 256)), dim3(256), 0, stream, (uint8_t *)out,
                     pattern, es, count);
  return mrl::plan::last_error();
}

}  // namespace mrl
