// f32 Softmax over a contiguous innermost dim: y = exp(x - max) / sum(exp(x - max))
// (morello/src/spec.rs:86-90; oracle morello/src/verification.rs:166-184).
//
// Morello decomposes Softmax into max / denominator / normalise passes over the row
// (morello/src/scheduling/to_softmax_parts.rs:33-181, examples/softmax2.rs:47-113: three
// trips through memory).  Here one wavefront owns a row, keeps it in registers between the
// passes (one HBM read, one HBM write per element) and reduces with cross-lane shuffles;
// rows too long for that are taken in chunks by whole workgroups, whose partial (max, denom)
// pairs are merged with the reference's online formula
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
      const f4 t = MRL_LOAD_ONCE((const f4 *)src + idx);
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

// The same for rows that are not whole 16-byte vectors (cols not a multiple of 4, so rows start
// on any 4 bytes): NE scalars per lane, element i * 64 + lane, cols <= NE * 64.
template <int NE, bool OUT_BF16>
__global__ __launch_bounds__(256) void k_softmax_regs1(const float *__restrict__ in, void *__restrict__ out_any,
                                                       uint64_t rows, uint32_t cols) {
  const uint64_t row = uint64_t(blockIdx.x) * 4 + (threadIdx.x >> 6);
  if (row >= rows) return;
  const uint32_t lane = threadIdx.x & 63;
  const float *src = in + row * cols;
  float v[NE];
  float mx = F32_MIN;
  bool nan = false;
#pragma unroll
  for (int i = 0; i < NE; i++) {
    const uint32_t e = i * 64 + lane;
    v[i] = e < cols ? MRL_LOAD_ONCE(src + e) : F32_MIN;
    nan |= v[i] != v[i];
    mx = fmaxf(mx, v[i]);
  }
  mx = wave_max(mx);
  if (__any(nan)) mx = __uint_as_float(0x7fc00000u);
  float sum = 0.0f;
#pragma unroll
  for (int i = 0; i < NE; i++) {
    v[i] = expf(v[i] - mx);
    sum += uint32_t(i * 64) + lane < cols ? v[i] : 0.0f;
  }
  sum = wave_sum(sum);
#pragma unroll
  for (int i = 0; i < NE; i++) {
    const uint32_t e = i * 64 + lane;
    if (e >= cols) continue;
    const float y = v[i] / sum;
    if constexpr (OUT_BF16) (static_cast<uint16_t *>(out_any) + row * cols)[e] = uint16_t(bf16_bits(y));
    else __builtin_nontemporal_store(y, static_cast<float *>(out_any) + row * cols + e);
  }
}

// Rows of up to 256 elements: L lanes per row (a power of two, 64 / L rows per wavefront), up to
// eight elements per lane in registers, the reductions by shuffles within the L lanes.  A wavefront
// per row would leave most lanes idle and cost a wavefront's fixed work for a handful of elements
// (2.7 million rows of 67: 1.28 ms).
template <int L, bool OUT_BF16>
__global__ __launch_bounds__(256) void k_softmax_short(const float *__restrict__ in, void *__restrict__ out_any,
                                                       uint64_t rows, uint32_t cols) {
  constexpr int PER = 8;
  const uint64_t thread = uint64_t(blockIdx.x) * 256 + threadIdx.x;
  const uint64_t row = thread / L;
  const uint32_t j = uint32_t(thread % L);
  const bool live = row < rows;
  const float *src = in + (live ? row : 0) * cols;
  float x[PER];
  float mx = F32_MIN;
  bool nan = false;
#pragma unroll
  for (int i = 0; i < PER; i++) {
    const uint32_t e = j + i * L;
    x[i] = (live && e < cols) ? src[e] : F32_MIN;
    nan |= x[i] != x[i];
    mx = fmaxf(mx, x[i]);
  }
#pragma unroll
  for (int o = L / 2; o > 0; o >>= 1) {
    mx = fmaxf(mx, __shfl_xor(mx, o));
    nan |= __shfl_xor(int(nan), o) != 0;
  }
  if (nan) mx = __uint_as_float(0x7fc00000u);
  float sum = 0.0f;
#pragma unroll
  for (int i = 0; i < PER; i++) {
    x[i] = expf(x[i] - mx);
    sum += (j + i * L < cols) ? x[i] : 0.0f;
  }
#pragma unroll
  for (int o = L / 2; o > 0; o >>= 1) sum += __shfl_xor(sum, o);
  if (!live) return;
#pragma unroll
  for (int i = 0; i < PER; i++) {
    const uint32_t e = j + i * L;
    if (e >= cols) continue;
    const float y = x[i] / sum;
    if constexpr (OUT_BF16) (static_cast<uint16_t *>(out_any) + row * cols)[e] = uint16_t(bf16_bits(y));
    else MRL_STORE_ONCE(y, static_cast<float *>(out_any) + row * cols + e);
  }
}

template <int L, bool OUT_BF16>
hipError_t launch_short(const float *in, void *out, uint64_t rows, uint32_t cols, hipStream_t stream) {
  const uint64_t blocks = (rows * L + 255) / 256;
  if (blocks > 0x7fffffffull) return hipErrorInvalidValue;
  MRL_LAUNCH((k_softmax_short<L, OUT_BF16>), dim3(uint32_t(blocks)), dim3(256), 0, stream, in, out, rows, cols);
  return mrl::plan::last_error();
}

// ---- rows longer than the register kernel takes: a workgroup per 4096-element chunk ----
// One wavefront per row leaves a few long rows (64 x 100000) on a handful of compute units, and
// its scalar loop waits out every load.  Here a workgroup owns SOFTMAX_CHUNK consecutive elements
// of one row, 16 per thread in registers: k_softmax_chunk_stats writes the chunk's (max,
// denominator) pair, k_softmax_chunk_write merges the pairs of its row with the parts formula
// (morello/src/spec.rs:107-132), reads its chunk again (from the cache, for tensors that fit
// it) and writes exp(x - max) / denominator.  V: floats per load (4 when cols is a multiple
// of 4, so that every chunk and row starts on 16 bytes; else 1).
constexpr uint32_t CHUNK = SOFTMAX_CHUNK, PER_THREAD = CHUNK / 256;

template <int V>
__device__ inline void load_chunk(const float *__restrict__ row, uint32_t first, uint32_t cols, float (&x)[PER_THREAD],
                                  uint32_t &valid) {
  valid = 0;
#pragma unroll
  for (uint32_t i = 0; i < PER_THREAD / V; i++) {
    const uint32_t idx = first + (i * 256 + threadIdx.x) * V;
    if (idx < cols) {
      valid |= ((1u << V) - 1) << (i * V);
      if constexpr (V == 4) {
        const f4 t = *(const f4 *)(row + idx);
        x[4 * i] = t[0], x[4 * i + 1] = t[1], x[4 * i + 2] = t[2], x[4 * i + 3] = t[3];
      } else {
        x[i] = row[idx];
      }
    } else {
#pragma unroll
      for (int j = 0; j < V; j++) x[i * V + j] = F32_MIN;
    }
  }
}

// (max, denominator) pairs of the four waves -> the workgroup's, in every thread.
__device__ inline void merge_waves(float &mx, float &den, bool &nan, float (*lds)[4]) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) {
    const float om = __shfl_xor(mx, o), od = __shfl_xor(den, o);
    const float nm = fmaxf(mx, om);
    den = den * expf(mx - nm) + od * expf(om - nm);
    mx = nm;
  }
  nan = __any(nan);
  const uint32_t w = threadIdx.x >> 6;
  if ((threadIdx.x & 63) == 0) lds[0][w] = mx, lds[1][w] = den, lds[2][w] = nan ? 1.0f : 0.0f;
  __syncthreads();
  mx = lds[0][0], den = lds[1][0], nan = lds[2][0] != 0.0f;
#pragma unroll
  for (int o = 1; o < 4; o++) {
    const float om = lds[0][o], od = lds[1][o];
    const float nm = fmaxf(mx, om);
    den = den * expf(mx - nm) + od * expf(om - nm);
    mx = nm;
    nan |= lds[2][o] != 0.0f;
  }
}

template <int V>
__global__ __launch_bounds__(256) void k_softmax_chunk_stats(const float *__restrict__ in, float2 *__restrict__ stats,
                                                             uint32_t cols, uint32_t chunks) {
  __shared__ float lds[3][4];
  const uint32_t chunk = blockIdx.x % chunks;
  const uint64_t row = blockIdx.x / chunks;
  float x[PER_THREAD];
  uint32_t valid;
  load_chunk<V>(in + row * cols, chunk * CHUNK, cols, x, valid);
  float mx = F32_MIN;
  bool nan = false;
#pragma unroll
  for (uint32_t i = 0; i < PER_THREAD; i++) {
    nan |= x[i] != x[i];
    mx = fmaxf(mx, x[i]);  // slots past the row hold f32::MIN
  }
  float den = 0.0f;
#pragma unroll
  for (uint32_t i = 0; i < PER_THREAD; i++) den += (valid >> i & 1) ? expf(x[i] - mx) : 0.0f;
  merge_waves(mx, den, nan, lds);
  if (threadIdx.x == 0) stats[blockIdx.x] = float2{nan ? __uint_as_float(0x7fc00000u) : mx, den};
}

template <int V, bool OUT_BF16>
__global__ __launch_bounds__(256) void k_softmax_chunk_write(const float *__restrict__ in, void *__restrict__ out_any,
                                                             const float2 *__restrict__ stats, uint32_t cols,
                                                             uint32_t chunks) {
  __shared__ float lds[3][4];
  const uint32_t chunk = blockIdx.x % chunks;
  const uint64_t row = blockIdx.x / chunks;
  // The chunk first: it may be overwritten below (the Spec's output can be its input's buffer).
  float x[PER_THREAD];
  uint32_t valid;
  load_chunk<V>(in + row * cols, chunk * CHUNK, cols, x, valid);
  float mx = F32_MIN, den = 0.0f;
  bool nan = false;
  for (uint32_t c = threadIdx.x; c < chunks; c += 256) {
    const float2 s = stats[row * chunks + c];
    nan |= s.x != s.x;
    const float nm = fmaxf(mx, s.x);
    den = den * expf(mx - nm) + s.y * expf(s.x - nm);
    mx = nm;
  }
  merge_waves(mx, den, nan, lds);
  if (nan) mx = __uint_as_float(0x7fc00000u);
#pragma unroll
  for (uint32_t i = 0; i < PER_THREAD / V; i++) {
    const uint32_t idx = chunk * CHUNK + (i * 256 + threadIdx.x) * V;
    if (idx >= cols) continue;
    float y[V];
#pragma unroll
    for (int j = 0; j < V; j++) y[j] = expf(x[i * V + j] - mx) / den;
    if constexpr (V == 4 && OUT_BF16) {
      typedef unsigned u2 __attribute__((ext_vector_type(2)));
      __builtin_nontemporal_store(u2{bf16_bits(y[0]) | (bf16_bits(y[1]) << 16), bf16_bits(y[2]) | (bf16_bits(y[3]) << 16)},
                                  reinterpret_cast<u2 *>(static_cast<uint16_t *>(out_any) + row * cols + idx));
    } else if constexpr (V == 4) {
      __builtin_nontemporal_store(f4{y[0], y[1], y[2], y[3]}, (f4 *)(static_cast<float *>(out_any) + row * cols + idx));
    } else if constexpr (OUT_BF16) {
      (static_cast<uint16_t *>(out_any) + row * cols)[idx] = uint16_t(bf16_bits(y[0]));
    } else {
      (static_cast<float *>(out_any) + row * cols)[idx] = y[0];
    }
  }
}

// Rows of 4096 < cols <= NV * 1024 (cols a multiple of 4) when there are rows enough to fill
// the chip with a workgroup each: the row stays in the workgroup's registers between the passes,
// as in k_softmax_regs, so it is read once.
template <int NV, bool OUT_BF16>
__global__ __launch_bounds__(256) void k_softmax_block(const float *__restrict__ in, void *__restrict__ out_any,
                                                       uint32_t cols) {
  __shared__ float lds[2][4];
  const uint64_t row = blockIdx.x;
  const uint32_t nvec = cols / 4, w = threadIdx.x >> 6;
  const f4 *src = (const f4 *)(in + row * cols);
  f4 v[NV];
  float mx = F32_MIN;
  bool nan = false;
#pragma unroll
  for (int i = 0; i < NV; i++) {
    const uint32_t idx = i * 256 + threadIdx.x;
    if (idx < nvec) {
      v[i] = MRL_LOAD_ONCE(src + idx);
      nan |= (v[i][0] != v[i][0]) | (v[i][1] != v[i][1]) | (v[i][2] != v[i][2]) | (v[i][3] != v[i][3]);
      mx = fmaxf(fmaxf(mx, fmaxf(v[i][0], v[i][1])), fmaxf(v[i][2], v[i][3]));
    }
  }
  mx = wave_max(mx);
  if ((threadIdx.x & 63) == 0) lds[0][w] = __any(nan) ? __uint_as_float(0x7fc00000u) : mx;
  __syncthreads();
  {
    const float a = lds[0][0], b = lds[0][1], c = lds[0][2], d = lds[0][3];
    mx = (a != a || b != b || c != c || d != d) ? __uint_as_float(0x7fc00000u) : fmaxf(fmaxf(a, b), fmaxf(c, d));
  }
  float sum = 0.0f;
#pragma unroll
  for (int i = 0; i < NV; i++) {
    const uint32_t idx = i * 256 + threadIdx.x;
    if (idx < nvec) {
#pragma unroll
      for (int j = 0; j < 4; j++) v[i][j] = expf(v[i][j] - mx);
      sum += (v[i][0] + v[i][1]) + (v[i][2] + v[i][3]);
    }
  }
  sum = wave_sum(sum);
  if ((threadIdx.x & 63) == 0) lds[1][w] = sum;
  __syncthreads();
  sum = (lds[1][0] + lds[1][1]) + (lds[1][2] + lds[1][3]);
#pragma unroll
  for (int i = 0; i < NV; i++) {
    const uint32_t idx = i * 256 + threadIdx.x;
    if (idx < nvec) {
      const f4 y = v[i] / sum;
      if constexpr (OUT_BF16) {
        typedef unsigned u2 __attribute__((ext_vector_type(2)));
        __builtin_nontemporal_store(u2{bf16_bits(y[0]) | (bf16_bits(y[1]) << 16), bf16_bits(y[2]) | (bf16_bits(y[3]) << 16)},
                                    reinterpret_cast<u2 *>(static_cast<uint16_t *>(out_any) + row * cols) + idx);
      } else {
        __builtin_nontemporal_store(y, (f4 *)(static_cast<float *>(out_any) + row * cols) + idx);
      }
    }
  }
}

template <int V, bool OUT_BF16>
hipError_t launch_chunks(const float *in, void *out, uint64_t rows, uint32_t cols, float2 *stats, hipStream_t stream) {
  const uint32_t chunks = (cols + CHUNK - 1) / CHUNK;
  const dim3 grid{uint32_t(rows * chunks)}, block{256};
  plan::work(plan::UNIT_STREAM, 0, 4.0 * rows * cols);
  MRL_LAUNCH(k_softmax_chunk_stats<V>, grid, block, 0, stream, in, stats, cols, chunks);
  plan::work(plan::UNIT_STREAM, 0, double(rows) * cols * (4 + (OUT_BF16 ? 2 : 4)));
  MRL_LAUNCH((k_softmax_chunk_write<V, OUT_BF16>), grid, block, 0, stream, in, out, stats, cols, chunks);
  return mrl::plan::last_error();
}

}  // namespace

namespace {
template <bool OUT_BF16>
hipError_t launch_rows(const float *in, void *out, uint64_t rows, uint32_t cols, void *scratch, hipStream_t stream) {
  if (rows == 0 || cols == 0) return hipSuccess;
  if (cols <= 256 && rows * 32 <= 0x7fffffffull * 256) {
    plan::work(plan::UNIT_STREAM, 0, double(rows) * cols * (4 + (OUT_BF16 ? 2 : 4)));
    if (cols <= 8) return launch_short<1, OUT_BF16>(in, out, rows, cols, stream);
    if (cols <= 16) return launch_short<2, OUT_BF16>(in, out, rows, cols, stream);
    if (cols <= 32) return launch_short<4, OUT_BF16>(in, out, rows, cols, stream);
    if (cols <= 64) return launch_short<8, OUT_BF16>(in, out, rows, cols, stream);
    if (cols <= 128) return launch_short<16, OUT_BF16>(in, out, rows, cols, stream);
    return launch_short<32, OUT_BF16>(in, out, rows, cols, stream);
  }
  // A workgroup per row with the row in registers: rows beyond the wavefront kernel's 4096
  // columns when there are 256 of them or more, and rows of more than 1024 columns when there are
  // too few of them to occupy the chip a wavefront each.
  if (cols % 4 == 0 && rows <= 0x7fffffffull &&
      ((cols > 16 * 256 && cols <= 16 * 1024 && rows >= 256) || (cols > 1024 && cols <= 16 * 256 && rows < 2048))) {
    plan::work(plan::UNIT_STREAM, 0, double(rows) * cols * (4 + (OUT_BF16 ? 2 : 4)));
    if (cols <= 8 * 1024) MRL_LAUNCH((k_softmax_block<8, OUT_BF16>), dim3(uint32_t(rows)), dim3(256), 0, stream, in, out, cols);
    else MRL_LAUNCH((k_softmax_block<16, OUT_BF16>), dim3(uint32_t(rows)), dim3(256), 0, stream, in, out, cols);
    return mrl::plan::last_error();
  }
  if (cols % 4 != 0 && cols <= 64 * 64 && rows >= 512 && (rows + 3) / 4 <= 0x7fffffffull) {
    const dim3 grid{uint32_t((rows + 3) / 4)}, block{256};
    plan::work(plan::UNIT_STREAM, 0, double(rows) * cols * (4 + (OUT_BF16 ? 2 : 4)));
    if (cols <= 16 * 64) MRL_LAUNCH((k_softmax_regs1<16, OUT_BF16>), grid, block, 0, stream, in, out, rows, cols);
    else if (cols <= 32 * 64) MRL_LAUNCH((k_softmax_regs1<32, OUT_BF16>), grid, block, 0, stream, in, out, rows, cols);
    else MRL_LAUNCH((k_softmax_regs1<64, OUT_BF16>), grid, block, 0, stream, in, out, rows, cols);
    return mrl::plan::last_error();
  }
  if (scratch && softmax_scratch_bytes(rows, cols)) {
    if (cols % 4 == 0) return launch_chunks<4, OUT_BF16>(in, out, rows, cols, static_cast<float2 *>(scratch), stream);
    return launch_chunks<1, OUT_BF16>(in, out, rows, cols, static_cast<float2 *>(scratch), stream);
  }
  const uint64_t blocks64 = (rows + 3) / 4;
  if (blocks64 > 0x7fffffffull) return hipErrorInvalidValue;
  const dim3 grid{uint32_t(blocks64)}, block{256};
  plan::work(plan::UNIT_STREAM, 0, double(rows) * cols * (4 + (OUT_BF16 ? 2 : 4)));
  if (cols % 4 == 0 && cols <= 16 * 256) {
    const uint32_t nv = (cols / 4 + 63) / 64;
    if (nv <= 1) MRL_LAUNCH((k_softmax_regs<1, OUT_BF16>), grid, block, 0, stream, in, out, rows, cols);
    else if (nv <= 2) MRL_LAUNCH((k_softmax_regs<2, OUT_BF16>), grid, block, 0, stream, in, out, rows, cols);
    else if (nv <= 4) MRL_LAUNCH((k_softmax_regs<4, OUT_BF16>), grid, block, 0, stream, in, out, rows, cols);
    else if (nv <= 8) MRL_LAUNCH((k_softmax_regs<8, OUT_BF16>), grid, block, 0, stream, in, out, rows, cols);
    else MRL_LAUNCH((k_softmax_regs<16, OUT_BF16>), grid, block, 0, stream, in, out, rows, cols);
  } else {
    return hipErrorInvalidValue;  // rows in chunks, and no scratch was passed for them
  }
  return mrl::plan::last_error();
}
}  // namespace

// Scratch the chunked kernels want for this shape (0: the shape runs without).
size_t softmax_scratch_bytes(uint64_t rows, uint32_t cols) {
  // Up to 4096 columns the register kernels serve; fewer than 512 rows that are not whole
  // vectors go in chunks too (a single one), with scalar loads.
  if (cols <= 16 * 256 && (cols % 4 == 0 || cols <= 256 || rows >= 512)) return 0;
  const uint64_t chunks = (cols + SOFTMAX_CHUNK - 1) / SOFTMAX_CHUNK;
  if (rows * chunks > 0x7fffffffull) return 0;
  return size_t(rows * chunks * sizeof(float2));
}

hipError_t launch_softmax_rows(const float *in, float *out, uint64_t rows, uint32_t cols, void *scratch,
                               hipStream_t stream) {
  return launch_rows<false>(in, out, rows, cols, scratch, stream);
}

hipError_t launch_softmax_rows_bf16(const float *in, void *out, uint64_t rows, uint32_t cols, void *scratch,
                                    hipStream_t stream) {
  return launch_rows<true>(in, out, rows, cols, scratch, stream);
}

}  // namespace mrl
