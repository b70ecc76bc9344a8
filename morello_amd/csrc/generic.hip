// Correctness-first kernels: any dtype combination, any strides, any size.  The MFMA
// kernels cover the shapes that matter for throughput; everything else lands here so that
// every Spec the descriptor can express still runs on the GPU.
//
// Arithmetic follows the reference's oracle (morello/src/verification.rs:115-134,
// 547-569, 603-643): both inputs are converted to the output dtype, then multiplied and
// accumulated in that dtype.  Integer outputs are computed modulo 2^32 and truncated on
// store, which equals wrapping arithmetic in the narrower type.
#include <algorithm>
#include <type_traits>
#include <utility>

#include "kernels.h"
#include "layout_factor.h"

namespace mrl {
namespace {

__device__ inline float bf16_bits_to_f32(uint16_t v) { return __uint_as_float(uint32_t(v) << 16); }

__device__ inline uint32_t narrow_int(int dtype, uint32_t v) {
  switch (dtype) {
    case MRL_U8: return v & 0xffu;
    case MRL_I8: return uint32_t(int32_t(int8_t(uint8_t(v))));
    case MRL_U16: return v & 0xffffu;
    case MRL_I16: return uint32_t(int32_t(int16_t(uint16_t(v))));
    default: return v;
  }
}

__device__ inline float load_f32(const void *p, int dtype, int64_t off) {
  switch (dtype) {
    case MRL_U8: return float(((const uint8_t *)p)[off]);
    case MRL_I8: return float(((const int8_t *)p)[off]);
    case MRL_U16: return float(((const uint16_t *)p)[off]);
    case MRL_I16: return float(((const int16_t *)p)[off]);
    case MRL_U32: return float(((const uint32_t *)p)[off]);
    case MRL_I32: return float(((const int32_t *)p)[off]);
    case MRL_F32: return ((const float *)p)[off];
    default: return bf16_bits_to_f32(((const uint16_t *)p)[off]);
  }
}

// Rust `as` for narrow integer targets saturates floats at the target's own bounds.
__device__ inline uint32_t float_to_int(float f, int dt) {
  if (f != f) return 0;
  float lo, hi;
  switch (dt) {
    case MRL_U8: lo = 0.f, hi = 255.f; break;
    case MRL_I8: lo = -128.f, hi = 127.f; break;
    case MRL_U16: lo = 0.f, hi = 65535.f; break;
    case MRL_I16: lo = -32768.f, hi = 32767.f; break;
    case MRL_U32: return f <= 0.f ? 0u : f >= 4294967296.f ? 0xffffffffu : uint32_t(f);
    default: return f <= -2147483648.f ? 0x80000000u : f >= 2147483648.f ? 0x7fffffffu : uint32_t(int32_t(f));
  }
  f = fminf(fmaxf(f, lo), hi);
  return uint32_t(int32_t(f));
}

// Rust `as` semantics (verification.rs:547-569, `x.as_()` into the output dtype): integers wrap,
// floats saturate at the bounds of the dtype they are cast to and NaN becomes 0.
__device__ inline uint32_t load_u32(const void *p, int dtype, int64_t off, int out_dtype) {
  uint32_t v;
  switch (dtype) {
    case MRL_U8: v = ((const uint8_t *)p)[off]; break;
    case MRL_I8: v = uint32_t(int32_t(((const int8_t *)p)[off])); break;
    case MRL_U16: v = ((const uint16_t *)p)[off]; break;
    case MRL_I16: v = uint32_t(int32_t(((const int16_t *)p)[off])); break;
    case MRL_U32: v = ((const uint32_t *)p)[off]; break;
    case MRL_I32: v = uint32_t(((const int32_t *)p)[off]); break;
    default: v = float_to_int(load_f32(p, dtype, off), out_dtype);
  }
  return narrow_int(out_dtype, v);
}

__device__ inline void store_u32(void *p, int dtype, int64_t off, uint32_t v) {
  switch (dtype) {
    case MRL_U8: case MRL_I8: ((uint8_t *)p)[off] = uint8_t(v); break;
    case MRL_U16: case MRL_I16: case MRL_BF16: ((uint16_t *)p)[off] = uint16_t(v); break;
    default: ((uint32_t *)p)[off] = v; break;
  }
}

// ------------------------------------------------------------------ relayout
__global__ void k_relayout(const uint8_t *src, uint8_t *dst, LayoutEval sl, LayoutEval dl,
                           uint32_t es, uint64_t count) {
  const uint64_t i = uint64_t(blockIdx.x) * blockDim.x + threadIdx.x;
  if (i >= count) return;
  uint32_t pt[MRL_MAX_RANK];
  uint64_t rem = i;
  for (int d = int(sl.rank) - 1; d >= 0; d--) {
    pt[d] = uint32_t(rem % sl.shape[d]);
    rem /= sl.shape[d];
  }
  const int64_t so = layout_offset(sl, pt), d_o = layout_offset(dl, pt);
  if (es == 1) dst[d_o] = src[so];
  else if (es == 2) ((uint16_t *)dst)[d_o] = ((const uint16_t *)src)[so];
  else ((uint32_t *)dst)[d_o] = ((const uint32_t *)src)[so];
}

// ---------------------------------------------------------------------- move
__device__ inline uint16_t f32_to_bf16_bits(float f) {
  uint32_t bits = __float_as_uint(f);
  if ((bits & 0x7fffffffu) > 0x7f800000u) return uint16_t((bits >> 16) | 0x40u);
  bits += 0x7fffu + ((bits >> 16) & 1u);  // round to nearest even
  return uint16_t(bits >> 16);
}

// One element: read as `sdt`, converted with Rust `as` semantics, returned as the bits of `ddt`.
__device__ inline uint32_t move_bits(const void *src, int sdt, int64_t so, int ddt) {
  if (sdt == ddt) {  // bits as they are (a NaN keeps its payload)
    const size_t size = sdt == MRL_U8 || sdt == MRL_I8 ? 1 : sdt == MRL_U16 || sdt == MRL_I16 || sdt == MRL_BF16 ? 2 : 4;
    return size == 1 ? ((const uint8_t *)src)[so] : size == 2 ? ((const uint16_t *)src)[so] : ((const uint32_t *)src)[so];
  }
  const bool src_float = sdt == MRL_F32 || sdt == MRL_BF16;
  if (ddt == MRL_F32) return __float_as_uint(load_f32(src, sdt, so));
  if (ddt == MRL_BF16) return f32_to_bf16_bits(load_f32(src, sdt, so));
  if (src_float) return float_to_int(load_f32(src, sdt, so), ddt);
  return load_u32(src, sdt, so, MRL_U32);  // int -> int wraps
}

// An element's bits, zero-extended, by element size alone (no dtype switch around the load).
template <int SIZE>
__device__ inline uint32_t load_sized(const void *p, int64_t off) {
  if constexpr (SIZE == 1) return static_cast<const uint8_t *>(p)[off];
  else if constexpr (SIZE == 2) return static_cast<const uint16_t *>(p)[off];
  else return static_cast<const uint32_t *>(p)[off];
}
template <int SIZE>
__device__ inline void store_sized(void *p, int64_t off, uint32_t v) {
  if constexpr (SIZE == 1) static_cast<uint8_t *>(p)[off] = uint8_t(v);
  else if constexpr (SIZE == 2) static_cast<uint16_t *>(p)[off] = uint16_t(v);
  else static_cast<uint32_t *>(p)[off] = v;
}

// The same conversions on an element already in a register (`raw`: its bits, zero-extended).
__device__ inline float raw_to_f32(uint32_t raw, int dtype) {
  switch (dtype) {
    case MRL_U8: return float(raw & 0xffu);
    case MRL_I8: return float(int8_t(uint8_t(raw)));
    case MRL_U16: return float(raw & 0xffffu);
    case MRL_I16: return float(int16_t(uint16_t(raw)));
    case MRL_U32: return float(raw);
    case MRL_I32: return float(int32_t(raw));
    case MRL_F32: return __uint_as_float(raw);
    default: return bf16_bits_to_f32(uint16_t(raw));
  }
}
__device__ inline uint32_t convert_raw(uint32_t raw, int sdt, int ddt) {
  if (sdt == ddt) return raw;
  const bool src_float = sdt == MRL_F32 || sdt == MRL_BF16;
  if (ddt == MRL_F32) return __float_as_uint(raw_to_f32(raw, sdt));
  if (ddt == MRL_BF16) return f32_to_bf16_bits(raw_to_f32(raw, sdt));
  if (src_float) return float_to_int(raw_to_f32(raw, sdt), ddt);
  return narrow_int(sdt, raw);  // int -> int: extend by the source's sign, the store truncates
}

// Calls f(source dtype, destination dtype) with the two as compile-time constants
// (std::integral_constant), chosen once by a switch over the dtypes of SE and of DE bytes: inside
// f a conversion is the few instructions it needs, where a switch around every element costs more
// than the conversion (u8 -> bf16 over 64 Mi elements: 60 us that way, 30 this way).
template <int SE, int DE, class F>
__device__ inline void with_dtypes(int sdt, int ddt, F &&f) {
  // (u, i) of one and four bytes, (u, i, bf16) of two
  constexpr int S0 = SE == 1 ? MRL_U8 : SE == 2 ? MRL_U16 : MRL_U32, S1 = S0 + 1, S2 = SE == 2 ? MRL_BF16 : MRL_F32;
  constexpr int D0 = DE == 1 ? MRL_U8 : DE == 2 ? MRL_U16 : MRL_U32, D1 = D0 + 1, D2 = DE == 2 ? MRL_BF16 : MRL_F32;
  const int si = sdt == S0 ? 0 : sdt == S1 ? 1 : 2, di = ddt == D0 ? 0 : ddt == D1 ? 1 : 2;
#define MRL_CASE(A, B)                                                                   \
  case A * 3 + B:                                                                        \
    f(std::integral_constant<int, (A == 0 ? S0 : A == 1 ? S1 : S2)>{},                  \
      std::integral_constant<int, (B == 0 ? D0 : B == 1 ? D1 : D2)>{});                 \
    break;
  switch (si * 3 + di) {
    MRL_CASE(0, 0) MRL_CASE(0, 1) MRL_CASE(0, 2) MRL_CASE(1, 0) MRL_CASE(1, 1) MRL_CASE(1, 2)
    MRL_CASE(2, 0) MRL_CASE(2, 1) MRL_CASE(2, 2)
  }
#undef MRL_CASE
}

// Move of a contiguous run with a dtype conversion: N elements per thread, one vector load
// and one vector store (SE, DE: element sizes in bytes).  N = 4 where an element of four bytes is
// involved, 8 or 16 between narrower ones, so that the wider side moves 16 bytes a thread (u8 ->
// bf16 over 64 Mi elements: 68 us with four elements a thread).
typedef unsigned v2u __attribute__((ext_vector_type(2)));
typedef unsigned v4u_t __attribute__((ext_vector_type(4)));
template <int SE, int DE, int N = 4>
__global__ __launch_bounds__(256) void k_convert4(const void *__restrict__ src, void *__restrict__ dst, int sdt,
                                                  int ddt, uint64_t count) {
  // A pack travels as whole dwords (loads and stores of 4, 8 or 16 bytes, two of 16 for a pack of
  // 32), and an element is cut out of its dword by shifts: through arrays of bytes the compiler
  // narrowed the load of a u16 -> u8 pack to the sixteen bytes the conversion keeps, one load each.
  constexpr int SW = SE * N / 4, DW = DE * N / 4;   // dwords of a pack on either side
  static_assert(SE * N % 4 == 0 && DE * N % 4 == 0, "packs are whole dwords");
  struct alignas(SW >= 4 ? 16 : SW * 4) SrcPack { uint32_t w[SW]; };
  struct alignas(DW >= 4 ? 16 : DW * 4) DstPack { uint32_t w[DW]; };
  const uint64_t packs = count / N, step = uint64_t(gridDim.x) * 256;
  // (the dtypes are switched on once per pack: with_dtypes)
  auto convert_pack = [&](const SrcPack &in, DstPack &out, auto sd, auto dd) {
#pragma unroll
    for (int w = 0; w < DW; w++) out.w[w] = 0;
#pragma unroll
    for (int e = 0; e < N; e++) {
      const uint32_t raw = SE == 4 ? in.w[e] : (in.w[e * SE / 4] >> (8 * (e * SE % 4))) & (SE == 1 ? 0xffu : 0xffffu);
      const uint32_t v = convert_raw(raw, decltype(sd)::value, decltype(dd)::value);
      if constexpr (DE == 4) out.w[e] = v;
      else out.w[e * DE / 4] |= (v & (DE == 1 ? 0xffu : 0xffffu)) << (8 * (e * DE % 4));
    }
  };
  for (uint64_t i = uint64_t(blockIdx.x) * 256 + threadIdx.x; i < packs; i += step) {
    SrcPack in;
    if constexpr (SW == 1) in.w[0] = static_cast<const uint32_t *>(src)[i];
    else if constexpr (SW == 2) { const v2u v = static_cast<const v2u *>(src)[i]; in.w[0] = v[0], in.w[1] = v[1]; }
    else {
#pragma unroll
      for (int q = 0; q < SW / 4; q++) {
        const v4u_t v = static_cast<const v4u_t *>(src)[i * (SW / 4) + q];
#pragma unroll
        for (int k = 0; k < 4; k++) in.w[q * 4 + k] = v[k];
      }
    }
    DstPack out;
    with_dtypes<SE, DE>(sdt, ddt, [&](auto sd, auto dd) { convert_pack(in, out, sd, dd); });
    // the converted elements as one store of 4, 8 or 16 bytes
    static_assert(DW == 1 || DW == 2 || DW == 4, "a pack is stored by one instruction");
    if constexpr (DW == 1) MRL_STORE_ONCE(out.w[0], static_cast<uint32_t *>(dst) + i);
    else if constexpr (DW == 2) MRL_STORE_ONCE((v2u{out.w[0], out.w[1]}), static_cast<v2u *>(dst) + i);
    else MRL_STORE_ONCE((v4u_t{out.w[0], out.w[1], out.w[2], out.w[3]}), static_cast<v4u_t *>(dst) + i);
  }
  // The elements past the last whole pack.
  if (blockIdx.x == 0 && threadIdx.x < count % N) {
    const int64_t at = int64_t(packs * N + threadIdx.x);
    store_u32(dst, ddt, at, move_bits(src, sdt, at, ddt));
  }
}

__global__ void k_move_generic(const void *src, void *dst, LayoutEval sl, LayoutEval dl, int sdt,
                               int ddt, uint64_t count) {
  const uint64_t i = uint64_t(blockIdx.x) * blockDim.x + threadIdx.x;
  if (i >= count) return;
  uint32_t pt[MRL_MAX_RANK];
  uint64_t rem = i;
  for (int d = int(sl.rank) - 1; d >= 0; d--) {
    pt[d] = uint32_t(rem % sl.shape[d]);
    rem /= sl.shape[d];
  }
  const int64_t so = layout_offset(sl, pt), d_o = layout_offset(dl, pt);
  store_u32(dst, ddt, d_o, move_bits(src, sdt, so, ddt));
}

// Move between two layouts that are permutations of the logical dims (element strides on both
// sides).  `order` lists the dims slowest to fastest for the index decode.
struct MoveStrided {
  const void *src;
  void *dst;
  int sdt, ddt;
  uint32_t rank;
  uint32_t shape[MOVE_MAX_RANK];
  int64_t ss[MOVE_MAX_RANK], ds[MOVE_MAX_RANK];
  uint32_t order[MOVE_MAX_RANK];
  uint32_t dim_s, dim_d;      // the dim each side stores contiguously
  uint32_t tiles_s, tiles_d;  // 64-element tiles along them
  uint64_t count;
};

// Both sides contiguous along the same dim: consecutive threads take consecutive elements of
// that dim, so reads and writes are both coalesced.
__global__ __launch_bounds__(256) void k_move_rows(MoveStrided p) {
  const uint64_t i = uint64_t(blockIdx.x) * blockDim.x + threadIdx.x;
  if (i >= p.count) return;
  uint32_t rem = uint32_t(i);  // a tensor has fewer than 2^31 elements
  int64_t so = 0, d_o = 0;
  for (int o = int(p.rank) - 1; o >= 0; o--) {
    const uint32_t d = p.order[o], c = rem % p.shape[d];
    rem /= p.shape[d];
    so += int64_t(c) * p.ss[d], d_o += int64_t(c) * p.ds[d];
  }
  store_u32(p.dst, p.ddt, d_o, move_bits(p.src, p.sdt, so, p.ddt));
}

// The same when nothing is converted and every run along the shared contiguous dim is whole
// 16-byte vectors on both sides: shapes and strides count vectors.
__global__ __launch_bounds__(256) void k_move_rows16(MoveStrided p) {
  const uint64_t i = uint64_t(blockIdx.x) * blockDim.x + threadIdx.x;
  if (i >= p.count) return;
  uint32_t rem = uint32_t(i);
  int64_t so = 0, d_o = 0;
  for (int o = int(p.rank) - 1; o >= 0; o--) {
    const uint32_t d = p.order[o], c = rem % p.shape[d];
    rem /= p.shape[d];
    so += int64_t(c) * p.ss[d], d_o += int64_t(c) * p.ds[d];
  }
  MRL_STORE_ONCE(static_cast<const v4u_t *>(p.src)[so], static_cast<v4u_t *>(p.dst) + d_o);
}

// The two sides are contiguous along different dims: a 64 x 64 tile of (dim_d, dim_s) goes
// through LDS, read with dim_s fastest and written with dim_d fastest, so both sides see
// whole contiguous runs (move_relayout of morello/src/scheduling/moves.rs as a transpose).
template <int SE, int DE>
__global__ __launch_bounds__(256) void k_move_tiled(MoveStrided p) {
  __shared__ uint32_t tile[64][65];
  uint64_t blk = blockIdx.x;
  const uint32_t ts = uint32_t(blk % p.tiles_s);
  blk /= p.tiles_s;
  // Diagonal order: workgroups that run together differ in both tile coordinates.  In row or
  // column order they would all read (or all write) addresses a whole number of rows apart,
  // which with power-of-two row lengths is one memory channel for all of them.
  const uint32_t td = uint32_t((blk + ts) % p.tiles_d);
  blk /= p.tiles_d;
  // The remaining dims, slowest to fastest in `order` (dim_s and dim_d are skipped).
  int64_t so = 0, d_o = 0;
  for (int o = int(p.rank) - 1; o >= 0; o--) {
    const uint32_t d = p.order[o];
    if (d == p.dim_s || d == p.dim_d) continue;
    const uint32_t c = uint32_t(blk % p.shape[d]);
    blk /= p.shape[d];
    so += int64_t(c) * p.ss[d], d_o += int64_t(c) * p.ds[d];
  }
  const uint32_t lane = threadIdx.x & 63, quad = threadIdx.x >> 6;
  const uint32_t s0 = ts * 64, d0 = td * 64, ns = p.shape[p.dim_s], nd = p.shape[p.dim_d];
  // All sixteen loads of a thread are issued before the first is used: a small tensor is a
  // handful of tiles, and their time is these loads' latency.
  uint32_t v[16];
#pragma unroll
  for (uint32_t i = 0; i < 16; i++) {
    const uint32_t r = quad + 4 * i;
    v[i] = 0;
    if (d0 + r < nd && s0 + lane < ns)
      v[i] = load_sized<SE>(p.src, so + int64_t(d0 + r) * p.ss[p.dim_d] + int64_t(s0 + lane) * p.ss[p.dim_s]);
  }
  // The conversion is arithmetic on registers, after the loads: a dtype switch around each load
  // would put a branch between any two of them.
  with_dtypes<SE, DE>(p.sdt, p.ddt, [&](auto sd, auto dd) {
#pragma unroll
    for (uint32_t i = 0; i < 16; i++) tile[quad + 4 * i][lane] = convert_raw(v[i], decltype(sd)::value, decltype(dd)::value);
  });
  __syncthreads();
#pragma unroll
  for (uint32_t i = 0; i < 16; i++) {
    const uint32_t r = quad + 4 * i;
    if (s0 + r < ns && d0 + lane < nd)
      store_sized<DE>(p.dst, d_o + int64_t(s0 + r) * p.ds[p.dim_s] + int64_t(d0 + lane) * p.ds[p.dim_d], tile[lane][r]);
  }
}

// The same with nothing converted: typed loads and stores (the dtype switch of the converting
// form puts a branch between any two loads, so none of them overlap).
template <class E>
__global__ __launch_bounds__(256) void k_move_tiled_as(MoveStrided p) {
  __shared__ uint32_t tile[64][65];
  const E *src = static_cast<const E *>(p.src);
  E *dst = static_cast<E *>(p.dst);
  uint64_t blk = blockIdx.x;
  const uint32_t ts = uint32_t(blk % p.tiles_s);
  blk /= p.tiles_s;
  const uint32_t td = uint32_t((blk + ts) % p.tiles_d);
  blk /= p.tiles_d;
  // The remaining dims, slowest to fastest in `order` (dim_s and dim_d are skipped).
  int64_t so = 0, d_o = 0;
  for (int o = int(p.rank) - 1; o >= 0; o--) {
    const uint32_t d = p.order[o];
    if (d == p.dim_s || d == p.dim_d) continue;
    const uint32_t c = uint32_t(blk % p.shape[d]);
    blk /= p.shape[d];
    so += int64_t(c) * p.ss[d], d_o += int64_t(c) * p.ds[d];
  }
  const uint32_t lane = threadIdx.x & 63, quad = threadIdx.x >> 6;
  const uint32_t s0 = ts * 64, d0 = td * 64, ns = p.shape[p.dim_s], nd = p.shape[p.dim_d];
  uint32_t v[16];
#pragma unroll
  for (uint32_t i = 0; i < 16; i++) {
    const uint32_t r = quad + 4 * i;
    v[i] = 0;
    if (d0 + r < nd && s0 + lane < ns)
      v[i] = src[so + int64_t(d0 + r) * p.ss[p.dim_d] + int64_t(s0 + lane) * p.ss[p.dim_s]];
  }
#pragma unroll
  for (uint32_t i = 0; i < 16; i++) tile[quad + 4 * i][lane] = v[i];
  __syncthreads();
#pragma unroll
  for (uint32_t i = 0; i < 16; i++) {
    const uint32_t r = quad + 4 * i;
    if (s0 + r < ns && d0 + lane < nd)
      dst[d_o + int64_t(s0 + r) * p.ds[p.dim_s] + int64_t(d0 + lane) * p.ds[p.dim_d]] = E(tile[lane][r]);
  }
}

// The same transpose for 16-bit elements that are not converted: 128 x 128 tiles, two elements
// (one dword) per lane on both sides.  Needs even extents along both contiguous dims and even
// strides elsewhere, so that every dword is whole and aligned.
__global__ __launch_bounds__(256) void k_move_tiled16(MoveStrided p) {
  __shared__ uint16_t tile[128][130];
  uint64_t blk = blockIdx.x;
  const uint32_t ts = uint32_t(blk % p.tiles_s);
  blk /= p.tiles_s;
  const uint32_t td = uint32_t((blk + ts) % p.tiles_d);  // diagonal order, see k_move_tiled
  blk /= p.tiles_d;
  int64_t so = 0, d_o = 0;
  for (int o = int(p.rank) - 1; o >= 0; o--) {
    const uint32_t d = p.order[o];
    if (d == p.dim_s || d == p.dim_d) continue;
    const uint32_t c = uint32_t(blk % p.shape[d]);
    blk /= p.shape[d];
    so += int64_t(c) * p.ss[d], d_o += int64_t(c) * p.ds[d];
  }
  const uint32_t lane = threadIdx.x & 63, quad = threadIdx.x >> 6;
  const uint32_t s0 = ts * 128, d0 = td * 128, ns = p.shape[p.dim_s], nd = p.shape[p.dim_d];
  const uint16_t *src = static_cast<const uint16_t *>(p.src);
  uint16_t *dst = static_cast<uint16_t *>(p.dst);
#pragma unroll 4
  for (uint32_t r = quad; r < 128; r += 4)
    if (d0 + r < nd && s0 + 2 * lane < ns) {
      const uint32_t pair = *(const uint32_t *)(src + so + int64_t(d0 + r) * p.ss[p.dim_d] + (s0 + 2 * lane));
      tile[r][2 * lane] = uint16_t(pair), tile[r][2 * lane + 1] = uint16_t(pair >> 16);
    }
  __syncthreads();
#pragma unroll 4
  for (uint32_t r = quad; r < 128; r += 4)
    if (s0 + r < ns && d0 + 2 * lane < nd) {
      const uint32_t pair = uint32_t(tile[2 * lane][r]) | (uint32_t(tile[2 * lane + 1][r]) << 16);
      *(uint32_t *)(dst + d_o + int64_t(s0 + r) * p.ds[p.dim_s] + (d0 + 2 * lane)) = pair;
    }
}

// 16-bit elements whose source rows are whole 16-byte vectors: the 128 x 128 tile sits in LDS as
// dwords (pairs along the source's contiguous dim), loaded eight elements per lane; a lane then
// takes the dwords of two neighbouring tile rows and regroups their halves into the two dwords
// it stores (pairs along the destination's contiguous dim).  No 16-bit LDS access, no bank
// conflict beyond the two passes 64 lanes need anyway.
__global__ __launch_bounds__(256) void k_move_tiled16v(MoveStrided p) {
  __shared__ uint32_t tile[128][65];
  uint64_t blk = blockIdx.x;
  const uint32_t ts = uint32_t(blk % p.tiles_s);
  blk /= p.tiles_s;
  const uint32_t td = uint32_t((blk + ts) % p.tiles_d);  // diagonal order, see k_move_tiled
  blk /= p.tiles_d;
  int64_t so = 0, d_o = 0;
  for (int o = int(p.rank) - 1; o >= 0; o--) {
    const uint32_t d = p.order[o];
    if (d == p.dim_s || d == p.dim_d) continue;
    const uint32_t c = uint32_t(blk % p.shape[d]);
    blk /= p.shape[d];
    so += int64_t(c) * p.ss[d], d_o += int64_t(c) * p.ds[d];
  }
  typedef uint32_t quad_t __attribute__((ext_vector_type(4)));
  const uint32_t s0 = ts * 128, d0 = td * 128, ns = p.shape[p.dim_s], nd = p.shape[p.dim_d];
  const uint16_t *src = static_cast<const uint16_t *>(p.src);
  uint16_t *dst = static_cast<uint16_t *>(p.dst);
  const uint32_t col = (threadIdx.x & 15) * 8, row = threadIdx.x >> 4;
  quad_t v[8];
#pragma unroll
  for (int i = 0; i < 8; i++) {
    const uint32_t r = row + 16 * i;
    v[i] = quad_t{0, 0, 0, 0};
    if (d0 + r < nd && s0 + col < ns)
      v[i] = MRL_LOAD_ONCE((const quad_t *)(src + so + int64_t(d0 + r) * p.ss[p.dim_d] + (s0 + col)));
  }
#pragma unroll
  for (int i = 0; i < 8; i++) {
    const uint32_t r = row + 16 * i;
#pragma unroll
    for (int j = 0; j < 4; j++) tile[r][col / 2 + j] = v[i][j];
  }
  __syncthreads();
  const uint32_t lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const uint32_t d = d0 + 2 * lane;
  if (d >= nd) return;
#pragma unroll 4
  for (uint32_t sp = wave; sp < 64; sp += 4) {
    const uint32_t a = tile[2 * lane][sp], b = tile[2 * lane + 1][sp];
    const uint32_t sidx = s0 + 2 * sp;
    if (sidx < ns) MRL_STORE_ONCE((a & 0xffffu) | (b << 16), (uint32_t *)(dst + d_o + int64_t(sidx) * p.ds[p.dim_s] + d));
    if (sidx + 1 < ns) MRL_STORE_ONCE((a >> 16) | (b & 0xffff0000u), (uint32_t *)(dst + d_o + int64_t(sidx + 1) * p.ds[p.dim_s] + d));
  }
}

// Bytes whose source rows are whole 16-byte vectors: a 128 x 128 tile as dwords (four bytes along
// the source's contiguous dim each), loaded sixteen bytes per lane.  A lane then takes the dwords
// of four neighbouring tile rows at one column, transposes the 4 x 4 bytes in registers (byte
// permutes) and stores the four dwords into four destination rows.  The four rows are read in
// an order rotated by the lane's group, which spreads the 32 lanes of a half-wave over all banks.
__global__ __launch_bounds__(256) void k_move_tiled8v(MoveStrided p) {
  __shared__ uint32_t tile[128][33];
  uint64_t blk = blockIdx.x;
  const uint32_t ts = uint32_t(blk % p.tiles_s);
  blk /= p.tiles_s;
  const uint32_t td = uint32_t((blk + ts) % p.tiles_d);  // diagonal order, see k_move_tiled
  blk /= p.tiles_d;
  int64_t so = 0, d_o = 0;
  for (int o = int(p.rank) - 1; o >= 0; o--) {
    const uint32_t d = p.order[o];
    if (d == p.dim_s || d == p.dim_d) continue;
    const uint32_t c = uint32_t(blk % p.shape[d]);
    blk /= p.shape[d];
    so += int64_t(c) * p.ss[d], d_o += int64_t(c) * p.ds[d];
  }
  typedef uint32_t quad_t __attribute__((ext_vector_type(4)));
  const uint32_t s0 = ts * 128, d0 = td * 128, ns = p.shape[p.dim_s], nd = p.shape[p.dim_d];
  const uint8_t *src = static_cast<const uint8_t *>(p.src);
  uint8_t *dst = static_cast<uint8_t *>(p.dst);
  const uint32_t col = (threadIdx.x & 7) * 16, row = threadIdx.x >> 3;  // 8 lanes per 128-byte row
  quad_t v[4];
#pragma unroll
  for (int i = 0; i < 4; i++) {
    const uint32_t r = row + 32 * i;
    v[i] = quad_t{0, 0, 0, 0};
    if (d0 + r < nd && s0 + col < ns)
      v[i] = MRL_LOAD_ONCE((const quad_t *)(src + so + int64_t(d0 + r) * p.ss[p.dim_d] + (s0 + col)));
  }
#pragma unroll
  for (int i = 0; i < 4; i++) {
    const uint32_t r = row + 32 * i;
#pragma unroll
    for (int j = 0; j < 4; j++) tile[r][col / 4 + j] = v[i][j];
  }
  __syncthreads();
  const uint32_t lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const uint32_t group = lane & 31, half = lane >> 5;  // four tile rows 4 * group .. + 3
  const uint32_t turn = group >> 3;
  const uint32_t d = d0 + 4 * group;
#pragma unroll
  for (uint32_t it = 0; it < 4; it++) {
    const uint32_t sq = it * 8 + wave * 2 + half;  // which four source bytes (one dword of a tile row)
    uint32_t x[4];
#pragma unroll
    for (uint32_t j = 0; j < 4; j++) x[j] = tile[4 * group + ((j + turn) & 3)][sq];
    // x[j] is tile row (j + turn) % 4: undo the rotation.
    uint32_t a[4];
#pragma unroll
    for (uint32_t k = 0; k < 4; k++) {
      const uint32_t from = (k - turn) & 3;
      a[k] = from == 0 ? x[0] : from == 1 ? x[1] : from == 2 ? x[2] : x[3];
    }
    const uint32_t lo01 = __builtin_amdgcn_perm(a[1], a[0], 0x05010400u), hi01 = __builtin_amdgcn_perm(a[1], a[0], 0x07030602u);
    const uint32_t lo23 = __builtin_amdgcn_perm(a[3], a[2], 0x05010400u), hi23 = __builtin_amdgcn_perm(a[3], a[2], 0x07030602u);
    const uint32_t out[4] = {__builtin_amdgcn_perm(lo23, lo01, 0x05040100u), __builtin_amdgcn_perm(lo23, lo01, 0x07060302u),
                             __builtin_amdgcn_perm(hi23, hi01, 0x05040100u), __builtin_amdgcn_perm(hi23, hi01, 0x07060302u)};
    if (d < nd) {
#pragma unroll
      for (uint32_t k = 0; k < 4; k++) {
        const uint32_t sidx = s0 + 4 * sq + k;
        if (sidx < ns) MRL_STORE_ONCE(out[k], (uint32_t *)(dst + d_o + int64_t(sidx) * p.ds[p.dim_s] + d));
      }
    }
  }
}

// The same for 32-bit elements that are not converted: 64 x 64 tiles, four elements (16 bytes)
// per lane on both sides.  Needs extents along both contiguous dims and all other strides in
// multiples of 4 elements and 16-byte aligned bases, so that every vector is whole and aligned.
__global__ __launch_bounds__(256) void k_move_tiled32(MoveStrided p) {
  __shared__ uint32_t tile[64][65];
  uint64_t blk = blockIdx.x;
  const uint32_t ts = uint32_t(blk % p.tiles_s);
  blk /= p.tiles_s;
  const uint32_t td = uint32_t((blk + ts) % p.tiles_d);  // diagonal order, see k_move_tiled
  blk /= p.tiles_d;
  int64_t so = 0, d_o = 0;
  for (int o = int(p.rank) - 1; o >= 0; o--) {
    const uint32_t d = p.order[o];
    if (d == p.dim_s || d == p.dim_d) continue;
    const uint32_t c = uint32_t(blk % p.shape[d]);
    blk /= p.shape[d];
    so += int64_t(c) * p.ss[d], d_o += int64_t(c) * p.ds[d];
  }
  const uint32_t col = (threadIdx.x & 15) * 4, row = threadIdx.x >> 4;  // 16 lanes per 64-element row
  const uint32_t s0 = ts * 64, d0 = td * 64, ns = p.shape[p.dim_s], nd = p.shape[p.dim_d];
  const uint32_t *src = static_cast<const uint32_t *>(p.src);
  uint32_t *dst = static_cast<uint32_t *>(p.dst);
  typedef uint32_t quad_t __attribute__((ext_vector_type(4)));
  quad_t v[4];
#pragma unroll
  for (int i = 0; i < 4; i++) {
    const uint32_t r = row + 16 * i;
    v[i] = quad_t{0, 0, 0, 0};
    if (d0 + r < nd && s0 + col < ns)
      v[i] = MRL_LOAD_ONCE((const quad_t *)(src + so + int64_t(d0 + r) * p.ss[p.dim_d] + (s0 + col)));
  }
#pragma unroll
  for (int i = 0; i < 4; i++) {
    const uint32_t r = row + 16 * i;
    tile[r][col] = v[i][0], tile[r][col + 1] = v[i][1], tile[r][col + 2] = v[i][2], tile[r][col + 3] = v[i][3];
  }
  __syncthreads();
#pragma unroll
  for (int i = 0; i < 4; i++) {
    const uint32_t r = row + 16 * i;
    if (s0 + r < ns && d0 + col < nd) {
      const quad_t out{tile[col][r], tile[col + 1][r], tile[col + 2][r], tile[col + 3][r]};
      __builtin_nontemporal_store(out, (quad_t *)(dst + d_o + int64_t(s0 + r) * p.ds[p.dim_s] + (d0 + col)));
    }
  }
}

// Any other pair of contiguous dims (a Packed(8) digit on one side, say, too short for the
// 64 x 64 transpose): a tile of up to 4096 elements, `ext[d]` along each digit, chosen on the host
// so that it holds runs of 64 contiguous elements on both sides.  Read in source order into LDS,
// written in destination order.  Element t of the tile in source order has digit
// (t / tstride_s[d]) % ext[d] along d, likewise tstride_d in destination order; the divisions are
// multiplications by precomputed reciprocals (exact for operands below 2^16).
struct MoveTile {
  MoveStrided m;
  uint32_t ext[MOVE_MAX_RANK], chunks[MOVE_MAX_RANK];
  uint32_t tstride_s[MOVE_MAX_RANK], tstride_d[MOVE_MAX_RANK];
  uint32_t inv_s[MOVE_MAX_RANK], inv_d[MOVE_MAX_RANK], inv_ext[MOVE_MAX_RANK];  // ceil(2^32 / x)
  uint32_t tile;  // elements per tile
  FastDiv by_chunks[MOVE_MAX_RANK];   // a block number into tile coordinates without dividing (blocks number below 2^31)
  // Runs of V > 1 elements per thread: the LDS distance between neighbours along the
  // destination's fastest digit, and whether whole runs may be loaded / stored as one vector.
  uint32_t lds_step;
  bool vec_s, vec_d;
};
constexpr uint32_t MOVE_TILE_MAX = 4096;

__device__ inline uint32_t div_small(uint32_t n, uint32_t d, uint32_t inv) {
  return d == 1 ? n : __umulhi(n, inv);
}

// E: the element type when nothing is converted (typed loads and stores), void when the dtypes
// differ (conversion per element).  Offsets fit 32 bits: a tensor has fewer than 2^31 elements.
// V: elements per thread and step, a run along the fastest digit of the side being walked (the
// host picks V > 1 only when those digits, their tile extents and their sizes are multiples of
// V): one digit extraction serves V elements.
// NACT: the digits along which the tile extends come first (the host orders them so) and number
// at most NACT; the per-element digit loops run over exactly those, unrolled, with no test of
// which digits matter.
// E void: elements are converted, SSIZE and DSIZE their sizes in bytes on the two sides.
template <class E, int V, int NACT, int SSIZE = 0, int DSIZE = 0>
__global__ __launch_bounds__(256) void k_move_gather(MoveTile p) {
  constexpr bool CONVERT = std::is_void<E>::value;
  typedef typename std::conditional<CONVERT, uint32_t, E>::type Cell;
  static_assert(V == 1 || !CONVERT, "runs are for elements that are not converted");
  typedef Cell Run __attribute__((ext_vector_type(V == 1 ? 2 : V)));  // used only when V > 1
  __shared__ Cell lds[MOVE_TILE_MAX + MOVE_TILE_MAX / 64];
  uint32_t blk = blockIdx.x;
  int64_t base_s = 0, base_d = 0;
  uint32_t room[MOVE_MAX_RANK];  // how much of each digit is left from this tile's origin on
#pragma unroll
  for (uint32_t d = 0; d < MOVE_MAX_RANK; d++) {
    room[d] = 1;
    if (d < p.m.rank) {
      const uint32_t rest = p.by_chunks[d].div(blk);
      const uint32_t origin = (blk - rest * p.chunks[d]) * p.ext[d];
      blk = rest;
      room[d] = p.m.shape[d] - origin;
      base_s += int64_t(origin) * p.m.ss[d], base_d += int64_t(origin) * p.m.ds[d];
    }
  }
#pragma unroll 4
  for (uint32_t t = threadIdx.x * V; t < p.tile; t += 256 * V) {
    uint32_t so = 0;
    bool inside = true;
#pragma unroll
    for (uint32_t d = 0; d < uint32_t(NACT); d++) {
      const uint32_t q = div_small(t, p.tstride_s[d], p.inv_s[d]);
      const uint32_t c = q - div_small(q, p.ext[d], p.inv_ext[d]) * p.ext[d];
      inside = inside && c < room[d];
      so += c * uint32_t(p.m.ss[d]);
    }
    if (inside) {
      if constexpr (CONVERT) {
        lds[t + t / 64] = load_sized<SSIZE ? SSIZE : 4>(p.m.src, base_s + so);
      } else if constexpr (V == 1) {
        lds[t + t / 64] = static_cast<const E *>(p.m.src)[base_s + so];
      } else {
        const E *from = static_cast<const E *>(p.m.src) + base_s + so;
        Run run;
        if (p.vec_s) run = *reinterpret_cast<const Run *>(from);
        else
#pragma unroll
          for (int e = 0; e < V; e++) run[e] = from[e];
#pragma unroll
        for (int e = 0; e < V; e++) lds[t + t / 64 + e] = run[e];
      }
    }
  }
  __syncthreads();
#pragma unroll 4
  for (uint32_t t = threadIdx.x * V; t < p.tile; t += 256 * V) {
    uint32_t d_o = 0, at = 0;
    bool inside = true;
#pragma unroll
    for (uint32_t d = 0; d < uint32_t(NACT); d++) {
      const uint32_t q = div_small(t, p.tstride_d[d], p.inv_d[d]);
      const uint32_t c = q - div_small(q, p.ext[d], p.inv_ext[d]) * p.ext[d];
      inside = inside && c < room[d];
      d_o += c * uint32_t(p.m.ds[d]);
      at += c * p.tstride_s[d];
    }
    if (inside) {
      if constexpr (CONVERT) {
        const uint32_t v = convert_raw(lds[at + at / 64], p.m.sdt, p.m.ddt);
        store_sized<DSIZE ? DSIZE : 4>(p.m.dst, base_d + d_o, v);
      } else if constexpr (V == 1) {
        static_cast<E *>(p.m.dst)[base_d + d_o] = lds[at + at / 64];
      } else {
        Run run;
#pragma unroll
        for (int e = 0; e < V; e++) {
          const uint32_t from = at + e * p.lds_step;  // the next element along the destination's fastest digit
          run[e] = lds[from + from / 64];
        }
        E *to = static_cast<E *>(p.m.dst) + base_d + d_o;
        if (p.vec_d) *reinterpret_cast<Run *>(to) = run;
        else
#pragma unroll
          for (int e = 0; e < V; e++) to[e] = run[e];
      }
    }
  }
}

// Four 16-byte vectors per thread in flight, streamed past the caches: 6.5 TB/s on a 256 MiB
// copy against 5.7 TB/s for one cached vector per thread.
constexpr int COPY_UNROLL = 4;
typedef unsigned v4u __attribute__((ext_vector_type(4)));
__global__ __launch_bounds__(256) void k_copy16(const v4u *__restrict__ src, v4u *__restrict__ dst,
                                                uint64_t vecs) {
  const uint64_t step = uint64_t(gridDim.x) * 256 * COPY_UNROLL;
  for (uint64_t i = uint64_t(blockIdx.x) * 256 * COPY_UNROLL + threadIdx.x; i < vecs; i += step) {
    v4u v[COPY_UNROLL];
#pragma unroll
    for (int u = 0; u < COPY_UNROLL; u++)
      if (i + u * 256 < vecs) v[u] = MRL_LOAD_ONCE(src + i + u * 256);
#pragma unroll
    for (int u = 0; u < COPY_UNROLL; u++)
      if (i + u * 256 < vecs) __builtin_nontemporal_store(v[u], dst + i + u * 256);
  }
}

// bf16 -> f32 of a whole buffer, position by position (exact: a 16-bit shift).
__global__ __launch_bounds__(256) void k_widen_bf16(const uint16_t *__restrict__ src, uint32_t *__restrict__ dst,
                                                    uint64_t count) {
  const uint64_t step = uint64_t(gridDim.x) * blockDim.x;
  for (uint64_t i = uint64_t(blockIdx.x) * blockDim.x + threadIdx.x; i < count; i += step)
    dst[i] = uint32_t(src[i]) << 16;
}

// Copies [batch][rows][cols] with contiguous rows into rows of `dst_ld` elements (a whole number
// of dwords), writing zeros from the end of each row to its leading dimension.  One thread per
// destination dword, assembled from element-sized loads (the source rows need not be aligned
// beyond their element size).
template <class E>
__global__ __launch_bounds__(256) void k_pad_rows(const E *__restrict__ src, uint32_t *__restrict__ dst,
                                                  uint32_t rows, uint32_t cols, int64_t src_batch,
                                                  int64_t src_ld, uint32_t dst_ld, uint64_t dwords) {
  constexpr uint32_t PER = 4 / sizeof(E);
  const uint32_t row_dwords = dst_ld / PER;
  const uint64_t step = uint64_t(gridDim.x) * blockDim.x;
  for (uint64_t i = uint64_t(blockIdx.x) * blockDim.x + threadIdx.x; i < dwords; i += step) {
    const uint64_t line = i / row_dwords;
    const uint32_t col0 = uint32_t(i % row_dwords) * PER;
    const E *from = src + int64_t(line / rows) * src_batch + int64_t(line % rows) * src_ld;
    uint32_t word = 0;
#pragma unroll
    for (uint32_t e = 0; e < PER; e++)
      if (col0 + e < cols) word |= uint32_t(from[col0 + e]) << (8 * sizeof(E) * e);
    dst[i] = word;
  }
}

// Two such copies in one launch (blockIdx.y names the copy): the two operands of a Matmul whose rows
// are not whole 16-byte chunks each took a launch of about 2.4 us for their padded copy (int8 1000^3).
struct PadJob {
  const void *src;
  uint32_t *dst;
  uint32_t rows, cols, dst_ld;
  int64_t src_batch, src_ld;
  uint64_t dwords;
};
template <class E>
__global__ __launch_bounds__(256) void k_pad_rows_pair(PadJob j0, PadJob j1) {
  const PadJob &j = blockIdx.y ? j1 : j0;
  constexpr uint32_t PER = 4 / sizeof(E);
  const uint32_t row_dwords = j.dst_ld / PER;
  const uint64_t step = uint64_t(gridDim.x) * blockDim.x;
  for (uint64_t i = uint64_t(blockIdx.x) * blockDim.x + threadIdx.x; i < j.dwords; i += step) {
    const uint64_t line = i / row_dwords;
    const uint32_t col0 = uint32_t(i % row_dwords) * PER;
    const E *from = static_cast<const E *>(j.src) + int64_t(line / j.rows) * j.src_batch + int64_t(line % j.rows) * j.src_ld;
    uint32_t word = 0;
#pragma unroll
    for (uint32_t e = 0; e < PER; e++)
      if (col0 + e < j.cols) word |= uint32_t(from[col0 + e]) << (8 * sizeof(E) * e);
    j.dst[i] = word;
  }
}

// The same when rows start on 16 bytes on both sides and `cols` is whole 16-byte vectors: one
// thread per destination vector (sizes and strides here count vectors).
__global__ __launch_bounds__(256) void k_pad_rows16(const v4u *__restrict__ src, v4u *__restrict__ dst, uint32_t rows,
                                                    uint32_t cols, int64_t src_batch, int64_t src_ld, uint32_t dst_ld,
                                                    uint64_t vectors) {
  const uint64_t i = uint64_t(blockIdx.x) * blockDim.x + threadIdx.x;
  if (i >= vectors) return;
  const uint64_t line = i / dst_ld;
  const uint32_t col = uint32_t(i % dst_ld);
  v4u v{0, 0, 0, 0};
  if (col < cols) v = MRL_LOAD_ONCE(src + int64_t(line / rows) * src_batch + int64_t(line % rows) * src_ld + col);
  __builtin_nontemporal_store(v, dst + i);
}

__global__ void k_copy1(const uint8_t *src, uint8_t *dst, uint64_t bytes) {
  const uint64_t i = uint64_t(blockIdx.x) * blockDim.x + threadIdx.x;
  if (i < bytes) dst[i] = src[i];
}

// -------------------------------------------------------------------- matmul
struct MM {
  const void *a, *b;
  void *c;
  int dta, dtb, dtc;
  uint32_t B, M, K, N;
  int64_t sa[3], sb[3], sc[3];
  int accum;
};

template <bool FLOAT_OUT>
__global__ __launch_bounds__(256) void k_matmul_generic(MM p) {
  __shared__ uint32_t ta[16][17], tb[16][17];
  const uint32_t tx = threadIdx.x % 16, ty = threadIdx.x / 16;
  // One 16 x 16 output tile per workgroup, tiles numbered n-fastest, then m, then batch, in
  // grid.x alone (grid.y and grid.z stop at 65535, which 2^20 rows would pass).
  const uint32_t tiles_n = (p.N + 15) / 16, tiles_m = (p.M + 15) / 16;
  const uint32_t tile_j = blockIdx.x % tiles_n, tile_i = (blockIdx.x / tiles_n) % tiles_m;
  const uint32_t bi = blockIdx.x / tiles_n / tiles_m;
  const uint32_t j = tile_j * 16 + tx, i = tile_i * 16 + ty;
  const bool live = i < p.M && j < p.N;
  const int64_t coff = int64_t(bi) * p.sc[0] + int64_t(i) * p.sc[1] + int64_t(j) * p.sc[2];
  float facc = 0.0f;
  uint32_t iacc = 0;
  if (p.accum && live) {
    if (FLOAT_OUT) facc = ((const float *)p.c)[coff];
    else iacc = load_u32(p.c, p.dtc, coff, MRL_U32);
  }
  for (uint32_t k0 = 0; k0 < p.K; k0 += 16) {
    {  // A tile: row i, col k0+tx ; B tile: row k0+ty, col j
      const uint32_t ka = k0 + tx, kb = k0 + ty;
      uint32_t av = 0, bv = 0;
      if (i < p.M && ka < p.K) {
        const int64_t o = int64_t(bi) * p.sa[0] + int64_t(i) * p.sa[1] + int64_t(ka) * p.sa[2];
        av = FLOAT_OUT ? __float_as_uint(load_f32(p.a, p.dta, o)) : load_u32(p.a, p.dta, o, p.dtc);
      }
      if (kb < p.K && j < p.N) {
        const int64_t o = int64_t(bi) * p.sb[0] + int64_t(kb) * p.sb[1] + int64_t(j) * p.sb[2];
        bv = FLOAT_OUT ? __float_as_uint(load_f32(p.b, p.dtb, o)) : load_u32(p.b, p.dtb, o, p.dtc);
      }
      ta[ty][tx] = av;
      tb[ty][tx] = bv;
    }
    __syncthreads();
#pragma unroll
    for (uint32_t kk = 0; kk < 16; kk++) {
      if (FLOAT_OUT) facc += __uint_as_float(ta[ty][kk]) * __uint_as_float(tb[kk][tx]);
      else iacc += ta[ty][kk] * tb[kk][tx];
    }
    __syncthreads();
  }
  if (live) {
    if (FLOAT_OUT) ((float *)p.c)[coff] = facc;
    else store_u32(p.c, p.dtc, coff, iacc);
  }
}

// ---------------------------------------------------------------------- conv
struct CV {
  const void *img, *filt;
  void *out;
  int dti, dtf, dto;
  uint32_t B, F, C, OH, OW, FH, FW;
  int64_t si[4], sf[4], so[4];
  int accum;
};

template <bool FLOAT_OUT>
__global__ __launch_bounds__(256) void k_conv_generic(CV p) {
  const uint64_t total = uint64_t(p.B) * p.F * p.OH * p.OW;
  const uint64_t idx = uint64_t(blockIdx.x) * blockDim.x + threadIdx.x;
  if (idx >= total) return;
  // Decode with f fastest so that NHWC outputs are written contiguously.
  uint64_t r = idx;
  const uint32_t f = uint32_t(r % p.F); r /= p.F;
  const uint32_t x = uint32_t(r % p.OW); r /= p.OW;
  const uint32_t y = uint32_t(r % p.OH); r /= p.OH;
  const uint32_t b = uint32_t(r);
  const int64_t ooff = b * p.so[0] + f * p.so[1] + y * p.so[2] + x * p.so[3];
  float facc = 0.0f;
  uint32_t iacc = 0;
  if (p.accum) {
    if (FLOAT_OUT) facc = ((const float *)p.out)[ooff];
    else iacc = load_u32(p.out, p.dto, ooff, MRL_U32);
  }
  for (uint32_t c = 0; c < p.C; c++)
    for (uint32_t rr = 0; rr < p.FH; rr++)
      for (uint32_t s = 0; s < p.FW; s++) {
        const int64_t io = b * p.si[0] + c * p.si[1] + int64_t(y + rr) * p.si[2] + int64_t(x + s) * p.si[3];
        const int64_t fo = f * p.sf[0] + c * p.sf[1] + rr * p.sf[2] + s * p.sf[3];
        if (FLOAT_OUT) facc += load_f32(p.img, p.dti, io) * load_f32(p.filt, p.dtf, fo);
        else iacc += load_u32(p.img, p.dti, io, p.dto) * load_u32(p.filt, p.dtf, fo, p.dto);
      }
  if (FLOAT_OUT) ((float *)p.out)[ooff] = facc;
  else store_u32(p.out, p.dto, ooff, iacc);
}

// The same with one wavefront per output element, its lanes striding over the C * FH * FW
// products: for a handful of outputs with a long reduction (examples/simple_conv_x86.rs: 8 outputs
// of 72 products each) the one-thread-per-output kernel is a chain of dependent loads.
template <bool FLOAT_OUT>
__global__ __launch_bounds__(256) void k_conv_generic_wave(CV p) {
  const uint64_t total = uint64_t(p.B) * p.F * p.OH * p.OW;
  const uint64_t idx = uint64_t(blockIdx.x) * 4 + (threadIdx.x >> 6);
  if (idx >= total) return;
  const uint32_t lane = threadIdx.x & 63;
  uint64_t r = idx;
  const uint32_t f = uint32_t(r % p.F); r /= p.F;
  const uint32_t x = uint32_t(r % p.OW); r /= p.OW;
  const uint32_t y = uint32_t(r % p.OH); r /= p.OH;
  const uint32_t b = uint32_t(r);
  const int64_t ooff = b * p.so[0] + f * p.so[1] + y * p.so[2] + x * p.so[3];
  float facc = 0.0f;
  uint32_t iacc = 0;
  const uint32_t window = p.FH * p.FW, terms = p.C * window;
  for (uint32_t t = lane; t < terms; t += 64) {
    const uint32_t c = t / window, rr = (t % window) / p.FW, s = t % p.FW;
    const int64_t io = b * p.si[0] + c * p.si[1] + int64_t(y + rr) * p.si[2] + int64_t(x + s) * p.si[3];
    const int64_t fo = f * p.sf[0] + c * p.sf[1] + rr * p.sf[2] + s * p.sf[3];
    if (FLOAT_OUT) facc += load_f32(p.img, p.dti, io) * load_f32(p.filt, p.dtf, fo);
    else iacc += load_u32(p.img, p.dti, io, p.dto) * load_u32(p.filt, p.dtf, fo, p.dto);
  }
  for (int o = 32; o > 0; o >>= 1) {
    facc += __shfl_xor(facc, o);
    iacc += uint32_t(__shfl_xor(int(iacc), o));
  }
  if (lane != 0) return;
  if (p.accum) {
    if (FLOAT_OUT) facc += ((const float *)p.out)[ooff];
    else iacc += load_u32(p.out, p.dto, ooff, MRL_U32);
  }
  if (FLOAT_OUT) ((float *)p.out)[ooff] = facc;
  else store_u32(p.out, p.dto, ooff, iacc);
}

// ------------------------------------------------------------------- softmax
// One wavefront per line along an arbitrary-stride scan dim: max, then exp and sum, then
// divide (morello/src/verification.rs:166-184).
struct SM {
  const float *in;
  float *out;
  uint32_t rank, scan_dim;
  uint32_t shape[MRL_MAX_RANK];
  int64_t si[MRL_MAX_RANK], so[MRL_MAX_RANK];
  uint64_t lines;
};

__device__ inline float wave_max(float v) {
  for (int o = 32; o > 0; o >>= 1) v = fmaxf(v, __shfl_xor(v, o));
  return v;
}
__device__ inline float wave_sum(float v) {
  for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o);
  return v;
}

__global__ __launch_bounds__(256) void k_softmax_generic(SM p) {
  const uint64_t line = uint64_t(blockIdx.x) * 4 + threadIdx.x / 64;
  const uint32_t lane = threadIdx.x % 64;
  if (line >= p.lines) return;
  uint64_t r = line;
  int64_t ibase = 0, obase = 0;
  for (int d = int(p.rank) - 1; d >= 0; d--) {
    if (uint32_t(d) == p.scan_dim) continue;
    const uint32_t c = uint32_t(r % p.shape[d]);
    r /= p.shape[d];
    ibase += c * p.si[d];
    obase += c * p.so[d];
  }
  const uint32_t n = p.shape[p.scan_dim];
  const int64_t is = p.si[p.scan_dim], os = p.so[p.scan_dim];
  float mx = -3.40282347e+38f;
  bool nan = false;
  for (uint32_t i = lane; i < n; i += 64) {
    const float v = p.in[ibase + i * is];
    nan |= v != v;
    mx = fmaxf(mx, v);
  }
  mx = wave_max(mx);
  if (__any(nan)) mx = __uint_as_float(0x7fc00000u);
  float sum = 0.0f;
  for (uint32_t i = lane; i < n; i += 64) {
    const float e = expf(p.in[ibase + i * is] - mx);
    p.out[obase + i * os] = e;
    sum += e;
  }
  sum = wave_sum(sum);
  for (uint32_t i = lane; i < n; i += 64) p.out[obase + i * os] /= sum;
}

// The scan dim is strided but another dim (`fast`) is contiguous on both sides: a workgroup
// takes 64 consecutive positions of `fast` (one per lane, so every access is a 256-byte run)
// and its WAVES waves (16 for long scan dims) split the scan dim; each lane keeps the online (max, denominator) pair of
// morello/src/spec.rs:96-106 over its share, the shares are merged through LDS with the
// parts formula (spec.rs:107-132), and a second sweep writes exp(x - max) / denominator.
// With few columns (fewer workgroups than compute units) the scan dim is also cut into `chunks`
// pieces of chunk_len steps, blockIdx.y naming the piece, and the work into two launches
// (morello/src/scheduling/parallel_softmax.rs:24-223 on the GPU's grid): PHASE 1 leaves every
// piece's pair in `pairs` ([column tile][piece][lane]), PHASE 2 merges a column's pairs and writes
// its own piece.  PHASE 0 is the whole Softmax in one launch.
struct SMC {
  SM s;
  uint32_t fast, fast_tiles;
  uint32_t chunks, chunk_len;
  float2 *pairs;
};
// exp(x) for x <= 0 (and NaN) as 2^t (one instruction at a quarter of the vector rate) with t = x log2(e)
// formed in two parts, the low part applied as a first-order factor: within two units in the last
// place, where libm's expf costs about twenty instructions.  The column kernel is bound by those:
// 2048 x 4096 over dim 0 took 27 us with expf.  Arguments below -150 give 0 like anything below -104.
__device__ inline float exp_nonpositive(float x) {
  x = x < -150.0f ? -150.0f : x;
  const float t = x * 1.44269504f;
  const float lo = __builtin_fmaf(x, 1.44269504f, -t) + x * 1.92596299e-8f;
  return __builtin_amdgcn_exp2f(t) * __builtin_fmaf(lo, 0.693147181f, 1.0f);
}
__device__ inline void merge_pair(float &m, float &d, float om, float od) {
  const float nm = (om != om || m != m) ? __uint_as_float(0x7fc00000u) : fmaxf(m, om);
  d = d * expf(m - nm) + od * expf(om - nm);
  m = nm;
}
// A scan dim of at most 16 elements beside a contiguous dim: a thread per column, the column in
// registers, 256 consecutive columns per workgroup (q.fast_tiles counts tiles of 256 here).  The
// kernel below would give each handful of rows a workgroup of its own, with its start-up and its
// exchange through LDS: 8 x 8 x 1024 x 1024 over dim 1 took 295 us that way.
__global__ __launch_bounds__(256) void k_softmax_cols_short(SMC q) {
  const SM &p = q.s;
  uint64_t r = blockIdx.x;
  const uint32_t f = uint32_t(r % q.fast_tiles) * 256 + threadIdx.x;
  r /= q.fast_tiles;
  int64_t ibase = 0, obase = 0;
  for (int d = int(p.rank) - 1; d >= 0; d--) {
    if (uint32_t(d) == p.scan_dim || uint32_t(d) == q.fast) continue;
    const uint32_t c = uint32_t(r % p.shape[d]);
    r /= p.shape[d];
    ibase += c * p.si[d];
    obase += c * p.so[d];
  }
  if (f >= p.shape[q.fast]) return;
  ibase += f, obase += f;  // unit stride on both sides
  const uint32_t n = p.shape[p.scan_dim];
  const int64_t is = p.si[p.scan_dim], os = p.so[p.scan_dim];
  float x[16];
  float m = -3.40282347e+38f;
  bool nan = false;
#pragma unroll
  for (int j = 0; j < 16; j++) {
    x[j] = uint32_t(j) < n ? p.in[ibase + j * is] : -3.40282347e+38f;
    nan |= x[j] != x[j];
    m = fmaxf(m, x[j]);
  }
  if (nan) m = __uint_as_float(0x7fc00000u);
  float den = 0.0f;
#pragma unroll
  for (int j = 0; j < 16; j++) {
    x[j] = exp_nonpositive(x[j] - m);
    den += uint32_t(j) < n ? x[j] : 0.0f;
  }
  const float inv = 1.0f / den;
#pragma unroll
  for (int j = 0; j < 16; j++)
    if (uint32_t(j) < n) MRL_STORE_ONCE(x[j] * inv, p.out + obase + j * os);
}

template <int WAVES, int PHASE>
__global__ __launch_bounds__(64 * WAVES) void k_softmax_cols(SMC q) {
  const SM &p = q.s;
  __shared__ float sm_max[WAVES][64], sm_den[WAVES][64];
  const uint32_t lane = threadIdx.x % 64, w = threadIdx.x / 64;
  uint64_t r = blockIdx.x;
  const uint32_t f = uint32_t(r % q.fast_tiles) * 64 + lane;
  r /= q.fast_tiles;
  int64_t ibase = 0, obase = 0;
  for (int d = int(p.rank) - 1; d >= 0; d--) {
    if (uint32_t(d) == p.scan_dim || uint32_t(d) == q.fast) continue;
    const uint32_t c = uint32_t(r % p.shape[d]);
    r /= p.shape[d];
    ibase += c * p.si[d];
    obase += c * p.so[d];
  }
  const bool live = f < p.shape[q.fast];
  ibase += f, obase += f;  // unit stride on both sides
  const uint32_t first = PHASE == 0 ? 0 : blockIdx.y * q.chunk_len;
  const uint32_t n = PHASE == 0 ? p.shape[p.scan_dim] : min(p.shape[p.scan_dim], first + q.chunk_len);
  const int64_t is = p.si[p.scan_dim], os = p.so[p.scan_dim];
  constexpr int UNROLL = 8;
  float m, d;
  if (PHASE != 2) {
    float mx = -3.40282347e+38f, den = 0.0f;
    bool nan = false;
    // Eight loads in flight per lane, then one rescale of the running denominator for the eight.
    if (live)
      for (uint32_t i0 = first + w; i0 < n; i0 += WAVES * UNROLL) {
        float x[UNROLL];
        float nm = mx;
#pragma unroll
        for (int j = 0; j < UNROLL; j++) {
          const uint32_t i = i0 + j * WAVES;
          x[j] = i < n ? p.in[ibase + i * is] : -3.40282347e+38f;
          nan |= x[j] != x[j];
          nm = fmaxf(nm, x[j]);
        }
        float add = 0.0f;
#pragma unroll
        for (int j = 0; j < UNROLL; j++) add += i0 + j * WAVES < n ? exp_nonpositive(x[j] - nm) : 0.0f;
        den = den * exp_nonpositive(mx - nm) + add;
        mx = nm;
      }
    if (nan) mx = __uint_as_float(0x7fc00000u);
    sm_max[w][lane] = mx, sm_den[w][lane] = den;
    __syncthreads();
    m = sm_max[0][lane], d = sm_den[0][lane];
#pragma unroll
    for (int o = 1; o < WAVES; o++) merge_pair(m, d, sm_max[o][lane], sm_den[o][lane]);
    if (PHASE == 1) {
      if (w == 0) q.pairs[(uint64_t(blockIdx.x) * q.chunks + blockIdx.y) * 64 + lane] = make_float2(m, d);
      return;
    }
  } else {
    // The column's pairs: every wave merges its share of the pieces, eight loads in flight at a
    // time, and the waves' results meet in LDS.
    const float2 *mine = q.pairs + uint64_t(blockIdx.x) * q.chunks * 64 + lane;
    m = -3.40282347e+38f, d = 0.0f;
    for (uint32_t c0 = w; c0 < q.chunks; c0 += WAVES * UNROLL) {
      float2 pc[UNROLL];
#pragma unroll
      for (int j = 0; j < UNROLL; j++) {
        const uint32_t c = c0 + j * WAVES;
        pc[j] = c < q.chunks ? mine[uint64_t(c) * 64] : make_float2(-3.40282347e+38f, 0.0f);
      }
#pragma unroll
      for (int j = 0; j < UNROLL; j++) merge_pair(m, d, pc[j].x, pc[j].y);
    }
    sm_max[w][lane] = m, sm_den[w][lane] = d;
    __syncthreads();
    m = sm_max[0][lane], d = sm_den[0][lane];
#pragma unroll
    for (int o = 1; o < WAVES; o++) merge_pair(m, d, sm_max[o][lane], sm_den[o][lane]);
  }
  const float inv_d = 1.0f / d;
  if (live)
    for (uint32_t i0 = first + w; i0 < n; i0 += WAVES * UNROLL) {
      float x[UNROLL];
#pragma unroll
      for (int j = 0; j < UNROLL; j++) {
        const uint32_t i = i0 + j * WAVES;
        x[j] = i < n ? p.in[ibase + i * is] : 0.0f;
      }
#pragma unroll
      for (int j = 0; j < UNROLL; j++) {
        const uint32_t i = i0 + j * WAVES;
        if (i < n) MRL_STORE_ONCE(exp_nonpositive(x[j] - m) * inv_d, p.out + obase + i * os);
      }
    }
}

__global__ void k_fill_zero(uint32_t *p, uint64_t words, uint8_t *tail, uint32_t tail_bytes) {
  const uint64_t i = uint64_t(blockIdx.x) * blockDim.x + threadIdx.x;
  const uint64_t step = uint64_t(gridDim.x) * blockDim.x;
  for (uint64_t w = i; w < words; w += step) p[w] = 0;
  if (i < tail_bytes) tail[i] = 0;
}

bool float_out(int dt) { return dt == MRL_F32; }

}  // namespace

hipError_t launch_relayout(const void *src, void *dst, const LayoutEval &sl, const LayoutEval &dl,
                           uint32_t es, uint64_t count, hipStream_t stream) {
  if (count == 0) return hipSuccess;
  const uint32_t blocks = uint32_t((count + 255) / 256);
  plan::work(plan::UNIT_VALU, 40.0 * count, 2.0 * count * es);  // index arithmetic per element
  MRL_LAUNCH(k_relayout, dim3(blocks), dim3(256), 0, stream, (const uint8_t *)src,
                     (uint8_t *)dst, sl, dl, es, count);
  return mrl::plan::last_error();
}

hipError_t launch_move_generic(const void *src, void *dst, const LayoutEval &sl, const LayoutEval &dl,
                               int sdt, int ddt, uint64_t count, hipStream_t stream) {
  if (count == 0) return hipSuccess;
  const uint32_t blocks = uint32_t((count + 255) / 256);
  plan::work(plan::UNIT_VALU, 40.0 * count, double(count) * (mrl_dtype_size(sdt) + mrl_dtype_size(ddt)));
  MRL_LAUNCH(k_move_generic, dim3(blocks), dim3(256), 0, stream, src, dst, sl, dl, sdt, ddt, count);
  return mrl::plan::last_error();
}

hipError_t launch_copy(const void *src, void *dst, uint64_t bytes, hipStream_t stream) {
  const uint64_t vecs = bytes / 16, tail = bytes % 16;
  if (vecs) {
    uint64_t blocks = (vecs + 256 * COPY_UNROLL - 1) / (256 * COPY_UNROLL);
    if (blocks > 8192) blocks = 8192;  // grid-stride: 32 blocks per CU on a 256-CU part
    plan::work(plan::UNIT_STREAM, 0, 2.0 * bytes);
    MRL_LAUNCH(k_copy16, dim3(uint32_t(blocks)), dim3(256), 0, stream, (const v4u *)src,
                       (v4u *)dst, vecs);
  }
  if (tail)
    MRL_LAUNCH(k_copy1, dim3(1), dim3(16), 0, stream, (const uint8_t *)src + vecs * 16,
                       (uint8_t *)dst + vecs * 16, tail);
  return mrl::plan::last_error();
}

// Move over a common strided view of the two sides (layout_factor.h).  Returns
// hipErrorInvalidValue when the view does not fit the kernels' index ranges (the caller then
// takes the generic path).
hipError_t launch_move_view(const void *src, int src_dtype, void *dst, int dst_dtype,
                            const MoveDim *dims, uint32_t rank, hipStream_t stream) {
  if (rank > MOVE_MAX_RANK) return hipErrorInvalidValue;
  {
    double count = 1;
    for (uint32_t d = 0; d < rank; d++) count *= dims[d].size;
    plan::work(plan::UNIT_STREAM, 0, count * (mrl_dtype_size(src_dtype) + mrl_dtype_size(dst_dtype)));
  }
  // Elements narrower than 4 bytes that travel together (a digit contiguous on both sides, no
  // conversion) are moved as 2- or 4-byte units: a Packed(4) digit of bytes becomes one u32.
  MoveDim wide[MOVE_MAX_RANK];
  if (src_dtype == dst_dtype && mrl_dtype_size(src_dtype) < 4) {
    const uint32_t elem = uint32_t(mrl_dtype_size(src_dtype));
    for (uint32_t unit = 4; unit > elem; unit /= 2) {
      const uint32_t per = unit / elem;
      int shared = -1;
      bool fits = (reinterpret_cast<uintptr_t>(src) % unit) == 0 && (reinterpret_cast<uintptr_t>(dst) % unit) == 0;
      for (uint32_t d = 0; d < rank; d++)
        if (dims[d].size > 1 && dims[d].ss == 1 && dims[d].ds == 1) shared = int(d);
      for (uint32_t d = 0; fits && d < rank; d++)
        fits = int(d) == shared ? dims[d].size % per == 0 : (dims[d].ss % per == 0 && dims[d].ds % per == 0);
      if (shared < 0 || !fits) continue;
      uint32_t n = 0;
      for (uint32_t d = 0; d < rank; d++) {
        MoveDim m = dims[d];
        if (int(d) == shared) m.size /= per;
        else m.ss /= per, m.ds /= per;
        if (m.size > 1) wide[n++] = m;
      }
      if (n == 0) wide[n++] = {1, 1, 1};
      dims = wide, rank = n;
      src_dtype = dst_dtype = unit == 4 ? MRL_U32 : MRL_U16;
      break;
    }
  }
  MoveStrided p;
  p.src = src, p.dst = dst, p.sdt = src_dtype, p.ddt = dst_dtype, p.rank = rank;
  p.count = 1;
  int dim_s = -1, dim_d = -1;
  for (uint32_t d = 0; d < MOVE_MAX_RANK; d++) {
    p.shape[d] = d < rank ? dims[d].size : 1;
    p.ss[d] = d < rank ? dims[d].ss : 0;
    p.ds[d] = d < rank ? dims[d].ds : 0;
    p.count *= p.shape[d];
    if (d < rank && p.shape[d] > 1 && p.ss[d] == 1) dim_s = int(d);
    if (d < rank && p.shape[d] > 1 && p.ds[d] == 1) dim_d = int(d);
  }
  if (p.count == 0) return hipSuccess;
  if (p.count > 0xffffffffull) return hipErrorInvalidValue;  // the kernels index elements with 32 bits
  // Decode order: by decreasing destination stride, the destination's contiguous dim last.
  for (uint32_t d = 0; d < MOVE_MAX_RANK; d++) p.order[d] = d;
  for (uint32_t i = 0; i < p.rank; i++)
    for (uint32_t j = i + 1; j < p.rank; j++)
      if (p.ds[p.order[j]] > p.ds[p.order[i]]) std::swap(p.order[i], p.order[j]);
  // A shared contiguous dim serves both sides when its runs are at least 64 bytes long.
  const bool shared_runs = dim_s >= 0 && dim_s == dim_d &&
                           (rank == 1 || uint64_t(p.shape[dim_s]) * mrl_dtype_size(src_dtype) >= 64);
  // A tensor this small is one round of workgroups either way: an element per thread finishes
  // in a third of the time the tiled kernels' loops over a handful of tiles take.
  const bool tiny = p.count <= 65536;
  if (dim_s < 0 || dim_d < 0 || shared_runs || tiny) {
    // Whole 16-byte vectors along the shared dim, everywhere: move vectors, not elements.
    const int64_t per = 16 / int64_t(mrl_dtype_size(src_dtype));
    bool vectors = dim_s >= 0 && dim_s == dim_d && src_dtype == dst_dtype && p.shape[dim_s] % per == 0 &&
                   (reinterpret_cast<uintptr_t>(src) & 15) == 0 && (reinterpret_cast<uintptr_t>(dst) & 15) == 0;
    for (uint32_t d = 0; vectors && d < rank; d++)
      vectors = int(d) == dim_s || (p.ss[d] % per == 0 && p.ds[d] % per == 0);
    if (vectors && rank == 1)
      return launch_copy(src, dst, p.count * mrl_dtype_size(src_dtype), stream);
    // One contiguous run with a conversion: four elements per thread.
    const size_t se = mrl_dtype_size(src_dtype), de = mrl_dtype_size(dst_dtype);
    if (rank == 1 && dim_s == 0 && dim_d == 0 && src_dtype != dst_dtype && p.count >= 1024 &&
        (reinterpret_cast<uintptr_t>(src) % (4 * se)) == 0 && (reinterpret_cast<uintptr_t>(dst) % (4 * de)) == 0) {
      // sixteen bytes a thread on the wider side where both buffers are aligned for it
      // (two-byte to one-byte elements: sixteen, two 16-byte loads and a 16-byte store)
      const uint32_t wide = se == 2 && de == 1 ? 16u : uint32_t(16 / std::max(se, de));
      const uint32_t n = (reinterpret_cast<uintptr_t>(src) % (wide * se)) == 0 && (reinterpret_cast<uintptr_t>(dst) % (wide * de)) == 0 ? wide : 4;
      const uint32_t blocks = uint32_t(std::min<uint64_t>((p.count / n + 255) / 256, 1u << 20));
      const dim3 grid{blocks}, block{256};
#define MRL_CONVERT(SE, DE)                                                                                                  \
  if (se == SE && de == DE) {                                                                                                \
    constexpr int WIDE = SE == 2 && DE == 1 ? 16 : 16 / (SE > DE ? SE : DE);                                                 \
    if (n == WIDE) MRL_LAUNCH((k_convert4<SE, DE, WIDE>), grid, block, 0, stream, src, dst, src_dtype, dst_dtype, p.count);   \
    else MRL_LAUNCH((k_convert4<SE, DE, 4>), grid, block, 0, stream, src, dst, src_dtype, dst_dtype, p.count);               \
  }
      MRL_CONVERT(1, 1) MRL_CONVERT(1, 2) MRL_CONVERT(1, 4)
      MRL_CONVERT(2, 1) MRL_CONVERT(2, 2) MRL_CONVERT(2, 4)
      MRL_CONVERT(4, 1) MRL_CONVERT(4, 2) MRL_CONVERT(4, 4)
#undef MRL_CONVERT
      return mrl::plan::last_error();
    }
    if (vectors) {
      for (uint32_t d = 0; d < rank; d++) {
        if (int(d) == dim_s) p.shape[d] /= uint32_t(per);
        else p.ss[d] /= per, p.ds[d] /= per;
      }
      p.count /= uint64_t(per);
    }
    const uint64_t blocks = (p.count + 255) / 256;
    if (blocks > 0x7fffffffull) return hipErrorInvalidValue;
    if (vectors) MRL_LAUNCH(k_move_rows16, dim3(uint32_t(blocks)), dim3(256), 0, stream, p);
    else MRL_LAUNCH(k_move_rows, dim3(uint32_t(blocks)), dim3(256), 0, stream, p);
    return mrl::plan::last_error();
  }
  // Two long contiguous dims: the 64 x 64 transpose.
  if (dim_s != dim_d && p.shape[dim_s] >= 32 && p.shape[dim_d] >= 32) {
    p.dim_s = uint32_t(dim_s), p.dim_d = uint32_t(dim_d);
    // 16-bit elements, nothing converted, every dword whole and aligned: two elements per lane.
    bool pairs = src_dtype == dst_dtype && mrl_dtype_size(src_dtype) == 2 && p.shape[dim_s] % 2 == 0 &&
                 p.shape[dim_d] % 2 == 0 && (reinterpret_cast<uintptr_t>(src) & 3) == 0 &&
                 (reinterpret_cast<uintptr_t>(dst) & 3) == 0;
    for (uint32_t d = 0; pairs && d < p.rank; d++)
      pairs = (int(d) == dim_s || p.ss[d] % 2 == 0) && (int(d) == dim_d || p.ds[d] % 2 == 0);
    // ... and the source side in whole 16-byte vectors.
    bool octets = pairs && p.shape[dim_s] % 8 == 0 && (reinterpret_cast<uintptr_t>(src) & 15) == 0;
    for (uint32_t d = 0; octets && d < p.rank; d++) octets = int(d) == dim_s || p.ss[d] % 8 == 0;
    // Bytes: sixteen per lane on the source side, four on the destination side.
    bool bytes16 = src_dtype == dst_dtype && mrl_dtype_size(src_dtype) == 1 && p.shape[dim_s] % 16 == 0 &&
                   p.shape[dim_d] % 4 == 0 && (reinterpret_cast<uintptr_t>(src) & 15) == 0 &&
                   (reinterpret_cast<uintptr_t>(dst) & 3) == 0;
    for (uint32_t d = 0; bytes16 && d < p.rank; d++)
      bytes16 = (int(d) == dim_s || p.ss[d] % 16 == 0) && (int(d) == dim_d || p.ds[d] % 4 == 0);
    // 32-bit elements likewise, four per lane.
    bool quads = src_dtype == dst_dtype && mrl_dtype_size(src_dtype) == 4 && p.shape[dim_s] % 4 == 0 &&
                 p.shape[dim_d] % 4 == 0 && (reinterpret_cast<uintptr_t>(src) & 15) == 0 &&
                 (reinterpret_cast<uintptr_t>(dst) & 15) == 0;
    for (uint32_t d = 0; quads && d < p.rank; d++)
      quads = (int(d) == dim_s || p.ss[d] % 4 == 0) && (int(d) == dim_d || p.ds[d] % 4 == 0);
    const uint32_t side = pairs || bytes16 ? 128 : 64;
    p.tiles_s = (p.shape[dim_s] + side - 1) / side, p.tiles_d = (p.shape[dim_d] + side - 1) / side;
    uint64_t blocks = uint64_t(p.tiles_s) * p.tiles_d;
    for (uint32_t d = 0; d < p.rank; d++)
      if (int(d) != dim_s && int(d) != dim_d) blocks *= p.shape[d];
    if (blocks > 0x7fffffffull) return hipErrorInvalidValue;
    if (bytes16) MRL_LAUNCH(k_move_tiled8v, dim3(uint32_t(blocks)), dim3(256), 0, stream, p);
    else if (octets) MRL_LAUNCH(k_move_tiled16v, dim3(uint32_t(blocks)), dim3(256), 0, stream, p);
    else if (pairs) MRL_LAUNCH(k_move_tiled16, dim3(uint32_t(blocks)), dim3(256), 0, stream, p);
    else if (quads) MRL_LAUNCH(k_move_tiled32, dim3(uint32_t(blocks)), dim3(256), 0, stream, p);
    else if (src_dtype != dst_dtype) {
      const int se = int(mrl_dtype_size(src_dtype)), de = int(mrl_dtype_size(dst_dtype));
#define MRL_TILED(SE, DE) \
  if (se == SE && de == DE) MRL_LAUNCH((k_move_tiled<SE, DE>), dim3(uint32_t(blocks)), dim3(256), 0, stream, p)
      MRL_TILED(1, 1); MRL_TILED(1, 2); MRL_TILED(1, 4);
      MRL_TILED(2, 1); MRL_TILED(2, 2); MRL_TILED(2, 4);
      MRL_TILED(4, 1); MRL_TILED(4, 2); MRL_TILED(4, 4);
#undef MRL_TILED
    }
    else if (mrl_dtype_size(src_dtype) == 1) MRL_LAUNCH(k_move_tiled_as<uint8_t>, dim3(uint32_t(blocks)), dim3(256), 0, stream, p);
    else if (mrl_dtype_size(src_dtype) == 2) MRL_LAUNCH(k_move_tiled_as<uint16_t>, dim3(uint32_t(blocks)), dim3(256), 0, stream, p);
    else MRL_LAUNCH(k_move_tiled_as<uint32_t>, dim3(uint32_t(blocks)), dim3(256), 0, stream, p);
    return mrl::plan::last_error();
  }
  // Neither pattern above, up to a million elements: an element per thread again (a [45, 1963, 4]
  // tensor turned to [45, 4, 1963] took 20 us through the tile below, 4 us this way).
  if (p.count <= (1u << 20)) {
    MRL_LAUNCH(k_move_rows, dim3(uint32_t((p.count + 255) / 256)), dim3(256), 0, stream, p);
    return mrl::plan::last_error();
  }
  // Otherwise a tile grown digit by digit: along the destination's fastest digits until they
  // make a run of 64, along the source's fastest until they do, then along the destination's
  // again while the tile stays within MOVE_TILE_MAX.
  MoveTile t;
  t.m = p;
  uint32_t by_ss[MOVE_MAX_RANK], by_ds[MOVE_MAX_RANK];  // digits, fastest first
  for (uint32_t d = 0; d < MOVE_MAX_RANK; d++) by_ss[d] = by_ds[d] = d, t.ext[d] = 1;
  std::sort(by_ss, by_ss + rank, [&](uint32_t x, uint32_t y) { return p.ss[x] < p.ss[y]; });
  std::sort(by_ds, by_ds + rank, [&](uint32_t x, uint32_t y) { return p.ds[x] < p.ds[y]; });
  uint32_t tile = 1;
  auto grow = [&](const uint32_t *order, uint32_t run_target, uint32_t tile_cap) {
    uint32_t run = 1;
    for (uint32_t i = 0; i < rank && run < run_target; i++) {
      const uint32_t d = order[i];
      run *= t.ext[d];
      if (t.ext[d] == p.shape[d] || run >= run_target) continue;
      const uint32_t want = std::min<uint32_t>({p.shape[d] / t.ext[d], (run_target + run - 1) / run,
                                                std::max<uint32_t>(1, tile_cap / tile)});
      if (want <= 1) break;
      tile = tile / t.ext[d] * (t.ext[d] * want), run *= want, t.ext[d] *= want;
      if (t.ext[d] != p.shape[d]) break;  // a partly covered digit ends the contiguous run
    }
  };
  grow(by_ds, 64, MOVE_TILE_MAX / 64);
  grow(by_ss, 64, MOVE_TILE_MAX);
  grow(by_ds, MOVE_TILE_MAX, MOVE_TILE_MAX);
  // The runs are as long as they get; a tile still far below the cap (a digit covered in part
  // ends the growth above: 4 of 6 strips of an OddEven(16) dim left a tile of 64 elements, 20000
  // workgroups for 5 MB) is filled along whatever digits have room, more runs per workgroup.
  for (uint32_t i = 0; i < rank && tile < MOVE_TILE_MAX; i++) {
    const uint32_t d = by_ds[i];
    const uint32_t grown = std::min<uint32_t>(p.shape[d], uint32_t(uint64_t(t.ext[d]) * (MOVE_TILE_MAX / tile)));
    if (grown > t.ext[d]) tile = tile / t.ext[d] * grown, t.ext[d] = grown;
  }
  t.tile = tile;
  uint64_t blocks = 1;
  uint32_t stride_s = 1, stride_d = 1;
  auto inverse = [](uint32_t x) { return x <= 1 ? 0u : uint32_t(((uint64_t(1) << 32) + x - 1) / x); };
  for (uint32_t i = 0; i < rank; i++) {
    t.tstride_s[by_ss[i]] = stride_s, stride_s *= t.ext[by_ss[i]];
    t.tstride_d[by_ds[i]] = stride_d, stride_d *= t.ext[by_ds[i]];
  }
  for (uint32_t d = 0; d < MOVE_MAX_RANK; d++) {
    if (d >= rank) t.tstride_s[d] = t.tstride_d[d] = 1;
    t.chunks[d] = d < rank ? (p.shape[d] + t.ext[d] - 1) / t.ext[d] : 1;
    t.inv_s[d] = inverse(t.tstride_s[d]), t.inv_d[d] = inverse(t.tstride_d[d]), t.inv_ext[d] = inverse(t.ext[d]);
    blocks *= t.chunks[d];
  }
  if (blocks > 0x7fffffffull || tile > MOVE_TILE_MAX) return hipErrorInvalidValue;
  const dim3 grid{uint32_t(blocks)};
  const size_t elem = mrl_dtype_size(src_dtype);
  // Runs of 4 or 2 elements per thread (any element size) where both sides' fastest digits allow.
  const uint32_t fs = by_ss[0], fd = by_ds[0];
  uint32_t run = 1;
  if (src_dtype == dst_dtype && p.ss[fs] == 1 && p.ds[fd] == 1)
    for (uint32_t v : {4u, 2u})
      if (run == 1 && t.ext[fs] % v == 0 && p.shape[fs] % v == 0 && t.ext[fd] % v == 0 && p.shape[fd] % v == 0) run = v;
  t.lds_step = t.tstride_s[fd];
  if (elem == 1 && run == 2) run = 1;  // bytes travel in fours or alone
  t.vec_s = (reinterpret_cast<uintptr_t>(src) % (elem * run)) == 0;
  t.vec_d = (reinterpret_cast<uintptr_t>(dst) % (elem * run)) == 0;
  for (uint32_t d = 0; d < rank; d++) {
    if (d != fs && p.ss[d] % run != 0) t.vec_s = false;
    if (d != fd && p.ds[d] % run != 0) t.vec_d = false;
  }
  // Digits the tile extends along first (any order of the digits serves the kernel, as long as
  // every per-digit array follows it).
  uint32_t perm[MOVE_MAX_RANK], n_act = 0, n_rest = 0;
  for (uint32_t d = 0; d < MOVE_MAX_RANK; d++)
    if (t.ext[d] > 1) perm[n_act++] = d;
  for (uint32_t d = 0; d < MOVE_MAX_RANK; d++)
    if (t.ext[d] <= 1) perm[n_act + n_rest++] = d;
  {
    const MoveTile o = t;
    for (uint32_t i = 0; i < MOVE_MAX_RANK; i++) {
      const uint32_t d = perm[i];
      t.m.shape[i] = o.m.shape[d], t.m.ss[i] = o.m.ss[d], t.m.ds[i] = o.m.ds[d];
      t.ext[i] = o.ext[d], t.chunks[i] = o.chunks[d], t.by_chunks[i] = FastDiv(o.chunks[d]);
      t.tstride_s[i] = o.tstride_s[d], t.tstride_d[i] = o.tstride_d[d];
      t.inv_s[i] = o.inv_s[d], t.inv_d[i] = o.inv_d[d], t.inv_ext[i] = o.inv_ext[d];
    }
    t.m.rank = MOVE_MAX_RANK;  // size-one digits fill the tail: shape 1, one chunk
  }
#define MRL_GATHER(E, V)                                                                              \
  do {                                                                                                \
    if (n_act <= 3) MRL_LAUNCH((k_move_gather<E, V, 3>), grid, dim3(256), 0, stream, t);              \
    else if (n_act <= 5) MRL_LAUNCH((k_move_gather<E, V, 5>), grid, dim3(256), 0, stream, t);         \
    else MRL_LAUNCH((k_move_gather<E, V, int(MOVE_MAX_RANK)>), grid, dim3(256), 0, stream, t);        \
  } while (0)
  if (src_dtype != dst_dtype) {
    const int se = int(elem), de = int(mrl_dtype_size(dst_dtype));
#define MRL_GATHER_CV(SE, DE)                                                                                      \
  if (se == SE && de == DE) {                                                                                      \
    if (n_act <= 5) MRL_LAUNCH((k_move_gather<void, 1, 5, SE, DE>), grid, dim3(256), 0, stream, t);                \
    else MRL_LAUNCH((k_move_gather<void, 1, int(MOVE_MAX_RANK), SE, DE>), grid, dim3(256), 0, stream, t);          \
  }
    MRL_GATHER_CV(1, 1) MRL_GATHER_CV(1, 2) MRL_GATHER_CV(1, 4)
    MRL_GATHER_CV(2, 1) MRL_GATHER_CV(2, 2) MRL_GATHER_CV(2, 4)
    MRL_GATHER_CV(4, 1) MRL_GATHER_CV(4, 2) MRL_GATHER_CV(4, 4)
#undef MRL_GATHER_CV
  }
  else if (elem == 4 && run == 4) MRL_GATHER(uint32_t, 4);
  else if (elem == 4 && run == 2) MRL_GATHER(uint32_t, 2);
  else if (elem == 4) MRL_GATHER(uint32_t, 1);
  else if (elem == 2 && run == 4) MRL_GATHER(uint16_t, 4);
  else if (elem == 2 && run == 2) MRL_GATHER(uint16_t, 2);
  else if (elem == 2) MRL_GATHER(uint16_t, 1);
  else if (run == 4) MRL_GATHER(uint8_t, 4);
  else MRL_GATHER(uint8_t, 1);
#undef MRL_GATHER
  return mrl::plan::last_error();
}

// Move between two strided layouts of the same logical shape.
hipError_t launch_move_strided(const Strided &src, const Strided &dst, hipStream_t stream) {
  // Dims of size one address nothing; neighbours that continue each other on both sides (h and w
  // of an image between NCHW and NHWC) are one dim: the tiled kernels then see its whole length
  // (56 x 56 pixels as 3136, whole 16-byte vectors, where a row of 56 is not).
  MoveDim dims[MRL_MAX_RANK];
  uint32_t n = 0;
  for (uint32_t d = 0; d < src.rank; d++) {
    if (src.shape[d] == 1) continue;
    const MoveDim next = {src.shape[d], src.stride[d], dst.stride[d]};
    if (n > 0 && dims[n - 1].ss == next.ss * int64_t(next.size) && dims[n - 1].ds == next.ds * int64_t(next.size) &&
        uint64_t(dims[n - 1].size) * next.size <= 0xffffffffull)
      dims[n - 1] = {dims[n - 1].size * next.size, next.ss, next.ds};
    else
      dims[n++] = next;
  }
  if (n == 0) dims[n++] = {1, 1, 1};
  return launch_move_view(src.ptr, src.dtype, dst.ptr, dst.dtype, dims, n, stream);
}

hipError_t launch_pad_rows(const Strided &src, void *dst, uint32_t dst_ld, uint32_t elem_size,
                           hipStream_t stream) {
  if (src.rank != 3 || (src.shape[2] != 1 && src.stride[2] != 1) || dst_ld * elem_size % 4 != 0 ||
      dst_ld < src.shape[2])
    return hipErrorInvalidValue;
  const uint32_t batch = src.shape[0], rows = src.shape[1], cols = src.shape[2];
  const uint64_t dwords = uint64_t(batch) * rows * (dst_ld * elem_size / 4);
  if (dwords == 0) return hipSuccess;
  const uint32_t blocks = uint32_t(std::min<uint64_t>((dwords + 255) / 256, 65536));
  const int64_t sb = batch == 1 ? 0 : src.stride[0], sl = rows == 1 ? 0 : src.stride[1];
  plan::work(plan::UNIT_STREAM, 0, double(batch) * rows * cols * elem_size + 4.0 * dwords);
  const uint32_t per16 = 16 / elem_size;
  if (cols % per16 == 0 && dst_ld % per16 == 0 && sb % per16 == 0 && sl % per16 == 0 &&
      (reinterpret_cast<uintptr_t>(src.ptr) & 15) == 0 && (reinterpret_cast<uintptr_t>(dst) & 15) == 0 &&
      dwords / 4 <= 0x7fffffffull * 256) {
    const uint64_t vectors = dwords / 4;
    MRL_LAUNCH(k_pad_rows16, dim3(uint32_t((vectors + 255) / 256)), dim3(256), 0, stream, (const v4u *)src.ptr, (v4u *)dst,
               rows, cols / per16, sb / per16, sl / per16, dst_ld / per16, vectors);
    return mrl::plan::last_error();
  }
  if (elem_size == 1)
    MRL_LAUNCH(k_pad_rows<uint8_t>, dim3(blocks), dim3(256), 0, stream, (const uint8_t *)src.ptr,
                       (uint32_t *)dst, rows, cols, sb, sl, dst_ld, dwords);
  else if (elem_size == 2)
    MRL_LAUNCH(k_pad_rows<uint16_t>, dim3(blocks), dim3(256), 0, stream, (const uint16_t *)src.ptr,
                       (uint32_t *)dst, rows, cols, sb, sl, dst_ld, dwords);
  else if (elem_size == 4)
    MRL_LAUNCH(k_pad_rows<uint32_t>, dim3(blocks), dim3(256), 0, stream, (const uint32_t *)src.ptr,
                       (uint32_t *)dst, rows, cols, sb, sl, dst_ld, dwords);
  else
    return hipErrorInvalidValue;
  return mrl::plan::last_error();
}

hipError_t launch_pad_rows_pair(const Strided &src0, void *dst0, uint32_t dst_ld0, const Strided &src1, void *dst1,
                                uint32_t dst_ld1, uint32_t elem_size, hipStream_t stream) {
  PadJob jobs[2];
  const Strided *srcs[2] = {&src0, &src1};
  void *dsts[2] = {dst0, dst1};
  const uint32_t lds[2] = {dst_ld0, dst_ld1};
  uint64_t most = 0;
  double bytes = 0;
  for (int i = 0; i < 2; i++) {
    const Strided &src = *srcs[i];
    if (src.rank != 3 || (src.shape[2] != 1 && src.stride[2] != 1) || lds[i] * elem_size % 4 != 0 || lds[i] < src.shape[2])
      return hipErrorInvalidValue;
    const uint32_t batch = src.shape[0], rows = src.shape[1], cols = src.shape[2];
    jobs[i].src = src.ptr, jobs[i].dst = static_cast<uint32_t *>(dsts[i]);
    jobs[i].rows = rows, jobs[i].cols = cols, jobs[i].dst_ld = lds[i];
    jobs[i].src_batch = batch == 1 ? 0 : src.stride[0], jobs[i].src_ld = rows == 1 ? 0 : src.stride[1];
    jobs[i].dwords = uint64_t(batch) * rows * (lds[i] * elem_size / 4);
    most = std::max(most, jobs[i].dwords);
    bytes += double(batch) * rows * cols * elem_size + 4.0 * jobs[i].dwords;
  }
  if (most == 0) return hipSuccess;
  plan::work(plan::UNIT_STREAM, 0, bytes);
  const dim3 grid(uint32_t(std::min<uint64_t>((most + 255) / 256, 65536)), 2);
  if (elem_size == 1) MRL_LAUNCH(k_pad_rows_pair<uint8_t>, grid, dim3(256), 0, stream, jobs[0], jobs[1]);
  else if (elem_size == 2) MRL_LAUNCH(k_pad_rows_pair<uint16_t>, grid, dim3(256), 0, stream, jobs[0], jobs[1]);
  else if (elem_size == 4) MRL_LAUNCH(k_pad_rows_pair<uint32_t>, grid, dim3(256), 0, stream, jobs[0], jobs[1]);
  else return hipErrorInvalidValue;
  return mrl::plan::last_error();
}

hipError_t launch_widen_bf16(const void *src, void *dst, uint64_t count, hipStream_t stream) {
  if (count == 0) return hipSuccess;
  uint64_t blocks = (count + 255) / 256;
  if (blocks > 16384) blocks = 16384;
  plan::work(plan::UNIT_STREAM, 0, 6.0 * count);
  MRL_LAUNCH(k_widen_bf16, dim3(uint32_t(blocks)), dim3(256), 0, stream, (const uint16_t *)src,
                     (uint32_t *)dst, count);
  return mrl::plan::last_error();
}

hipError_t launch_matmul_generic(const Strided &a, const Strided &b, const Strided &c, int accum,
                                 hipStream_t stream) {
  MM p;
  p.a = a.ptr, p.b = b.ptr, p.c = c.ptr;
  p.dta = a.dtype, p.dtb = b.dtype, p.dtc = c.dtype;
  p.B = a.shape[0], p.M = a.shape[1], p.K = a.shape[2], p.N = b.shape[2];
  for (int d = 0; d < 3; d++) p.sa[d] = a.stride[d], p.sb[d] = b.stride[d], p.sc[d] = c.stride[d];
  p.accum = accum;
  const uint64_t tiles = uint64_t((p.N + 15) / 16) * ((p.M + 15) / 16) * p.B;
  if (tiles > 0x7fffffffull) return hipErrorInvalidValue;
  dim3 grid{uint32_t(tiles)};
  {
    const double mn = double(p.B) * p.M * p.N;
    plan::work(plan::UNIT_VALU, 2.0 * mn * p.K,
               double(p.B) * (double(p.M) * p.K * mrl_dtype_size(a.dtype) + double(p.K) * p.N * mrl_dtype_size(b.dtype)) +
                   mn * mrl_dtype_size(c.dtype));
  }
  if (float_out(c.dtype)) MRL_LAUNCH(k_matmul_generic<true>, grid, dim3(256), 0, stream, p);
  else MRL_LAUNCH(k_matmul_generic<false>, grid, dim3(256), 0, stream, p);
  return mrl::plan::last_error();
}

hipError_t launch_conv_generic(const Strided &img, const Strided &filt, const Strided &out,
                               int accum, hipStream_t stream) {
  CV p;
  p.img = img.ptr, p.filt = filt.ptr, p.out = out.ptr;
  p.dti = img.dtype, p.dtf = filt.dtype, p.dto = out.dtype;
  p.B = out.shape[0], p.F = out.shape[1], p.OH = out.shape[2], p.OW = out.shape[3];
  p.C = filt.shape[1], p.FH = filt.shape[2], p.FW = filt.shape[3];
  for (int d = 0; d < 4; d++) p.si[d] = img.stride[d], p.sf[d] = filt.stride[d], p.so[d] = out.stride[d];
  p.accum = accum;
  const uint64_t total = uint64_t(p.B) * p.F * p.OH * p.OW;
  plan::work(plan::UNIT_VALU, 2.0 * total * p.C * p.FH * p.FW,
             double(p.B) * p.C * (p.OH + p.FH - 1) * (p.OW + p.FW - 1) * mrl_dtype_size(img.dtype) +
                 double(total) * mrl_dtype_size(out.dtype));
  if (total <= 16384 && uint64_t(p.C) * p.FH * p.FW >= 32) {  // few outputs, long reductions
    const uint32_t wave_blocks = uint32_t((total + 3) / 4);
    if (float_out(out.dtype)) MRL_LAUNCH(k_conv_generic_wave<true>, dim3(wave_blocks), dim3(256), 0, stream, p);
    else MRL_LAUNCH(k_conv_generic_wave<false>, dim3(wave_blocks), dim3(256), 0, stream, p);
    return mrl::plan::last_error();
  }
  const uint32_t blocks = uint32_t((total + 255) / 256);
  if (float_out(out.dtype)) MRL_LAUNCH(k_conv_generic<true>, dim3(blocks), dim3(256), 0, stream, p);
  else MRL_LAUNCH(k_conv_generic<false>, dim3(blocks), dim3(256), 0, stream, p);
  return mrl::plan::last_error();
}

// Pieces the scan dim is cut into when the column kernel would have `blocks` workgroups: none
// (1) when those fill the chip or the scan dim is short; else enough for about 1024 workgroups,
// each piece at least 32 steps (a 256-thread workgroup takes 32 steps in one unrolled pass).
uint32_t softmax_cols_chunks(uint64_t blocks, uint32_t scan) {
  if (blocks >= 256 || scan < 128) return 1;
  const uint64_t want = (1024 + blocks - 1) / blocks;
  return uint32_t(std::max<uint64_t>(1, std::min<uint64_t>({want, scan / 32, 256})));
}

size_t softmax_cols_scratch_bytes(uint64_t blocks, uint32_t scan) {
  const uint32_t chunks = softmax_cols_chunks(blocks, scan);
  return chunks > 1 ? size_t(blocks) * chunks * 64 * sizeof(float2) : 0;
}

hipError_t launch_softmax_generic(const Strided &in, const Strided &out, uint32_t scan_dim, void *scratch,
                                  hipStream_t stream) {
  SM p;
  p.in = (const float *)in.ptr, p.out = (float *)out.ptr;
  p.rank = in.rank, p.scan_dim = scan_dim;
  uint64_t lines = 1;
  for (uint32_t d = 0; d < MRL_MAX_RANK; d++) {
    p.shape[d] = d < in.rank ? in.shape[d] : 1;
    p.si[d] = d < in.rank ? in.stride[d] : 0;
    p.so[d] = d < in.rank ? out.stride[d] : 0;
    if (d < in.rank && d != scan_dim) lines *= in.shape[d];
  }
  p.lines = lines;
  plan::work(plan::UNIT_VALU, 20.0 * lines * in.shape[scan_dim], 8.0 * lines * in.shape[scan_dim]);
  // A dim other than the scan dim that both sides store contiguously: the column kernel.
  for (uint32_t d = 0; d < in.rank; d++)
    if (d != scan_dim && in.shape[d] >= 16 && in.stride[d] == 1 && out.stride[d] == 1) {
      SMC q;
      q.s = p, q.fast = d, q.fast_tiles = (in.shape[d] + 63) / 64;
      q.chunks = 1, q.chunk_len = in.shape[scan_dim], q.pairs = nullptr;
      if (in.shape[scan_dim] <= 16 && lines >= 65536) {
        q.fast_tiles = (in.shape[d] + 255) / 256;
        const uint64_t wgs = lines / in.shape[d] * q.fast_tiles;
        if (wgs > 0x7fffffffull) break;
        MRL_LAUNCH(k_softmax_cols_short, dim3(uint32_t(wgs)), dim3(256), 0, stream, q);
        return mrl::plan::last_error();
      }
      const uint64_t blocks = lines / in.shape[d] * q.fast_tiles;
      if (blocks > 0x7fffffffull) break;
      const uint32_t chunks = scratch ? softmax_cols_chunks(blocks, in.shape[scan_dim]) : 1;
      if (chunks > 1) {
        // Few columns: the scan dim shared out over blockIdx.y as well, in two launches.
        q.chunks = chunks, q.chunk_len = (in.shape[scan_dim] + chunks - 1) / chunks, q.pairs = (float2 *)scratch;
        const double count = double(lines) * in.shape[scan_dim];
        // Measured 2.5-4.4 TB/s over their 12 bytes an element; a workgroup's chain of passes over
        // its piece (32 steps a pass) is what small problems take: 2149 x 172 11 us, 100000 x 64 45 us.
        const double chain_ns = 2500.0 + 700.0 * ((q.chunk_len + 31) / 32);
        plan::work(plan::UNIT_STREAM, 0, 5.2 * count, 0, chain_ns);
        MRL_LAUNCH((k_softmax_cols<4, 1>), dim3(uint32_t(blocks), chunks), dim3(256), 0, stream, q);
        plan::work(plan::UNIT_STREAM, 0, 10.4 * count, 0, chain_ns);
        MRL_LAUNCH((k_softmax_cols<4, 2>), dim3(uint32_t(blocks), chunks), dim3(256), 0, stream, q);
        return mrl::plan::last_error();
      }
      if (in.shape[scan_dim] >= 512) MRL_LAUNCH((k_softmax_cols<16, 0>), dim3(uint32_t(blocks)), dim3(1024), 0, stream, q);
      else MRL_LAUNCH((k_softmax_cols<4, 0>), dim3(uint32_t(blocks)), dim3(256), 0, stream, q);
      return mrl::plan::last_error();
    }
  const uint32_t blocks = uint32_t((lines + 3) / 4);
  MRL_LAUNCH(k_softmax_generic, dim3(blocks), dim3(256), 0, stream, p);
  return mrl::plan::last_error();
}

namespace {
// One thread per 32-bit element of C.
template <class T>
__global__ __launch_bounds__(256) void k_sum_splits(const T *__restrict__ partial, T *__restrict__ c, uint32_t splits,
                                                    uint32_t n, uint64_t count, int64_t ldc, int accum) {
  const uint64_t i = uint64_t(blockIdx.x) * 256 + threadIdx.x;
  if (i >= count) return;
  T *to = c + int64_t(i / n) * ldc + int64_t(i % n);
  T sum = accum ? *to : T(0);
  constexpr uint32_t U = 8;  // loads in flight together
  for (uint32_t s0 = 0; s0 < splits; s0 += U) {
    T v[U];
#pragma unroll
    for (uint32_t u = 0; u < U; u++) v[u] = partial[uint64_t(s0 + u < splits ? s0 + u : s0) * count + i];
#pragma unroll
    for (uint32_t u = 0; u < U; u++) sum += s0 + u < splits ? v[u] : T(0);
  }
  *to = sum;
}
}  // namespace

hipError_t launch_sum_splits(const void *partial, void *c, uint32_t splits, uint32_t m, uint32_t n, int64_t ldc,
                             bool accum, bool integers, hipStream_t stream) {
  const uint64_t count = uint64_t(m) * n;
  if (count == 0) return hipSuccess;
  const uint64_t blocks = (count + 255) / 256;
  if (blocks > 0x7fffffffull) return hipErrorInvalidValue;
  plan::work(plan::UNIT_STREAM, 0, 4.0 * count * (splits + 1 + (accum ? 1 : 0)));
  if (integers)
    MRL_LAUNCH(k_sum_splits<int>, dim3(uint32_t(blocks)), dim3(256), 0, stream, (const int *)partial, (int *)c, splits, n,
               count, ldc, int(accum));
  else
    MRL_LAUNCH(k_sum_splits<float>, dim3(uint32_t(blocks)), dim3(256), 0, stream, (const float *)partial, (float *)c, splits,
               n, count, ldc, int(accum));
  return mrl::plan::last_error();
}

hipError_t launch_fill_zero(void *ptr, uint64_t bytes, hipStream_t stream) {
  if (bytes == 0) return hipSuccess;
  const uint64_t words = bytes / 4;
  const uint32_t tail = uint32_t(bytes % 4);
  uint64_t blocks = (words + 255) / 256;
  if (blocks > 65536) blocks = 65536;
  if (blocks == 0) blocks = 1;
  plan::work(plan::UNIT_STREAM, 0, double(bytes));
  MRL_LAUNCH(k_fill_zero, dim3(uint32_t(blocks)), dim3(256), 0, stream, (uint32_t *)ptr,
                     words, (uint8_t *)ptr + words * 4, tail);
  return mrl::plan::last_error();
}

}  // namespace mrl
