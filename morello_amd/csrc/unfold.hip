// Conv as a Matmul on the matrix cores, for the shapes the fused implicit-GEMM kernel of
// conv_i8.hip is not built for.  The Conv Spec (morello/src/spec.rs:486-494; no stride, no
// padding) is
//     out[b, f, y, x] (+)= sum_{c, r, s} image[b, c, y + r, x + s] * filters[f, c, r, s].
// With channels-last tensors the window of one output pixel is FH runs of FW * C contiguous
// elements of the image, and a filter in KRSC order is those same FH * FW * C weights in a row.
// So "unfolding" every window into a row gives U[b * OH * OW][FH * FW * C], the filters are a B
// operand stored k-fastest as they lie, and the channels-last output is C[b * OH * OW][F].
#include <algorithm>

#include "kernels.h"

namespace mrl {
namespace {

struct Unfold {
  const void *image;
  void *rows;
  uint32_t h, w, c, oh, ow, fh, fw;
  uint32_t run;        // fw * c: elements of one contiguous run of a window
  uint32_t k;          // fh * run: elements of a window
  uint32_t row_units;  // units (of sizeof(V) bytes) per row of U, padding included
  uint64_t units;      // all of U
};

// One thread per unit V of U (V = 16 or 4 bytes; runs and rows are whole units).
// Units from a window's end to the row's leading dimension are zeros.
template <class V>
__global__ __launch_bounds__(256) void k_unfold(Unfold p, uint32_t elem_size) {
  const uint32_t per = sizeof(V) / elem_size;  // elements per unit
  const uint64_t step = uint64_t(gridDim.x) * blockDim.x;
  const V *image = static_cast<const V *>(p.image);
  V *rows = static_cast<V *>(p.rows);
  for (uint64_t i = uint64_t(blockIdx.x) * blockDim.x + threadIdx.x; i < p.units; i += step) {
    const uint64_t pixel = i / p.row_units;
    const uint32_t col = uint32_t(i % p.row_units) * per;  // element within the row
    V v{};
    if (col < p.k) {
      const uint32_t r = col / p.run, within = col % p.run;
      const uint32_t x = uint32_t(pixel % p.ow);
      const uint64_t by = pixel / p.ow;  // b * oh + y
      const uint32_t y = uint32_t(by % p.oh);
      const uint64_t b = by / p.oh;
      const uint64_t src = ((b * p.h + y + r) * p.w + x) * p.c + within;  // in elements
      v = image[src / per];
    }
    rows[i] = v;
  }
}

// The same for channel vectors that are not whole dwords (three u8 channels, say): one thread per
// dword of U, assembled from element loads.  row_units counts dwords here.
template <class E>
__global__ __launch_bounds__(256) void k_unfold_gather(Unfold p) {
  constexpr uint32_t PER = 4 / sizeof(E);
  const uint64_t step = uint64_t(gridDim.x) * blockDim.x;
  const E *image = static_cast<const E *>(p.image);
  uint32_t *rows = static_cast<uint32_t *>(p.rows);
  for (uint64_t i = uint64_t(blockIdx.x) * blockDim.x + threadIdx.x; i < p.units; i += step) {
    const uint64_t pixel = i / p.row_units;
    const uint32_t col = uint32_t(i % p.row_units) * PER;
    const uint32_t x = uint32_t(pixel % p.ow);
    const uint64_t by = pixel / p.ow;
    const uint32_t y = uint32_t(by % p.oh);
    const uint64_t corner = ((by / p.oh * p.h + y) * p.w + x) * p.c;  // the window's first element
    uint32_t r = col / p.run, within = col % p.run;
    uint32_t word = 0;
#pragma unroll
    for (uint32_t e = 0; e < PER; e++) {
      if (col + e < p.k) word |= uint32_t(image[corner + uint64_t(r) * p.w * p.c + within]) << (8 * sizeof(E) * e);
      if (++within == p.run) within = 0, r++;
    }
    rows[i] = word;
  }
}

}  // namespace

hipError_t launch_unfold(const void *image, void *rows, uint32_t batch, uint32_t c, uint32_t oh,
                         uint32_t ow, uint32_t fh, uint32_t fw, uint32_t row_elems,
                         uint32_t elem_size, hipStream_t stream) {
  Unfold p;
  p.image = image, p.rows = rows;
  p.h = oh + fh - 1, p.w = ow + fw - 1, p.c = c, p.oh = oh, p.ow = ow, p.fh = fh, p.fw = fw;
  p.run = fw * c, p.k = fh * p.run;
  if (row_elems < p.k) return hipErrorInvalidValue;
  // The widest unit that divides a channel vector (so every run starts on a unit and is whole
  // units long) and the row.
  const uint64_t c_bytes = uint64_t(c) * elem_size, row_bytes = uint64_t(row_elems) * elem_size;
  if (row_bytes % 4 != 0) return hipErrorInvalidValue;
  const uint32_t unit = (c_bytes % 16 == 0 && row_bytes % 16 == 0) ? 16 : 4;
  const bool gather = c_bytes % 4 != 0;
  p.row_units = uint32_t(row_bytes / unit);
  p.units = uint64_t(batch) * oh * ow * p.row_units;
  if (p.units == 0) return hipSuccess;
  const uint32_t blocks = uint32_t(std::min<uint64_t>((p.units + 255) / 256, 1u << 20));
  plan::work(plan::UNIT_STREAM, 0, 2.0 * p.units * (gather ? 4 : unit));
  if (gather && elem_size == 1) MRL_LAUNCH(k_unfold_gather<uint8_t>, dim3(blocks), dim3(256), 0, stream, p);
  else if (gather) MRL_LAUNCH(k_unfold_gather<uint16_t>, dim3(blocks), dim3(256), 0, stream, p);
  else if (unit == 16) MRL_LAUNCH(k_unfold<uint4>, dim3(blocks), dim3(256), 0, stream, p, elem_size);
  else MRL_LAUNCH(k_unfold<uint32_t>, dim3(blocks), dim3(256), 0, stream, p, elem_size);
  return mrl::plan::last_error();
}

}  // namespace mrl
