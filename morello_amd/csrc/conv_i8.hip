// Conv Spec, NHWC u8|i8 image x KRSC i8 filters -> NHWC i32, on the int8 MFMA
// (v_mfma_i32_16x16x64_i8) as an implicit GEMM.
//
// Semantics (morello/src/spec.rs:486-498, 741-776; morello/src/scheduling/
// spatial_split.rs:73-118): stride 1, no padding, cross-correlation,
//   out[b,y,x,f] (=0 unless accum) += sum_{r,s,c} img[b,y+r,x+s,c] * filt[f,r,s,c].
// spatial_split turns every filter position (r,s) into a MatmulAccum[1, pixels, C, F] of
// the shifted image against filt[:, r, s, :]; that is exactly one k slab here.
//
// Memory-level mapping: the whole filter bank (F x FH x FW x C bytes, 36 KiB for the
// 64x3x3x64 case) is moved once per wavefront into VGPRs (move_param(1, VRF) hoisted out of
// every loop); image pixels go straight from global memory into MFMA operand registers
// (channels are the fastest NHWC dim, so one pixel's 64 channels are 64 contiguous bytes
// = four lanes x 16 B); the accumulators start at zero (to_accum) and each output pixel is
// written once, 16 B per lane.  The kernel is bound by the 4-byte-per-element output
// stream, not by the MFMA.
//
// u8 images: a' = a xor 0x80 and the per-filter correction 128 * sum_{r,s,c} filt[f,r,s,c]
// is added at the end (exact in i32).
#include "kernels.h"

namespace mrl {
namespace {

typedef int v4i __attribute__((ext_vector_type(4)));

constexpr int FT = 4;  // filter tiles of 16 -> F = 64

template <int SLABS, bool IMG_UNSIGNED>
__global__ __launch_bounds__(256) void k_conv_i8(ConvArgs p, uint32_t pixels, uint32_t tiles) {
  const int lane = threadIdx.x & 63;
  const uint32_t wave = blockIdx.x * 4 + (threadIdx.x >> 6);
  const uint32_t nwaves = gridDim.x * 4;
  const int li = lane & 15, lg = lane >> 4;
  const int H = p.oh + p.fh - 1, W = p.ow + p.fw - 1;
  const int sub = p.c / 64;  // 64-channel slabs per filter position

  // Filter bank -> registers.  Slab s covers filter position (s / sub) and channels
  // 64*(s % sub) .. +63; lane (li, lg) holds filter row ft*16+li, bytes 16*lg .. +15.
  v4i filt[FT][SLABS];
  const uint8_t *fbase = (const uint8_t *)p.filters;
  const int krow = p.fh * p.fw * p.c;  // bytes per filter
#pragma unroll
  for (int ft = 0; ft < FT; ft++)
#pragma unroll
    for (int s = 0; s < SLABS; s++)
      filt[ft][s] = *(const v4i *)(fbase + (ft * 16 + li) * krow + s * 64 + lg * 16);

  int corr[FT][4];
  if (IMG_UNSIGNED) {
#pragma unroll
    for (int ft = 0; ft < FT; ft++) {
      int sum = 0;
#pragma unroll
      for (int s = 0; s < SLABS; s++)
#pragma unroll
        for (int w = 0; w < 4; w++) sum = __builtin_amdgcn_sdot4(filt[ft][s][w], 0x01010101, sum, false);
      sum += __shfl_xor(sum, 16);
      sum += __shfl_xor(sum, 32);  // every lane with the same li now has filter ft*16+li
#pragma unroll
      for (int r = 0; r < 4; r++) corr[ft][r] = 128 * __shfl(sum, lg * 4 + r);
    }
  }

  // Byte offset of each slab's source relative to the pixel's own (y, x) position.
  int slab_off[SLABS];
#pragma unroll
  for (int s = 0; s < SLABS; s++) {
    const int pos = s / sub, r = pos / p.fw, q = pos % p.fw;
    slab_off[s] = (r * W + q) * p.c + (s % sub) * 64 + lg * 16;
  }

  for (uint32_t t = wave; t < tiles; t += nwaves) {
    uint32_t pix = t * 16 + li;
    const bool live = pix < pixels;
    if (!live) pix = pixels - 1;  // clamp: loads stay in bounds, the store is masked
    const uint32_t x = pix % p.ow, y = (pix / p.ow) % p.oh, b = pix / (p.ow * p.oh);
    const uint8_t *src = (const uint8_t *)p.image + (int64_t(b) * H * W + int64_t(y) * W + x) * p.c;
    v4i img[SLABS];
#pragma unroll
    for (int s = 0; s < SLABS; s++) {
      img[s] = *(const v4i *)(src + slab_off[s]);
      if (IMG_UNSIGNED) img[s] ^= v4i{int(0x80808080), int(0x80808080), int(0x80808080), int(0x80808080)};
    }
    v4i acc[FT];
#pragma unroll
    for (int ft = 0; ft < FT; ft++) acc[ft] = v4i{0, 0, 0, 0};
#pragma unroll
    for (int s = 0; s < SLABS; s++)
#pragma unroll
      for (int ft = 0; ft < FT; ft++)
        acc[ft] = __builtin_amdgcn_mfma_i32_16x16x64_i8(filt[ft][s], img[s], acc[ft], 0, 0, 0);
    // D[row = filter 4*lg + r][col = pixel li]: lane owns 4 consecutive filters of its pixel.
    if (live) {
      int32_t *dst = (int32_t *)p.out + int64_t(pix) * p.f + lg * 4;
#pragma unroll
      for (int ft = 0; ft < FT; ft++) {
        v4i v = acc[ft];
        if (IMG_UNSIGNED) v += v4i{corr[ft][0], corr[ft][1], corr[ft][2], corr[ft][3]};
        v4i *d = (v4i *)(dst + ft * 16);
        if (p.accum) v += *d;
        *d = v;
      }
    }
  }
}

template <int SLABS>
hipError_t launch_slabs(const ConvArgs &c, bool img_unsigned, hipStream_t stream) {
  const uint64_t pixels = uint64_t(c.b) * c.oh * c.ow;
  const uint32_t tiles = uint32_t((pixels + 15) / 16);
  // Two workgroups of four waves per CU on a 256-CU part; never more waves than tiles.
  uint32_t blocks = 512;
  if (blocks * 4 > tiles) blocks = (tiles + 3) / 4;
  if (img_unsigned)
    hipLaunchKernelGGL((k_conv_i8<SLABS, true>), dim3(blocks), dim3(256), 0, stream, c, uint32_t(pixels), tiles);
  else
    hipLaunchKernelGGL((k_conv_i8<SLABS, false>), dim3(blocks), dim3(256), 0, stream, c, uint32_t(pixels), tiles);
  return hipGetLastError();
}

int slabs_of(const ConvArgs &c) { return int(c.fh * c.fw * (c.c / 64)); }

}  // namespace

bool conv_i8_applicable(const ConvArgs &c) {
  auto al16 = [](const void *p) { return (reinterpret_cast<uintptr_t>(p) & 15) == 0; };
  if (c.f != 64 || c.c == 0 || c.c % 64 != 0) return false;
  const int s = slabs_of(c);
  if (s != 1 && s != 9) return false;
  const uint64_t pixels = uint64_t(c.b) * c.oh * c.ow;
  const uint64_t in_bytes = uint64_t(c.b) * (c.oh + c.fh - 1) * (c.ow + c.fw - 1) * c.c;
  return pixels > 0 && pixels < (1ull << 31) && in_bytes < (1ull << 31) && al16(c.image) &&
         al16(c.filters) && al16(c.out);
}

hipError_t launch_conv_i8(const ConvArgs &c, bool img_unsigned, hipStream_t stream) {
  switch (slabs_of(c)) {
    case 1: return launch_slabs<1>(c, img_unsigned, stream);
    case 9: return launch_slabs<9>(c, img_unsigned, stream);
    default: return hipErrorInvalidValue;
  }
}

}  // namespace mrl
