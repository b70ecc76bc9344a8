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
// every loop, staged through LDS so the bank crosses L2 once per workgroup); image pixels
// go straight from global memory into MFMA operand registers, one tile ahead of the MFMAs
// (channels are the fastest NHWC dim, so one pixel's 64 channels are 64 contiguous bytes
// = four lanes x 16 B); the accumulators start at zero (to_accum) and each output pixel is
// written once, 16 B per lane.  The kernel is bound by the 4-byte-per-element output
// stream, not by the MFMA.
//
// u8 images: a' = a xor 0x80 and the per-filter correction 128 * sum_{r,s,c} filt[f,r,s,c]
// is added at the end (exact in i32).
#include <algorithm>

#include "kernels.h"

namespace mrl {
namespace {

typedef int v4i __attribute__((ext_vector_type(4)));

constexpr int FT = 4;          // filter tiles of 16 -> F = 64
constexpr int CONV_WAVES = 4;  // waves per workgroup: 4 measured fastest (8: 9.8 us against 9.4 at 32x64x56x56)

template <int SLABS, bool IMG_UNSIGNED, int WAVES>
__global__ __launch_bounds__(64 * WAVES) void k_conv_i8(const void *image, const void *filters_all, void *out_all, uint32_t c, uint32_t f,
                                                         uint32_t oh, uint32_t ow, uint32_t fh, uint32_t fw, int accum, uint32_t pixels,
                                                         uint32_t tiles) {
  // Scalar arguments, fifteen dwords: few enough to arrive preloaded in SGPRs with the wave
  // instead of through a load the first instructions would wait for.
  struct {
    const void *image, *filters;
    void *out;
    uint32_t c, f, oh, ow, fh, fw;
    int accum;
  } const p = {image, filters_all, out_all, c, f, oh, ow, fh, fw, accum};
  // The filter bank, staged once per workgroup: rows of krow bytes, 16-byte chunks.
  extern __shared__ __attribute__((aligned(16))) uint8_t filt_lds[];
  const int lane = threadIdx.x & 63;
  constexpr int NT = 64 * WAVES;
  const uint32_t wave = blockIdx.x * WAVES + (threadIdx.x >> 6);
  const uint32_t nwaves = gridDim.x * WAVES;
  const int li = lane & 15, lg = lane >> 4;
  const int H = p.oh + p.fh - 1, W = p.ow + p.fw - 1;
  const int sub = p.c / 64;  // 64-channel slabs per filter position
  const int krow = p.fh * p.fw * p.c;  // bytes per filter
  // blockIdx.y: which group of 64 filters (= 64 output channels) this workgroup computes.
  const uint8_t *filters = (const uint8_t *)p.filters + int64_t(blockIdx.y) * (FT * 16) * krow;
  int32_t *out = (int32_t *)p.out + blockIdx.y * (FT * 16);

  // Filter bank: global -> LDS (coalesced, once per workgroup) -> registers (per wave).
  // 64 filters x (SLABS * 64) bytes = SLABS * 256 chunks of 16 bytes.  These loads need
  // nothing but the pointer and the thread index, so they go out first and are in flight
  // during the address arithmetic of the first pixel tile.
  constexpr int PER_THREAD = (SLABS * 256 + NT - 1) / NT;
  v4i stage[PER_THREAD];
#pragma unroll
  for (int i = 0; i < PER_THREAD; i++) {
    const int c = i * NT + threadIdx.x;
    if (c < SLABS * 256) stage[i] = *(const v4i *)(filters + c * 16);
  }

  // Byte offset of each slab's source relative to the pixel's own (y, x) position.
  int slab_off[SLABS];
#pragma unroll
  for (int s = 0; s < SLABS; s++) {
    const int pos = s / sub, r = pos / p.fw, q = pos % p.fw;
    slab_off[s] = (r * W + q) * p.c + (s % sub) * 64 + lg * 16;
  }
  // Pixel operand of one tile: lane (li, lg) holds pixel t*16+li, channels 16*lg .. +15 of
  // every slab.  Out-of-range pixels of the last tile are clamped for the loads and masked
  // for the store.
  auto load_tile = [&](uint32_t t, v4i *img) {
    uint32_t pix = min(t * 16 + li, pixels - 1);
    const uint32_t x = pix % p.ow, y = (pix / p.ow) % p.oh, b = pix / (p.ow * p.oh);
    const uint8_t *src = (const uint8_t *)p.image + (int64_t(b) * H * W + int64_t(y) * W + x) * p.c;
#pragma unroll
    for (int s = 0; s < SLABS; s++) img[s] = *(const v4i *)(src + slab_off[s]);
  };

  // First tile's pixels are requested before anything else: their latency overlaps the
  // filter staging below.
  v4i img[SLABS];
  uint32_t t = wave;
  if (t < tiles) load_tile(t, img);

  // Filter bank, second half of its staging: registers -> LDS.
#pragma unroll
  for (int i = 0; i < PER_THREAD; i++) {
    const int c = i * NT + threadIdx.x;
    if (c < SLABS * 256) *(v4i *)(filt_lds + c * 16) = stage[i];
  }
  __syncthreads();
  v4i filt[FT][SLABS];
#pragma unroll
  for (int ft = 0; ft < FT; ft++)
#pragma unroll
    for (int s = 0; s < SLABS; s++)
      filt[ft][s] = *(const v4i *)(filt_lds + (ft * 16 + li) * krow + s * 64 + lg * 16);

  // u8 correction 128 * sum_k filt[f][k]: the same MFMAs against an all-ones pixel leave, in
  // every column, the filter sums in exactly the accumulator layout the stores use.  They are
  // parked in LDS past the filter bank.  With a multiple of the filter tiles in waves each wave forms one
  // tile's sums (a quarter of the MFMAs, which sit on every wave's path to its first store) and a
  // barrier hands them round; otherwise every wave writes the same 64 numbers and reads back its
  // own writes.
  int *corr_lds = (int *)(filt_lds + FT * 16 * krow);
  // Per wave: 16 pixel rows of 64 results, rows 68 dwords apart (16-byte aligned, banks shifted).
  constexpr int TURN_ROW = 68;
  int *turn_lds = corr_lds + FT * 16 + (threadIdx.x >> 6) * (16 * TURN_ROW);
  if (IMG_UNSIGNED) {
    const v4i ones = v4i{0x01010101, 0x01010101, 0x01010101, 0x01010101};
    constexpr bool SHARED = WAVES % FT == 0;  // several waves per filter tile write the same numbers
    const int my_ft = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6) % FT;
#pragma unroll
    for (int ft = 0; ft < FT; ft++) {
      if (SHARED && ft != my_ft) continue;
      v4i sum = v4i{0, 0, 0, 0};
#pragma unroll
      for (int s = 0; s < SLABS; s++) sum = __builtin_amdgcn_mfma_i32_16x16x64_i8(filt[ft][s], ones, sum, 0, 0, 0);
      if (li == 0) *(v4i *)(corr_lds + ft * 16 + lg * 4) = sum * 128;
    }
    if (SHARED) __syncthreads();
  }

  // The pixel registers are refilled slab by slab with the next tile as soon as the MFMAs
  // of the current tile have consumed them, so the next tile's loads are in flight under
  // the rest of this tile's MFMAs and its stores.
  while (t < tiles) {
    const uint32_t tn = t + nwaves;
    const uint32_t pix_n = min(min(tn, tiles - 1) * 16 + li, pixels - 1);  // clamped: always loadable
    const uint32_t xn = pix_n % p.ow, yn = (pix_n / p.ow) % p.oh, bn = pix_n / (p.ow * p.oh);
    const uint8_t *src_n = (const uint8_t *)p.image + (int64_t(bn) * H * W + int64_t(yn) * W + xn) * p.c;
    v4i acc[FT];
#pragma unroll
    for (int ft = 0; ft < FT; ft++) acc[ft] = v4i{0, 0, 0, 0};
#pragma unroll
    for (int s = 0; s < SLABS; s++) {
      v4i px = img[s];
      if (IMG_UNSIGNED) px ^= v4i{int(0x80808080), int(0x80808080), int(0x80808080), int(0x80808080)};
#pragma unroll
      for (int ft = 0; ft < FT; ft++)
        acc[ft] = __builtin_amdgcn_mfma_i32_16x16x64_i8(filt[ft][s], px, acc[ft], 0, 0, 0);
      img[s] = *(const v4i *)(src_n + slab_off[s]);
    }
    // D[row = filter 4*lg + r][col = pixel li]: lane owns 4 consecutive filters of its pixel in
    // each filter tile, i.e. 16-byte pieces 64 bytes apart.  The tile's 16 x 64 results go through
    // this wave's own patch of LDS so that the stores are whole 256-byte pixel rows, four
    // pixels per instruction (1 KiB contiguous when F = 64), instead of 64-byte segments.
#pragma unroll
    for (int ft = 0; ft < FT; ft++) {
      v4i v = acc[ft];
      if (IMG_UNSIGNED) v += *(const v4i *)(corr_lds + ft * 16 + lg * 4);
      *(v4i *)(turn_lds + li * TURN_ROW + ft * 16 + lg * 4) = v;
    }
    __builtin_amdgcn_wave_barrier();  // LDS operations of a wave complete in order
#pragma unroll
    for (int i = 0; i < 4; i++) {
      const uint32_t row = i * 4 + lg, pix = t * 16 + row;  // lane (li, lg): pixel row, filters 4*li .. +3
      v4i v = *(const v4i *)(turn_lds + row * TURN_ROW + li * 4);
      if (pix < pixels) {
        v4i *d = (v4i *)(out + int64_t(pix) * p.f + li * 4);
        if (p.accum) v += *d;
        __builtin_nontemporal_store(v, d);  // written once, never re-read by this kernel
      }
    }
    __builtin_amdgcn_wave_barrier();
    t = tn;
  }
}

template <int SLABS>
hipError_t launch_slabs(const ConvArgs &c, bool img_unsigned, hipStream_t stream) {
  const uint64_t pixels = uint64_t(c.b) * c.oh * c.ow;
  const uint32_t tiles = uint32_t((pixels + 15) / 16);
  // 2048 waves = two per SIMD of a 256-CU part at ~250 VGPRs each, as workgroups of
  // CONV_WAVES waves; never more waves than tiles.
  constexpr int WAVES = CONV_WAVES;
  const uint32_t groups = c.f / (FT * 16);
  uint32_t blocks = std::max<uint32_t>(1, 2048 / WAVES / groups);
  if (blocks * WAVES > tiles) blocks = (tiles + WAVES - 1) / WAVES;
  // the filter bank + corrections + a 16 x 68-dword patch per wave for the output rows
  const size_t lds = size_t(FT) * 16 * c.fh * c.fw * c.c + FT * 16 * sizeof(int) + size_t(WAVES) * 16 * 68 * sizeof(int);
  plan::work(plan::UNIT_MFMA_I8, 2.0 * pixels * c.f * c.fh * c.fw * c.c,
             double(c.b) * (c.oh + c.fh - 1) * (c.ow + c.fw - 1) * c.c + double(c.f) * c.fh * c.fw * c.c +
                 4.0 * pixels * c.f * (c.accum ? 2 : 1));
  if (img_unsigned)
    MRL_LAUNCH((k_conv_i8<SLABS, true, WAVES>), dim3(blocks, groups), dim3(64 * WAVES), lds, stream, c.image, c.filters, c.out, c.c, c.f, c.oh, c.ow,
               c.fh, c.fw, c.accum, uint32_t(pixels), tiles);
  else
    MRL_LAUNCH((k_conv_i8<SLABS, false, WAVES>), dim3(blocks, groups), dim3(64 * WAVES), lds, stream, c.image, c.filters, c.out, c.c, c.f, c.oh, c.ow,
               c.fh, c.fw, c.accum, uint32_t(pixels), tiles);
  return mrl::plan::last_error();
}

int slabs_of(const ConvArgs &c) { return int(c.fh * c.fw * (c.c / 64)); }

}  // namespace

bool conv_i8_applicable(const ConvArgs &c) {
  auto al16 = [](const void *p) { return (reinterpret_cast<uintptr_t>(p) & 15) == 0; };
  if (c.f == 0 || c.f % 64 != 0 || c.f > 64 * 65535 || c.c == 0 || c.c % 64 != 0) return false;
  const int s = slabs_of(c);  // 16 VGPRs of filter operands per slab and lane
  if (s != 1 && s != 2 && s != 3 && s != 4 && s != 6 && s != 9) return false;
  const uint64_t pixels = uint64_t(c.b) * c.oh * c.ow;
  const uint64_t in_bytes = uint64_t(c.b) * (c.oh + c.fh - 1) * (c.ow + c.fw - 1) * c.c;
  return pixels > 0 && pixels < (1ull << 31) && in_bytes < (1ull << 31) && al16(c.image) &&
         al16(c.filters) && al16(c.out);
}

hipError_t launch_conv_i8(const ConvArgs &c, bool img_unsigned, hipStream_t stream) {
  switch (slabs_of(c)) {
    case 1: return launch_slabs<1>(c, img_unsigned, stream);
    case 2: return launch_slabs<2>(c, img_unsigned, stream);
    case 3: return launch_slabs<3>(c, img_unsigned, stream);
    case 4: return launch_slabs<4>(c, img_unsigned, stream);
    case 6: return launch_slabs<6>(c, img_unsigned, stream);
    case 9: return launch_slabs<9>(c, img_unsigned, stream);
    default: return hipErrorInvalidValue;
  }
}

}  // namespace mrl
