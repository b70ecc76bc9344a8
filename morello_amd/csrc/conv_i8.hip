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

template <int SLABS, bool IMG_UNSIGNED, int WAVES, bool OUT_PLANES>
__global__ __launch_bounds__(64 * WAVES) void k_conv_i8(const void *image, const void *filters_all, void *out_all, uint32_t f, uint32_t oh,
                                                         uint32_t ow, uint32_t packed, uint32_t pixels, uint32_t ow_mul, uint32_t oh_mul,
                                                         uint32_t nwaves) {
  // Scalar arguments, fourteen dwords: what arrives preloaded in SGPRs with the wave instead of
  // through a load the first instructions would wait for (the waves of the whole grid included,
  // which the launch would otherwise leave behind the explicit arguments).  `packed`: fh, fw in
  // four bits each, accum in bit 8, the 64-channel slabs of a pixel from bit 9, the two divisions'
  // shifts in bits 16-21 and 24-29.
  struct {
    const void *image, *filters;
    void *out;
    uint32_t c, f, oh, ow, fh, fw;
    int accum;
  } const p = {image, filters_all, out_all, ((packed >> 9) & 15) * 64, f, oh, ow, packed & 15, (packed >> 4) & 15, int((packed >> 8) & 1)};
  const uint32_t tiles = (pixels + 15) / 16;
  // pixel number -> (image, row, column) by multiply-and-shift (FastDiv: exact below 2^31)
  FastDiv by_ow, by_oh;
  by_ow.mul = ow_mul, by_ow.shift = (packed >> 16) & 63, by_oh.mul = oh_mul, by_oh.shift = (packed >> 24) & 63;
  // (byte offset of the pixel's window corner in the image: below 2^31, conv_i8_applicable)
  auto corner = [&](uint32_t pix) {
    const uint32_t row = by_ow.div(pix), b = by_oh.div(row);
    return ((b * (p.oh + p.fh - 1) + (row - b * p.oh)) * (p.ow + p.fw - 1) + (pix - row * p.ow)) * p.c;
  };
  // The filter bank, staged once per workgroup: rows of krow bytes, 16-byte chunks.
  extern __shared__ __attribute__((aligned(16))) uint8_t filt_lds[];
  const int lane = threadIdx.x & 63;
  constexpr int NT = 64 * WAVES;
  const uint32_t wave = blockIdx.x * WAVES + (threadIdx.x >> 6);
  const int li = lane & 15, lg = lane >> 4;
  const int W = p.ow + p.fw - 1;
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
  constexpr bool EVEN_SHARES = SLABS * 256 % NT == 0;   // every thread moves PER_THREAD chunks: no bounds to test
  v4i stage[PER_THREAD];
#pragma unroll
  for (int i = 0; i < PER_THREAD; i++) {
    const int c = i * NT + threadIdx.x;
    if (EVEN_SHARES || c < SLABS * 256) stage[i] = *(const v4i *)(filters + c * 16);
  }

  // Byte offset of each slab's source relative to the pixel's own (y, x) position.
  // Slab s is channels 64 * (s % sub) .. of filter position s / sub.  The fw * sub slabs of a
  // filter row are consecutive bytes of the image (channels fastest, then pixels), and the next
  // row starts (W - fw) pixels further on: counted up, not divided.
  uint32_t slab_off[SLABS];
  {
    uint32_t off = 0, in_row = 0;
    const uint32_t row_slabs = p.fw * sub, skip = (W - p.fw) * p.c;
#pragma unroll
    for (int s = 0; s < SLABS; s++) {
      slab_off[s] = off + lg * 16;
      off += 64;
      if (++in_row == row_slabs) in_row = 0, off += skip;
    }
  }
  // Pixel operand of one tile: lane (li, lg) holds pixel t*16+li, channels 16*lg .. +15 of
  // every slab.  Out-of-range pixels of the last tile are clamped for the loads and masked
  // for the store.
  auto load_tile = [&](uint32_t t, v4i *img) {
    uint32_t pix = min(t * 16 + li, pixels - 1);
    const uint32_t src = corner(pix);
#pragma unroll
    for (int s = 0; s < SLABS; s++) img[s] = *(const v4i *)((const uint8_t *)p.image + (src + slab_off[s]));
  };

  // First tile's pixels are requested before anything else: their latency overlaps the
  // filter staging below.
  v4i img[SLABS];
  // Which tiles: dealt round-robin over all waves, or (MRL_CONV_XCD_RUNS, bit 30 of `packed`) each
  // XCD's workgroups (every eighth one) over a contiguous eighth of the tiles, so that an XCD's L2
  // holds an eighth of the image instead of all of it.  Measured no faster (7.78 against 7.84 us
  // at 32 x 56 x 56 x 64): the image's second and third readers find it in the memory-side cache.
  uint32_t t = wave, t_end = tiles, t_step = nwaves;
  if (packed & (1u << 30)) {
    const uint32_t per_xcd = (tiles + 7) / 8, xcd = blockIdx.x & 7;
    t = xcd * per_xcd + (blockIdx.x >> 3) * WAVES + (threadIdx.x >> 6);
    t_end = min(tiles, (xcd + 1) * per_xcd);
    t_step = nwaves >> 3;
  }
  if (t < t_end) load_tile(t, img);

  // Filter bank, second half of its staging: registers -> LDS.
#pragma unroll
  for (int i = 0; i < PER_THREAD; i++) {
    const int c = i * NT + threadIdx.x;
    if (EVEN_SHARES || c < SLABS * 256) *(v4i *)(filt_lds + c * 16) = stage[i];
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
  while (t < t_end) {
    const uint32_t tn = t + t_step;
    const uint32_t pix_n = min(min(tn, tiles - 1) * 16 + li, pixels - 1);  // clamped: always loadable
    const uint32_t src_n = corner(pix_n);
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
      img[s] = *(const v4i *)((const uint8_t *)p.image + (src_n + slab_off[s]));
    }
    // D[row = filter 4*lg + r][col = pixel li]: lane owns 4 consecutive filters of its pixel in
    // each filter tile.  An output stored as planes of filters takes them as they are: register r
    // of the 16 lanes of a group is 16 consecutive pixels of one filter's plane, 64 contiguous
    // bytes (a tile that crosses into the next image continues in that image's plane).
    if constexpr (OUT_PLANES) {
      const uint32_t pix = t * 16 + li;
      if (pix < pixels) {
        const uint32_t plane = p.oh * p.ow, b = by_oh.div(by_ow.div(pix));
        int32_t *first = (int32_t *)p.out + (int64_t(b) * p.f + blockIdx.y * (FT * 16) + lg * 4) * plane + (pix - b * plane);
#pragma unroll
        for (int ft = 0; ft < FT; ft++) {
          v4i v = acc[ft];
          if (p.accum) {   // a filter tile's four old values requested together (all sixteen: too many registers beside nine slabs of filters)
            v4i old;
#pragma unroll
            for (int r = 0; r < 4; r++) old[r] = first[int64_t(ft * 16 + r) * plane];
            v += old;
          }
          if (IMG_UNSIGNED) v += *(const v4i *)(corr_lds + ft * 16 + lg * 4);
          // ordinary stores: half a cache line each, the other half comes from the neighbouring tile
          // (non-temporal ones measured 16.1 against 11.7 us at 32 x 64 x 56 x 56)
#pragma unroll
          for (int r = 0; r < 4; r++) first[int64_t(ft * 16 + r) * plane] = v[r];
        }
      }
      t = tn;
      continue;
    }
    // Channels-last: 16-byte pieces 64 bytes apart.  The tile's 16 x 64 results go through
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


// ---- 64 channels, whole output rows per workgroup ----------------------------------------------
// The same Conv with the roles of a workgroup's four waves turned round: wave w holds 16 of the 64
// filters (TAPS x 4 operand registers instead of TAPS x 16: a quarter of the start-up, and room
// for four waves per SIMD), and all four multiply them with the SAME pixels, which therefore come
// through LDS once per workgroup instead of once per wave: the input rows that a run of output
// rows touches are one contiguous piece of the NHWC image (also across an image boundary), moved
// by direct-to-LDS loads (no staging registers), and the fh x fw taps of a pixel tile are reads
// of that piece at different offsets, so the taps' overlap is served by LDS instead of by the
// vector cache (the image crosses it 1.5-2 times instead of fh * fw / 1.2 times).  A u8 image is
// made signed (xor 0x80) once per byte in LDS instead of once per tap and wave in registers.
//   move_param(image, L1) -> global_load_lds_dwordx4, rows padded to 16 pixels, a pixel's four
//   16-byte chunks rotated by (pixel / 2) % 4, which is what lets the 16 lanes of an operand read
//   (pixels 64 bytes apart) run at the full LDS rate (measured: 2.75 cycles a read for 16 waves of a
//   compute unit, as for a contiguous read; 4.27 with no rotation or with (pixel / 4) % 4); applied
//   on the source side of the loads.
// Output: a lane holds 4 consecutive filters of one pixel (16 bytes); the four waves' pieces of a
// tile meet in LDS and are written as whole pixel rows.
typedef __attribute__((address_space(3))) void lds_void_t;

__device__ inline void conv_dma16(const uint8_t *base, uint32_t voff, uint32_t lds_addr) {
  asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2" : : "s"(lds_addr), "v"(voff), "s"(base) : "memory");
}

template <int TAPS, bool IMG_UNSIGNED>
__global__ __launch_bounds__(256) void k_conv_rows_i8(const void *image, const void *filters_all, void *out_all, uint32_t f,
                                                      uint32_t oh, uint32_t ow, uint32_t fh, uint32_t fw, int accum,
                                                      uint32_t total_rows, uint32_t rows_per_wg) {
  struct {
    const void *image, *filters;
    void *out;
    uint32_t f, oh, ow, fh, fw;
    int accum;
    uint32_t total_rows, rows_per_wg;
  } const p = {image, filters_all, out_all, f, oh, ow, fh, fw, accum, total_rows, rows_per_wg};
  extern __shared__ __attribute__((aligned(1024))) uint8_t rows_lds[];
  const int lane = threadIdx.x & 63, li = lane & 15, lg = lane >> 4;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const uint32_t H = p.oh + p.fh - 1, W = p.ow + p.fw - 1, W16 = (W + 15) & ~15u;
  const uint32_t row_bytes = W16 * 64, kb_per_row = W16 / 16;
  // Output rows [g0, g1) (row g = image g / oh, line g % oh) and the input rows they read: input
  // row b * H + y is row-major memory, and the last rows of one image are followed by the first of
  // the next, so the piece is contiguous whatever the run crosses.
  const uint32_t g0 = blockIdx.x * p.rows_per_wg, g1 = min(g0 + p.rows_per_wg, p.total_rows);
  const uint32_t in_first = (g0 / p.oh) * H + g0 % p.oh;
  const uint32_t in_last = ((g1 - 1) / p.oh) * H + (g1 - 1) % p.oh + p.fh - 1;
  const uint32_t nkb = (in_last - in_first + 1) * kb_per_row;
  const uint32_t lds0 = uint32_t(reinterpret_cast<uintptr_t>((lds_void_t *)rows_lds));
  {
    // KiB k of the piece: 16 pixels of input row in_first + k / kb_per_row; lane L fills 16-byte
    // position L % 4 of pixel L / 4 with the chunk that belongs there.  Pixels past the row's end
    // (the padding) fetch the row's last pixel again.
    const uint32_t pl = lane >> 2, cp = lane & 3;
    for (uint32_t k = wave; k < nkb; k += 4) {
      const uint32_t ku = __builtin_amdgcn_readfirstlane(k);
      const uint32_t row = in_first + ku / kb_per_row, xp = 16 * (ku % kb_per_row) + pl;
      const uint32_t chunk = (cp - (xp >> 1)) & 3;
      conv_dma16((const uint8_t *)p.image, (row * W + min(xp, W - 1)) * 64 + chunk * 16, lds0 + ku * 1024);
    }
  }
  // This wave's 16 filters as MFMA operands: lane (li, lg) holds channels 16 lg .. + 15 of filter li, per tap.
  const uint8_t *filters = (const uint8_t *)p.filters + (int64_t(blockIdx.y) * 64 + wave * 16 + li) * (TAPS * 64) + lg * 16;
  v4i filt[TAPS];
#pragma unroll
  for (int t = 0; t < TAPS; t++) filt[t] = *(const v4i *)(filters + t * 64);
  // Per tap the lane's address within an output row's first tile: pixel li + s of input row r.
  uint32_t tap_addr[TAPS];
#pragma unroll
  for (int t = 0; t < TAPS; t++) {
    const uint32_t r = t / p.fw, s0 = t % p.fw, xp = li + s0;
    tap_addr[t] = r * row_bytes + xp * 64 + (((lg + (xp >> 1)) & 3) << 4);
  }
  __builtin_amdgcn_s_waitcnt(0x0F70);  // the piece and the filters are in
  if (IMG_UNSIGNED) {
    // a - 128 for every byte this wave fetched (its own KiBs: no barrier needed before)
    for (uint32_t k = wave; k < nkb; k += 4) {
      unsigned long long *q = (unsigned long long *)(rows_lds + k * 1024) + lane;
      __hip_atomic_fetch_xor(q, 0x8080808080808080ull, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
      __hip_atomic_fetch_xor(q + 64, 0x8080808080808080ull, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
    }
  }
  // u8 correction 128 * sum filt[f]: the same MFMAs against an all-ones pixel leave the filter sums
  // in the accumulator layout; the accumulators start from it.
  v4i corr = v4i{0, 0, 0, 0};
  if (IMG_UNSIGNED) {
    const v4i ones = v4i{0x01010101, 0x01010101, 0x01010101, 0x01010101};
#pragma unroll
    for (int t = 0; t < TAPS; t++) corr = __builtin_amdgcn_mfma_i32_16x16x64_i8(filt[t], ones, corr, 0, 0, 0);
    corr *= 128;
  }
  __syncthreads();
  const uint32_t ntiles = (p.ow + 15) / 16, count = (g1 - g0) * ntiles;
  int32_t *out = (int32_t *)p.out + blockIdx.y * 64 + li * 4;
  // The run's tiles in order: 16 pixels each, tile j of output row g.  A cursor walks them (no
  // division per tile): LDS offset of the row's first input row and of the tile in it, and the
  // output offset of the row's first pixel.  Past the last tile it stays on it.
  struct Cursor {
    uint32_t j, y, lds_off, left;   // tile within the row, line within the image, LDS offset of tile 0's pixel 0, tiles left
    int64_t out_off;                // elements from `out` to the row's pixel 0
  };
  Cursor cur = {0, g0 % p.oh, 0, count, int64_t(g0) * p.ow * p.f};
  auto advance = [&](Cursor &c) {
    if (c.left <= 1) return;
    c.left--;
    if (++c.j < ntiles) return;
    c.j = 0;
    c.out_off += int64_t(p.ow) * p.f;
    // the next output row's first input row: the next LDS row, or fh rows on where a new image begins
    const bool wrap = c.y + 1 == p.oh;
    c.lds_off += (wrap ? p.fh : 1u) * row_bytes;
    c.y = wrap ? 0 : c.y + 1;
  };
  // The operands of the next tile are read from LDS while the current one is multiplied: two
  // register sets taken in turn, every read and every MFMA issued whatever the tile (a tile past
  // the end repeats the last one and stores nothing), so that the loop body is one straight line
  // and a wait can be for one set's reads alone.
  auto read_tile = [&](const Cursor &c, v4i *px) {
    const uint8_t *at = rows_lds + c.lds_off + c.j * 1024;
#pragma unroll
    for (int t = 0; t < TAPS; t++) px[t] = *(const v4i *)(at + tap_addr[t]);
  };
  // A tile's 16 x 64 results are the four waves' 16 x 16 blocks side by side (a lane holds 4
  // consecutive filters of one pixel, 16 bytes of its 256-byte row).  They meet in LDS (rows 272
  // bytes apart: 16 bytes of padding shift the banks) and leave as whole rows, wave w the four
  // pixels 4 w .. 4 w + 3: 1 KiB contiguous per store instruction when F = 64, where four waves
  // writing their 64-byte pieces cost 3 us of a 9.7 us launch.  Two exchange buffers in turn,
  // one barrier per tile.
  constexpr int XROW = 272;
  uint8_t *xbuf = rows_lds + (in_last - in_first + 1) * row_bytes + 1024;
  uint32_t turn = 0;
  auto finish_tile = [&](const Cursor &c, bool live, const v4i *px) {
    v4i acc = corr;
#pragma unroll
    for (int t = 0; t < TAPS; t++) acc = __builtin_amdgcn_mfma_i32_16x16x64_i8(filt[t], px[t], acc, 0, 0, 0);
    uint8_t *xb = xbuf + turn * (16 * XROW);
    turn ^= 1;
    *(v4i *)(xb + li * XROW + wave * 64 + lg * 16) = acc;
    __syncthreads();
    const uint32_t pixel = 4 * wave + lg, x = 16 * c.j + pixel;
    v4i v = *(const v4i *)(xb + pixel * XROW + li * 16);
    if (live && x < p.ow) {
      v4i *d = (v4i *)(out + c.out_off + int64_t(x) * p.f);
      if (p.accum) v += *d;
      __builtin_nontemporal_store(v, d);
    }
  };
  v4i px_a[TAPS], px_b[TAPS];
  read_tile(cur, px_a);
  for (uint32_t i = 0; i < count; i += 2) {
    Cursor nxt = cur;
    advance(nxt);
    read_tile(nxt, px_b);
    finish_tile(cur, true, px_a);
    cur = nxt;
    advance(nxt);
    read_tile(nxt, px_a);
    finish_tile(cur, i + 1 < count, px_b);
    cur = nxt;
  }
}

// Output rows per workgroup and the LDS the piece of the image takes, or 0 when the kernel does
// not apply (the piece of the smallest run does not fit).
struct RowsPlan {
  uint32_t rows_per_wg, lds_bytes;
};
RowsPlan conv_rows_plan(const ConvArgs &c) {
  const uint32_t W = c.ow + c.fw - 1, W16 = (W + 15) & ~15u, row_bytes = W16 * 64;
  const uint64_t total_rows = uint64_t(c.b) * c.oh;
  // four workgroups of four waves per compute unit when there are rows enough
  uint32_t rows = uint32_t(std::min<uint64_t>(8, std::max<uint64_t>(1, (total_rows + 4 * g_compute_units - 1) / (4 * g_compute_units))));
  for (; rows >= 1; rows--) {
    const uint32_t crossings = (rows + c.oh - 2) / c.oh;   // image boundaries a run of `rows` can cross
    const uint64_t in_rows = rows + uint64_t(c.fh - 1) * (1 + crossings);
    const uint64_t lds = in_rows * row_bytes + 1024 + 2 * 16 * 272;   // the piece, slack for reads past it, two exchange buffers
    if (lds <= 40 * 1024) return RowsPlan{rows, uint32_t(lds)};
  }
  return RowsPlan{0, 0};
}

template <int TAPS>
hipError_t launch_rows(const ConvArgs &c, bool img_unsigned, const RowsPlan &rp, hipStream_t stream) {
  const uint32_t total_rows = c.b * c.oh;
  const dim3 grid((total_rows + rp.rows_per_wg - 1) / rp.rows_per_wg, c.f / 64);
  const double pixels = double(total_rows) * c.ow;
  plan::work(plan::UNIT_MFMA_I8, 2.0 * pixels * c.f * c.fh * c.fw * c.c,
             double(c.b) * (c.oh + c.fh - 1) * (c.ow + c.fw - 1) * c.c + double(c.f) * c.fh * c.fw * c.c +
                 4.0 * pixels * c.f * (c.accum ? 2 : 1));
  if (img_unsigned)
    MRL_LAUNCH((k_conv_rows_i8<TAPS, true>), grid, dim3(256), rp.lds_bytes, stream, c.image, c.filters, c.out, c.f, c.oh, c.ow, c.fh,
               c.fw, c.accum, total_rows, rp.rows_per_wg);
  else
    MRL_LAUNCH((k_conv_rows_i8<TAPS, false>), grid, dim3(256), rp.lds_bytes, stream, c.image, c.filters, c.out, c.f, c.oh, c.ow, c.fh,
               c.fw, c.accum, total_rows, rp.rows_per_wg);
  return mrl::plan::last_error();
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
  const FastDiv by_ow(c.ow), by_oh(c.oh);
  // (a window of at most nine slabs: fh, fw and the slabs of a pixel are at most nine each)
  uint32_t packed = c.fh | c.fw << 4 | uint32_t(c.accum != 0) << 8 | (c.c / 64) << 9 | by_ow.shift << 16 | by_oh.shift << 24;
#ifdef MRL_CONV_XCD_RUNS
  if (blocks % 8 == 0 && groups == 1) packed |= 1u << 30;
#endif
#define MRL_CONV_I8(U, PLANES)                                                                                                      \
  MRL_LAUNCH((k_conv_i8<SLABS, U, WAVES, PLANES>), dim3(blocks, groups), dim3(64 * WAVES), lds, stream, c.image, c.filters, c.out, c.f, \
             c.oh, c.ow, packed, uint32_t(pixels), by_ow.mul, by_oh.mul, blocks * WAVES)
  if (img_unsigned && c.out_planes) MRL_CONV_I8(true, true);
  else if (img_unsigned) MRL_CONV_I8(true, false);
  else if (c.out_planes) MRL_CONV_I8(false, true);
  else MRL_CONV_I8(false, false);
#undef MRL_CONV_I8
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

bool conv_rows_applicable(const ConvArgs &c) {
  return conv_i8_applicable(c) && !c.out_planes && c.c == 64 && uint64_t(c.b) * c.oh < (1u << 31) && conv_rows_plan(c).rows_per_wg > 0;
}

hipError_t launch_conv_i8(const ConvArgs &c, bool img_unsigned, hipStream_t stream, bool whole_rows) {
  // The kernel that shares a workgroup's pixels through LDS (64 channels: a tap is one k step)
  // is taken when asked for: on the benchmark's Conv the two kernels measure the same (8.8-8.9 us:
  // both are a launch, a start-up of one trip to memory and the 24 MB of output at HBM's rate).
  if (whole_rows) {
    if (!conv_rows_applicable(c)) return hipErrorInvalidValue;
    const RowsPlan rp = conv_rows_plan(c);
    switch (slabs_of(c)) {
      case 1: return launch_rows<1>(c, img_unsigned, rp, stream);
      case 2: return launch_rows<2>(c, img_unsigned, rp, stream);
      case 3: return launch_rows<3>(c, img_unsigned, rp, stream);
      case 4: return launch_rows<4>(c, img_unsigned, rp, stream);
      case 6: return launch_rows<6>(c, img_unsigned, rp, stream);
      default: return launch_rows<9>(c, img_unsigned, rp, stream);
    }
  }
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
