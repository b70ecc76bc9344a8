// Conv NHWC u8|i8 x KRSC i8 -> i32, bf16 x bf16 -> f32 and f32 x f32 -> f32 for pixels of few channels (a first layer: 3 channels, 7 x 7
// filters), where a pixel's channels are not whole 16-byte chunks and the implicit Matmul of
// conv_gemm.hip does not apply (morello/src/spec.rs:486-494: no stride, no padding).  The other
// route for such shapes writes every window to memory first (unfold.hip) and multiplies the rows:
// 64 MB of windows for 32 x 3 x 118 x 118 -> 64 x 112 x 112.  Here the windows are formed in LDS.
//
// A workgroup of four waves takes tiles of 8 x 16 output pixels of one image, one after the other:
//   1. the tile's input patch ((8 + fh - 1) x (16 + fw - 1) pixels) goes into LDS (u8 as a - 128);
//      its bytes are fetched into registers while the previous tile is multiplied;
//   2. every output pixel's window is copied out of the patch into a row of its own: fh runs of
//      fw * c contiguous bytes, each run padded to whole dwords (so that the copies are dwords: two
//      aligned reads and a byte alignment per dword written), the row to whole MFMA k steps of 64 bytes;
//   3. each wave multiplies two rows of the tile (16 pixels each: a B operand block) with the
//      filters (A operands from LDS, staged once per workgroup in the same padded order, zeros in
//      the padding, so that whatever the windows hold there counts for nothing):
//      v_mfma_i32_16x16x64_i8 / v_mfma_f32_16x16x32_bf16 (the same 64 bytes of window a step, the
//      same 16 bytes a lane group), a lane ends up with 4 consecutive filters of one pixel, 16
//      contiguous bytes of the channels-last output.  f32: four v_mfma_f32_16x16x4_f32 per
//      64 bytes, the j-th on the j-th of the 16 bytes' four values (a lane group's 16 bytes are
//      four k indices; which ones is free as long as both operands agree).  Floats: the padding
//      of the windows is zeros as well (a NaN there times a zero weight would not be zero).
// The u8 correction 128 * sum of a filter's weights comes from the same MFMAs against an operand
// of ones, once per workgroup.  Rows of windows and filters lie 16 bytes more than their length
// apart, which spreads the 16 lanes of an operand read over all banks.
#include "kernels.h"
#include "plan.h"

namespace mrl {
namespace {

typedef int v4i __attribute__((ext_vector_type(4)));
typedef float v4f __attribute__((ext_vector_type(4)));
typedef __bf16 v8bf __attribute__((ext_vector_type(8)));
enum { IMG_I8 = 0, IMG_U8 = 1, IMG_BF16 = 2, IMG_F32 = 3 };

constexpr int TILE_H = 8, TILE_W = 16, TILE_PIXELS = TILE_H * TILE_W;
constexpr int PATCH_REGS = 8;   // patch bytes a thread holds in flight: patches of up to 2 KiB

struct WindowsArgs {
  const uint8_t *image, *filters;
  int32_t *out;
  uint32_t b, f, c, oh, ow, fh, fw;   // c: BYTES of one pixel's channels
  int accum;
  uint32_t tiles_x, tiles_y, tiles;   // per image, per image, in all
  uint32_t seg, seg_padded;           // fw * c: bytes of one run of a window; the same in whole dwords
  uint32_t patch_stride;              // bytes between the patch's rows in LDS (whole dwords)
  // The image / the output as planes ([b][c][h][w], [b][f][oh][ow]: dense NCHW) instead of channels-last.
  // A patch's bytes are fetched one by one either way, so planes only change where a byte comes
  // from; the accumulators hold 16 consecutive pixels of a filter per register and lane group,
  // 64 contiguous bytes of that filter's plane, and are stored as they are.
  int in_planes, out_planes;
};

// KS: MFMA k steps per window (fh * seg_padded bytes, padded to 64 KS).
template <int KS, int KIND>
__global__ __launch_bounds__(256) void k_conv_windows(WindowsArgs p) {
  constexpr bool IMG_UNSIGNED = KIND == IMG_U8, FLOATS = KIND == IMG_BF16 || KIND == IMG_F32, HALVES = KIND == IMG_BF16;
  typedef typename std::conditional<FLOATS, v4f, v4i>::type Acc;
  auto mfma = [](v4i a, v4i b, Acc c) {
    if constexpr (KIND == IMG_F32) {
      const v4f fa = __builtin_bit_cast(v4f, a), fb = __builtin_bit_cast(v4f, b);
#pragma unroll
      for (int j = 0; j < 4; j++) c = __builtin_amdgcn_mfma_f32_16x16x4f32(fa[j], fb[j], c, 0, 0, 0);
      return c;
    } else if constexpr (KIND == IMG_BF16) {
      return __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(v8bf, a), __builtin_bit_cast(v8bf, b), c, 0, 0, 0);
    } else {
      return __builtin_amdgcn_mfma_i32_16x16x64_i8(a, b, c, 0, 0, 0);
    }
  };
  extern __shared__ __attribute__((aligned(16))) uint8_t win_lds[];
  // Rows of windows and filters: 16 bytes more than their length apart (144 at least: two pixel
  // blocks' rows also hold a block's 16 x 272 bytes of results on their way out).
  constexpr int KPAD = 64 * KS, ROW = KS == 1 ? 144 : KPAD + 16;
  const int tid = threadIdx.x, lane = tid & 63, li = lane & 15, lg = lane >> 4;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  uint8_t *filt = win_lds;                    // [64][ROW]
  uint8_t *rows = filt + 64 * ROW;            // [128][ROW]
  uint8_t *patch = rows + TILE_PIXELS * ROW;  // [TILE_H + fh - 1][patch_stride] + 4
  const uint32_t f0 = blockIdx.y * 64, nf = min(64u, p.f - f0);   // this workgroup's filters (a multiple of 16)
  const int nfb = int(nf / 16);
  const uint32_t k = p.fh * p.seg;

  const uint32_t patch_h = TILE_H + p.fh - 1, patch_wb = (TILE_W + p.fw - 1) * p.c, patch_bytes = patch_h * patch_wb;
  const uint32_t h = p.oh + p.fh - 1, w = p.ow + p.fw - 1;
  // A tile's patch: rows y0 .. of the image from pixel x0 on; past the image's edge (a ragged
  // tile) the last row / the row's last byte again, which only reaches pixels that are not stored.
  // Which row and byte of the patch a thread's j-th byte is does not depend on the tile: the
  // divisions are done once.
  uint8_t held[PATCH_REGS];
  uint32_t held_row[PATCH_REGS], held_byte[PATCH_REGS];
#pragma unroll
  for (int j = 0; j < PATCH_REGS; j++) {
    const uint32_t i = tid + j * 256;
    held_row[j] = i / patch_wb, held_byte[j] = i % patch_wb;
  }
  struct Corner {
    uint32_t img, y0, x0;
  };
  auto corner_of = [&](uint32_t t) {
    const uint32_t per_image = p.tiles_x * p.tiles_y, img = t / per_image, in_img = t - img * per_image, ty = in_img / p.tiles_x;
    return Corner{img, ty * TILE_H, (in_img - ty * p.tiles_x) * TILE_W};
  };
  constexpr uint32_t ES = KIND == IMG_F32 ? 4 : KIND == IMG_BF16 ? 2 : 1;   // bytes of an element
  auto patch_source = [&](const Corner &at, uint32_t r, uint32_t xb) {
    const uint32_t y = min(at.y0 + r, h - 1), x = min(at.x0 * p.c + xb, w * p.c - 1);
    if (p.in_planes) {
      const uint32_t pixel = x / p.c, in_pixel = x - pixel * p.c, channel = in_pixel / ES;
      return p.image + ((uint64_t(at.img) * (p.c / ES) + channel) * h + y) * w * ES + pixel * ES + (in_pixel - channel * ES);
    }
    return p.image + (uint64_t(at.img) * h + y) * w * p.c + x;
  };
  auto fetch_patch = [&](uint32_t t) {
    const Corner at = corner_of(t);
#pragma unroll
    for (int j = 0; j < PATCH_REGS; j++)
      if (tid + j * 256 < patch_bytes) held[j] = *patch_source(at, held_row[j], held_byte[j]);
  };
  auto put = [&](uint32_t r, uint32_t xb, uint8_t v) { patch[r * p.patch_stride + xb] = IMG_UNSIGNED ? uint8_t(v ^ 0x80) : v; };
  if (blockIdx.x < p.tiles) fetch_patch(blockIdx.x);   // the first tile's patch: in flight while the filters are staged
  // The filters, once: run r of filter f at r * seg_padded of the filter's row, zeros everywhere
  // else.  Their nf * k bytes are one contiguous piece of memory: fetched with every load in
  // flight at once into the space the window rows will take, then copied from there run by run
  // as dwords (as the windows are below), the bytes behind a run's end masked to zero.
  {
    const uint32_t raw_bytes = nf * k;
    const uint8_t *from = p.filters + uint64_t(f0) * k;
    const uint32_t head = uint32_t(-reinterpret_cast<uintptr_t>(from)) & 15;   // bytes up to the first 16-byte boundary
    uint8_t *raw = rows + 16;                                                   // raw[i] for byte i; raw + head is 16-byte aligned
    raw -= head;
    const uint32_t chunks = raw_bytes > head ? (raw_bytes - head) / 16 : 0;
    constexpr int FILTER_LOADS = 4;   // 16 KiB with all loads in flight; the rest in further rounds
    for (uint32_t c0 = 0; c0 < chunks; c0 += FILTER_LOADS * 256) {
      v4i got[FILTER_LOADS];
#pragma unroll
      for (int j = 0; j < FILTER_LOADS; j++) {
        const uint32_t ch = c0 + j * 256 + tid;
        if (ch < chunks) got[j] = *(const v4i *)(from + head + ch * 16);
      }
#pragma unroll
      for (int j = 0; j < FILTER_LOADS; j++) {
        const uint32_t ch = c0 + j * 256 + tid;
        if (ch < chunks) *(v4i *)(raw + head + ch * 16) = got[j];
      }
    }
    // the bytes before the first and behind the last whole chunk
    if (uint32_t(tid) < 32) {
      const uint32_t i = uint32_t(tid) < 16 ? uint32_t(tid) : head + chunks * 16 + (tid - 16);
      if ((uint32_t(tid) < 16 ? i < min(head, raw_bytes) : i < raw_bytes)) raw[i] = from[i];
    }
    for (uint32_t i = tid; i < 64 * ROW / 16; i += 256) ((v4i *)filt)[i] = v4i{0, 0, 0, 0};
    __syncthreads();
    const uint32_t dwords = p.seg_padded / 4;
    for (uint32_t run = tid; run < nf * p.fh; run += 256) {
      const uint32_t fi = run / p.fh, r = run % p.fh;
      const uint32_t at = uint32_t(raw - rows) + fi * k + r * p.seg, shift = at & 3;   // byte offset within `rows` (16-byte aligned)
      const uint32_t *src = (const uint32_t *)rows + (at >> 2);
      uint32_t *dst = (uint32_t *)(filt + fi * ROW + r * p.seg_padded);
      for (uint32_t d = 0; d < dwords; d++) {
        uint32_t v = __builtin_amdgcn_alignbyte(src[d + 1], src[d], shift);
        const uint32_t valid = p.seg - 4 * d;   // bytes of this dword that belong to the run
        if (valid < 4) v &= (1u << (8 * valid)) - 1;
        dst[d] = v;
      }
    }
    __syncthreads();   // the raw bytes are no longer needed: the rows are free for the windows
  }
  Acc corr[4] = {};
  if constexpr (IMG_UNSIGNED) {
    const v4i ones = v4i{0x01010101, 0x01010101, 0x01010101, 0x01010101};
#pragma unroll
    for (int fb = 0; fb < 4; fb++) {
#pragma unroll
      for (int ks = 0; ks < KS; ks++)
        corr[fb] = __builtin_amdgcn_mfma_i32_16x16x64_i8(*(const v4i *)(filt + (fb * 16 + li) * ROW + ks * 64 + lg * 16), ones,
                                                         corr[fb], 0, 0, 0);
      corr[fb] *= 128;
    }
  }
  for (uint32_t t = blockIdx.x; t < p.tiles; t += gridDim.x) {
    const Corner at = corner_of(t);
    const uint32_t img = at.img, y0 = at.y0, x0 = at.x0;
    // 1. the patch out of the registers (what they do not hold, straight from memory)
#pragma unroll
    for (int j = 0; j < PATCH_REGS; j++)
      if (tid + j * 256 < patch_bytes) put(held_row[j], held_byte[j], held[j]);
    for (uint32_t i = tid + PATCH_REGS * 256; i < patch_bytes; i += 256) put(i / patch_wb, i % patch_wb, *patch_source(at, i / patch_wb, i % patch_wb));
    __syncthreads();   // also: every wave is done with the previous tile's windows
    // 2. the windows: thread (pixel, half) copies every other run of the pixel's window, eight
    //    dwords at a time (nine aligned dwords read, shifted by the run's byte offset)
    {
      const uint32_t px = tid & 127, ty = px >> 4, tx = px & 15;
      const uint32_t *__restrict__ patch32 = (const uint32_t *)patch;
      uint32_t *__restrict__ dst = (uint32_t *)(rows + px * ROW);
      const uint32_t dwords = p.seg_padded / 4;
      for (uint32_t r = tid >> 7; r < p.fh; r += 2) {
        const uint32_t from = (ty + r) * p.patch_stride + tx * p.c, shift = from & 3;
        const uint32_t *src = patch32 + (from >> 2);
        for (uint32_t d0 = 0; d0 < dwords; d0 += 8) {
          uint32_t v[9];
#pragma unroll
          for (int d = 0; d < 9; d++) v[d] = d0 + d <= dwords ? src[d0 + d] : 0;
#pragma unroll
          for (int d = 0; d < 8; d++)
            if (d0 + d < dwords) {
              uint32_t out = __builtin_amdgcn_alignbyte(v[d + 1], v[d], shift);
              if (HALVES && p.seg - 4 * (d0 + d) < 4) out &= 0xffffu;   // the run ends with half a dword: its padding is zero
              dst[r * dwords + d0 + d] = out;
            }
        }
      }
      // floats: zeros behind the last run too (the results that left through these rows lie there)
      if (FLOATS)
        for (uint32_t d = p.fh * dwords + (tid >> 7); d < KPAD / 4; d += 2) dst[d] = 0;
    }
    __syncthreads();
    const uint32_t next = t + gridDim.x;
    if (next < p.tiles) fetch_patch(next);   // in flight under the MFMAs and the stores
    // 3. two rows of the tile per wave against the group's filters
    Acc acc[2][4];
#pragma unroll
    for (int pb = 0; pb < 2; pb++)
#pragma unroll
      for (int fb = 0; fb < 4; fb++) acc[pb][fb] = corr[fb];
#pragma unroll
    for (int ks = 0; ks < KS; ks++) {
      v4i a[4], bop[2];
#pragma unroll
      for (int fb = 0; fb < 4; fb++) a[fb] = *(const v4i *)(filt + (fb * 16 + li) * ROW + ks * 64 + lg * 16);
#pragma unroll
      for (int pb = 0; pb < 2; pb++) bop[pb] = *(const v4i *)(rows + ((2 * wave + pb) * 16 + li) * ROW + ks * 64 + lg * 16);
#pragma unroll
      for (int pb = 0; pb < 2; pb++)
#pragma unroll
        for (int fb = 0; fb < 4; fb++) acc[pb][fb] = mfma(a[fb], bop[pb], acc[pb][fb]);
    }
    // A lane holds filters 16 fb + 4 lg .. + 3 of pixel (y0 + 2 wave + pb, x0 + li): 16-byte pieces
    // 64 bytes apart.  A pixel block's 16 x 64 results go through the wave's own window rows (no
    // other wave reads them, and this wave is done with them) and leave as whole rows: four pixels
    // per store instruction, 1 KiB contiguous when the Spec has 64 filters.
    if (p.out_planes) {
#pragma unroll
      for (int pb = 0; pb < 2; pb++) {
        const uint32_t y = y0 + 2 * wave + pb, x = x0 + li;
        if (y < p.oh && x < p.ow) {
          const uint64_t plane = uint64_t(p.oh) * p.ow;
          typedef typename std::conditional<FLOATS, float, int32_t>::type Out;
          Out *first = (Out *)p.out + (uint64_t(img) * p.f + f0 + 4 * lg) * plane + uint64_t(y) * p.ow + x;
#pragma unroll
          for (int fb = 0; fb < 4; fb++)
            if (fb < nfb) {
              Acc v = acc[pb][fb];
              if (p.accum) {
                Acc old;
#pragma unroll
                for (int r = 0; r < 4; r++) old[r] = first[(16 * fb + r) * plane];
                v += old;
              }
#pragma unroll
              for (int r = 0; r < 4; r++) first[(16 * fb + r) * plane] = v[r];
            }
        }
      }
      continue;
    }
    uint8_t *xb = rows + (2 * wave) * 16 * ROW;
    constexpr int XROW = 272;
#pragma unroll
    for (int pb = 0; pb < 2; pb++) {
#pragma unroll
      for (int fb = 0; fb < 4; fb++) *(Acc *)(xb + li * XROW + fb * 64 + lg * 16) = acc[pb][fb];
      const uint32_t y = y0 + 2 * wave + pb;
#pragma unroll
      for (int j = 0; j < 4; j++) {
        const uint32_t pixel = 4 * j + lg, x = x0 + pixel;
        Acc v = *(const Acc *)(xb + pixel * XROW + li * 16);
        if (y < p.oh && x < p.ow && li < 4 * nfb) {
          Acc *d = (Acc *)(p.out + ((uint64_t(img) * p.oh + y) * p.ow + x) * p.f + f0 + 4 * li);
          if (p.accum) v += *d;
          __builtin_nontemporal_store(v, d);
        }
      }
    }
  }
}

template <int KS, int KIND>
hipError_t launch_kind(const WindowsArgs &p, dim3 grid, size_t lds, hipStream_t stream) {
  static std::atomic<uint64_t> limit{0};
  if (!plan::recording()) {
    hipError_t e = raise_lds_limit(limit, (const void *)k_conv_windows<KS, KIND>, int(lds));
    if (e != hipSuccess) return e;
  }
  MRL_LAUNCH((k_conv_windows<KS, KIND>), grid, dim3(256), lds, stream, p);
  return plan::last_error();
}
template <int KS>
hipError_t launch_ks(const WindowsArgs &p, int kind, dim3 grid, size_t lds, hipStream_t stream) {
  switch (kind) {
    case IMG_I8: return launch_kind<KS, IMG_I8>(p, grid, lds, stream);
    case IMG_U8: return launch_kind<KS, IMG_U8>(p, grid, lds, stream);
    case IMG_BF16: return launch_kind<KS, IMG_BF16>(p, grid, lds, stream);
    case IMG_F32: return launch_kind<KS, IMG_F32>(p, grid, lds, stream);
    default: return hipErrorInvalidValue;
  }
}

constexpr uint32_t MAX_KS = 6;       // windows of up to 384 bytes: 75 KiB of rows, two workgroups to a compute unit
constexpr uint32_t MAX_KS_F32 = 10;  // f32: up to 640 bytes (3 channels, 7 x 7: 588), 126 KiB of rows, one workgroup

}  // namespace

// kind: 0 i8 x i8 -> i32, 1 u8 x i8 -> i32, 2 bf16 x bf16 -> f32, 3 f32 x f32 -> f32.  Filters in 16s, pixels that are
// not whole 16-byte chunks (those conv_gemm.hip reads in place), windows of at most 64 MAX_KS
// bytes with their runs padded to dwords.
bool conv_windows_applicable(const ConvArgs &c, int kind) {
  // (The same for an image or an output stored as planes: only the alignment of the output's 16-byte
  // stores does not apply to planes, which are written a dword at a time.)
  if (kind < 0 || kind > 3) return false;
  const uint64_t es = kind == 3 ? 4 : kind == 2 ? 2 : 1, c_bytes = c.c * es, seg_padded = (uint64_t(c.fw) * c_bytes + 3) & ~3ull;
  // Pixels that are not whole 16-byte chunks: the implicit Matmul cannot read those in place.  With
  // whole chunks it is the faster one, pixels of a single chunk included (32 x (16 -> 16) x 110^2
  // 3 x 3 int8: 33.8 us against 45.8 here, 16 -> 64 31.8 against 47.7, bf16 8 -> 32 29.1 against
  // 31.0, 8 x (8 -> 32) x 56^2 4.9 against 8.9; int8 32 -> 32 3 x 3: 44 against 60).
#ifdef MRL_WINDOWS_ANY_C   // measurement builds: every pixel width
  const bool c_ok = true;
#else
  const bool c_ok = c_bytes % 16 != 0;
#endif
  return c.f % 16 == 0 && c.f / 64 < 65535 && c_ok && uint64_t(c.fh) * seg_padded <= 64 * (kind == 3 ? MAX_KS_F32 : MAX_KS) &&
         uint64_t(c.b) * ((c.oh + TILE_H - 1) / TILE_H) * ((c.ow + TILE_W - 1) / TILE_W) < (1ull << 31) &&
         (reinterpret_cast<uintptr_t>(c.out) & (c.out_planes ? 3 : 15)) == 0 && (reinterpret_cast<uintptr_t>(c.image) & (es - 1)) == 0 &&
         (reinterpret_cast<uintptr_t>(c.filters) & (es - 1)) == 0;
}

hipError_t launch_conv_windows(const ConvArgs &c, int kind, hipStream_t stream) {
  if (!conv_windows_applicable(c, kind)) return hipErrorInvalidValue;
  const uint32_t es = kind == 3 ? 4 : kind == 2 ? 2 : 1;
  WindowsArgs p;
  p.image = (const uint8_t *)c.image, p.filters = (const uint8_t *)c.filters, p.out = (int32_t *)c.out;
  p.b = c.b, p.f = c.f, p.c = c.c * es, p.oh = c.oh, p.ow = c.ow, p.fh = c.fh, p.fw = c.fw, p.accum = c.accum;
  p.tiles_x = (c.ow + TILE_W - 1) / TILE_W, p.tiles_y = (c.oh + TILE_H - 1) / TILE_H, p.tiles = c.b * p.tiles_x * p.tiles_y;
  p.seg = c.fw * p.c, p.seg_padded = (p.seg + 3) & ~3u;
  p.patch_stride = ((TILE_W + c.fw - 1) * p.c + 3) & ~3u;
  p.in_planes = c.in_planes, p.out_planes = c.out_planes;
  const int ks = int((c.fh * p.seg_padded + 63) / 64);
  const size_t row = ks == 1 ? 144 : 64 * ks + 16;
  // the copies read one dword past a run's last: four bytes behind the patch
  const size_t lds = (64 + TILE_PIXELS) * row + size_t(TILE_H + c.fh - 1) * p.patch_stride + 16;
  // Workgroups walk the tiles with the grid's stride: as many as fit the chip at once, so that
  // the filters are staged once each.
  const uint32_t per_cu = uint32_t(std::max<size_t>(1, std::min<size_t>(4, (160 * 1024) / lds)));
  const uint32_t groups = (c.f + 63) / 64;
  const uint32_t wgs = std::min<uint32_t>(p.tiles, std::max(1u, g_compute_units * per_cu / groups));
  const double pixels = double(c.b) * c.oh * c.ow;
  plan::work(plan::UNIT_STREAM, 0, 1.5 * (pixels * c.f * 4 * (c.accum ? 2 : 1) + double(c.b) * (c.oh + c.fh - 1) * (c.ow + c.fw - 1) * p.c),
             0, 6000.0 + (1500.0 + 1000.0 * ks) * double((p.tiles + wgs - 1) / wgs));   // staging the filters; a tile
  const dim3 grid(wgs, groups);
  switch (ks) {
    case 1: return launch_ks<1>(p, kind, grid, lds, stream);
    case 2: return launch_ks<2>(p, kind, grid, lds, stream);
    case 3: return launch_ks<3>(p, kind, grid, lds, stream);
    case 4: return launch_ks<4>(p, kind, grid, lds, stream);
    case 5: return launch_ks<5>(p, kind, grid, lds, stream);
    case 6: return launch_ks<6>(p, kind, grid, lds, stream);
    case 7: return launch_kind<7, IMG_F32>(p, grid, lds, stream);
    case 8: return launch_kind<8, IMG_F32>(p, grid, lds, stream);
    case 9: return launch_kind<9, IMG_F32>(p, grid, lds, stream);
    case 10: return launch_kind<10, IMG_F32>(p, grid, lds, stream);
    default: return hipErrorInvalidValue;
  }
}

}  // namespace mrl
