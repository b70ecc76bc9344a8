// Conv NHWC x KRSC with short windows (at most 576 bytes: nine MFMA k steps of 64) and pixels of
// whole 16-byte chunks, u8|i8 x i8 -> i32 and bf16 x bf16 -> f32: the design of conv_i8.hip's
// tile-per-wave kernel (the filter bank resident in a wave's registers, pixels straight from
// global memory into operand registers one tile ahead, results out through the wave's patch of
// LDS as whole pixel rows) for any such window, where that kernel wants 64-channel slabs
// (morello/src/spec.rs:486-498, 741-776: stride 1, no padding, cross-correlation).
//
// A window is fh runs of fw * c contiguous bytes, K bytes in all, and KRSC filters are the same K
// bytes in a row, so the contraction runs over the window's 16-byte chunks in that order: chunk
// q lies in run q / (fw * c / 16).  A k step takes four chunks (one per lane group), whichever
// runs they fall in; the chunks past K of the last step have zero filter operands (and zero
// pixel operands for floats: an infinity there times zero would not be zero).
//
// Taken for early layers of 16 or 32 channels with at most 48 filters and windows of at most 320
// bytes, where the implicit Matmul (conv_gemm.hip) pads its 64-wide tiles: 32 x (32 -> 32) x 112^2,
// 3 x 3, int8 44 -> 34 us, bf16 16 -> 16 40 -> 23 us.  A wave's loads of its next pixels are
// counted complete only behind the stores it issued before them (a wave's vector memory
// operations complete in order), so a round lasts about as long as a store's acknowledgement
// whatever is in flight; with more filters or longer windows the implicit kernel's workgroups
// hide more of that, and the dispatch keeps those there.
#include <algorithm>

#include "kernels.h"
#include "plan.h"

namespace mrl {
namespace {

typedef int v4i __attribute__((ext_vector_type(4)));
typedef float v4f __attribute__((ext_vector_type(4)));
typedef __bf16 v8bf __attribute__((ext_vector_type(8)));
enum { SMALL_I8 = 0, SMALL_U8 = 1, SMALL_BF16 = 2 };

constexpr int FT = 4;       // filter tiles of 16 per workgroup: groups of 64 filters
constexpr int WAVES = 4;
constexpr int TURN_ROW = 68;  // dwords between the pixel rows of a wave's patch of results

// Tiles a wave has in flight per round: two while their pixel registers fit beside the filters'.
constexpr int tiles_per_round(int slabs) { return slabs <= 5 ? 2 : 1; }

struct SmallArgs {
  const uint8_t *image, *filters;
  void *out;
  uint32_t c_bytes, f, oh, ow, fh, fw;
  int accum;
  uint32_t pixels, tiles;
  uint32_t k_bytes;   // fh * fw * c_bytes, a multiple of 16
};

// SLABS: k steps of 64 bytes per window, ceil(k_bytes / 64).  TILES: tiles of 16 pixels a wave takes
// per round (their pixels are all requested before the first is used: with short windows a
// tile's MFMAs are too few to cover the next tile's trip to memory).
template <int SLABS, int KIND, int TILES>
__global__ __launch_bounds__(64 * WAVES) void k_conv_small(SmallArgs p) {
  constexpr bool IMG_UNSIGNED = KIND == SMALL_U8, FLOATS = KIND == SMALL_BF16;
  typedef typename std::conditional<FLOATS, v4f, v4i>::type Acc;
  auto mfma = [](v4i a, v4i b, Acc c) {
    if constexpr (FLOATS) return __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(v8bf, a), __builtin_bit_cast(v8bf, b), c, 0, 0, 0);
    else return __builtin_amdgcn_mfma_i32_16x16x64_i8(a, b, c, 0, 0, 0);
  };
  extern __shared__ __attribute__((aligned(16))) uint8_t small_lds[];
  constexpr int NT = 64 * WAVES;
  const int lane = threadIdx.x & 63, li = lane & 15, lg = lane >> 4;
  const int wave_in_group = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const uint32_t wave = blockIdx.x * WAVES + wave_in_group, nwaves = gridDim.x * WAVES;
  const int W = p.ow + p.fw - 1, H = p.oh + p.fh - 1;
  const uint32_t f0 = blockIdx.y * (FT * 16), nf = min(uint32_t(FT * 16), p.f - f0);   // a multiple of 16
  const int nft = int(nf / 16);
  const uint32_t k_chunks = p.k_bytes / 16, run_chunks = p.fw * p.c_bytes / 16;

  // The group's filters: nf rows of k_bytes, one contiguous piece of memory, into LDS as they lie.
  uint8_t *filt_lds = small_lds;
  {
    const uint8_t *from = p.filters + uint64_t(f0) * p.k_bytes;
    const uint32_t chunks = nf * k_chunks;
    constexpr int PER_THREAD = (SLABS * 256 + NT - 1) / NT;   // 64 filters x SLABS x 4 chunks at most
    v4i stage[PER_THREAD];
#pragma unroll
    for (int i = 0; i < PER_THREAD; i++) {
      const uint32_t c = i * NT + threadIdx.x;
      if (c < chunks) stage[i] = *(const v4i *)(from + c * 16);
    }
#pragma unroll
    for (int i = 0; i < PER_THREAD; i++) {
      const uint32_t c = i * NT + threadIdx.x;
      if (c < chunks) *(v4i *)(filt_lds + c * 16) = stage[i];
    }
  }
  // Where the lane's chunk of every k step lies relative to the window's first byte, and whether
  // the chunk exists (only the last step can run past K).
  int slab_off[SLABS];
  bool chunk_valid[SLABS];
#pragma unroll
  for (int s = 0; s < SLABS; s++) {
    const uint32_t q = 4 * s + lg;
    chunk_valid[s] = q < k_chunks;
    const uint32_t qc = chunk_valid[s] ? q : 0, r = qc / run_chunks;
    slab_off[s] = int((r * W) * p.c_bytes + (qc - r * run_chunks) * 16);
  }
  // The lane's pixel of tile t (past the end: the last pixel again, which is not stored).
  auto pixel_of = [&](uint32_t t) {
    const uint32_t pix = min(min(t, p.tiles - 1) * 16 + li, p.pixels - 1);
    const uint32_t x = pix % p.ow, y = (pix / p.ow) % p.oh, b = pix / (p.ow * p.oh);
    return p.image + (int64_t(b) * H * W + int64_t(y) * W + x) * p.c_bytes;
  };
  v4i img[TILES][SLABS];
  uint32_t t = wave * TILES;   // a round's tiles follow one another
  if (t < p.tiles) {
#pragma unroll
    for (int u = 0; u < TILES; u++) {
      const uint8_t *src = pixel_of(t + u);
#pragma unroll
      for (int s = 0; s < SLABS; s++) img[u][s] = *(const v4i *)(src + slab_off[s]);
    }
  }
  __syncthreads();
  v4i filt[FT][SLABS];
#pragma unroll
  for (int ft = 0; ft < FT; ft++)
#pragma unroll
    for (int s = 0; s < SLABS; s++)
      filt[ft][s] = ft < nft && chunk_valid[s] ? *(const v4i *)(filt_lds + (ft * 16 + li) * p.k_bytes + (4 * s + lg) * 16) : v4i{0, 0, 0, 0};

  // u8: a - 128 in the operands, 128 * (sum of a filter's weights) added back; the sums come from
  // the same MFMAs against a pixel of ones, each wave forming one filter tile's.
  uint8_t *after_bank = filt_lds + FT * 16 * p.k_bytes;
  int *corr_lds = (int *)after_bank;
  int *turn_lds = corr_lds + FT * 16 + wave_in_group * (16 * TURN_ROW);
  if constexpr (IMG_UNSIGNED) {
    const v4i ones = v4i{0x01010101, 0x01010101, 0x01010101, 0x01010101};
#pragma unroll
    for (int ft = 0; ft < FT; ft++) {
      if (ft != wave_in_group) continue;
      v4i sum = v4i{0, 0, 0, 0};
#pragma unroll
      for (int s = 0; s < SLABS; s++) sum = __builtin_amdgcn_mfma_i32_16x16x64_i8(filt[ft][s], ones, sum, 0, 0, 0);
      if (li == 0) *(v4i *)(corr_lds + ft * 16 + lg * 4) = sum * 128;
    }
    __syncthreads();
  }

  while (t < p.tiles) {
    const uint32_t tn = t + nwaves * TILES;
#pragma unroll
    for (int u = 0; u < TILES; u++) {
      const uint8_t *src_n = pixel_of(tn + u);
      Acc acc[FT] = {};
#pragma unroll
      for (int s = 0; s < SLABS; s++) {
        v4i px = img[u][s];
        if constexpr (IMG_UNSIGNED) px ^= v4i{int(0x80808080), int(0x80808080), int(0x80808080), int(0x80808080)};
        if constexpr (FLOATS)
          if (s == SLABS - 1 && !chunk_valid[s]) px = v4i{0, 0, 0, 0};
#pragma unroll
        for (int ft = 0; ft < FT; ft++)
          if (ft < nft) acc[ft] = mfma(filt[ft][s], px, acc[ft]);
        img[u][s] = *(const v4i *)(src_n + slab_off[s]);   // the next round's, as soon as this one's is used
      }
      // A lane holds filters 16 ft + 4 lg .. + 3 of pixel li: through the wave's patch of LDS, then
      // out as whole pixel rows (lane (li, lg): pixel 4 i + lg, filters 4 li .. + 3).
#pragma unroll
      for (int ft = 0; ft < FT; ft++) {
        Acc v = acc[ft];
        if constexpr (IMG_UNSIGNED) v += *(const v4i *)(corr_lds + ft * 16 + lg * 4);
        *(Acc *)(turn_lds + li * TURN_ROW + ft * 16 + lg * 4) = v;
      }
      __builtin_amdgcn_wave_barrier();
#pragma unroll
      for (int i = 0; i < 4; i++) {
        const uint32_t row = i * 4 + lg, pix = (t + u) * 16 + row;
        Acc v = *(const Acc *)(turn_lds + row * TURN_ROW + li * 4);
        if (pix < p.pixels && uint32_t(li * 4) < nf) {
          Acc *d = (Acc *)((uint32_t *)p.out + int64_t(pix) * p.f + f0 + li * 4);
          if (p.accum) v += *d;
          __builtin_nontemporal_store(v, d);
        }
      }
      __builtin_amdgcn_wave_barrier();
    }
    t = tn;
  }
}

template <int SLABS>
hipError_t launch_slabs(const SmallArgs &p, int kind, dim3 grid, size_t lds, hipStream_t stream) {
  constexpr int TILES = tiles_per_round(SLABS);
  switch (kind) {
    case SMALL_I8: MRL_LAUNCH((k_conv_small<SLABS, SMALL_I8, TILES>), grid, dim3(64 * WAVES), lds, stream, p); break;
    case SMALL_U8: MRL_LAUNCH((k_conv_small<SLABS, SMALL_U8, TILES>), grid, dim3(64 * WAVES), lds, stream, p); break;
    case SMALL_BF16: MRL_LAUNCH((k_conv_small<SLABS, SMALL_BF16, TILES>), grid, dim3(64 * WAVES), lds, stream, p); break;
    default: return hipErrorInvalidValue;
  }
  return plan::last_error();
}

}  // namespace

// kind: 0 i8 x i8 -> i32, 1 u8 x i8 -> i32, 2 bf16 x bf16 -> f32.
bool conv_small_applicable(const ConvArgs &c, int kind) {
  if (kind < 0 || kind > 2) return false;
  auto al16 = [](const void *p) { return (reinterpret_cast<uintptr_t>(p) & 15) == 0; };
  const uint64_t es = kind == 2 ? 2 : 1, c_bytes = c.c * es, k_bytes = uint64_t(c.fh) * c.fw * c_bytes;
  const uint64_t pixels = uint64_t(c.b) * c.oh * c.ow;
  const uint64_t in_bytes = uint64_t(c.b) * (c.oh + c.fh - 1) * (c.ow + c.fw - 1) * c_bytes;
  return c_bytes != 0 && c_bytes % 16 == 0 && k_bytes <= 576 && c.f != 0 && c.f % 16 == 0 && (c.f + 63) / 64 <= 65535 &&
         pixels > 0 && pixels < (1ull << 31) && in_bytes < (1ull << 31) && al16(c.image) && al16(c.filters) && al16(c.out);
}

hipError_t launch_conv_small(const ConvArgs &c, int kind, hipStream_t stream) {
  if (!conv_small_applicable(c, kind)) return hipErrorInvalidValue;
  const uint32_t es = kind == 2 ? 2 : 1;
  SmallArgs p;
  p.image = (const uint8_t *)c.image, p.filters = (const uint8_t *)c.filters, p.out = c.out;
  p.c_bytes = c.c * es, p.f = c.f, p.oh = c.oh, p.ow = c.ow, p.fh = c.fh, p.fw = c.fw, p.accum = c.accum;
  const uint64_t pixels = uint64_t(c.b) * c.oh * c.ow;
  p.pixels = uint32_t(pixels), p.tiles = uint32_t((pixels + 15) / 16);
  p.k_bytes = c.fh * c.fw * p.c_bytes;
  const int slabs = int((p.k_bytes + 63) / 64);
  const uint32_t groups = (c.f + 63) / 64;
  // as many waves as the chip holds at this kernel's register count, never more than tiles
  uint32_t blocks = std::max<uint32_t>(1, 2048u / WAVES / groups);
  const uint32_t rounds = (p.tiles + tiles_per_round(slabs) - 1) / tiles_per_round(slabs);
  if (blocks * WAVES > rounds) blocks = (rounds + WAVES - 1) / WAVES;
  const size_t lds = size_t(FT) * 16 * p.k_bytes + FT * 16 * sizeof(int) + size_t(WAVES) * 16 * TURN_ROW * sizeof(int);
  plan::work(kind == 2 ? plan::UNIT_MFMA_BF16 : plan::UNIT_MFMA_I8, 2.0 * pixels * c.f * c.fh * c.fw * c.c,
             double(c.b) * (c.oh + c.fh - 1) * (c.ow + c.fw - 1) * p.c_bytes + double(c.f) * p.k_bytes +
                 4.0 * pixels * c.f * (c.accum ? 2 : 1));
  const dim3 grid(blocks, groups);
  switch (slabs) {
    case 1: return launch_slabs<1>(p, kind, grid, lds, stream);
    case 2: return launch_slabs<2>(p, kind, grid, lds, stream);
    case 3: return launch_slabs<3>(p, kind, grid, lds, stream);
    case 4: return launch_slabs<4>(p, kind, grid, lds, stream);
    case 5: return launch_slabs<5>(p, kind, grid, lds, stream);
    case 6: return launch_slabs<6>(p, kind, grid, lds, stream);
    case 7: return launch_slabs<7>(p, kind, grid, lds, stream);
    case 8: return launch_slabs<8>(p, kind, grid, lds, stream);
    case 9: return launch_slabs<9>(p, kind, grid, lds, stream);
    default: return hipErrorInvalidValue;
  }
}

}  // namespace mrl
