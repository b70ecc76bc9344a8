// Internal interface between the host dispatcher and the kernel translation units.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#include <atomic>

#include "layout_math.h"
#include "plan.h"

namespace mrl {

// Raises a kernel's limit of dynamic LDS to `bytes`, once per device: the attribute belongs to
// the device the calling thread has selected, and launches may come from several threads.
// `done` is the kernel's own flag word, one bit per device.
inline hipError_t raise_lds_limit(std::atomic<uint64_t> &done, const void *kernel, int bytes) {
  int device = 0;
  hipError_t e = hipGetDevice(&device);
  if (e != hipSuccess) return e;
  const uint64_t bit = 1ull << (device & 63);
  if (done.load(std::memory_order_acquire) & bit) return hipSuccess;
  e = hipFuncSetAttribute(kernel, hipFuncAttributeMaxDynamicSharedMemorySize, bytes);
  if (e == hipSuccess) done.fetch_or(bit, std::memory_order_release);
  return e;
}


// A tensor whose layout is a pure permutation of its logical dims.
// Accesses of kernels that touch their data once.  Loads are ordinary ones and stores non-temporal:
// measured on the Softmax of 16 x 2048 rows of 2048 f32 (one read, one write of 268 MB each), that
// pairing took 83 us, non-temporal loads and stores 89, ordinary loads and stores 104, non-temporal
// loads with ordinary stores 85.  Non-temporal stores leave what the loads brought in where it is:
// a launch repeated on the same buffers (a benchmark's loop) then finds part of its input still in
// the memory-side cache, which ordinary stores would have displaced -- a conversion of 256 MB
// i32 to f32 measured 64 us that way, more than HBM alone delivers, against 86 us with ordinary
// stores.  On inputs that no launch has touched the ordinary loads cost 4 % against non-temporal
// ones (Softmax 97 against 93 us); on inputs a producer left in the cache they gain 8 to 16 %.
// (The switches are for such measurements.)
#ifdef MRL_NT_LOADS
#define MRL_LOAD_ONCE(p) __builtin_nontemporal_load(p)
#else
#define MRL_LOAD_ONCE(p) (*(p))
#endif
#ifdef MRL_PLAIN_STORES
#define MRL_STORE_ONCE(v, p) (*(p) = (v))
#else
#define MRL_STORE_ONCE(v, p) __builtin_nontemporal_store(v, p)
#endif

struct Strided {
  void *ptr;
  int dtype;
  uint32_t rank;
  uint32_t shape[MRL_MAX_RANK];
  int64_t stride[MRL_MAX_RANK];  // in elements
};

// ---- generic.hip: correctness-first kernels for any dtype / stride combination ----------
hipError_t launch_relayout(const void *src, void *dst, const LayoutEval &src_l,
                           const LayoutEval &dst_l, uint32_t elem_size, uint64_t count,
                           hipStream_t stream);
hipError_t launch_matmul_generic(const Strided &a, const Strided &b, const Strided &c, int accum,
                                 hipStream_t stream);
hipError_t launch_conv_generic(const Strided &img, const Strided &filt, const Strided &out,
                               int accum, hipStream_t stream);
// `scratch`: softmax_cols_scratch_bytes(blocks, scan) bytes when the caller wants a scan over an
// outer dim of few columns shared out over workgroups (blocks = lines / columns * ceil(columns / 64)
// for the contiguous dim the column kernel would take); nullptr: one launch whatever the shape.
uint32_t softmax_cols_chunks(uint64_t blocks, uint32_t scan);
size_t softmax_cols_scratch_bytes(uint64_t blocks, uint32_t scan);
hipError_t launch_softmax_generic(const Strided &in, const Strided &out, uint32_t scan_dim, void *scratch,
                                  hipStream_t stream);
hipError_t launch_fill_zero(void *ptr, uint64_t bytes, hipStream_t stream);
// Move Spec: element-wise copy with dtype conversion between two arbitrary layouts.
hipError_t launch_move_generic(const void *src, void *dst, const LayoutEval &src_l,
                               const LayoutEval &dst_l, int src_dtype, int dst_dtype,
                               uint64_t count, hipStream_t stream);
// Move between two layouts that are permutations of the logical dims (strides in elements):
// coalesced on both sides, through an LDS transpose when their contiguous dims differ.
hipError_t launch_move_strided(const Strided &src, const Strided &dst, hipStream_t stream);
// The same over a common strided view of two layouts (layout_factor.h): `rank` digits.
struct MoveDim;
hipError_t launch_move_view(const void *src, int src_dtype, void *dst, int dst_dtype,
                            const MoveDim *dims, uint32_t rank, hipStream_t stream);
// Copy of a [batch][rows][cols] tensor with contiguous rows into dense rows of `dst_ld` elements
// (a whole number of dwords), zeros from each row's end to `dst_ld`.
hipError_t launch_pad_rows(const Strided &src, void *dst, uint32_t dst_ld, uint32_t elem_size,
                           hipStream_t stream);
// Two such copies (elements of the same size) in one launch.
hipError_t launch_pad_rows_pair(const Strided &src0, void *dst0, uint32_t dst_ld0, const Strided &src1, void *dst1,
                                uint32_t dst_ld1, uint32_t elem_size, hipStream_t stream);
// bf16 -> f32 of a whole buffer, position by position.
hipError_t launch_widen_bf16(const void *src, void *dst, uint64_t count, hipStream_t stream);
// Move Spec fast path: same bytes on both sides (16-byte aligned buffers).
hipError_t launch_copy(const void *src, void *dst, uint64_t bytes, hipStream_t stream);

// Division of a number below 2^31 by a divisor fixed at launch: with s = ceil(log2 d) and
// mul = floor(2^(31+s) / d) + 1, n / d = (n * mul) >> (31 + s) exactly (the error term
// n * (mul * d - 2^(31+s)) stays below 2^(31+s) because n < 2^31 and mul * d - 2^(31+s) <= d <= 2^s).
// A multiply-high, a multiply-low and a shift where the hardware's division takes some thirty
// instructions.
struct FastDiv {
  uint32_t mul = 0, shift = 0;
  FastDiv() = default;
  explicit FastDiv(uint32_t d) {
    uint32_t s = 0;
    while ((1ull << s) < d) s++;
    mul = uint32_t((1ull << (31 + s)) / d + 1);
    shift = 31 + s;
  }
  __host__ __device__ uint32_t div(uint32_t n) const { return uint32_t((uint64_t(n) * mul) >> shift); }
};

// ---- gemm_mfma.hip / gemm_nt.hip: Matmul on the matrix cores (kernel: gemm_mfma_kernel.h) ----
// A and C row-major, B row-major or k-fastest; leading dimensions and batch strides in elements.
struct GemmArgs {
  const void *a;
  const void *b;
  void *c;
  uint32_t batch, m, n, k;
  int64_t lda, ldb, ldc;
  int64_t sa, sb, sc;  // batch strides
  int accum;
  // false: B rows run along N (`ldb` = elements between k rows); true: B rows run along K
  // (`ldb` = elements between n rows), as col_major / layout![0,2,1] store it.
  bool b_kmajor = false;
  // Conv as an implicit Matmul (the CONV build of the kernel): `a` is a channels-last image
  // [batch][h][w][c], row p of the left operand is the window of output pixel p (fh runs of
  // fw * c contiguous elements), never materialised.  m = batch * oh * ow, k = fh * fw * c.
  struct {
    uint32_t h, w, oh, ow, fw;
    uint32_t c_bytes;       // bytes of one pixel's channels (a whole number of 16-byte chunks)
    uint64_t image_bytes;   // all of `a`
    // K shared out over batch entries (each a slice of the windows, a partial result of its own):
    // bytes of a window a slice starts behind the previous one; 0 = one entry, the whole window.
    uint32_t slice_bytes;
    // Filled in by launch_conv_gemm: the divisions of the window arithmetic.
    FastDiv by_ow, by_oh, by_c_bytes, by_fw;
  } conv = {};
};
// kind: 0 = i8 x i8, 1 = u8 x i8, 2 = bf16 x bf16, 3 = f32 x f32; B stored k-fastest (gemm_nt.hip).
// tile: 64, 128 or 256 (square workgroup tiles).
hipError_t launch_gemm_nt(const GemmArgs &g, int kind, uint32_t tile, hipStream_t stream);
// Conv as an implicit Matmul (g.conv filled in, B = the KRSC filters, k-fastest); tile chosen by size.
bool conv_gemm_applicable(const GemmArgs &g, int kind);
// `tile`: side of the workgroup tile (64, 128, 256), or 0 for the choice by problem size.
hipError_t launch_conv_gemm(const GemmArgs &g, int kind, hipStream_t stream, uint32_t tile = 0);
// kind: 0 = i8 x i8 -> i32, 1 = u8 x i8 -> i32, 2 = bf16 x bf16 -> f32, 3 = f32 x f32 -> f32.
// Shapes, leading dimensions and alignment the kernel can walk.
bool gemm_possible(const GemmArgs &g, int kind);
// Whether the matrix-core kernel is the faster choice for this size (else the generic kernel).
bool gemm_pays(const GemmArgs &g, int kind);
// Tile chosen by size: 256 x 256 with enough tiles to occupy the chip, else 128 x 128 or 64 x 64.
hipError_t launch_gemm(const GemmArgs &g, int kind, hipStream_t stream);
// Side of the square tile launch_gemm would take for this size: 64, 128 or 256.
uint32_t gemm_tile_side(const GemmArgs &g, int kind);
// A single Matmul with few output tiles and a long K runs as `splits` batch entries over slices
// of K whose partial results are summed afterwards (1: as it is).  The slices are whole k steps.
uint32_t gemm_k_splits(const GemmArgs &g, int kind, uint32_t *remainder = nullptr);
// c[r][col] (+)= sum over s of partial[s][r][col]; partial is dense [splits][m][n], 32-bit
// elements (int32 when `integers`, else f32), summed in order of s.
hipError_t launch_sum_splits(const void *partial, void *c, uint32_t splits, uint32_t m, uint32_t n, int64_t ldc,
                             bool accum, bool integers, hipStream_t stream);
// Always the 256 x 256 tile, 128 bytes of K per step.
// staging: 0 = whichever of the 256 x 256 kernels applies (four waves, eight waves, compiler-scheduled),
// 1 / 2 / 3 = mrl_staging's REGISTERS / DIRECT_B / DIRECT_B_WIDE only (hipErrorInvalidValue where that one does not apply).
hipError_t launch_gemm_big(const GemmArgs &g, int kind, hipStream_t stream, uint32_t staging = 0);

// ---- gemv.hip: at most four rows of A against a k-fastest B, as dot products (a stream over B) ----
bool gemv_applicable(const GemmArgs &g, int kind);
hipError_t launch_gemv(const GemmArgs &g, int kind, hipStream_t stream);

// ---- gemm_sched.hip: the same kernel under a caller-chosen tile_out / split schedule -----
uint32_t gemm_schedule_count();
void gemm_schedule_at(uint32_t i, int elem_size, uint32_t *tile_m, uint32_t *tile_n, uint32_t *split_k, uint32_t *staging);
hipError_t launch_gemm_scheduled(const GemmArgs &g, int kind, uint32_t tile_m, uint32_t tile_n,
                                 uint32_t split_k, hipStream_t stream, uint32_t staging = 0);

// ---- conv_i8.hip: NHWC u8|i8 image x KRSC i8 filters -> NHWC i32, implicit GEMM --------
struct ConvArgs {
  const void *image;
  const void *filters;
  void *out;
  uint32_t b, f, c, oh, ow, fh, fw;
  int accum;
  // The output as planes of filters, [b][f][oh][ow] dense (row-major NCHW), instead of channels-last:
  // written in place by the kernels that can (conv_i8.hip's tile-per-wave kernel), where the
  // others write channels-last into scratch and a Move turns it.
  bool out_planes = false;
  // The image as planes of channels, [b][c][h][w] dense (conv_windows.hip fetches its patches from either).
  bool in_planes = false;
};
bool conv_i8_applicable(const ConvArgs &c);
// whole_rows: the kernel whose workgroups take whole output rows and share their pixels through LDS
// (conv_rows_applicable: 64 channels, a run's piece of the image fits LDS); else a wave per 16-pixel tile.
bool conv_rows_applicable(const ConvArgs &c);
hipError_t launch_conv_i8(const ConvArgs &c, bool img_unsigned, hipStream_t stream, bool whole_rows = false);

// ---- conv_windows.hip: Conv u8|i8 x i8 -> i32 and bf16 x bf16 -> f32 (kind 0, 1, 2 as for a Matmul),
// channels-last, pixels of few channels (not whole 16-byte chunks), windows of at most 384
// bytes, filters in 16s: the windows are formed in LDS.
// conv_small.hip: windows of at most 576 bytes over pixels of whole 16-byte chunks, the filters
// resident in registers (kind: 0 i8, 1 u8, 2 bf16 operands).
bool conv_small_applicable(const ConvArgs &c, int kind);
hipError_t launch_conv_small(const ConvArgs &c, int kind, hipStream_t stream);
bool conv_windows_applicable(const ConvArgs &c, int kind);
hipError_t launch_conv_windows(const ConvArgs &c, int kind, hipStream_t stream);

// ---- unfold.hip: the windows of a channels-last image as rows, for Conv as a Matmul ---------
// image: [batch][oh+fh-1][ow+fw-1][c]; rows: [batch*oh*ow][row_elems], each row the fh*fw*c
// elements of one window in (r, s, c) order followed by zeros.
hipError_t launch_unfold(const void *image, void *rows, uint32_t batch, uint32_t c, uint32_t oh,
                         uint32_t ow, uint32_t fh, uint32_t fw, uint32_t row_elems,
                         uint32_t elem_size, hipStream_t stream);

// ---- softmax.hip: f32 softmax over a contiguous innermost scan dim ---------------------
// Rows longer than 4096 run a workgroup per SOFTMAX_CHUNK elements and want
// softmax_scratch_bytes() of device scratch for the chunks' (max, denominator) pairs
// (hipErrorInvalidValue without it).  `out` may be `in`.
constexpr uint32_t SOFTMAX_CHUNK = 4096;
size_t softmax_scratch_bytes(uint64_t rows, uint32_t cols);
hipError_t launch_softmax_rows(const float *in, float *out, uint64_t rows, uint32_t cols, void *scratch,
                               hipStream_t stream);
// The same with the result rounded to bf16 (rows of `cols` 16-bit values).
hipError_t launch_softmax_rows_bf16(const float *in, void *out, uint64_t rows, uint32_t cols, void *scratch,
                                    hipStream_t stream);

// ---- parts.hip: the primitive Specs of the Softmax decomposition, Broadcast, Fill ----------
struct PartsArgs {
  int kind;  // mrl_spec_kind
  int accum;
  uint32_t rank, scan_dim, n_params;
  uint32_t shape[MRL_MAX_RANK];           // the Spec shape (full tensor)
  float *ptr[4];
  int64_t stride[4][MRL_MAX_RANK];        // element strides per parameter (0 on reduced dims)
  uint64_t lines;                         // product of the dims other than scan_dim
  FastDiv by_shape[MRL_MAX_RANK];         // filled in by launch_parts: a line number into coordinates without dividing
};
hipError_t launch_parts(const PartsArgs &p, hipStream_t stream);
hipError_t launch_broadcast(const void *in, void *out, const LayoutEval &il, const LayoutEval &ol,
                            uint32_t dim, uint32_t elem_size, uint64_t count, hipStream_t stream);
// Broadcast between row-major tensors as out[before][n][after] <- in[before][after], elements of es
// bytes: true (and *err set) if one of the 16-byte forms took it, false if the shape or the
// pointers' alignment leave it to launch_broadcast.
bool launch_broadcast_rows(const void *in, void *out, uint64_t before, uint32_t n, uint64_t after, uint32_t es,
                           hipStream_t stream, hipError_t *err);
hipError_t launch_fill(void *out, int dtype, int fill_value, uint64_t count, hipStream_t stream);

// ---- mfma_rate.hip: sustained matrix-core rate of this board (measurement, not a Spec) ----
hipError_t measure_mfma_rate(int kind, bool random_operands, uint32_t iters, hipStream_t stream,
                             double *ops_per_second);

// Compute units of the selected device (mrl_init sets it; 256 on an MI355X).  Heuristics read
// this instead of asking the runtime, so that planning a Spec makes no runtime call.
extern uint32_t g_compute_units;

// ---- attention.hip: fused Matmul -> Softmax -> Matmul on bf16 inputs -------------------
struct AttnArgs {
  const void *q;   // [b, m, k]   bf16 row-major
  const void *kt;  // logical [b, k, n2]: stored as [b, n2, k] (K row-major), or as it reads when kt_rows
  const void *v;   // [b, n2, n]  bf16 row-major
  float *out;      // [b, m, n_out] f32 row-major
  uint32_t b, m, k, n2, n;
  // Columns of the result that exist in `out` (its rows are n_out floats): n, or fewer when V
  // was padded with zero columns up to a head dim the kernel is built for.
  uint32_t n_out;
  bool kt_rows = false;  // KT stored row-major, n2 fastest (n2 a multiple of 8)
  // Queries per workgroup: 128 (eight waves) or 64 (four).
  uint32_t query_block = 128;
  // More than 1: the keys are shared out over that many workgroups per query block and the
  // partial results merged afterwards; `partials` holds attn_partial_bytes() of scratch.
  uint32_t key_splits = 1;
  float *partials = nullptr;
};
uint32_t attn_key_splits(const AttnArgs &a);
size_t attn_partial_bytes(const AttnArgs &a, uint32_t splits);
bool attn_applicable(const AttnArgs &a);
hipError_t launch_attn(const AttnArgs &a, hipStream_t stream);

}  // namespace mrl
