/*
 * CPU oracle for the Morello Spec execution path.  TEST INFRASTRUCTURE ONLY.
 *
 * This is a plain-C restatement of what a Morello Matmul / Conv / Softmax Spec and the
 * Matmul->Softmax->Matmul Compose compute, used to check the GPU library.  It is never
 * linked into, loaded by, or called from the shipped library: only tests, the smoke check
 * and the benchmark's CPU-baseline leg may use it.
 *
 * Reference anchors (paths relative to the reference checkout):
 *   dtypes .................. morello/src/common.rs:15-36
 *   layout index math ....... morello/src/layout.rs:221-272 (buffer_indexing_expr),
 *                             :769-810 (expand_physical_shape)
 *   parameter shapes ........ morello/src/spec.rs:467-583
 *   Matmul / Softmax / Compose closed forms ... morello/src/verification.rs:105-337
 *   Conv semantics .......... morello/src/spec.rs:486-498,741-776 and
 *                             morello/src/scheduling/spatial_split.rs:18-129
 *                             (NOT verification.rs:153-162, which is defective: it
 *                             indexes the output by input channel, overwrites instead of
 *                             accumulating and zero-pads)
 *   check-mode inputs ....... morello/src/verification.rs:893-952
 *
 * Pinning status (what independent evidence each function is tested against):
 *   orc_layout_*  ........ expectations asserted in morello/src/layout.rs:1452-1551,
 *                          2391-2452, book/src/data_layouts.md:59-99, plus bijection
 *                          brute force.
 *   orc_matmul  .......... numpy int64/float64 matmul, identity/extreme cases, and the
 *                          emitted kernel quoted in examples/simple_matmul_x86.rs:146-178
 *                          (compiled into oracle/_ref when the reference is present).
 *   orc_conv  ............ scipy.signal.correlate (valid mode), 1x1-filter == Matmul,
 *                          oh=ow=1 == dot product.  The reference's own tests do not
 *                          execute a Conv: parity with the reference *implementation*
 *                          is unpinned; parity with the Spec semantics is pinned.
 *   orc_softmax  ......... scipy.special.softmax in float64, row-sum / shift invariants.
 *   orc_compose_msm  ..... composition of the three above in float64 (numpy).
 *   u8*i8->i32 and bf16 execution are not exercised by any test in the reference
 *   (its CI skips bf16 execution): parity there is pinned by mathematics only.
 *   bf16 OUTPUTS of orc_matmul / orc_conv: PARITY UNPINNED.  Inputs are cast to bf16
 *   (verification.rs:629-631), products summed in f32, the sum rounded to bf16 once; the
 *   reference's interpreter works in bf16 arithmetic (a rounding after every operation)
 *   and its own comparison for bf16 is `todo!` (verification.rs:597).  What is pinned is
 *   the arithmetic stated here: hand-computed known answers (exact small integers, the
 *   ties 257 -> 256 and 259 -> 260, input rounding) in tests/test_oracle.py.
 */
#ifndef MORELLO_ORACLE_H
#define MORELLO_ORACLE_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* morello/src/common.rs:15-24, in declaration order. */
enum {
  ORC_U8 = 0,
  ORC_I8 = 1,
  ORC_U16 = 2,
  ORC_I16 = 3,
  ORC_U32 = 4,
  ORC_I32 = 5,
  ORC_F32 = 6,
  ORC_BF16 = 7
};

/* morello/src/layout.rs:74-81 */
enum { ORC_DYNAMIC = 0, ORC_PACKED = 1, ORC_ODDEVEN = 2 };

#define ORC_MAX_PHYS 10
#define ORC_MAX_RANK 5

typedef struct {
  uint8_t logical_dim;
  uint8_t kind;
  uint32_t size; /* pack / strip size; ignored for ORC_DYNAMIC */
} orc_physdim;

typedef struct {
  uint32_t ndims;
  orc_physdim dims[ORC_MAX_PHYS];
} orc_layout;

/* Status codes. */
enum { ORC_OK = 0, ORC_BAD_LAYOUT = 1, ORC_UNSUPPORTED = 2, ORC_BAD_ARG = 3 };

size_t orc_dtype_size(int dtype);

/* layout.rs:769-810.  Writes layout->ndims sizes.  Returns ORC_BAD_LAYOUT for shapes the
 * layout does not apply to. */
int orc_layout_physical_shape(const orc_layout *layout, const uint32_t *shape, uint32_t rank,
                              uint32_t *phys_shape);

/* layout.rs:221-272 evaluated at a concrete logical point.  Returns -1 on a bad layout. */
int64_t orc_layout_buffer_index(const orc_layout *layout, const uint32_t *shape, uint32_t rank,
                                const uint32_t *point);

/* layout.rs:1234-1247: row-major over `shape`, dropping size-one dims. */
void orc_layout_row_major(const uint32_t *shape, uint32_t rank, orc_layout *out);

/* bf16 helpers: widening is a 16-bit shift (partials/x86/cvtbf16_fp32.c); narrowing is
 * round-to-nearest-even, as the `half` crate and clang's __bf16 do. */
float orc_bf16_to_f32(uint16_t v);
uint16_t orc_f32_to_bf16(float f);

/* Matmul Spec.  spec_shape = [b, m, k, n]; A[b,m,k], B[b,k,n], C[b,m,n]
 * (spec.rs:480-485).  Both inputs are converted to the output dtype, then
 * C (=0 unless accum) += A.B (verification.rs:115-134, 603-643).  A NULL layout means
 * row-major.  Integer outputs wrap modulo 2^bits. */
int orc_matmul(const uint32_t spec_shape[4], const int dtypes[3], const orc_layout *layouts[3],
               int accum, const void *a, const void *b, void *c);

/* As orc_matmul, but only rows [row_begin, row_end) of every batch entry of C are computed
 * and written; other elements of C are left untouched.  Used to spot-check full-size runs. */
int orc_matmul_rows(const uint32_t spec_shape[4], const int dtypes[3],
                    const orc_layout *layouts[3], int accum, const void *a, const void *b,
                    void *c, uint32_t row_begin, uint32_t row_end);

/* Conv Spec.  spec_shape = [b, f, c, oh, ow, fh, fw]; image [b,c,oh+fh-1,ow+fw-1],
 * filters [f,c,fh,fw], out [b,f,oh,ow] (spec.rs:486-498).  Stride 1, no padding,
 * cross-correlation:  out[b,f,y,x] (=0 unless accum) +=
 *     sum_{c,r,s} img[b,c,y+r,x+s] * filt[f,c,r,s]. */
int orc_conv(const uint32_t spec_shape[7], const int dtypes[3], const orc_layout *layouts[3],
             int accum, const void *image, const void *filters, void *out);

/* Softmax Spec over `scan_dim` of an f32 tensor (spec.rs:86-90, verification.rs:166-184):
 * max, subtract, expf, sum, divide. */
int orc_softmax(const uint32_t *shape, uint32_t rank, uint32_t scan_dim,
                const orc_layout *layouts[2], const float *in, float *out);

/* Compose [Matmul[b,m,n2,n] , Softmax{scan_dim 2}[b,m,n2], Matmul[b,m,k,n2]] listed
 * last-executed first (spec.rs:1532); external parameters [V, Q, KT, out]
 * (spec.rs:3329-3365): Q[b,m,k], KT[b,k,n2], V[b,n2,n], out[b,m,n] f32.
 * dtypes = {V, Q, KT, out}.  The intermediates are f32 (verification.rs:225-286). */
int orc_compose_msm(uint32_t b, uint32_t m, uint32_t k, uint32_t n2, uint32_t n,
                    const int dtypes[4], const orc_layout *layouts[4], const void *v,
                    const void *q, const void *kt, float *out);

/* Move Spec (verification.rs:521-532, 547-569: assign_cast = element-wise Rust `as`):
 * ints wrap to the destination width, floats saturate at the destination's bounds with
 * NaN -> 0, f32 -> bf16 rounds to nearest even, everything -> f32 as C converts.
 * Pinned by: numpy `astype` for int->int and int->float, known answers for saturation,
 * identity and layout round trips. */
int orc_move(const uint32_t *shape, uint32_t rank, const int dtypes[2], const orc_layout *layouts[2],
             const void *in, void *out);

/* The primitives Softmax decomposes into (spec.rs:86-162), numbered as in the GPU library's
 * ABI.  f32, dense row-major; `params` in Spec parameter order; a "reduced" parameter is
 * dense over the shape with scan_dim set to one.  Each line is updated element by element
 * exactly as the emitter's scalar kernels would be (codegen/cpu.rs:1350-1433).
 * Pinned by: numpy max / logsumexp identities in float64, scipy.special.softmax for
 * Complete, splitting a row into tiles and merging for FromParts, and accum == running the
 * non-accumulating form on the concatenated input.  The reference's interpreter leaves
 * these as todo!() (verification.rs:185-205) except DivideVec/DivideVecScalar, so parity
 * with a reference *execution* is unpinned; the arithmetic is pinned. */
enum {
  ORC_PART_MAX = 6,
  ORC_PART_DENOMINATOR = 7,
  ORC_PART_DENOMINATOR_AND_MAX = 8,
  ORC_PART_DENOMINATOR_AND_MAX_FROM_PARTS = 9,
  ORC_PART_DENOMINATOR_AND_UNSCALED = 10,
  ORC_PART_DENOMINATOR_AND_UNSCALED_FROM_MAX = 11,
  ORC_PART_COMPLETE = 12,
  ORC_PART_DIVIDE_VEC = 13,
  ORC_PART_DIVIDE_VEC_SCALAR = 14
};
int orc_softmax_part(int kind, int accum, const uint32_t *shape, uint32_t rank, uint32_t scan_dim,
                     float *const params[4]);

/* Broadcast{dim} (spec.rs:70-75, 499-507): out[.., i, ..] = in[.., 0, ..]; dense row-major. */
int orc_broadcast(const uint32_t *shape, uint32_t rank, uint32_t dim, size_t elem_size,
                  const void *in, void *out);

/* Fill{value} (spec.rs:143-170; verification.rs:214-222): value 0 Zero, 1 NegInf (floats
 * only), 2 Min (the dtype's minimum; f32::MIN / bf16::MIN for floats). */
int orc_fill(int dtype, int value, void *dst, size_t count);

/* verification.rs:893-952: ints count up from the dtype minimum and wrap at the maximum;
 * f32 and bf16 cycle 0,1,2,3.  Fills `count` elements in logical row-major order. */
int orc_fill_check_pattern(int dtype, void *dst, size_t count);

#ifdef __cplusplus
}
#endif
#endif
