/*
 * CPU oracle for the Morello Spec execution path.  TEST INFRASTRUCTURE ONLY: see
 * morello_oracle.h for scope, reference anchors and what pins each function.
 *
 * Strategy: every tensor is gathered out of its layout into a dense logical row-major
 * array already converted to the output dtype's arithmetic class (wrapping 32-bit
 * integers, or f32), the closed form is evaluated with plain loops, and the result is
 * scattered back through the output layout.
 */
#include "morello_oracle.h"

#include <float.h>
#include <math.h>
#include <stdlib.h>
#include <string.h>

size_t orc_dtype_size(int dtype) {
  /* common.rs:30-36 */
  switch (dtype) {
    case ORC_U8:
    case ORC_I8:
      return 1;
    case ORC_U16:
    case ORC_I16:
    case ORC_BF16:
      return 2;
    case ORC_U32:
    case ORC_I32:
    case ORC_F32:
      return 4;
    default:
      return 0;
  }
}

float orc_bf16_to_f32(uint16_t v) {
  uint32_t bits = (uint32_t)v << 16;
  float f;
  memcpy(&f, &bits, 4);
  return f;
}

uint16_t orc_f32_to_bf16(float f) {
  uint32_t bits;
  memcpy(&bits, &f, 4);
  if ((bits & 0x7fffffffu) > 0x7f800000u) { /* NaN: keep it quiet */
    return (uint16_t)((bits >> 16) | 0x0040u);
  }
  uint32_t lsb = (bits >> 16) & 1u;
  bits += 0x7fffu + lsb;
  return (uint16_t)(bits >> 16);
}

/* ---------------------------------------------------------------- layouts */

int orc_layout_physical_shape(const orc_layout *layout, const uint32_t *shape, uint32_t rank,
                              uint32_t *phys_shape) {
  /* layout.rs:769-810: walk physical dims fastest-first, peeling sizes off each logical
   * dim.  0 marks "a Dynamic dim already consumed this logical dim". */
  uint32_t remaining[ORC_MAX_RANK];
  int tiled_packing[ORC_MAX_RANK];
  if (rank > ORC_MAX_RANK || layout->ndims > ORC_MAX_PHYS) return ORC_BAD_LAYOUT;
  for (uint32_t d = 0; d < rank; d++) {
    if (shape[d] == 0) return ORC_BAD_LAYOUT;
    remaining[d] = shape[d];
    tiled_packing[d] = 0;
  }
  for (int i = (int)layout->ndims - 1; i >= 0; i--) {
    const orc_physdim *pd = &layout->dims[i];
    if (pd->logical_dim >= rank) return ORC_BAD_LAYOUT;
    uint32_t *rem = &remaining[pd->logical_dim];
    if (*rem == 0) return ORC_BAD_LAYOUT;
    if (pd->kind == ORC_DYNAMIC) {
      phys_shape[i] = *rem;
      *rem = 0;
    } else {
      if (pd->size == 0) return ORC_BAD_LAYOUT;
      if (*rem < pd->size) {
        int smaller_ok = (pd->kind == ORC_PACKED) || (*rem == 1);
        if (!smaller_ok || tiled_packing[pd->logical_dim]) return ORC_BAD_LAYOUT;
        phys_shape[i] = *rem;
        *rem = 1;
        tiled_packing[pd->logical_dim] = 1;
      } else if (*rem % pd->size != 0) {
        return ORC_BAD_LAYOUT;
      } else {
        phys_shape[i] = pd->size;
        *rem /= pd->size;
      }
    }
  }
  for (uint32_t d = 0; d < rank; d++)
    if (remaining[d] > 1) return ORC_BAD_LAYOUT;
  return ORC_OK;
}

int64_t orc_layout_buffer_index(const orc_layout *layout, const uint32_t *shape, uint32_t rank,
                                const uint32_t *point) {
  /* layout.rs:221-272 with every variable bound to a number. */
  uint32_t phys[ORC_MAX_PHYS];
  if (orc_layout_physical_shape(layout, shape, rank, phys) != ORC_OK) return -1;
  int64_t remaining[ORC_MAX_RANK];
  for (uint32_t d = 0; d < rank; d++) remaining[d] = shape[d];
  int64_t working = 0;
  for (uint32_t i = 0; i < layout->ndims; i++) {
    const orc_physdim *pd = &layout->dims[i];
    uint32_t ld = pd->logical_dim;
    int64_t psize = phys[i];
    int64_t prev = remaining[ld];
    int64_t next = prev / psize;
    remaining[ld] = next;
    int64_t term = point[ld];
    if (prev != (int64_t)shape[ld]) term %= prev;
    if (pd->kind == ORC_ODDEVEN) {
      int64_t strip = pd->size;
      int64_t half = strip / 2;
      int64_t alternating = ((term % strip) % 2) * half;
      int64_t linear = (term % strip) / 2;
      term = (linear + alternating) / next;
    } else if ((int64_t)shape[ld] != psize) {
      term /= next;
    }
    working = working * psize + term;
  }
  return working;
}

void orc_layout_row_major(const uint32_t *shape, uint32_t rank, orc_layout *out) {
  out->ndims = 0;
  for (uint32_t d = 0; d < rank; d++) {
    if (shape[d] == 1) continue;
    out->dims[out->ndims].logical_dim = (uint8_t)d;
    out->dims[out->ndims].kind = ORC_DYNAMIC;
    out->dims[out->ndims].size = 0;
    out->ndims++;
  }
}

static size_t volume(const uint32_t *shape, uint32_t rank) {
  size_t v = 1;
  for (uint32_t d = 0; d < rank; d++) v *= shape[d];
  return v;
}

/* Table mapping each logical row-major position to its buffer offset.  A NULL layout is
 * row-major (identity).  Returns NULL on a bad layout (and sets *bad). */
static int64_t *offset_table(const orc_layout *layout, const uint32_t *shape, uint32_t rank,
                             int *bad) {
  size_t n = volume(shape, rank);
  *bad = 0;
  if (!layout) return NULL;
  uint32_t phys[ORC_MAX_PHYS];
  if (orc_layout_physical_shape(layout, shape, rank, phys) != ORC_OK) {
    *bad = 1;
    return NULL;
  }
  int64_t *tab = (int64_t *)malloc(sizeof(int64_t) * (n ? n : 1));
  uint32_t pt[ORC_MAX_RANK] = {0};
  for (size_t i = 0; i < n; i++) {
    tab[i] = orc_layout_buffer_index(layout, shape, rank, pt);
    for (int d = (int)rank - 1; d >= 0; d--) {
      if (++pt[d] < shape[d]) break;
      pt[d] = 0;
    }
  }
  return tab;
}

/* ------------------------------------------------------------ conversions */

static int is_float(int dtype) { return dtype == ORC_F32 || dtype == ORC_BF16; }

/* Rust `as` from any dtype to a 32-bit integer class value (wrapping for ints,
 * saturating for floats; verification.rs:547-569). */
static uint32_t load_as_u32(const void *buf, int dtype, int64_t off, int out_signed) {
  switch (dtype) {
    case ORC_U8:
      return ((const uint8_t *)buf)[off];
    case ORC_I8:
      return (uint32_t)(int32_t)((const int8_t *)buf)[off];
    case ORC_U16:
      return ((const uint16_t *)buf)[off];
    case ORC_I16:
      return (uint32_t)(int32_t)((const int16_t *)buf)[off];
    case ORC_U32:
      return ((const uint32_t *)buf)[off];
    case ORC_I32:
      return (uint32_t)((const int32_t *)buf)[off];
    case ORC_F32:
    case ORC_BF16: {
      float f = dtype == ORC_F32 ? ((const float *)buf)[off]
                                 : orc_bf16_to_f32(((const uint16_t *)buf)[off]);
      if (f != f) return 0;
      if (out_signed) {
        if (f <= -2147483648.0f) return 0x80000000u;
        if (f >= 2147483648.0f) return 0x7fffffffu;
        return (uint32_t)(int32_t)f;
      }
      if (f <= 0.0f) return 0;
      if (f >= 4294967296.0f) return 0xffffffffu;
      return (uint32_t)f;
    }
    default:
      return 0;
  }
}

static float load_as_f32(const void *buf, int dtype, int64_t off) {
  switch (dtype) {
    case ORC_U8:
      return (float)((const uint8_t *)buf)[off];
    case ORC_I8:
      return (float)((const int8_t *)buf)[off];
    case ORC_U16:
      return (float)((const uint16_t *)buf)[off];
    case ORC_I16:
      return (float)((const int16_t *)buf)[off];
    case ORC_U32:
      return (float)((const uint32_t *)buf)[off];
    case ORC_I32:
      return (float)((const int32_t *)buf)[off];
    case ORC_F32:
      return ((const float *)buf)[off];
    case ORC_BF16:
      return orc_bf16_to_f32(((const uint16_t *)buf)[off]);
    default:
      return 0.0f;
  }
}

/* Float outputs: f32 as it is; bf16 read by widening and written by one rounding to nearest even. */
static float load_out_f32(const void *buf, int dtype, int64_t off) {
  return dtype == ORC_BF16 ? orc_bf16_to_f32(((const uint16_t *)buf)[off]) : ((const float *)buf)[off];
}
static void store_out_f32(void *buf, int dtype, int64_t off, float v) {
  if (dtype == ORC_BF16) ((uint16_t *)buf)[off] = orc_f32_to_bf16(v);
  else ((float *)buf)[off] = v;
}
/* Inputs are cast to the output dtype first (verification.rs:629-631): for a bf16 output that
 * rounds f32 inputs to bf16. */
static void round_inputs_to(float *v, size_t n, int dt_out) {
  if (dt_out != ORC_BF16) return;
  for (size_t i = 0; i < n; i++) v[i] = orc_bf16_to_f32(orc_f32_to_bf16(v[i]));
}

static void store_from_u32(void *buf, int dtype, int64_t off, uint32_t v) {
  switch (dtype) {
    case ORC_U8:
    case ORC_I8:
      ((uint8_t *)buf)[off] = (uint8_t)v;
      break;
    case ORC_U16:
    case ORC_I16:
      ((uint16_t *)buf)[off] = (uint16_t)v;
      break;
    default:
      ((uint32_t *)buf)[off] = v;
      break;
  }
}

static int out_is_signed(int dtype) {
  return dtype == ORC_I8 || dtype == ORC_I16 || dtype == ORC_I32;
}

/* Sign- or zero-extend an integer of the output dtype held in the low bits. */
static uint32_t narrow_to(int dtype, uint32_t v) {
  switch (dtype) {
    case ORC_U8:
      return v & 0xffu;
    case ORC_I8:
      return (uint32_t)(int32_t)(int8_t)(uint8_t)v;
    case ORC_U16:
      return v & 0xffffu;
    case ORC_I16:
      return (uint32_t)(int32_t)(int16_t)(uint16_t)v;
    default:
      return v;
  }
}

/* Rust `as` from a float to an integer dtype: saturates at that dtype's own bounds, NaN -> 0
 * (verification.rs:547-569 casts every operand with `x.as_()` into the output dtype). */
static uint32_t float_as_int(float f, int out_dtype) {
  float lo, hi;
  if (f != f) return 0;
  switch (out_dtype) {
    case ORC_U8: lo = 0.0f, hi = 255.0f; break;
    case ORC_I8: lo = -128.0f, hi = 127.0f; break;
    case ORC_U16: lo = 0.0f, hi = 65535.0f; break;
    case ORC_I16: lo = -32768.0f, hi = 32767.0f; break;
    case ORC_U32: return f <= 0.0f ? 0u : f >= 4294967296.0f ? 0xffffffffu : (uint32_t)f;
    default: return f <= -2147483648.0f ? 0x80000000u : f >= 2147483648.0f ? 0x7fffffffu : (uint32_t)(int32_t)f;
  }
  if (f < lo) f = lo;
  if (f > hi) f = hi;
  return (uint32_t)(int32_t)f;
}

static uint32_t *gather_u32(const void *buf, int dtype, const int64_t *tab, size_t n,
                            int out_dtype) {
  uint32_t *dst = (uint32_t *)malloc(sizeof(uint32_t) * (n ? n : 1));
  int sgn = out_is_signed(out_dtype);
  for (size_t i = 0; i < n; i++) {
    int64_t off = tab ? tab[i] : (int64_t)i;
    if (is_float(dtype))
      dst[i] = narrow_to(out_dtype, float_as_int(load_as_f32(buf, dtype, off), out_dtype));
    else
      dst[i] = narrow_to(out_dtype, load_as_u32(buf, dtype, off, sgn));
  }
  return dst;
}

static float *gather_f32(const void *buf, int dtype, const int64_t *tab, size_t n) {
  float *dst = (float *)malloc(sizeof(float) * (n ? n : 1));
  for (size_t i = 0; i < n; i++) dst[i] = load_as_f32(buf, dtype, tab ? tab[i] : (int64_t)i);
  return dst;
}

/* ------------------------------------------------------------------ matmul */

int orc_matmul_rows(const uint32_t spec_shape[4], const int dtypes[3],
                    const orc_layout *layouts[3], int accum, const void *a, const void *b,
                    void *c, uint32_t row_begin, uint32_t row_end) {
  const uint32_t B = spec_shape[0], M = spec_shape[1], K = spec_shape[2], N = spec_shape[3];
  const uint32_t sa[3] = {B, M, K}, sb[3] = {B, K, N}, sc[3] = {B, M, N};
  const int dt_out = dtypes[2];
  if (row_end > M || row_begin > row_end) return ORC_BAD_ARG;
  int bad_a, bad_b, bad_c;
  int64_t *ta = offset_table(layouts ? layouts[0] : NULL, sa, 3, &bad_a);
  int64_t *tb = offset_table(layouts ? layouts[1] : NULL, sb, 3, &bad_b);
  int64_t *tc = offset_table(layouts ? layouts[2] : NULL, sc, 3, &bad_c);
  if (bad_a || bad_b || bad_c) {
    free(ta), free(tb), free(tc);
    return ORC_BAD_LAYOUT;
  }
  const size_t na = (size_t)B * M * K, nb = (size_t)B * K * N;
  if (is_float(dt_out)) {
    /* A bf16 output: inputs cast to bf16, products summed in f32, one rounding at the end.  The
     * reference rounds after every operation (bf16 arithmetic) and has no comparison for it
     * (verification.rs:597 `todo!`): this is the documented, more accurate reading. */
    float *fa = gather_f32(a, dtypes[0], ta, na);
    float *fb = gather_f32(b, dtypes[1], tb, nb);
    round_inputs_to(fa, na, dt_out), round_inputs_to(fb, nb, dt_out);
    float *row = (float *)malloc(sizeof(float) * N);
    for (uint32_t bi = 0; bi < B; bi++) {
      for (uint32_t i = row_begin; i < row_end; i++) {
        for (uint32_t j = 0; j < N; j++) {
          size_t ci = ((size_t)bi * M + i) * N + j;
          row[j] = accum ? load_out_f32(c, dt_out, tc ? tc[ci] : (int64_t)ci) : 0.0f;
        }
        const float *ar = fa + ((size_t)bi * M + i) * K;
        for (uint32_t k = 0; k < K; k++) {
          const float av = ar[k];
          const float *br = fb + ((size_t)bi * K + k) * N;
          for (uint32_t j = 0; j < N; j++) row[j] += av * br[j];
        }
        for (uint32_t j = 0; j < N; j++) {
          size_t ci = ((size_t)bi * M + i) * N + j;
          store_out_f32(c, dt_out, tc ? tc[ci] : (int64_t)ci, row[j]);
        }
      }
    }
    free(row), free(fa), free(fb);
  } else {
    uint32_t *ia = gather_u32(a, dtypes[0], ta, na, dt_out);
    uint32_t *ib = gather_u32(b, dtypes[1], tb, nb, dt_out);
    uint32_t *row = (uint32_t *)malloc(sizeof(uint32_t) * N);
    for (uint32_t bi = 0; bi < B; bi++) {
      for (uint32_t i = row_begin; i < row_end; i++) {
        for (uint32_t j = 0; j < N; j++) {
          size_t ci = ((size_t)bi * M + i) * N + j;
          row[j] = accum ? load_as_u32(c, dt_out, tc ? tc[ci] : (int64_t)ci, 0) : 0u;
        }
        const uint32_t *ar = ia + ((size_t)bi * M + i) * K;
        for (uint32_t k = 0; k < K; k++) {
          const uint32_t av = ar[k];
          const uint32_t *br = ib + ((size_t)bi * K + k) * N;
          for (uint32_t j = 0; j < N; j++) row[j] += av * br[j];
        }
        for (uint32_t j = 0; j < N; j++) {
          size_t ci = ((size_t)bi * M + i) * N + j;
          store_from_u32(c, dt_out, tc ? tc[ci] : (int64_t)ci, row[j]);
        }
      }
    }
    free(row), free(ia), free(ib);
  }
  free(ta), free(tb), free(tc);
  return ORC_OK;
}

int orc_matmul(const uint32_t spec_shape[4], const int dtypes[3], const orc_layout *layouts[3],
               int accum, const void *a, const void *b, void *c) {
  return orc_matmul_rows(spec_shape, dtypes, layouts, accum, a, b, c, 0, spec_shape[1]);
}

/* -------------------------------------------------------------------- conv */

int orc_conv(const uint32_t spec_shape[7], const int dtypes[3], const orc_layout *layouts[3],
             int accum, const void *image, const void *filters, void *out) {
  const uint32_t B = spec_shape[0], F = spec_shape[1], C = spec_shape[2], OH = spec_shape[3],
                 OW = spec_shape[4], FH = spec_shape[5], FW = spec_shape[6];
  const uint32_t H = OH + FH - 1, W = OW + FW - 1;
  const uint32_t si[4] = {B, C, H, W}, sf[4] = {F, C, FH, FW}, so[4] = {B, F, OH, OW};
  const int dt_out = dtypes[2];
  int bad_i, bad_f, bad_o;
  int64_t *ti = offset_table(layouts ? layouts[0] : NULL, si, 4, &bad_i);
  int64_t *tf = offset_table(layouts ? layouts[1] : NULL, sf, 4, &bad_f);
  int64_t *to = offset_table(layouts ? layouts[2] : NULL, so, 4, &bad_o);
  if (bad_i || bad_f || bad_o) {
    free(ti), free(tf), free(to);
    return ORC_BAD_LAYOUT;
  }
  const size_t ni = (size_t)B * C * H * W, nf = (size_t)F * C * FH * FW;
  if (is_float(dt_out)) {
    float *im = gather_f32(image, dtypes[0], ti, ni);
    float *fl = gather_f32(filters, dtypes[1], tf, nf);
    round_inputs_to(im, ni, dt_out), round_inputs_to(fl, nf, dt_out);
    for (uint32_t b = 0; b < B; b++)
      for (uint32_t f = 0; f < F; f++)
        for (uint32_t y = 0; y < OH; y++)
          for (uint32_t x = 0; x < OW; x++) {
            size_t oi = (((size_t)b * F + f) * OH + y) * OW + x;
            int64_t off = to ? to[oi] : (int64_t)oi;
            float acc = accum ? load_out_f32(out, dt_out, off) : 0.0f;
            for (uint32_t c = 0; c < C; c++)
              for (uint32_t r = 0; r < FH; r++)
                for (uint32_t s = 0; s < FW; s++)
                  acc += im[(((size_t)b * C + c) * H + y + r) * W + x + s] *
                         fl[(((size_t)f * C + c) * FH + r) * FW + s];
            store_out_f32(out, dt_out, off, acc);
          }
    free(im), free(fl);
  } else {
    uint32_t *im = gather_u32(image, dtypes[0], ti, ni, dt_out);
    uint32_t *fl = gather_u32(filters, dtypes[1], tf, nf, dt_out);
    for (uint32_t b = 0; b < B; b++)
      for (uint32_t f = 0; f < F; f++)
        for (uint32_t y = 0; y < OH; y++)
          for (uint32_t x = 0; x < OW; x++) {
            size_t oi = (((size_t)b * F + f) * OH + y) * OW + x;
            int64_t off = to ? to[oi] : (int64_t)oi;
            uint32_t acc = accum ? load_as_u32(out, dt_out, off, 0) : 0u;
            for (uint32_t c = 0; c < C; c++)
              for (uint32_t r = 0; r < FH; r++)
                for (uint32_t s = 0; s < FW; s++)
                  acc += im[(((size_t)b * C + c) * H + y + r) * W + x + s] *
                         fl[(((size_t)f * C + c) * FH + r) * FW + s];
            store_from_u32(out, dt_out, off, acc);
          }
    free(im), free(fl);
  }
  free(ti), free(tf), free(to);
  return ORC_OK;
}

/* ----------------------------------------------------------------- softmax */

/* One softmax over `n` values spaced `stride` apart in a dense array
 * (verification.rs:166-184: max, subtract, exp, sum, divide). */
static void softmax_line(const float *in, float *out, size_t n, size_t stride) {
  float mx = -3.40282347e+38f; /* f32::MIN, verification.rs:842-861 */
  for (size_t i = 0; i < n; i++) {
    float v = in[i * stride];
    if (v != v) {
      mx = v;
      break;
    }
    if (v > mx) mx = v;
  }
  float denom = 0.0f;
  for (size_t i = 0; i < n; i++) {
    float e = expf(in[i * stride] - mx);
    out[i * stride] = e;
    denom += e;
  }
  for (size_t i = 0; i < n; i++) out[i * stride] /= denom;
}

int orc_softmax(const uint32_t *shape, uint32_t rank, uint32_t scan_dim,
                const orc_layout *layouts[2], const float *in, float *out) {
  if (scan_dim >= rank) return ORC_BAD_ARG;
  int bad_i, bad_o;
  int64_t *ti = offset_table(layouts ? layouts[0] : NULL, shape, rank, &bad_i);
  int64_t *to = offset_table(layouts ? layouts[1] : NULL, shape, rank, &bad_o);
  if (bad_i || bad_o) {
    free(ti), free(to);
    return ORC_BAD_LAYOUT;
  }
  size_t n = volume(shape, rank);
  float *dense_in = gather_f32(in, ORC_F32, ti, n);
  float *dense_out = (float *)malloc(sizeof(float) * (n ? n : 1));
  size_t inner = 1;
  for (uint32_t d = scan_dim + 1; d < rank; d++) inner *= shape[d];
  size_t len = shape[scan_dim];
  size_t outer = n / (inner * len);
  for (size_t o = 0; o < outer; o++)
    for (size_t i = 0; i < inner; i++)
      softmax_line(dense_in + o * len * inner + i, dense_out + o * len * inner + i, len, inner);
  for (size_t i = 0; i < n; i++) out[to ? to[i] : (int64_t)i] = dense_out[i];
  free(dense_in), free(dense_out), free(ti), free(to);
  return ORC_OK;
}

/* ----------------------------------------------------------------- compose */

int orc_compose_msm(uint32_t b, uint32_t m, uint32_t k, uint32_t n2, uint32_t n,
                    const int dtypes[4], const orc_layout *layouts[4], const void *v,
                    const void *q, const void *kt, float *out) {
  if (dtypes[3] != ORC_F32) return ORC_UNSUPPORTED;
  /* Innermost component: S = Q.KT into a zeroed f32 buffer (verification.rs:239-256). */
  const uint32_t s0[4] = {b, m, k, n2};
  const int d0[3] = {dtypes[1], dtypes[2], ORC_F32};
  const orc_layout *l0[3] = {layouts ? layouts[1] : NULL, layouts ? layouts[2] : NULL, NULL};
  size_t ns = (size_t)b * m * n2;
  float *s = (float *)calloc(ns ? ns : 1, sizeof(float));
  float *p = (float *)malloc(sizeof(float) * (ns ? ns : 1));
  int rc = orc_matmul(s0, d0, l0, 0, q, kt, s);
  if (rc == ORC_OK) {
    /* Softmax over scan_dim 2 (verification.rs:258-277). */
    const uint32_t ss[3] = {b, m, n2};
    rc = orc_softmax(ss, 3, 2, NULL, s, p);
  }
  if (rc == ORC_OK) {
    /* Head component: out = P.V (verification.rs:279-281). */
    const uint32_t s2[4] = {b, m, n2, n};
    const int d2[3] = {ORC_F32, dtypes[0], ORC_F32};
    const orc_layout *l2[3] = {NULL, layouts ? layouts[0] : NULL, layouts ? layouts[3] : NULL};
    rc = orc_matmul(s2, d2, l2, 0, p, v, out);
  }
  free(s), free(p);
  return rc;
}

/* -------------------------------------------------------------------- move */

int orc_move(const uint32_t *shape, uint32_t rank, const int dtypes[2], const orc_layout *layouts[2],
             const void *in, void *out) {
  int bad_i, bad_o;
  int64_t *ti = offset_table(layouts ? layouts[0] : NULL, shape, rank, &bad_i);
  int64_t *to = offset_table(layouts ? layouts[1] : NULL, shape, rank, &bad_o);
  if (bad_i || bad_o) {
    free(ti), free(to);
    return ORC_BAD_LAYOUT;
  }
  const size_t n = volume(shape, rank);
  const int sdt = dtypes[0], ddt = dtypes[1];
  for (size_t i = 0; i < n; i++) {
    const int64_t so = ti ? ti[i] : (int64_t)i, d_o = to ? to[i] : (int64_t)i;
    if (ddt == ORC_F32) ((float *)out)[d_o] = load_as_f32(in, sdt, so);
    else if (ddt == ORC_BF16) ((uint16_t *)out)[d_o] = orc_f32_to_bf16(load_as_f32(in, sdt, so));
    else if (is_float(sdt)) store_from_u32(out, ddt, d_o, float_as_int(load_as_f32(in, sdt, so), ddt));
    else store_from_u32(out, ddt, d_o, load_as_u32(in, sdt, so, 0));
  }
  free(ti), free(to);
  return ORC_OK;
}

/* ------------------------------------------------------------ input pattern */

int orc_fill_check_pattern(int dtype, void *dst, size_t count) {
  /* verification.rs:893-952 */
  switch (dtype) {
    case ORC_U8:
      for (size_t i = 0; i < count; i++) ((uint8_t *)dst)[i] = (uint8_t)i;
      return ORC_OK;
    case ORC_I8:
      for (size_t i = 0; i < count; i++) ((int8_t *)dst)[i] = (int8_t)(uint8_t)(i + 128u);
      return ORC_OK;
    case ORC_U16:
      for (size_t i = 0; i < count; i++) ((uint16_t *)dst)[i] = (uint16_t)i;
      return ORC_OK;
    case ORC_I16:
      for (size_t i = 0; i < count; i++) ((int16_t *)dst)[i] = (int16_t)(uint16_t)(i + 32768u);
      return ORC_OK;
    case ORC_U32:
      for (size_t i = 0; i < count; i++) ((uint32_t *)dst)[i] = (uint32_t)i;
      return ORC_OK;
    case ORC_I32:
      for (size_t i = 0; i < count; i++)
        ((int32_t *)dst)[i] = (int32_t)((uint32_t)i + 0x80000000u);
      return ORC_OK;
    case ORC_F32:
      for (size_t i = 0; i < count; i++) ((float *)dst)[i] = (float)(i & 3u);
      return ORC_OK;
    case ORC_BF16:
      for (size_t i = 0; i < count; i++) ((uint16_t *)dst)[i] = orc_f32_to_bf16((float)(i & 3u));
      return ORC_OK;
    default:
      return ORC_BAD_ARG;
  }
}

/* ------------------------------------------- primitives of the Softmax decomposition */

/* One line along the scan dim, visited element by element as the scalar kernels the
 * emitter prints are visited by the loops around them (codegen/cpu.rs:1350-1433,
 * 1968-2113).  `x`, `y`: full-shape parameters of the line with element stride `st`;
 * `r0`, `r1`: the line's entries of the reduced parameters. */
static void part_line(int kind, int accum, size_t n, size_t st, float *p0, float *p1, float *p2,
                      float *p3) {
  switch (kind) {
    case ORC_PART_MAX: /* [in, out] */
      if (!accum) *p1 = -INFINITY;
      for (size_t i = 0; i < n; i++) *p1 = fmaxf(*p1, p0[i * st]);
      break;
    case ORC_PART_DENOMINATOR: /* [in, max, denom]: cpu.rs:1414-1424 */
      if (!accum) *p2 = 0.0f;
      for (size_t i = 0; i < n; i++) *p2 += expf(p0[i * st] - *p1);
      break;
    case ORC_PART_DENOMINATOR_AND_MAX: /* [in, max, denom]: cpu.rs:1360-1389 */
      if (!accum) *p1 = -INFINITY, *p2 = 0.0f;
      for (size_t i = 0; i < n; i++) {
        const float old_max = *p1;
        const float new_max = fmaxf(old_max, p0[i * st]);
        *p2 = *p2 * expf(old_max - new_max) + expf(p0[i * st] - new_max);
        *p1 = new_max;
      }
      break;
    case ORC_PART_DENOMINATOR_AND_MAX_FROM_PARTS: /* [tile_max, tile_denom, max, denom]: cpu.rs:1390-1413 */
      if (!accum) *p2 = -INFINITY, *p3 = 0.0f;
      for (size_t i = 0; i < n; i++) {
        const float old_max = *p2;
        const float new_max = fmaxf(old_max, p0[i * st]);
        *p3 = *p3 * expf(old_max - new_max) + p1[i * st] * expf(p0[i * st] - new_max);
        *p2 = new_max;
      }
      break;
    case ORC_PART_DENOMINATOR_AND_UNSCALED: { /* [in, denom, unscaled]: spec.rs:133-136 */
      float m = -INFINITY;
      for (size_t i = 0; i < n; i++) m = fmaxf(m, p0[i * st]);
      *p1 = 0.0f;
      for (size_t i = 0; i < n; i++) {
        const float e = expf(p0[i * st] - m);
        *p1 += e;
        p2[i * st] = e;
      }
      break;
    }
    case ORC_PART_DENOMINATOR_AND_UNSCALED_FROM_MAX: /* [in, max, denom, unscaled]: cpu.rs:1425-1433 */
      if (!accum) *p2 = 0.0f;
      for (size_t i = 0; i < n; i++) {
        const float e = expf(p0[i * st] - *p1);
        *p2 += e;
        p3[i * st] = e;
      }
      break;
    case ORC_PART_COMPLETE: /* [in, max, denom, out]: cpu.rs:1350-1359 */
      for (size_t i = 0; i < n; i++) p3[i * st] = expf(p0[i * st] - *p1) / *p2;
      break;
    case ORC_PART_DIVIDE_VEC: /* [numer, denom]: verification.rs:191-197 */
      for (size_t i = 0; i < n; i++) p0[i * st] /= p1[i * st];
      break;
    case ORC_PART_DIVIDE_VEC_SCALAR: /* [numer, denom]: verification.rs:198-204 */
      for (size_t i = 0; i < n; i++) p0[i * st] /= *p1;
      break;
  }
}

int orc_softmax_part(int kind, int accum, const uint32_t *shape, uint32_t rank, uint32_t scan_dim,
                     float *const params[4]) {
  /* Which parameters have size one on the scan dim (spec.rs:499-583). */
  static const unsigned reduced[] = {
      [ORC_PART_MAX] = 2u,
      [ORC_PART_DENOMINATOR] = 6u,
      [ORC_PART_DENOMINATOR_AND_MAX] = 6u,
      [ORC_PART_DENOMINATOR_AND_MAX_FROM_PARTS] = 12u,
      [ORC_PART_DENOMINATOR_AND_UNSCALED] = 2u,
      [ORC_PART_DENOMINATOR_AND_UNSCALED_FROM_MAX] = 6u,
      [ORC_PART_COMPLETE] = 6u,
      [ORC_PART_DIVIDE_VEC] = 0u,
      [ORC_PART_DIVIDE_VEC_SCALAR] = 2u,
  };
  static const unsigned nparams[] = {
      [ORC_PART_MAX] = 2, [ORC_PART_DENOMINATOR] = 3, [ORC_PART_DENOMINATOR_AND_MAX] = 3,
      [ORC_PART_DENOMINATOR_AND_MAX_FROM_PARTS] = 4, [ORC_PART_DENOMINATOR_AND_UNSCALED] = 3,
      [ORC_PART_DENOMINATOR_AND_UNSCALED_FROM_MAX] = 4, [ORC_PART_COMPLETE] = 4,
      [ORC_PART_DIVIDE_VEC] = 2, [ORC_PART_DIVIDE_VEC_SCALAR] = 2,
  };
  if (kind < ORC_PART_MAX || kind > ORC_PART_DIVIDE_VEC_SCALAR || rank == 0 || rank > ORC_MAX_RANK)
    return ORC_BAD_ARG;
  if (kind == ORC_PART_DIVIDE_VEC) scan_dim = rank - 1;
  if (scan_dim >= rank) return ORC_BAD_ARG;
  if (kind == ORC_PART_DENOMINATOR_AND_UNSCALED && accum) return ORC_UNSUPPORTED;
  size_t outer = 1, inner = 1;
  for (uint32_t d = 0; d < scan_dim; d++) outer *= shape[d];
  for (uint32_t d = scan_dim + 1; d < rank; d++) inner *= shape[d];
  const size_t n = shape[scan_dim];
  for (size_t o = 0; o < outer; o++)
    for (size_t in = 0; in < inner; in++) {
      float *p[4] = {0, 0, 0, 0};
      for (unsigned t = 0; t < nparams[kind]; t++)
        p[t] = (reduced[kind] >> t) & 1 ? params[t] + o * inner + in : params[t] + o * n * inner + in;
      part_line(kind, accum, n, inner, p[0], p[1], p[2], p[3]);
    }
  return ORC_OK;
}

int orc_broadcast(const uint32_t *shape, uint32_t rank, uint32_t dim, size_t elem_size,
                  const void *in, void *out) {
  if (rank == 0 || rank > ORC_MAX_RANK || dim >= rank) return ORC_BAD_ARG;
  size_t outer = 1, inner = 1;
  for (uint32_t d = 0; d < dim; d++) outer *= shape[d];
  for (uint32_t d = dim + 1; d < rank; d++) inner *= shape[d];
  for (size_t o = 0; o < outer; o++)
    for (size_t i = 0; i < shape[dim]; i++)
      memcpy((char *)out + ((o * shape[dim] + i) * inner) * elem_size,
             (const char *)in + o * inner * elem_size, inner * elem_size);
  return ORC_OK;
}

int orc_fill(int dtype, int value, void *dst, size_t count) {
  /* verification.rs:214-222 with DynArray::zero / fill_neg_inf / fill_min (:521-545). */
  uint32_t pattern = 0;
  if (value == 1) {
    if (!is_float(dtype)) return ORC_BAD_ARG;
    const float ninf = -INFINITY;
    memcpy(&pattern, &ninf, 4);
    if (dtype == ORC_BF16) pattern >>= 16;
  } else if (value == 2) {
    const float fmin_ = -FLT_MAX;
    switch (dtype) {
      case ORC_I8: pattern = (uint8_t)INT8_MIN; break;
      case ORC_I16: pattern = (uint16_t)INT16_MIN; break;
      case ORC_I32: pattern = (uint32_t)INT32_MIN; break;
      case ORC_F32: memcpy(&pattern, &fmin_, 4); break;
      case ORC_BF16: pattern = 0xff7fu; break; /* half::bf16::MIN */
      default: pattern = 0; break;
    }
  } else if (value != 0) {
    return ORC_BAD_ARG;
  }
  const size_t es = orc_dtype_size(dtype);
  if (es == 0) return ORC_BAD_ARG;
  for (size_t i = 0; i < count; i++) memcpy((char *)dst + i * es, &pattern, es); /* little endian */
  return ORC_OK;
}
