/*
 * Build-time wrapper that compiles the reference's own x86 C partials (they are
 * `inline`/file-local snippets meant to be pasted into emitted programs) and exports them
 * under stable names, so tests can compare the oracle's arithmetic with the arithmetic the
 * reference's emitted C really uses.  TEST INFRASTRUCTURE ONLY.  The partials are included
 * from the reference checkout by path (-DREF_PARTIALS=...); nothing is copied.
 */
#include <immintrin.h>
#include <stdint.h>

#define REF_STR2(x) #x
#define REF_STR(x) REF_STR2(x)
#define REF_FILE(name) REF_STR(REF_PARTIALS/x86/name)

#include REF_FILE(expf_avx2.c)
#include REF_FILE(sum8.c)
#include REF_FILE(max8.c)
#include REF_FILE(max4.c)
#include REF_FILE(cvtbf16_fp32.c)

/* exp256_ps applied to n floats (n a multiple of 8). */
void ref_exp256(const float *in, float *out, int n) {
  for (int i = 0; i < n; i += 8) _mm256_storeu_ps(out + i, exp256_ps(_mm256_loadu_ps(in + i)));
}

void ref_exp128(const float *in, float *out, int n) {
  for (int i = 0; i < n; i += 4) _mm_storeu_ps(out + i, exp128_ps(_mm_loadu_ps(in + i)));
}

float ref_sum8(const float *in) { return sum8(_mm256_loadu_ps(in)); }
float ref_sum4(const float *in) { return sum4(_mm_loadu_ps(in)); }
float ref_max8(const float *in) { return horizontal_max_f32(_mm256_loadu_ps(in)); }
float ref_max4(const float *in) { return horizontal_max4_f32(_mm_loadu_ps(in)); }

/* 8 bf16 bit patterns -> 8 floats. */
void ref_cvtbf16_fp32(const uint16_t *in, float *out) {
  _mm256_storeu_ps(out, cvtbf16_fp32(_mm_loadu_si128((const __m128i *)in)));
}
