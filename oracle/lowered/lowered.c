/* See lowered.h.  TEST INFRASTRUCTURE ONLY. */
#include "lowered.h"

#include <math.h>
#include <omp.h>
#include <stdlib.h>
#include <string.h>

typedef int32_t vsi8 __attribute__((vector_size(32)));
typedef float vf8 __attribute__((vector_size(32)));

int lowered_num_procs(void) { return omp_get_num_procs(); }

static int clamp_threads(int threads, int steps) {
  /* partials/x86/cores_clamp.c: never more threads than loop steps or cores. */
  int procs = omp_get_num_procs();
  if (threads <= 0 || threads > procs) threads = procs;
  return threads < steps ? threads : (steps > 0 ? steps : 1);
}

void lowered_matmul_f32(const float *restrict n000, const float *restrict n001,
                        float *restrict n002, int m, int k, int n) {
  for (int n003 = 0; n003 < m / 16; n003++) {
  for (int n004 = 0; n004 < n / 16; n004++) {
    for (int n005 = 0; n005 < 16; n005++) {
    for (int n006 = 0; n006 < 16; n006++) {
      float n007;
      memset((void *)(&n007), 0, 4);
      n002[(n * n005 + 16 * n * n003 + n006 + 16 * n004)] = n007;
      for (int n008 = 0; n008 < k / 4; n008++) {
        float n009[4] __attribute__((aligned (128)));
        for (int n010 = 0; n010 < 4; n010++) {
          n009[(n010)] = n000[(k * n005 + 16 * k * n003 + n010 + 4 * n008)];
        }
        float n011[4] __attribute__((aligned (128)));
        for (int n012 = 0; n012 < 4; n012++) {
          n011[(n012)] = n001[(n * n012 + 4 * n * n008 + n006 + 16 * n004)];
        }
        float n013;
        n013 = n002[(n * n005 + 16 * n * n003 + n006 + 16 * n004)];
        for (int n014 = 0; n014 < 4; n014++) {
          n013 += n009[(n014)] * n011[(n014)];  /* MultAdd */
        }
        n002[(n * n005 + 16 * n * n003 + n006 + 16 * n004)] = n013;
      }
    }
    }
  }
  }
}

void lowered_matmul_u8i8i32(const uint8_t *restrict n000, const int8_t *restrict n001,
                            int32_t *restrict n002, int m, int k, int n, int row_begin,
                            int row_end, int threads) {
  (void)m;
  const int steps = row_end - row_begin;
#pragma omp parallel for num_threads(clamp_threads(threads, steps)) proc_bind(spread) schedule(static)
  for (int n003 = row_begin; n003 < row_end; n003++) {
  for (int n004 = 0; n004 < n / 16; n004++) {
    vsi8 n005[2];  /* move_param(2, VRF): 16 i32 = two 8-lane vectors */
    memcpy(n005, &n002[(n * n003 + 16 * n004)], 64);
    for (int n006 = 0; n006 < k; n006++) {
      int32_t n007;
      n007 = n000[(k * n003 + n006)];  /* Assign u8 -> i32 */
      int32_t n008[16] __attribute__((aligned (128)));
      for (int n009 = 0; n009 < 16; n009++) {
        n008[(n009)] = n001[(n * n006 + 16 * n004 + n009)];  /* Assign i8 -> i32 */
      }
      n005[0] += n007 * (*(vsi8 *)(&n008[0]));  /* BroadcastVecMultAdd */
      n005[1] += n007 * (*(vsi8 *)(&n008[8]));  /* BroadcastVecMultAdd */
    }
    memcpy(&n002[(n * n003 + 16 * n004)], n005, 64);
  }
  }
}

static inline float bf16_as_f32(uint16_t v) {
  uint32_t bits = (uint32_t)v << 16;  /* CastBf16F32: same value as (float)(__bf16) */
  float f;
  memcpy(&f, &bits, 4);
  return f;
}

void lowered_matmul_bf16f32(const uint16_t *restrict n000, const uint16_t *restrict n001,
                            float *restrict n002, int m, int k, int n, int row_begin,
                            int row_end, int threads) {
  (void)m;
  const int steps = row_end - row_begin;
#pragma omp parallel for num_threads(clamp_threads(threads, steps)) proc_bind(spread) schedule(static)
  for (int n003 = row_begin; n003 < row_end; n003++) {
  for (int n004 = 0; n004 < n / 16; n004++) {
    vf8 n005[2];
    memcpy(n005, &n002[(n * n003 + 16 * n004)], 64);
    for (int n006 = 0; n006 < k; n006++) {
      float n007;
      n007 = bf16_as_f32(n000[(k * n003 + n006)]);  /* CastBf16F32 */
      float n008[16] __attribute__((aligned (128)));
      for (int n009 = 0; n009 < 16; n009++) {
        n008[(n009)] = bf16_as_f32(n001[(n * n006 + 16 * n004 + n009)]);  /* VectorCastBf16F32 */
      }
      n005[0] += n007 * (*(vf8 *)(&n008[0]));  /* BroadcastVecMultAdd */
      n005[1] += n007 * (*(vf8 *)(&n008[8]));  /* BroadcastVecMultAdd */
    }
    memcpy(&n002[(n * n003 + 16 * n004)], n005, 64);
  }
  }
}

void lowered_conv_u8i8i32(const uint8_t *restrict n000, const int8_t *restrict n001,
                          int32_t *restrict n002, int b, int f, int c, int oh, int ow, int fh,
                          int fw, int img_begin, int img_end, int threads) {
  (void)b;
  const int h = oh + fh - 1, w = ow + fw - 1;
  const int steps = (img_end - img_begin) * oh;
#pragma omp parallel for collapse(2) num_threads(clamp_threads(threads, steps)) proc_bind(spread) schedule(static)
  for (int n003 = img_begin; n003 < img_end; n003++) {
  for (int n004 = 0; n004 < oh; n004++) {
    for (int n005 = 0; n005 < ow; n005++) {
    for (int n006 = 0; n006 < f; n006++) {
      int32_t n007;
      memset((void *)(&n007), 0, 4);  /* to_accum: Zero through a register */
      for (int n008 = 0; n008 < fh; n008++) {   /* spatial_split rows */
      for (int n009 = 0; n009 < fw; n009++) {   /* spatial_split cols */
        for (int n010 = 0; n010 < c; n010++) {  /* MatmulAccum[1,1,C,1], split(1) */
          int32_t n011;
          n011 = n000[(((n003 * h + n004 + n008) * w + n005 + n009) * c + n010)];  /* Assign */
          int32_t n012;
          n012 = n001[(((n006 * fh + n008) * fw + n009) * c + n010)];  /* Assign */
          n007 += n011 * n012;  /* MultAdd */
        }
      }
      }
      n002[(((n003 * oh + n004) * ow + n005) * f + n006)] = n007;
    }
    }
  }
  }
}

void lowered_compose_msm(const uint16_t *restrict v, const uint16_t *restrict q,
                         const uint16_t *restrict kmat, float *restrict out, int b, int m,
                         int k, int n2, int n, int head_begin, int head_end, int threads) {
  (void)b;
  const int steps = head_end - head_begin;
#pragma omp parallel for num_threads(clamp_threads(threads, steps)) proc_bind(spread) schedule(static)
  for (int n003 = head_begin; n003 < head_end; n003++) {
    /* bufferize x2 (matmul_chain.rs:60-63): two GL intermediates per batch entry */
    float *n004, *n005;  /* posix_memalign(.., 128, ..) as c_utils.rs:77-93 */
    if (posix_memalign((void **)&n004, 128, sizeof(float) * (size_t)m * n2) != 0) abort();
    if (posix_memalign((void **)&n005, 128, sizeof(float) * (size_t)m * n2) != 0) abort();
    const uint16_t *qh = q + (size_t)n003 * m * k, *kh = kmat + (size_t)n003 * n2 * k;
    const uint16_t *vh = v + (size_t)n003 * n2 * n;
    float *oh = out + (size_t)n003 * m * n;
    /* stage 1: S = Q.KT, to_accum + split(1) + casts + MultAdd */
    for (int n006 = 0; n006 < m; n006++) {
    for (int n007 = 0; n007 < n2; n007++) {
      float n008;
      memset((void *)(&n008), 0, 4);
      for (int n009 = 0; n009 < k; n009++) {
        float n010;
        n010 = bf16_as_f32(qh[(k * n006 + n009)]);   /* CastBf16F32 */
        float n011;
        n011 = bf16_as_f32(kh[(k * n007 + n009)]);   /* CastBf16F32 (layout![0,2,1]) */
        n008 += n010 * n011;  /* MultAdd */
      }
      n004[(n2 * n006 + n007)] = n008;
    }
    }
    /* stage 2: Softmax rows: to_softmax_parts -> to_max_and_unscaled -> divide
     * (softmax2.rs:47-113) with the scalar value kernels */
    for (int n006 = 0; n006 < m; n006++) {
      float n012 = -INFINITY;  /* ValueNegInf */
      for (int n007 = 0; n007 < n2; n007++) {
        n012 = fmaxf(n012, n004[(n2 * n006 + n007)]);  /* ValueMax */
      }
      float n013;
      memset((void *)(&n013), 0, 4);  /* ValueZero */
      for (int n007 = 0; n007 < n2; n007++) {
        float n014 = expf(n004[(n2 * n006 + n007)] - n012);  /* ValueSoftmaxDenominatorAndUnscaledFromMax */
        n013 += n014;
        n005[(n2 * n006 + n007)] = n014;
      }
      for (int n007 = 0; n007 < n2; n007++) {
        n005[(n2 * n006 + n007)] /= n013;  /* ValueDivideVecScalar */
      }
    }
    /* stage 3: out = P.V, f32 x bf16 -> f32 */
    for (int n006 = 0; n006 < m; n006++) {
    for (int n015 = 0; n015 < n / 8; n015++) {
      vf8 n016 = {0};  /* VectorZero */
      for (int n007 = 0; n007 < n2; n007++) {
        float n017;
        n017 = n005[(n2 * n006 + n007)];
        float n018[8] __attribute__((aligned (128)));
        for (int n019 = 0; n019 < 8; n019++) {
          n018[(n019)] = bf16_as_f32(vh[(n * n007 + 8 * n015 + n019)]);  /* VectorCastBf16F32 */
        }
        n016 += n017 * (*(vf8 *)(&n018[0]));  /* BroadcastVecMultAdd */
      }
      memcpy(&oh[(n * n006 + 8 * n015)], &n016, 32);
    }
    }
    free(n004);
    free(n005);
  }
}
