/*
 * Hand-restated "Morello-lowered" C: what Morello's C emitter (morello/src/codegen/cpu.rs)
 * prints for a stated manual schedule of each benchmark Spec, written by hand because the
 * Rust toolchain that would generate it is not available.  TEST INFRASTRUCTURE ONLY: these
 * are the CPU baseline that is timed beside the GPU kernels and a second, independently
 * structured implementation the oracle is compared with.  Shapes are run-time arguments
 * here (the emitter bakes them in as constants); loop structure, staging buffers, widening
 * assignments and leaf statements follow the emitter's rules:
 *   - one `for` per tiled axis (cpu.rs:3251-3376), parallel outer tiles carry the OpenMP
 *     pragma of cpu.rs:3283-3289;
 *   - a Move into RF/VRF becomes a local scalar / vector variable loaded before and stored
 *     after the body (moves.rs:487-511, cpu.rs:1076-1135);
 *   - dtype casts are widening Assigns (target/cpu.rs:2860-2872, cpu.rs:2125-2169,
 *     CastBf16F32 cpu.rs:2170-2188);
 *   - leaves: MultAdd `c += a * b` (cpu.rs:2114-2124), BroadcastVecMultAdd
 *     `out_vec += scalar * vec` (cpu.rs:2254-2296), the softmax value kernels
 *     (cpu.rs:1350-1433) and DivideVecScalar (cpu.rs:3103-3227).
 * Built with the reference's flags (codegen/mod.rs:37-48) plus -fopenmp.
 */
#ifndef MORELLO_LOWERED_H
#define MORELLO_LOWERED_H
#include <stdint.h>

/* C1: f32 Matmul, schedule of examples/simple_matmul_x86.rs:60-100 (tile_out 16x16,
 * tile_out 1x1, to_accum, split 4, RF moves, MultAdd); m, n multiples of 16, k of 4. */
void lowered_matmul_f32(const float *a, const float *b, float *c, int m, int k, int n);

/* C2: u8 x i8 -> i32 MatmulAccum rows [row_begin,row_end): tile_out_parallel(1 x 16) ->
 * move_param(2, VRF) -> split(1) -> cast(0, i32, RF), cast(1, i32, VRF) ->
 * BroadcastVecMultAdd.  n multiple of 16.  threads <= 0 means all cores. */
void lowered_matmul_u8i8i32(const uint8_t *a, const int8_t *b, int32_t *c, int m, int k, int n,
                            int row_begin, int row_end, int threads);

/* C3: bf16 x bf16 -> f32 MatmulAccum, same schedule with CastBf16F32 moves. */
void lowered_matmul_bf16f32(const uint16_t *a, const uint16_t *b, float *c, int m, int k, int n,
                            int row_begin, int row_end, int threads);

/* C4: Conv NHWC/KRSC u8 x i8 -> i32 for images [img_begin,img_end): to_accum -> loops over
 * batch / output pixel -> spatial_split -> per (r,s) MatmulAccum[1,1,C,F] -> widening
 * casts -> MultAdd.  (The reference cannot emit this Spec: views.rs:888-899.) */
void lowered_conv_u8i8i32(const uint8_t *img, const int8_t *filt, int32_t *out, int b, int f,
                          int c, int oh, int ow, int fh, int fw, int img_begin, int img_end,
                          int threads);

/* C5: Matmul -> Softmax -> Matmul for heads [head_begin,head_end), staged through two
 * full f32 intermediates as examples/matmul_chain.rs:60-81 does.  kt is K stored
 * row-major [b, n2, k].  scratch holds 2*m*n2 floats per thread. */
void lowered_compose_msm(const uint16_t *v, const uint16_t *q, const uint16_t *kmat, float *out,
                         int b, int m, int k, int n2, int n, int head_begin, int head_end,
                         int threads);

int lowered_num_procs(void);
#endif
