/*
 * morello_amd: MI355X (gfx950) execution backend for Morello Specs -- C ABI.
 *
 * This header is the drop-in boundary.  Morello lowers a scheduled Spec to a C function
 *
 *     void kernel(const T0 *restrict p0, ..., Tk *restrict pk);
 *
 * with one pointer per Spec parameter in Spec parameter order
 * (morello/src/codegen/cpu.rs:131-219), compiles it (codegen/mod.rs:207-266) and runs it
 * through a generated `main` (codegen/cpu.rs:284-409).  The entry points below stand where
 * that emitted kernel and the build/run step stand: they take a plain-C description of the
 * Spec (type, shape, dtypes, per-parameter layout: morello/src/spec.rs:33-162,
 * common.rs:15-24, layout.rs:67-81) plus the parameter pointers in the same order, and run
 * hand-written HIP kernels instead of emitted C.
 *
 * Differences from the emitted kernel, all deliberate:
 *   - every call returns an int status instead of aborting (cpu.rs:1157, :1338);
 *   - shapes and layouts are run-time arguments, not constants baked into the body;
 *   - pointers are device (HBM) pointers for mrl_run / mrl_run_async, host pointers for
 *     mrl_run_host (which stages through device memory and is the literal stand-in for
 *     calling kernel(...) from the emitted main).
 * The caller owns every parameter buffer (cpu.rs:399-403); parameters must not alias
 * (the emitted signature is all-restrict); an accumulating Spec accumulates across calls
 * exactly as the reference's benchmark loop does (cpu.rs:541-550).
 *
 * No type from any framework appears here: plain pointers, sizes and small structs only.
 */
#ifndef MORELLO_AMD_H
#define MORELLO_AMD_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* ------------------------------------------------------------------ types */

/* morello/src/common.rs:15-24, same order. */
typedef enum {
  MRL_U8 = 0,
  MRL_I8 = 1,
  MRL_U16 = 2,
  MRL_I16 = 3,
  MRL_U32 = 4,
  MRL_I32 = 5,
  MRL_F32 = 6,
  MRL_BF16 = 7
} mrl_dtype;

/* morello/src/layout.rs:74-81 */
typedef enum { MRL_DYNAMIC = 0, MRL_PACKED = 1, MRL_ODDEVEN = 2 } mrl_physdim_kind;

#define MRL_MAX_PHYS 10
#define MRL_MAX_RANK 5
#define MRL_MAX_SPEC_RANK 7
#define MRL_MAX_PARAMS 4

typedef struct {
  uint8_t logical_dim;
  uint8_t kind; /* mrl_physdim_kind */
  uint32_t size; /* Packed / OddEven size; ignored for Dynamic */
} mrl_physdim;

/* Physical dims listed slowest to fastest (layout.rs:67-70).  ndims == 0 with
 * `row_major_default` semantics is requested by passing a NULL layout pointer where one is
 * accepted; inside mrl_spec every parameter carries an explicit layout. */
typedef struct {
  uint32_t ndims;
  mrl_physdim dims[MRL_MAX_PHYS];
} mrl_layout;

/* The Specs this backend executes (subset of PrimitiveSpecType, spec.rs:57-162, plus the
 * three-component Compose of examples/matmul_chain.rs). */
typedef enum {
  MRL_SPEC_MATMUL = 0,     /* spec_shape [b,m,k,n]; params A[b,m,k] B[b,k,n] C[b,m,n]   */
  MRL_SPEC_CONV = 1,       /* spec_shape [b,f,c,oh,ow,fh,fw]; params image, filters, out.
                              Both: any dtype triple; inputs are cast to the output dtype
                              (verification.rs:547-569, 629-631), integer outputs wrap, f32
                              outputs sum in f32.  bf16 outputs: PARITY UNPINNED -- the
                              products are summed in f32 and rounded once, and an accumulating
                              Spec adds the old output before that single rounding; the
                              reference's interpreter rounds to bf16 after every operation
                              and again after `o += intermed` (verification.rs:629-642), and
                              holds no comparison for bf16 (verification.rs:597 is todo!)    */
  MRL_SPEC_SOFTMAX = 2,    /* spec_shape = tensor shape; params in, out; uses scan_dim   */
  MRL_SPEC_COMPOSE_MSM = 3,/* Matmul->Softmax->Matmul; spec_shape [b,m,k,n2,n];
                              params V[b,n2,n] Q[b,m,k] KT[b,k,n2] out[b,m,n]
                              (Compose parameter order, spec.rs:3329-3365)               */
  MRL_SPEC_MOVE = 4,       /* Move (spec.rs:57-162; oracle verification.rs assign_cast):
                              spec_shape = tensor shape; params in, out; the two may
                              differ in layout and dtype (Rust `as` conversion)          */
  /* The primitives Softmax decomposes into (spec.rs:86-162).  spec_shape = the full tensor
   * shape (rank <= 5); "reduced" parameters have size one on scan_dim (spec.rs:524-583).
   * f32 only.  `accum` as in spec.rs:1214-1241: accumulating forms read their outputs. */
  MRL_SPEC_FILL = 5,       /* params out; scan_dim holds the mrl_fill_value; any dtype     */
  MRL_SPEC_MAX = 6,        /* params in, out(reduced): out = max(out?, in) over scan_dim  */
  MRL_SPEC_SOFTMAX_DENOMINATOR = 7,
                           /* params in, max(reduced), denom(reduced):
                              denom (+)= sum exp(in - max)                                */
  MRL_SPEC_SOFTMAX_DENOMINATOR_AND_MAX = 8,
                           /* params in, max(reduced), denom(reduced): online update of
                              (max, denom) (spec.rs:96-101; cpu.rs:1360-1389)             */
  MRL_SPEC_SOFTMAX_DENOMINATOR_AND_MAX_FROM_PARTS = 9,
                           /* params tile_max, tile_denom (full shape: one entry per tile
                              along scan_dim), out_max, out_denom (reduced): merges the
                              per-tile pairs (spec.rs:102-132; cpu.rs:1390-1413)          */
  MRL_SPEC_SOFTMAX_DENOMINATOR_AND_UNSCALED = 10,
                           /* params in, denom(reduced), unscaled: unscaled = exp(in-max),
                              denom = its sum; never accumulates (spec.rs:133-141)        */
  MRL_SPEC_SOFTMAX_DENOMINATOR_AND_UNSCALED_FROM_MAX = 11,
                           /* params in, max(reduced), denom(reduced), unscaled
                              (cpu.rs:1425-1433)                                          */
  MRL_SPEC_SOFTMAX_COMPLETE = 12,
                           /* params in, max(reduced), denom(reduced), out:
                              out = exp(in - max) / denom (cpu.rs:1350-1359)              */
  MRL_SPEC_DIVIDE_VEC = 13,/* params numer (InOut), denom, same shape: numer /= denom     */
  MRL_SPEC_DIVIDE_VEC_SCALAR = 14,
                           /* params numer (InOut), denom(reduced): numer /= denom        */
  MRL_SPEC_BROADCAST = 15, /* params in(size one on scan_dim), out: copies along scan_dim;
                              any dtype, both the same (spec.rs:70-75)                    */
  MRL_SPEC_ONE_PREFIX = 16 /* params in[shape], out[1, shape...]: a copy under a leading
                              unit dim (spec.rs:59, 469-479); rank <= 4; same dtype       */
} mrl_spec_kind;

/* spec.rs:165-170 */
typedef enum { MRL_FILL_ZERO = 0, MRL_FILL_NEG_INF = 1, MRL_FILL_MIN = 2 } mrl_fill_value;

typedef struct {
  int32_t kind;     /* mrl_spec_kind */
  int32_t accum;    /* 1 = accumulate into the output(s) (InOut), 0 = overwrite */
  uint32_t scan_dim; /* Softmax family, Max, DivideVecScalar, Broadcast: the dim; Fill: the value */
  uint32_t rank;    /* entries used in spec_shape */
  uint32_t spec_shape[MRL_MAX_SPEC_RANK];
  uint32_t n_params;
  int32_t dtypes[MRL_MAX_PARAMS]; /* mrl_dtype per parameter, Spec parameter order */
  mrl_layout layouts[MRL_MAX_PARAMS];
} mrl_spec;

/* Status codes (the emitted C aborts or asserts where these are returned). */
typedef enum {
  MRL_OK = 0,
  MRL_ERR_UNSUPPORTED = 1, /* Spec kind / dtype combination not implemented            */
  MRL_ERR_BAD_LAYOUT = 2,  /* layout does not apply to the parameter's shape            */
  MRL_ERR_BAD_SPEC = 3,    /* malformed descriptor: rank, zero dim, n_params, scan_dim  */
  MRL_ERR_HIP = 4,         /* a HIP runtime call failed; see mrl_last_error()           */
  MRL_ERR_NO_DEVICE = 5,   /* no gfx950 device visible                                  */
  MRL_ERR_NULL = 6,        /* NULL pointer argument                                     */
  MRL_ERR_TOO_LARGE = 7    /* a tensor exceeds the index range the kernels assume      */
} mrl_status;

/* ------------------------------------------------------------- life cycle */

/* Selects `device` and checks that it is a gfx950 part.  Idempotent.  (No counterpart in the
 * reference, whose target is the host CPU.) */
int mrl_init(int device);
const char *mrl_status_string(int status);
/* Text of the last HIP error seen by this thread ("" if none). */
const char *mrl_last_error(void);
/* "major.minor.patch" of this library. */
const char *mrl_version(void);
/* The layout of the structs of this header as the loaded library was built with them.  A binding
 * compares it with the MRL_ABI_VERSION it was written against before it passes a struct: the
 * number goes up whenever a struct gains or changes a field (2: mrl_matmul_schedule.staging,
 * mrl_action; 3: the Softmax actions).  Every struct is zero-initialised by the caller before
 * its fields are set: fields added later mean "default" when zero. */
#define MRL_ABI_VERSION 4u
uint32_t mrl_abi_version(void);

/* --------------------------------------------------- Spec surface (host) */

/* common.rs:30-36 */
size_t mrl_dtype_size(int dtype);
/* common.rs:52-65: "u8", "i8", ..., "f32", "bf16" */
const char *mrl_dtype_name(int dtype);

/* Layout constructors: layout.rs:1234-1247, :1249-1253, :1255-1271, :1273-1279. */
int mrl_layout_row_major(const uint32_t *shape, uint32_t rank, mrl_layout *out);
int mrl_layout_col_major(const uint32_t *shape, uint32_t rank, mrl_layout *out);
int mrl_layout_batched_col_major(const uint32_t *shape, uint32_t rank, mrl_layout *out);
int mrl_layout_nhwc(const uint32_t *shape, uint32_t rank, mrl_layout *out);
/* layout.rs:769-810 (expand_physical_shape). */
int mrl_layout_physical_shape(const mrl_layout *layout, const uint32_t *shape, uint32_t rank,
                              uint32_t *phys_shape);
/* layout.rs:221-272 (buffer_indexing_expr) evaluated at `point`; -1 on a bad layout. */
int64_t mrl_layout_buffer_index(const mrl_layout *layout, const uint32_t *shape, uint32_t rank,
                                const uint32_t *point);

/* spec.rs:467-583 (parameter_shape): logical shape of parameter `idx`. */
int mrl_spec_parameter_shape(const mrl_spec *spec, uint32_t idx, uint32_t *shape,
                             uint32_t *rank);
/* spec.rs:1204-1245: 0 = In, 1 = Out, 2 = InOut; negative on error. */
int mrl_spec_parameter_direction(const mrl_spec *spec, uint32_t idx);
/* tensorspec.rs:153-160 (bytes_used) of parameter `idx`; 0 on error. */
size_t mrl_spec_parameter_bytes(const mrl_spec *spec, uint32_t idx);
/* spec.rs:273-305 convention extended to every dtype: Matmul/Conv 2*MACs, Softmax 5/elem,
 * Compose = sum of its components. */
uint64_t mrl_spec_ops(const mrl_spec *spec);
/* MRL_OK if mrl_run would accept the Spec (validates shapes, dtypes, layouts). */
int mrl_spec_check(const mrl_spec *spec);
/* Bytes of device scratch mrl_run takes for staging this Spec's parameters out of layouts the
 * kernels do not walk in place (Packed / OddEven dims in another order than row-major); 0 when
 * every parameter is read in place.  A lower bound on the call's scratch: operand copies made
 * for speed (zero-padded rows, column-major operands made row-major, unfolded Conv windows, up
 * to 1 GiB), the f32 image of a bf16 Matmul/Conv output with the bf16 copies of its inputs, and
 * the intermediates of a Compose come from the same allocator on top of it. */
size_t mrl_spec_workspace_bytes(const mrl_spec *spec);

/* -------------------------------------------------------------- execution */

/* Stands where the emitted `kernel(p0, ..., pk)` stands (codegen/cpu.rs:131-219,
 * call site :497-514).  `params` holds n_params DEVICE pointers in Spec parameter order,
 * each to bytes_used(parameter) bytes laid out by that parameter's layout.  Synchronous:
 * returns after the work has finished. */
int mrl_run(const mrl_spec *spec, void *const *params);

/* As mrl_run but only enqueues on `stream` (a hipStream_t, NULL = default stream).  Scratch
 * memory (relayout staging, padded operands, a Compose's intermediates) comes from an arena
 * the library keeps per stream it has seen: 64 MiB at first; a call that needs more takes the
 * excess from the stream-ordered allocator and, before it returns, waits for the stream once and
 * replaces the arena by one that holds the whole call (up to 16 GiB), so that its next run
 * allocates nothing.  mrl_spec_plan tells the amount (scratch_bytes).  Calls from several host
 * threads onto one stream take turns for the arena.  That one wait and reallocation cannot
 * happen under stream capture: a capturing caller uses mrl_run_noalloc or runs the Spec once
 * beforehand.  mrl_stream_destroy releases the arena of its stream; for a stream the caller
 * created itself, mrl_stream_release does, and without it that arena stays until the process
 * ends. */
int mrl_run_async(const mrl_spec *spec, void *const *params, void *stream);

/* As mrl_run_async, for callers that cannot allocate device memory (code under HIP graph capture,
 * tight serving loops, harnesses that forbid it).  No counterpart in the reference, whose emitted
 * programs allocate their buffers up front.  Calls no hipMalloc / hipFree / stream-ordered
 * allocator: scratch comes out of one fixed array of MRL_NOALLOC_SCRATCH_BYTES per GPU, which the
 * library's code object brings along (each GPU the library runs on holds it until the process
 * ends).  mrl_init must have been called for the device (it looks the array up) and that device
 * must be the calling thread's current one (MRL_ERR_NO_DEVICE otherwise).  Parameters are 256-byte
 * aligned, as device allocations are (MRL_ERR_UNSUPPORTED otherwise: the scratch need of a
 * misaligned call is not the plan's).  A Spec whose scratch need (mrl_spec_plan: scratch_bytes)
 * exceeds the array is turned down with MRL_ERR_TOO_LARGE before anything is launched.  All calls
 * on one GPU share the array: two that
 * overlap in time (different streams, or different host threads on one stream) race; the caller
 * serialises them. */
#define MRL_NOALLOC_SCRATCH_BYTES (32u << 20)
int mrl_run_noalloc(const mrl_spec *spec, void *const *params, void *stream);

/* Literal stand-in for calling the emitted kernel from the emitted main
 * (codegen/cpu.rs:284-409): `params` are HOST pointers; inputs (and the output, when it
 * is read) are copied to the device, the Spec is run, written parameters are copied back. */
int mrl_run_host(const mrl_spec *spec, void *const *params);

/* Per-kind conveniences that build the descriptor themselves.  NULL layouts mean
 * row-major, except Conv where NULL means NHWC image/output and KRSC filters
 * (layout![0,2,3,1] on [n,c,h,w] and [f,c,fh,fw]; layout.rs:1273-1279). */
int mrl_matmul(uint32_t b, uint32_t m, uint32_t k, uint32_t n, int dt_a, int dt_b, int dt_c,
               int accum, const void *a, const void *bmat, void *c, void *stream);
int mrl_conv(uint32_t b, uint32_t f, uint32_t c, uint32_t oh, uint32_t ow, uint32_t fh,
             uint32_t fw, int dt_img, int dt_filt, int dt_out, int accum, const void *image,
             const void *filters, void *out, void *stream);
int mrl_softmax(const uint32_t *shape, uint32_t rank, uint32_t scan_dim, const void *in,
                void *out, void *stream);
/* Move (spec.rs:63, scheduling/moves.rs:16-22): copies `in` to `out` (dense row-major both
 * sides, same dtype). */
int mrl_move(const uint32_t *shape, uint32_t rank, int dtype, const void *in, void *out,
             void *stream);
/* KT is the B operand of the first Matmul, logical [b,k,n2]; kt_col_major != 0 says it is
 * stored with layout![0,2,1] (i.e. K stored row-major as [b,n2,k]). */
int mrl_compose_msm(uint32_t b, uint32_t m, uint32_t k, uint32_t n2, uint32_t n, int dt_v,
                    int dt_q, int dt_kt, int kt_col_major, const void *v, const void *q,
                    const void *kt, void *out, void *stream);

/* ------------------------------------------------ schedule-driven execution */

/* A Morello manual schedule for a Matmul Spec, reduced to the two steps that have a knob in
 * the GPU kernel: `tile_out([1, tile_m, tile_n])` (one workgroup per output tile) followed
 * by `split(split_k)` (elements of K per step of the k loop)
 * (morello/src/scheduling_sugar.rs:37-132; worked schedules in
 * morello/examples/simple_matmul_x86.rs:60-100, matmul_x86.rs:27-70), and `staging`: the
 * counterpart of the schedule's move_param steps (which operand is staged in which memory
 * level, how many buffers deep).  Every tile exists with both operands moved HBM -> VGPR -> LDS
 * -> VGPR through two LDS stages; the 256 x 256 tile with a 128-byte k step also with B moved
 * HBM -> LDS directly (three slots, no staging registers) and A through registers, on eight
 * waves of 128 x 64 outputs or on four waves of 128 x 128, one per SIMD. */
typedef enum {
  MRL_STAGING_DEFAULT = 0,        /* what the dispatch rules pick for the tile and shape           */
  MRL_STAGING_REGISTERS = 1,      /* A, B: HBM -> VGPR -> LDS (2 stages); eight waves (k_gemm)      */
  MRL_STAGING_DIRECT_B = 2,       /* B: HBM -> LDS (3 slots); eight waves of 128 x 64 (k_gemm_big)  */
  MRL_STAGING_DIRECT_B_WIDE = 3   /* B: HBM -> LDS (3 slots); four waves of 128 x 128 (k_gemm_wide) */
} mrl_staging;
/* Zero-initialise before setting fields (staging was added after the first three). */
typedef struct {
  uint32_t tile_m, tile_n; /* tile_out */
  uint32_t split_k;        /* split, in elements of K */
  uint32_t staging;        /* mrl_staging: the move_param steps */
} mrl_matmul_schedule;

/* Lists the schedules the matrix-core Matmul kernel is built for, for this Spec's dtypes
 * (u8|i8 x i8 -> i32, bf16 x bf16 -> f32, f32 x f32 -> f32).  Writes up to `cap` entries, returns how many
 * exist (0 if the Spec has no matrix-core kernel). */
uint32_t mrl_matmul_schedules(const mrl_spec *spec, mrl_matmul_schedule *out, uint32_t cap);

/* mrl_run_async under a caller-chosen schedule.  MRL_ERR_UNSUPPORTED if the schedule is not
 * in mrl_matmul_schedules() or the operands do not meet the kernel's alignment rules; the
 * result is identical to mrl_run's whatever the schedule (integer Specs bit for bit). */
int mrl_run_matmul_scheduled(const mrl_spec *spec, void *const *params,
                             const mrl_matmul_schedule *schedule, void *stream);

/* ------------------------------------------------ benchmark protocol (L5) */

/* Mirrors CodeGen::bench / the emitted benchmarking main (codegen/cpu.rs:516-568,
 * codegen/mod.rs:133-169,330-340): one warm-up launch, then `iters` back-to-back launches
 * between two HIP events on `stream`'s queue, repeated `repeats` times.  Writes the best
 * and the mean per-launch time in nanoseconds.  Accumulating Specs keep accumulating. */
int mrl_bench(const mrl_spec *spec, void *const *params, uint32_t iters, uint32_t repeats,
              double *best_ns_per_iter, double *mean_ns_per_iter);

/* Enqueues `steps` launches of the Spec back to back on the default stream, bracketed by
 * two HIP events recorded on that same stream, waits, and writes the elapsed device time
 * for all of them in milliseconds.  The timed region of the benchmark's inner loop
 * (codegen/cpu.rs:541-550) measured on the device's clock. */
int mrl_run_timed(const mrl_spec *spec, void *const *params, uint32_t steps,
                  double *device_ms_total);

/* ------------------------------------------------ general Compose Specs */

/* LogicalSpec::Compose (spec.rs:39-45, 1519-1590): a pipeline of primitive Specs listed
 * last-executed first, each consuming the output of the one listed after it as its first
 * input.  A component is a PrimitiveBasics (spec.rs:47-55): type, spec_shape, dtypes. */
#define MRL_MAX_COMPONENTS 8
#define MRL_MAX_COMPOSE_PARAMS 12

typedef struct {
  int32_t kind;      /* mrl_spec_kind with exactly one written parameter; not a Compose   */
  int32_t accum;     /* 1 only on components[0], the head: the Compose then accumulates
                        into its output (spec.rs:3829-3838); elsewhere it must be 0, a
                        side-effecting tail component is rejected (spec.rs:1760-1764)     */
  uint32_t scan_dim;
  uint32_t rank;
  uint32_t spec_shape[MRL_MAX_SPEC_RANK];
  uint32_t n_params;
  int32_t dtypes[MRL_MAX_PARAMS];
} mrl_component;

typedef struct {
  uint32_t n_components;
  mrl_component components[MRL_MAX_COMPONENTS];
  /* External parameters in the order of compose_parameter_visit (spec.rs:3329-3365): the
   * first-listed component's inputs after its first, the middle components' likewise, all
   * inputs of the last-listed component, then the first-listed component's output. */
  uint32_t n_params;                          /* set by mrl_compose_init */
  mrl_layout layouts[MRL_MAX_COMPOSE_PARAMS]; /* row-major after mrl_compose_init */
  /* The schedule knob of scheduling/bufferize.rs:24-116: bit i set = the tensor feeding
   * component i (the output of component i+1) is materialised in device memory, row-major,
   * as `bufferize(i, GL, row_major)` would.  Zero (what mrl_compose_init leaves) lets the
   * library fuse across every boundary it has a kernel for; any set bit runs the pipeline
   * component by component. */
  uint32_t bufferize_mask;
} mrl_compose;

/* Validates the chain (every component's first input has the shape and dtype of the next
 * component's output), counts the external parameters and gives each a row-major layout;
 * the caller may then replace layouts. */
int mrl_compose_init(mrl_compose *c);
/* Which (component, component parameter) external parameter `idx` is. */
int mrl_compose_parameter(const mrl_compose *c, uint32_t idx, uint32_t *component, uint32_t *param);
int mrl_compose_parameter_shape(const mrl_compose *c, uint32_t idx, uint32_t *shape, uint32_t *rank);
int mrl_compose_parameter_dtype(const mrl_compose *c, uint32_t idx);
/* Runs the pipeline on device pointers in external parameter order.  The attention-shaped
 * [Matmul, Softmax{2}, Matmul] runs on the fused kernel when its conditions hold; any other
 * chain runs component by component with row-major intermediates of each component's
 * output dtype in a stream-ordered scratch allocation (the reference's interpreter also
 * materialises them: verification.rs:239-285, 286-335). */
int mrl_run_compose(const mrl_compose *c, void *const *params, void *stream);

/* No counterpart in the reference.  Measures what the matrix cores of this board sustain
 * with every SIMD issuing back-to-back MFMAs on register operands and no memory traffic:
 * kind 0 = int8 (u8/i8 -> i32), 1 = bf16 (-> f32); random_operands 0 = all-zero operands (the
 * datapath barely toggles: close to the datasheet rate), 1 = operands distributed like a
 * benchmark's (the clock settles at the power limit: the ceiling a Matmul kernel can
 * approach on such data).  `iters` x 64 MFMAs of 16 x 16 x 64 bytes per wavefront (20000 runs about 20 ms).
 * Writes operations per second (2 per multiply-add). */
int mrl_measure_mfma_rate(int kind, int random_operands, uint32_t iters, double *ops_per_second);

/* ------------------------------------------- device memory (plumbing only) */

/* What the emitted main does around the kernel call on the host: 128-byte aligned buffers per
 * parameter (codegen/c_utils.rs:77-93, codegen/cpu.rs:38), filled from the parameter files
 * (cpu.rs:221-270) or with zeros (cpu.rs:320), freed after the call (cpu.rs:399-403).  Device
 * allocations are aligned to 256 bytes or more. */
int mrl_device_malloc(void **ptr, size_t bytes);
int mrl_device_free(void *ptr);
int mrl_memcpy_h2d(void *dst, const void *src, size_t bytes);
int mrl_memcpy_d2h(void *dst, const void *src, size_t bytes);
int mrl_memset(void *dst, int value, size_t bytes);
int mrl_device_synchronize(void);
/* Device memory not allocated at the moment, in bytes (hipMemGetInfo): what a caller sizing
 * its buffers against the arenas the library keeps per stream wants to know. */
int mrl_device_mem_free(size_t *free_bytes);
/* HIP streams (default priority) for callers that have no HIP binding of their own: the
 * handle is what mrl_run_async, mrl_run_compose and the per-kind conveniences take.
 * mrl_stream_destroy waits for the stream's work, then frees the stream and its scratch arena.
 * mrl_stream_release waits for the work of a stream the CALLER owns (any hipStream_t that was
 * passed to mrl_run_async, NULL included) and frees only the arena the library kept for it:
 * call it before hipStreamDestroy, or to give the memory back; the stream stays usable and its
 * next call starts a new arena. */
int mrl_stream_create(void **stream);
int mrl_stream_synchronize(void *stream);
int mrl_stream_release(void *stream);
int mrl_stream_destroy(void *stream);
/* Name, CU count, clock (kHz) and memory size of the selected device. */
int mrl_device_info(char *name, size_t name_len, int *compute_units, int *clock_khz,
                    size_t *total_mem_bytes);

/* ---- The backend as a search target -------------------------------------------------------
 * What morello's `Target` / `Memory` / `Kernel` traits ask of a backend
 * (morello/src/target/mod.rs:37-117), as data a Rust `impl Target for Gfx950Target` would
 * forward.  All of it is host code: none of these calls needs a GPU. */

/* Target::target_id (target/mod.rs:74): "Gfx950". */
const char *mrl_target_id(void);
/* Target::line_size (target/mod.rs:50): bytes of one L2 cache line. */
uint32_t mrl_target_line_size(void);
/* Target::processors (target/mod.rs:53): compute units (the reference's u8 cannot hold 256). */
uint32_t mrl_target_processors(void);

/* One level of Target::memories (target/mod.rs:55), fastest first, with the `Memory` trait's
 * answers (target/mod.rs:80-95), Target::max_mem's limit for it (target/mod.rs:52; per
 * processor for registers and LDS) and Target::cache_hit_cost (target/mod.rs:51). */
typedef struct {
  char name[8];               /* "ACC", "VGPR", "LDS", "HBM" */
  uint8_t is_addressed;       /* Memory::is_addressed */
  uint8_t can_parallel_tile;  /* Memory::can_parallel_tile */
  uint8_t counts_registers;   /* Memory::counts_registers: the limit counts registers, not bytes */
  uint8_t has_layout;         /* Memory::has_layout */
  uint32_t vector_bytes[4];   /* Memory::vector_bytes, 0-terminated */
  uint64_t limit;             /* Target::max_mem: registers per lane, or bytes */
  uint32_t cache_hit_cost;    /* Target::cache_hit_cost */
} mrl_target_memory;
/* Writes up to `cap` levels; returns how many there are (4, the reference's MEMORY_COUNT). */
uint32_t mrl_target_memories(mrl_target_memory *out, uint32_t cap);

/* Target::default_memory (target/mod.rs:54): index into mrl_target_memories of the level Spec
 * parameters live in (HBM). */
uint32_t mrl_target_default_memory(void);
/* Target::possible_destination_memories (target/mod.rs:56): where a Move out of level `slower`
 * may land, itself first; returns the count. */
uint32_t mrl_target_destination_memories(uint32_t slower, uint32_t *out, uint32_t cap);
/* Target::all_layouts_for_shape / move_destination_layouts (target/mod.rs:58-67), built as the
 * reference's CPU targets build theirs (target/cpu.rs:317-398): row-major, plus column-major
 * (rank 2), k-fastest `layout![0,2,1]` (rank 3; read in place by the Matmul and Compose kernels)
 * or NHWC (rank 4); each of those with one more Packed(n) dim for n = 2 and the register file's
 * vector widths in elements, and with one more OddEven(n) dim for twice those widths, wherever
 * the result applies to `shape`.  Writes up to `cap` layouts, returns how many there are. */
uint32_t mrl_target_layouts_for_shape(const uint32_t *shape, uint32_t rank, int dtype, mrl_layout *out, uint32_t cap);
/* Kernel::name of every kernel family of the backend (target/mod.rs:111); returns the count. */
uint32_t mrl_target_kernels(const char **names, uint32_t cap);

/* One kernel launch a Spec would make. */
typedef struct {
  char kernel[160];    /* the kernel and the template arguments it was built with,
                          "k_attn [D = 128, RAGGED = false, KT_ROWS = false]" */
  uint32_t grid[3], block[3];
  uint32_t lds_bytes;  /* dynamic LDS per workgroup: Kernel::memory_allocated's LDS figure */
  int32_t unit;        /* what bounds it besides traffic: 0 HBM stream, 1 int8 MFMA, 2 bf16 MFMA,
                          3 f32 MFMA, 4 vector ALU */
  double ops, bytes;   /* arithmetic (2 per multiply-add) and HBM traffic the kernel is charged */
  double cost_ns;      /* predicted duration, launch gap included */
} mrl_plan_step;
typedef struct {
  uint32_t n_steps;        /* launches the Spec makes (may exceed the `cap` that was passed) */
  uint64_t scratch_bytes;  /* device scratch the call takes: Kernel::memory_allocated's HBM figure */
  double cost_ns;          /* sum over the steps: Kernel::main_cost (target/mod.rs:109), in ns */
} mrl_plan;
/* Which kernels mrl_run would launch for `spec` with 256-byte-aligned parameters (what
 * mrl_device_alloc and hipMalloc return; a parameter aligned below 16 bytes makes a run take the
 * element-wise paths instead of the 16-byte ones listed here), and the cost
 * model's prediction for them (Kernel::applies_to_logical_spec + main_cost + memory_allocated,
 * target/mod.rs:103-109; Cost, cost.rs:13-17).  The plan is produced by the same dispatch code
 * that runs a Spec, with launches recorded instead of made, so it cannot disagree with a run.
 * MRL_ERR_UNSUPPORTED / MRL_ERR_BAD_SPEC as mrl_run. */
int mrl_spec_plan(const mrl_spec *spec, mrl_plan *plan, mrl_plan_step *steps, uint32_t cap);
/* Kernels the calling thread has launched through this library so far: after a run of a Spec the
 * count has grown by that Spec's plan.n_steps (tests hold the two against each other). */
uint64_t mrl_launch_count(void);
/* The same for a Matmul under a manual schedule (mrl_run_matmul_scheduled): what a search over
 * tile_out / split (scheduling_sugar.rs:37-132) compares. */
int mrl_matmul_scheduled_plan(const mrl_spec *spec, const mrl_matmul_schedule *schedule, mrl_plan *plan,
                              mrl_plan_step *steps, uint32_t cap);
/* The smallest search there is: the manual schedule of lowest predicted cost among those the
 * kernel is built for (what morello's top-down search does over its actions, search.rs, with
 * this backend's cost model in place of cost.rs).  MRL_ERR_UNSUPPORTED when none applies. */
int mrl_matmul_search_schedule(const mrl_spec *spec, mrl_matmul_schedule *best, double *cost_ns);
/* The same for a general Compose. */
int mrl_compose_plan(const mrl_compose *c, mrl_plan *plan, mrl_plan_step *steps, uint32_t cap);

/* Target::actions (target/mod.rs:69): the lowerings of a Spec this backend can run, each with what
 * Kernel::main_cost and Kernel::memory_allocated would say of it, for a search to choose among.
 * A CPU action rewrites one step of a schedule; the lowerings here are whole paths to a kernel, so
 * an action names the scheduling steps it stands for (scheduling_sugar.rs:37-132):
 *   SELECT          the dispatch rules' own choice for the Spec as it stands (Action::Select)
 *   TILE_OUT_SPLIT  Matmul: tile_out([1, tile_m, tile_n]).split(split_k), then the matrix-core kernel
 *   FUSED           Conv: the fused NHWC/KRSC kernel, a wave per 16-pixel tile (`tile_m` = 0) or, with
 *                   `tile_m` = the output width, tile_out over whole output rows: a workgroup's waves
 *                   share the rows' pixels through LDS and take 16 filters each (64 channels);
 *                   Compose Matmul->Softmax->Matmul: the fused kernel
 *                   with tile_out over the rows (`tile_m` = 128 or 64 queries per workgroup, 0 = the
 *                   dispatch rules' choice) and the keys in `parts` shares (parallel_softmax.rs:31-223;
 *                   1 = one workgroup per query block, more = partial results merged with the parts formula)
 *   SPATIAL_SPLIT   Conv as a Matmul over its windows read in place (spatial_split.rs:73-118),
 *                   tile_out([tile_m, tile_n]) on that Matmul
 *   UNFOLD          Conv: the windows materialised (a Move), then the Matmul
 *   BUFFERIZE       Compose: both intermediates materialised (bufferize.rs:24-116), a kernel per stage
 *   GENERIC         Conv on the any-dtype kernel
 *   TO_SOFTMAX_PARTS            Softmax (f32): SoftmaxDenominatorAndUnscaled into the output, then
 *                               DivideVecScalar (scheduling/to_softmax_parts.rs:33-108)
 *   TO_SOFTMAX_PARTS_RECOMPUTE  Softmax: SoftmaxDenominatorAndMax, then SoftmaxComplete
 *                               (to_softmax_parts.rs:110-181)
 *   PARALLEL_SOFTMAX            the same with the first stage split along the scan dim in `parts`
 *                               equal tiles (row-major input), a (max, denominator) pair per tile,
 *                               merged by SoftmaxDenominatorAndMaxFromParts
 *                               (scheduling/parallel_softmax.rs:24-223)
 *   TO_ACCUM        Matmul / Conv that overwrites: Fill{Zero} on the output, then the accumulating
 *                   Spec (scheduling/to_accum.rs:12-60)
 *   MOVE_RELAYOUT   parameter `tile_m` (not row-major) through a row-major copy: a Move before the
 *                   Spec when the parameter is read, the Spec on the copy, a Move back when it is
 *                   written (scheduling/moves.rs:16-130 with the source's dtype;
 *                   scheduling_sugar.rs move_relayout)
 *   CAST            input `tile_m` of a Matmul / Conv converted to dtype `tile_n` = the output's
 *                   (the conversion the Spec's own semantics apply to every input,
 *                   verification.rs:629-631, so the result is the same), in its own layout: a Move
 *                   with that dtype pair, then the Spec on the copy (moves.rs:16-130 with another
 *                   dtype; scheduling_sugar.rs cast)
 *   TO_MAX_AND_DENOMINATOR  SoftmaxDenominatorAndMax that overwrites: Max, then SoftmaxDenominator,
 *                   on the Spec's own parameters (scheduling/to_max_and_denom.rs:13-72)
 *   TO_MAX_AND_UNSCALED     SoftmaxDenominatorAndUnscaled: Max into a buffer, then
 *                   SoftmaxDenominatorAndUnscaledFromMax (scheduling/to_max_and_unscaled.rs:30-110)
 *   BROADCAST_FIRST DivideVecScalar: Broadcast of the denominators to the full shape, then
 *                   DivideVec (scheduling/broadcast_first.rs:24-130)
 * Every action runs the Spec to its result (mrl_run_action).  The reference's actions return a
 * partial Impl whose nested sub-Specs a search expands further: the three Softmax rewrites,
 * BUFFERIZE, TO_ACCUM, MOVE_RELAYOUT, CAST and the three of the Softmax primitives (TO_MAX_AND_*,
 * BROADCAST_FIRST) are such rewrites here too, and mrl_action_apply
 * (below) lists their sub-Specs; every other action is a leaf, a terminal lowering by the library
 * with a price.  There is no action for a partly tiled Conv or Softmax as steps of their own. */
typedef enum {
  MRL_ACTION_SELECT = 0,
  MRL_ACTION_TILE_OUT_SPLIT = 1,
  MRL_ACTION_FUSED = 2,
  MRL_ACTION_SPATIAL_SPLIT = 3,
  MRL_ACTION_UNFOLD = 4,
  MRL_ACTION_BUFFERIZE = 5,
  MRL_ACTION_GENERIC = 6,
  MRL_ACTION_TO_SOFTMAX_PARTS = 7,
  MRL_ACTION_TO_SOFTMAX_PARTS_RECOMPUTE = 8,
  MRL_ACTION_PARALLEL_SOFTMAX = 9,
  MRL_ACTION_TO_ACCUM = 10,
  MRL_ACTION_MOVE_RELAYOUT = 11,
  MRL_ACTION_CAST = 12,
  MRL_ACTION_TO_MAX_AND_DENOMINATOR = 13,
  MRL_ACTION_TO_MAX_AND_UNSCALED = 14,
  MRL_ACTION_BROADCAST_FIRST = 15
} mrl_action_kind;
typedef struct {
  int32_t kind;             /* mrl_action_kind */
  uint32_t tile_m, tile_n;  /* TILE_OUT_SPLIT, SPATIAL_SPLIT; FUSED on a Compose: tile_m = queries per workgroup;
                               FUSED on a Conv: tile_m = 0 or the output width (whole rows per workgroup);
                               MOVE_RELAYOUT, CAST: tile_m = index of the parameter moved; CAST: tile_n = mrl_dtype */
  uint32_t split_k;         /* TILE_OUT_SPLIT: elements of K per step */
  uint32_t parts;           /* FUSED on a Compose: shares of the keys; PARALLEL_SOFTMAX: tiles along the scan dim */
  uint32_t staging;         /* TILE_OUT_SPLIT: mrl_staging */
  uint32_t n_steps;         /* filled by mrl_target_actions: launches, */
  uint64_t scratch_bytes;   /*   device scratch (Kernel::memory_allocated) */
  double cost_ns;           /*   and predicted time (Kernel::main_cost) of the action */
} mrl_action;
/* Writes up to `cap` actions that apply to `spec` (those whose plan succeeds), priced; returns how
 * many there are.  Host code: needs no GPU. */
uint32_t mrl_target_actions(const mrl_spec *spec, mrl_action *out, uint32_t cap);
/* The plan of one action (its kernels, step by step). */
int mrl_action_plan(const mrl_spec *spec, const mrl_action *action, mrl_plan *plan, mrl_plan_step *steps, uint32_t cap);
/* mrl_run_async under the chosen action.  MRL_ERR_UNSUPPORTED if it does not apply to the Spec or
 * to these operands (alignment); the result is the Spec's whatever the action: integer Specs bit
 * for bit, floating-point ones within the Spec's tolerance. */
int mrl_run_action(const mrl_spec *spec, void *const *params, const mrl_action *action, void *stream);
/* The children of an action in Morello's sense.  ActionT::apply (scheduling/mod.rs:40-63) turns a
 * Spec into a partial Impl whose leaves are sub-Specs that the search schedules in turn; for the
 * actions here that are such rewrites, mrl_action_apply lists those sub-Specs in execution order
 * with where each of their parameters comes from, and the buffers between them:
 *   TO_SOFTMAX_PARTS            SoftmaxDenominatorAndUnscaled, DivideVecScalar
 *                               (scheduling/to_softmax_parts.rs:33-108)
 *   TO_SOFTMAX_PARTS_RECOMPUTE  SoftmaxDenominatorAndMax, SoftmaxComplete (to_softmax_parts.rs:110-181)
 *   PARALLEL_SOFTMAX            SoftmaxDenominatorAndMax over [.., parts, scan / parts, ..],
 *                               SoftmaxDenominatorAndMaxFromParts, SoftmaxComplete
 *                               (scheduling/parallel_softmax.rs:24-223)
 *   BUFFERIZE (on the Compose)  Matmul, Softmax, Matmul with the two tensors between them in
 *                               buffers of the components' output dtype (scheduling/bufferize.rs:24-116)
 *   TO_ACCUM                    Fill{Zero} of the output, the accumulating Spec
 *   MOVE_RELAYOUT, CAST         [Move into the copy,] the Spec on the copy [, Move back]
 *   TO_MAX_AND_DENOMINATOR      Max, SoftmaxDenominator
 *   TO_MAX_AND_UNSCALED         Max, SoftmaxDenominatorAndUnscaledFromMax
 *   BROADCAST_FIRST             Broadcast, DivideVec
 * Every other action is a leaf (n_subspecs = 0): the library runs it as one piece.  Running the
 * sub-Specs one after the other with mrl_run, each on the buffers its sources name, computes the
 * Spec; each sub-Spec has actions of its own (mrl_target_actions), which is how a search over this
 * backend recurses.  Host code: needs no GPU. */
#define MRL_MAX_SUBSPECS 4
typedef struct {
  mrl_spec spec;
  /* Per parameter of `spec`: i >= 0 = parameter i of the Spec the action was applied to;
   * -1 - j = intermediate buffer j of the rewrite. */
  int32_t source[MRL_MAX_PARAMS];
} mrl_subspec;
typedef struct {
  uint32_t n_subspecs;
  mrl_subspec subspecs[MRL_MAX_SUBSPECS];
  uint32_t n_intermediates;
  uint64_t intermediate_bytes[MRL_MAX_SUBSPECS]; /* dense tensors in the layout their sub-Specs name */
} mrl_rewrite;
int mrl_action_apply(const mrl_spec *spec, const mrl_action *action, mrl_rewrite *out);
/* mrl_run_timed for a chosen action: `steps` launches back to back on the default stream between
 * two events (what BuiltArtifact::measure_time does for one schedule, codegen/mod.rs:330-340). */
int mrl_run_action_timed(const mrl_spec *spec, void *const *params, const mrl_action *action, uint32_t steps,
                         double *device_ms_total);

#ifdef __cplusplus
}
#endif
#endif
