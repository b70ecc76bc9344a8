// Matmul on the gfx950 matrix cores: u8|i8 x i8 -> i32 (v_mfma_i32_32x32x32_i8),
// bf16 x bf16 -> f32 (v_mfma_f32_32x32x16_bf16) and f32 x f32 -> f32
// (v_mfma_f32_32x32x2_f32), one tile pipeline for all three.
//
// What it computes is Morello's MatmulAccum on row-major operands
// (morello/src/spec.rs:480-485): C[i,j] (=0 unless accum) += sum_k A[i,k]*B[k,j].  The
// integer form matches the emitted C bit for bit (widening Assign, morello/src/target/
// cpu.rs:2860-2872, then MultAdd, morello/src/codegen/cpu.rs:2114-2124): integer addition
// is associative, so any tiling of the sum gives the same bits.  The bf16 form widens
// exactly (a 16-bit shift, codegen/partials/x86/cvtbf16_fp32.c) and accumulates in f32 in
// a different order than the emitted loop nest, hence a tolerance rather than equality.
//
// Memory-level mapping of a Morello schedule onto this kernel:
//   tile_out(256x256)        -> one workgroup per 256x256 tile of C
//   split(128 bytes of K)    -> the k loop
//   move_param(A/B, L1)      -> global -> LDS staging, double buffered
//   move_param(A/B, VRF)     -> LDS -> MFMA operand registers: ds_read_b128 for A (rows
//                               run along K) and the transposing ds_read_b64_tr_b8/_b16
//                               for B (rows run along N), so no relayout pass is needed
//   to_accum + Zero          -> accumulator registers start at zero; C is read only when
//                               the Spec accumulates
//
// The int8 MFMA multiplies signed bytes.  A u8 operand is fed as a' = a xor 0x80
// (= a - 128 as i8) and the exact correction 128 * sum_k B[k,j] is added per column in the
// epilogue; the column sums are accumulated from the B operand registers with v_dot4.
#pragma once
#include <type_traits>

#include "kernels.h"


namespace mrl {
namespace gemm {

typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v2i __attribute__((ext_vector_type(2)));
typedef short v4s __attribute__((ext_vector_type(4)));
typedef int v16i __attribute__((ext_vector_type(16)));
typedef float v16f __attribute__((ext_vector_type(16)));
typedef __bf16 v8bf __attribute__((ext_vector_type(8)));

typedef unsigned v4u __attribute__((ext_vector_type(4)));

// Tile rows per L2 group.  The workgroups of a launch go to the 8 XCDs round-robin and each XCD
// gets a contiguous run of tiles (an eighth of them); taken group_m tile rows at a time, such a
// run covers a block of C whose perimeter is what that XCD's L2 has to fetch, so the block
// should be as close to square as the counts allow (8192^3 with 256-tiles: 8 x 16 tiles per XCD,
// not 4 x 32, which made every XCD read all of B).
inline int group_rows(int tiles_m, int tiles_n) {
  const int ntiles = tiles_m * tiles_n;
  if (ntiles % 8 != 0) return 4;
  const int run = ntiles / 8;
  int best = 0;
  for (int gm = 1; gm <= tiles_m && gm <= run; gm *= 2) {
    if (run % gm != 0 || (gm * tiles_n) % run != 0 || tiles_m % gm != 0) continue;
    if (gm * gm <= run) best = gm;
  }
  return best ? best : 4;
}

// Where a workgroup works, as scalars the launch works out and the kernel takes as its FIRST
// arguments: those arrive in SGPRs with the wave (the GemmArgs structure behind them is loaded),
// so the tile's coordinates are known, without a division, by the time the operands' addresses
// are.  The divisions by a run-time value that this replaces are some thirty instructions each as
// the compiler expands them, on the scalar unit one after the other, in front of the first load.
struct TileWalk {
  uint32_t tiles_m, tiles_n, group_m;
  uint32_t per_xcd;     // tiles per XCD when the tiles divide evenly among the eight, else 0
  uint32_t group_mul, full_mul, last_mul;   // FastDiv by group_m * tiles_n, by group_m, by the last group's rows
  uint32_t shifts;      // their shift counts, a byte each
};
inline TileWalk tile_walk(int tiles_m, int tiles_n) {
  TileWalk w;
  w.tiles_m = uint32_t(tiles_m), w.tiles_n = uint32_t(tiles_n), w.group_m = uint32_t(group_rows(tiles_m, tiles_n));
  const uint32_t ntiles = w.tiles_m * w.tiles_n;
  w.per_xcd = ntiles % 8 == 0 ? ntiles / 8 : 0;
  const FastDiv group(w.group_m * w.tiles_n), full(w.group_m), last(std::max(1u, w.tiles_m % w.group_m));
  w.group_mul = group.mul, w.full_mul = full.mul, w.last_mul = last.mul;
  w.shifts = group.shift | full.shift << 8 | last.shift << 16;
  return w;
}
#ifdef MRL_WIDE_XCD_SWAP  // experiment: neighbouring XCDs exchange their blocks of tiles
#define MRL_XCD_FLIP 1
#else
#define MRL_XCD_FLIP 0
#endif
#define MRL_WALK_PARAMS                                                                                              \
  uint32_t tiles_m, uint32_t tiles_n, uint32_t group_m, uint32_t per_xcd, uint32_t group_mul, uint32_t full_mul, \
      uint32_t last_mul, uint32_t walk_shifts
#define MRL_WALK_ARGS(w) (w).tiles_m, (w).tiles_n, (w).group_m, (w).per_xcd, (w).group_mul, (w).full_mul, (w).last_mul, (w).shifts
// Workgroups are handed to the 8 XCDs round-robin; each XCD gets a contiguous run of tiles,
// ordered so that a run, taken group_m tile rows at a time, covers a compact block of C (shared
// A rows and B columns stay in that XCD's L2).
#define MRL_WALK_TILE(tile_m, tile_n)                                                                     \
  uint32_t tile_m, tile_n;                                                                                \
  {                                                                                                       \
    uint32_t pid = blockIdx.x;                                                                            \
    if (per_xcd) pid = ((pid & 7) ^ MRL_XCD_FLIP) * per_xcd + (pid >> 3);                                 \
    FastDiv by;                                                                                           \
    by.mul = group_mul, by.shift = walk_shifts & 255;                                                     \
    const uint32_t group = by.div(pid), first_m = group * group_m, gsz = min(tiles_m - first_m, group_m); \
    const uint32_t in_group = pid - group * (group_m * tiles_n);                                          \
    const bool full = gsz == group_m;                                                                     \
    by.mul = full ? full_mul : last_mul, by.shift = (full ? walk_shifts >> 8 : walk_shifts >> 16) & 255;  \
    tile_n = by.div(in_group), tile_m = first_m + (in_group - tile_n * gsz);                              \
  }

// Ragged tiles (EDGE) address memory through buffer resources: `records` bytes from `base` on
// are in range, a load beyond them returns zeros and a store beyond them is dropped, both
// without a branch.  Offsets are unsigned 32-bit, which is why the EDGE kernels want every
// leading dimension below EDGE_MAX_ROW_BYTES: 256 rows of a tile then stay below 4 GiB.
constexpr int64_t EDGE_MAX_ROW_BYTES = int64_t(1) << 24;
constexpr uint32_t OUT_OF_RANGE = 0xffffffffu;  // an offset no resource holds
__device__ inline __amdgpu_buffer_rsrc_t buffer_of(const void *base, int64_t records) {
  const int64_t clamped = records < 0 ? 0 : records > int64_t(0xffffffffu) ? int64_t(0xffffffffu) : records;
  return __builtin_amdgcn_make_buffer_rsrc(const_cast<void *>(base), 0, int(uint32_t(clamped)), 0x00020000);
}

// Workgroup tile: BM x BN outputs, BKB bytes of K per k step, WAVES_M x WAVES_N waves.
template <int BM_, int BN_, int BKB_, int WAVES_M_, int WAVES_N_>
struct Tile {
  static constexpr int BM = BM_, BN = BN_, BKB = BKB_, WAVES_M = WAVES_M_, WAVES_N = WAVES_N_;
  static constexpr int NT = 64 * WAVES_M * WAVES_N;
  static constexpr int A_STAGE = BM * BKB;  // A tile: [BM][BKB B], 16-byte chunks XOR-swizzled
  // B tile: [BK][BN] elements in global orientation, rows padded so that the rows one
  // transposing read touches fall on different banks (see Traits::PAD).
  template <class T> static constexpr int b_row() { return BN * T::ES + T::PAD; }
  template <class T> static constexpr int stage() { return A_STAGE + (BKB / T::ES) * b_row<T>(); }
};
typedef Tile<256, 256, 128, 2, 4> TileBig;   // one workgroup per CU, 136 KiB of LDS
// The 128 x 128 tile with a 128-byte step: eight waves of 32 x 64 outputs each for int8 (either
// orientation of B) and for bf16 against a k-fastest B, four waves of 64 x 64 otherwise.  Twice the
// waves hide more of a step's trip through LDS behind the other waves' MFMAs (one workgroup of this
// tile is all a compute unit holds at mid sizes).  Measured, four / eight waves as 4 x 2 / as 2 x 4:
// int8 1792^3 15.3 / 14.0 / 14.7 us, 2560 x 640 x 1280 9.05 / 8.28 / 8.31, 3072 x 3072 x 1024 22.6 /
// 21.0 / 22.2, Conv 32 x (128 -> 128) x 28 x 28 3 x 3 13.2 / 11.1 / 11.6; bf16 row-major 2048^3 25.4 /
// 27.2 / 25.9 (stays at four), the same Conv in bf16 17.4 / 15.8 / 15.6.
template <class T, bool B_KMAJOR>
using Tile128 = std::conditional_t<T::ES == 1 || (T::ES == 2 && B_KMAJOR), Tile<128, 128, 128, 4, 2>, Tile<128, 128, 128, 2, 2>>;

typedef __attribute__((address_space(3))) v2i lds_v2i;
typedef __attribute__((address_space(3))) v4s lds_v4s;

struct I8 {
  typedef v16i Acc;
  typedef int32_t Out;
  static constexpr int ES = 1;             // element bytes
  static constexpr int PAD = 32;           // 8 k-rows x 32 B cover all 64 banks
  static constexpr int K_PER_READ = 8;     // k rows covered by one transposing read
  static constexpr bool TRANSPOSED_READ = true;
  __device__ static v2i read_tr(const uint8_t *p) {
    return __builtin_amdgcn_ds_read_tr8_b64_v2i32((lds_v2i *)p);
  }
  __device__ static Acc mfma(v4i a, v4i b, Acc c) {
    return __builtin_amdgcn_mfma_i32_32x32x32_i8(a, b, c, 0, 0, 0);
  }
};
struct BF16 {
  typedef v16f Acc;
  typedef float Out;
  static constexpr int ES = 2;
  static constexpr int PAD = 64;           // 4 k-rows x 64 B cover all 64 banks
  static constexpr int K_PER_READ = 4;
  static constexpr bool TRANSPOSED_READ = true;
  __device__ static v2i read_tr(const uint8_t *p) {
    const v4s r = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_v4s *)p);
    return __builtin_bit_cast(v2i, r);
  }
  __device__ static Acc mfma(v4i a, v4i b, Acc c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(v8bf, a),
                                                   __builtin_bit_cast(v8bf, b), c, 0, 0, 0);
  }
};

// f32 operands, f32 accumulation.  One 32-byte k step is 8 values of k = four MFMAs of k = 2:
// lane half h of MFMA j takes k = 4h + j from both operands (any pairing of k values is a
// valid order of the sum as long as A and B agree), which makes A's share 16 contiguous
// bytes like the other types.  B needs no transposition: a lane reads its column's value from
// each of its four k rows (32 lanes x 4 bytes = 128 contiguous bytes per row).
struct F32 {
  typedef v16f Acc;
  typedef float Out;
  static constexpr int ES = 4;
  static constexpr int PAD = 32;           // rows k and k+4 land on opposite bank halves
  static constexpr int K_PER_READ = 1;
  static constexpr bool TRANSPOSED_READ = false;
  __device__ static v2i read_tr(const uint8_t *) { return v2i{0, 0}; }
  __device__ static Acc mfma(v4i a, v4i b, Acc c) {
    typedef float v4f __attribute__((ext_vector_type(4)));
    const v4f fa = __builtin_bit_cast(v4f, a), fb = __builtin_bit_cast(v4f, b);
    c = __builtin_amdgcn_mfma_f32_32x32x2f32(fa[0], fb[0], c, 0, 0, 0);
    c = __builtin_amdgcn_mfma_f32_32x32x2f32(fa[1], fb[1], c, 0, 0, 0);
    c = __builtin_amdgcn_mfma_f32_32x32x2f32(fa[2], fb[2], c, 0, 0, 0);
    c = __builtin_amdgcn_mfma_f32_32x32x2f32(fa[3], fb[3], c, 0, 0, 0);
    return c;
  }
};

// Writes one wave's TM x TN blocks of 32 x 32 accumulators to C (adding the u8 correction
// and, for an accumulating Spec, the previous contents).  `colsum` holds this wave's partial
// column sums of B; the partials of the PARTS waves that share the columns (and of the two
// lane halves) are combined through LDS, which every wave must be done reading.
template <class T, bool A_UNSIGNED, bool EDGE, int BN, int PARTS, int TM, int TN>
__device__ inline void epilogue(const GemmArgs &g, typename T::Out *C, uint8_t *lds,
                                typename T::Acc (&acc)[TM][TN], int (&colsum)[TN], int lane,
                                int part_idx, int row0, int col0, int rows_left, int cols_left) {
  typedef typename T::Out Out;
  constexpr int WAVES_M = PARTS;
  const int wm = part_idx;
  // Epilogue.  Column sums: combine the partials of the WAVES_M waves and two lane halves.
  int corr[TN];
#pragma unroll
  for (int tn = 0; tn < TN; tn++) corr[tn] = 0;
  if (A_UNSIGNED) {
    int *part = (int *)lds;  // [WAVES_M * 2][BN]; the k loop ended on a barrier
    __syncthreads();         // ... and every wave is past its last LDS read of the tiles
#pragma unroll
    for (int tn = 0; tn < TN; tn++)
      part[(wm * 2 + (lane >> 5)) * BN + col0 + tn * 32 + (lane & 31)] = colsum[tn];
    __syncthreads();
#pragma unroll
    for (int tn = 0; tn < TN; tn++) {
      int sum = 0;
#pragma unroll
      for (int w = 0; w < WAVES_M * 2; w++) sum += part[w * BN + col0 + tn * 32 + (lane & 31)];
      corr[tn] = sum * 128;
    }
  }
  // Lane (l%32, l/32) of accumulator register r owns C[8*(r/4) + 4*(l/32) + r%4][l%32] of
  // each 32x32 block.  An accumulating Spec reads its whole block row of C first, so the
  // loads are in flight together instead of one round trip per element.
  // With EDGE the tile may hang over the bottom / right border of C: rows_left and
  // cols_left bound what this workgroup owns.  The rows are cut off by the range check of
  // the buffer resource (an offset in a row past the last lies beyond its records); a lane
  // whose column is past the last gets the out-of-range offset.
  // Streaming (non-temporal) stores suit a small C whose rows are whole cache lines (a 13 MB
  // output: 14.0 against 15.0 us); a large one, or rows that straddle lines, is written faster
  // through the cache, which joins the parts of a line (268 MB: 60 against 73 us; rows of 4425
  // floats: 28 against 43 us).
  const bool stream_c = double(g.m) * g.n * g.batch * sizeof(Out) <= 32.0 * 1024 * 1024 && (g.ldc * sizeof(Out)) % 128 == 0;
  const int lane_row = row0 + (lane >> 5) * 4, lane_col = col0 + (lane & 31);
  Out *c_lane = C + int64_t(lane_row) * g.ldc + lane_col;
  const uint32_t ldc_b = uint32_t(g.ldc) * sizeof(Out);
  const auto c_buf = buffer_of(C, EDGE ? int64_t(rows_left - 1) * ldc_b + int64_t(cols_left) * sizeof(Out) : 0);
  const uint32_t lane_off = uint32_t(lane_row) * ldc_b + uint32_t(lane_col) * sizeof(Out);
  auto offset_of = [&](int tm, int tn, int r) -> uint32_t {
    const uint32_t off = lane_off + uint32_t(tm * 32 + (r >> 2) * 8 + (r & 3)) * ldc_b + tn * 32 * sizeof(Out);
    return lane_col + tn * 32 < cols_left ? off : OUT_OF_RANGE;
  };
#pragma unroll
  for (int tm = 0; tm < TM; tm++) {
    Out prev[TN][16];
    if (g.accum) {
#pragma unroll
      for (int tn = 0; tn < TN; tn++)
#pragma unroll
        for (int r = 0; r < 16; r++) {
          if constexpr (EDGE)
            prev[tn][r] = __builtin_bit_cast(Out, __builtin_amdgcn_raw_buffer_load_b32(c_buf, offset_of(tm, tn, r), 0, 0));
          else
            prev[tn][r] = c_lane[int64_t(tm * 32 + (r >> 2) * 8 + (r & 3)) * g.ldc + tn * 32];
        }
    }
    // A row's TN segments of 128 bytes one after the other: when rows of C are not whole cache
    // lines every segment straddles two of them, and the other part of a line should follow
    // at once rather than sixteen stores later.
    auto store_rows = [&](auto streaming) {
#pragma unroll
      for (int r = 0; r < 16; r++)
#pragma unroll
        for (int tn = 0; tn < TN; tn++) {
          Out v = acc[tm][tn][r];
          if (A_UNSIGNED) v += Out(corr[tn]);
          if (g.accum) v += prev[tn][r];
          if constexpr (EDGE) {
            __builtin_amdgcn_raw_buffer_store_b32(__builtin_bit_cast(unsigned, v), c_buf, offset_of(tm, tn, r), 0,
                                                  decltype(streaming)::value ? 2 : 0);
          } else {
            Out *to = &c_lane[int64_t(tm * 32 + (r >> 2) * 8 + (r & 3)) * g.ldc + tn * 32];
            if constexpr (decltype(streaming)::value) __builtin_nontemporal_store(v, to);
            else *to = v;
          }
        }
    };
    if (stream_c) store_rows(std::true_type{});
    else store_rows(std::false_type{});
  }
}

// Pins the instruction order of one k step: slot I of N issues MFMA_PER MFMAs, then its even
// share of the step's DS_READS operand reads, then (in the step that stages the next tile)
// one LDS write and one global load while any of the MEM_OPS are left.
template <int I, int N, int MFMA_PER, int DS_READS, int MEM_OPS>
__device__ inline void sched_slots(bool staging) {
  if constexpr (I < N) {
    __builtin_amdgcn_sched_group_barrier(0x008, MFMA_PER, 0);  // MFMA
    constexpr int FIRST = DS_READS * I / N, END = DS_READS * (I + 1) / N;
    if constexpr (END > FIRST) __builtin_amdgcn_sched_group_barrier(0x100, END - FIRST, 0);  // DS read
    if (staging && I < MEM_OPS) {
      __builtin_amdgcn_sched_group_barrier(0x200, 1, 0);  // DS write
      __builtin_amdgcn_sched_group_barrier(0x020, 1, 0);  // VMEM read
    }
    sched_slots<I + 1, N, MFMA_PER, DS_READS, MEM_OPS>(staging);
  }
}

// EDGE = false: M, N multiples of the tile and K a multiple of the k step.  EDGE = true: any
// M, N and K, with leading dimensions that are whole 16-byte chunks (and below
// EDGE_MAX_ROW_BYTES); chunks past the last row or past K are fed as zeros and stores outside
// C are dropped, both by the range check of buffer loads and stores, so the k loop and the
// epilogue stay free of branches.  A chunk that straddles the end of K brings along the bytes
// between the row's end and its leading dimension: the caller keeps those zero (they are its
// own padding whenever K is not a whole number of chunks).  Chunks to the right of B's last
// column hold whatever follows in memory: they only reach columns of C that are not stored.
// B_KMAJOR: B is stored with k fastest (each of its n rows runs along K, `ldb` elements apart:
// Morello's col_major / batched_col_major layouts, or layout![0,2,1]).  Its tile is then staged
// and read exactly like A's, and no transposing read is involved.
// CONV (with EDGE and B_KMAJOR): the left operand is not a matrix in memory but the windows of
// a channels-last image, g.conv; row p's 16-byte chunk at k byte kb lies at
// corner(p) + ((r * w + s) * c_bytes + kb % c_bytes) with (r, s) = divmod(kb / c_bytes, fw).
template <class T, bool A_UNSIGNED, class TL, bool EDGE, bool B_KMAJOR = false, bool CONV = false>
__global__ __launch_bounds__(TL::NT) void k_gemm(MRL_WALK_PARAMS, GemmArgs g) {
  static_assert(!CONV || (EDGE && B_KMAJOR), "the implicit Conv operand is addressed through the buffer path");
  extern __shared__ __attribute__((aligned(16))) uint8_t lds[];
  constexpr int BM = TL::BM, BN = TL::BN, BKB = TL::BKB, WAVES_M = TL::WAVES_M, WAVES_N = TL::WAVES_N;
  constexpr int NT = TL::NT, A_STAGE = TL::A_STAGE;
  constexpr int WM = BM / WAVES_M, WN = BN / WAVES_N, TM = WM / 32, TN = WN / 32;
  constexpr int ES = T::ES, BK = BKB / ES, B_ROW = TL::template b_row<T>();
  constexpr int STAGE = TL::template stage<T>();
  constexpr int A_ROW_CH = BKB / 16;              // 16-byte chunks per A tile row
  constexpr int A_ROWS_PER_LINE = 256 / BKB;      // A tile rows per 256-byte bank line
  constexpr int A_CH = BM * BKB / 16 / NT;       // 16-byte chunks per thread, A tile
  constexpr int B_ROW_CH = B_KMAJOR ? BKB / 16 : BN * ES / 16;               // chunks per B tile row
  constexpr int B_CH = (B_KMAJOR ? BN : BK) * B_ROW_CH / NT;                  // chunks per thread, B tile
  constexpr int B_LDS_ROW = B_KMAJOR ? BKB : B_ROW;                          // bytes per B tile row in LDS
  constexpr int SLABS = BKB / 32;                 // MFMA k steps per tile (32 bytes each)
  constexpr int K_SLAB = 32 / ES;                 // elements of K per MFMA
  typedef typename T::Acc Acc;
  typedef typename T::Out Out;

  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);  // wave-uniform, lives in an SGPR
  const int wm = wave / WAVES_N, wn = wave % WAVES_N;

  MRL_WALK_TILE(tile_m, tile_n)
  const int64_t m0 = int64_t(tile_m) * BM, n0 = int64_t(tile_n) * BN;

  const uint8_t *A = (const uint8_t *)g.a + (int64_t(blockIdx.y) * g.sa + m0 * g.lda) * ES;
  const uint8_t *B = (const uint8_t *)g.b + (int64_t(blockIdx.y) * g.sb + (B_KMAJOR ? n0 * g.ldb : n0)) * ES;
  Out *C = (Out *)g.c + int64_t(blockIdx.y) * g.sc + m0 * g.ldc + n0;
  const int64_t lda_b = g.lda * ES, ldb_b = g.ldb * ES;

  // Per-thread staging assignments for one k step.  Thread `tid` moves 16-byte chunk
  // tid + i*NT of each tile; successive i differ by a whole number of rows (a multiple of
  // 16), so one base pointer / LDS offset per operand plus compile-time strides suffices.
  constexpr int A_ROWS_PER_I = NT / A_ROW_CH, B_ROWS_PER_I = NT / B_ROW_CH;
  static_assert(A_ROWS_PER_I % 16 == 0, "swizzle term must not depend on i");
  const uint8_t *a_src;
  int a_dst;
  {
    // 16 lanes of an operand read hit 16 consecutive rows at one chunk index; XOR-ing the
    // chunk with (row / rows-per-bank-line) spreads them over all 64 banks.
    const int row = tid / A_ROW_CH, ch = tid % A_ROW_CH;
    a_src = A + int64_t(row) * lda_b + ch * 16;
    a_dst = row * BKB + ((ch ^ ((row / A_ROWS_PER_LINE) & (A_ROW_CH - 1))) << 4);
  }
  const uint8_t *b_src;
  int b_dst;
  {
    const int row = tid / B_ROW_CH, ch = tid % B_ROW_CH;
    b_src = B + int64_t(row) * ldb_b + ch * 16;
    if constexpr (B_KMAJOR) b_dst = A_STAGE + row * BKB + ((ch ^ ((row / A_ROWS_PER_LINE) & (A_ROW_CH - 1))) << 4);
    else b_dst = A_STAGE + row * B_ROW + ch * 16;
  }
  const int64_t a_step_i = int64_t(A_ROWS_PER_I) * lda_b, b_step_i = int64_t(B_ROWS_PER_I) * ldb_b;
  const int64_t b_step_kt = B_KMAJOR ? int64_t(BKB) : int64_t(BK) * ldb_b;
  // Operand fragment offsets within a stage for MFMA k step 0.
  int a_frag[TM];
#pragma unroll
  for (int tm = 0; tm < TM; tm++) a_frag[tm] = (wm * WM + tm * 32 + (lane & 31)) * BKB;
  const int a_swz = ((lane & 31) / A_ROWS_PER_LINE) & (A_ROW_CH - 1);  // WM, 32 are multiples of 16
  const int a_half = lane >> 5;
  // Transposing read: a 16-lane group fetches a K_PER_READ x 16 element block; lane p of the
  // group supplies the address of 8 bytes of one k row, and receives the column it indexes.
  int b_frag[TN];
#pragma unroll
  for (int tn = 0; tn < TN; tn++) {
    if constexpr (B_KMAJOR) {
      b_frag[tn] = A_STAGE + (wn * WN + tn * 32 + (lane & 31)) * BKB;
    } else if constexpr (T::TRANSPOSED_READ) {
      constexpr int LANES_PER_ROW = 16 / (8 / ES);  // lanes that share one k row: 2 (i8), 4 (bf16)
      const int p = lane & 15;
      const int k = (K_SLAB / 2) * (lane >> 5) + p / LANES_PER_ROW;
      const int col = wn * WN + tn * 32 + 16 * ((lane >> 4) & 1) + (8 / ES) * (p % LANES_PER_ROW);
      b_frag[tn] = A_STAGE + k * B_ROW + col * ES;
    } else {
      b_frag[tn] = A_STAGE + (K_SLAB / 2) * (lane >> 5) * B_ROW + (wn * WN + tn * 32 + (lane & 31)) * ES;
    }
  }

  Acc acc[TM][TN];
#pragma unroll
  for (int tm = 0; tm < TM; tm++)
#pragma unroll
    for (int tn = 0; tn < TN; tn++)
#pragma unroll
      for (int r = 0; r < 16; r++) acc[tm][tn][r] = 0;
  int colsum[TN];
#pragma unroll
  for (int tn = 0; tn < TN; tn++) colsum[tn] = 0;

  v4i a_reg[A_CH], b_reg[B_CH];
  const int kt_count = int((g.k + BK - 1) / BK);
  // EDGE bookkeeping.  The tiles are addressed relative to `a_tile` / `b_tile` (wave-uniform,
  // advanced by one k step per load) with per-thread 32-bit offsets; what lies past the last
  // row of the tile is out of the resource's range.  The end of K inside a row is not (the
  // next row follows), so a thread whose chunk starts at or past K asks for the
  // out-of-range offset instead.
  const int k_bytes = int(g.k) * ES;
  const uint8_t *a_tile = A, *b_tile = B;
  const int a_rows = min(BM, int(g.m - m0)), b_rows = min(BN, int(g.n - n0));  // rows the tile owns
  const uint32_t a_off = uint32_t(tid / A_ROW_CH) * uint32_t(lda_b) + (tid % A_ROW_CH) * 16;
  // CONV: byte offset of the window corner of each of the thread's rows (out of range past M).
  uint32_t a_corner[A_CH];
  if constexpr (CONV) {
#pragma unroll
    for (int i = 0; i < A_CH; i++) {
      const int64_t p = m0 + tid / A_ROW_CH + i * A_ROWS_PER_I;
      const uint32_t q = uint32_t(min(p, int64_t(g.m) - 1));
      const uint32_t row = g.conv.by_ow.div(q), x = q - row * g.conv.ow, img = g.conv.by_oh.div(row), y = row - img * g.conv.oh;
      a_corner[i] = p < int64_t(g.m) ? ((img * g.conv.h + y) * g.conv.w + x) * g.conv.c_bytes : OUT_OF_RANGE;
    }
  }
  const uint32_t b_off = uint32_t(tid / B_ROW_CH) * uint32_t(ldb_b) + (tid % B_ROW_CH) * 16;
  const int a_kb0 = (tid % A_ROW_CH) * 16;  // the thread's k byte within a tile
  const int b_kb0 = (tid % B_ROW_CH) * 16;  // B_KMAJOR: likewise
  int ld_kb = 0;  // k byte offset of the tile the next load_global() fetches

  // Loads the next tile in sequence and advances the source pointers.
  auto load_global = [&]() {
    if constexpr (EDGE) {
      const bool a_in = ld_kb + a_kb0 < k_bytes;
      if constexpr (CONV) {
        const auto a_buf = buffer_of(g.a, int64_t(g.conv.image_bytes));
        const uint32_t kb = blockIdx.y * g.conv.slice_bytes + uint32_t(ld_kb + a_kb0), pos = g.conv.by_c_bytes.div(kb), r = g.conv.by_fw.div(pos);
        const uint32_t in_window = ((r * g.conv.w + (pos - r * g.conv.fw)) * g.conv.c_bytes) + (kb - pos * g.conv.c_bytes);
#pragma unroll
        for (int i = 0; i < A_CH; i++)
          a_reg[i] = __builtin_bit_cast(v4i, __builtin_amdgcn_raw_buffer_load_b128(
                                                 a_buf, a_in && a_corner[i] != OUT_OF_RANGE ? a_corner[i] + in_window : OUT_OF_RANGE, 0, 0));
      } else {
        const auto a_buf = buffer_of(a_tile, int64_t(a_rows) * lda_b - ld_kb);
#pragma unroll
        for (int i = 0; i < A_CH; i++)
          a_reg[i] = __builtin_bit_cast(v4i, __builtin_amdgcn_raw_buffer_load_b128(
                                                 a_buf, a_in ? a_off + i * uint32_t(a_step_i) : OUT_OF_RANGE, 0, 0));
      }
      if constexpr (B_KMAJOR) {
        const auto b_buf = buffer_of(b_tile, int64_t(b_rows) * ldb_b - ld_kb);
        const bool b_in = ld_kb + b_kb0 < k_bytes;
#pragma unroll
        for (int i = 0; i < B_CH; i++)
          b_reg[i] = __builtin_bit_cast(v4i, __builtin_amdgcn_raw_buffer_load_b128(
                                                 b_buf, b_in ? b_off + i * uint32_t(b_step_i) : OUT_OF_RANGE, 0, 0));
      } else {
        // k rows left from this tile's first on, each up to its leading dimension.
        const auto b_buf = buffer_of(b_tile, (int64_t(g.k) - ld_kb / ES) * ldb_b - n0 * ES);
#pragma unroll
        for (int i = 0; i < B_CH; i++)
          b_reg[i] = __builtin_bit_cast(v4i, __builtin_amdgcn_raw_buffer_load_b128(
                                                 b_buf, b_off + i * uint32_t(b_step_i), 0, 0));
      }
      a_tile += BKB;
      b_tile += b_step_kt;
    } else {
#pragma unroll
      for (int i = 0; i < A_CH; i++) a_reg[i] = *(const v4i *)(a_src + i * a_step_i);
#pragma unroll
      for (int i = 0; i < B_CH; i++) b_reg[i] = *(const v4i *)(b_src + i * b_step_i);
      a_src += BKB;
      b_src += b_step_kt;
    }
    ld_kb += BKB;
  };
  auto store_lds = [&](int stage) {
    uint8_t *base = lds + stage * STAGE;
#pragma unroll
    for (int i = 0; i < A_CH; i++) {
      v4i v = a_reg[i];
      if (A_UNSIGNED) v ^= v4i{int(0x80808080), int(0x80808080), int(0x80808080), int(0x80808080)};
      *(v4i *)(base + a_dst + i * A_ROWS_PER_I * BKB) = v;
    }
#pragma unroll
    for (int i = 0; i < B_CH; i++) *(v4i *)(base + b_dst + i * B_ROWS_PER_I * B_LDS_ROW) = b_reg[i];
  };
  // MFMA operands for one 32-byte k step, double buffered in registers.
  v4i af[2][TM], bf[2][TN];
  auto read_frags = [&](int stage, int s, int buf) {
    const uint8_t *base = lds + stage * STAGE;
#pragma unroll
    for (int tm = 0; tm < TM; tm++)
      af[buf][tm] = *(const v4i *)(base + a_frag[tm] + (((2 * s + a_half) ^ a_swz) << 4));
#pragma unroll
    for (int tn = 0; tn < TN; tn++) {
      if constexpr (B_KMAJOR) {
        bf[buf][tn] = *(const v4i *)(base + b_frag[tn] + (((2 * s + a_half) ^ a_swz) << 4));
      } else if constexpr (T::TRANSPOSED_READ) {
        const v2i lo = T::read_tr(base + b_frag[tn] + (s * K_SLAB) * B_ROW);
        const v2i hi = T::read_tr(base + b_frag[tn] + (s * K_SLAB + T::K_PER_READ) * B_ROW);
        bf[buf][tn] = v4i{lo[0], lo[1], hi[0], hi[1]};
      } else {
        const uint8_t *col = base + b_frag[tn] + (s * K_SLAB) * B_ROW;
        bf[buf][tn] = v4i{*(const int *)col, *(const int *)(col + B_ROW), *(const int *)(col + 2 * B_ROW),
                          *(const int *)(col + 3 * B_ROW)};
      }
    }
  };
  auto mfma_slab = [&](int s, int buf) {
    // Column sums of B for the u8 correction: each of the WAVES_M waves that share these
    // columns takes every WAVES_M-th k step (a scalar branch: `wm` is wave-uniform).
    if (A_UNSIGNED && (s % WAVES_M) == wm) {
#pragma unroll
      for (int tn = 0; tn < TN; tn++)
#pragma unroll
        for (int w = 0; w < 4; w++)
          colsum[tn] = __builtin_amdgcn_sdot4(bf[buf][tn][w], 0x01010101, colsum[tn], false);
    }
#pragma unroll
    for (int tm = 0; tm < TM; tm++)
#pragma unroll
      for (int tn = 0; tn < TN; tn++) acc[tm][tn] = T::mfma(af[buf][tm], bf[buf][tn], acc[tm][tn]);
  };

  // Software pipeline.  While tile kt is multiplied out of LDS stage kt&1, tile kt+1 sits
  // in registers (its global loads were issued one tile earlier) and is written to the
  // other stage during the second-to-last k step; the barrier comes before the last k
  // step's MFMAs, so the first operands of tile kt+1 are fetched under them and the matrix
  // core does not drain at the barrier.  The loop's body is branch-free; the last two tiles,
  // which have nothing left to fetch or to stage behind them, follow it straight-line.
  // sched_group_barrier pins the interleaving of LDS, VMEM and MFMA issue that the text below
  // spells out.
  load_global();
  store_lds(0);
  if (kt_count >= 2) load_global();
  __syncthreads();
  read_frags(0, 0, 0);

  // The loop covers the tiles that have two more behind them; the last two run straight-line
  // below, without the loads, the staging and the barrier that would only serve tiles past the
  // end of K (re-read and re-staged, they cost a 64^3 problem of two steps an eighth of its launch:
  // 3.93 -> 3.47 us).
  const int main_steps = max(kt_count - 2, 0);
  for (int kt = 0; kt < main_steps; kt++) {
    const int cur = kt & 1;
    // Tile kt+2 is loaded next.
#pragma unroll
    for (int s = 0; s < SLABS; s++) {
      if (s + 1 < SLABS) read_frags(cur, s + 1, (s + 1) & 1);
      if (s == SLABS - 2) {
        store_lds(cur ^ 1);
        load_global();
      }
      if (s == SLABS - 1) {
        __syncthreads();
        read_frags(cur ^ 1, 0, 0);
      }
      mfma_slab(s, s & 1);
      // One output block's MFMAs, then a share of this step's memory instructions, TM*TN times.
      sched_slots<0, TM * TN, T::TRANSPOSED_READ ? 1 : 4,
                  TM + (B_KMAJOR ? 1 : T::TRANSPOSED_READ ? 2 : 4) * TN, A_CH + B_CH>(
          s == SLABS - 2);
    }
  }

  if (kt_count >= 2) {  // the tile before the last: the last one, in registers, is staged under it
    const int cur = main_steps & 1;
#pragma unroll
    for (int s = 0; s < SLABS; s++) {
      if (s + 1 < SLABS) read_frags(cur, s + 1, (s + 1) & 1);
      if (s == SLABS - 2) store_lds(cur ^ 1);
      if (s == SLABS - 1) {
        __syncthreads();
        read_frags(cur ^ 1, 0, 0);
      }
      mfma_slab(s, s & 1);
    }
  }
  {
    const int cur = (kt_count - 1) & 1;
#pragma unroll
    for (int s = 0; s < SLABS; s++) {
      if (s + 1 < SLABS) read_frags(cur, s + 1, (s + 1) & 1);
      mfma_slab(s, s & 1);
    }
  }

  epilogue<T, A_UNSIGNED, EDGE, BN, WAVES_M, TM, TN>(g, C, lds, acc, colsum, lane, wm, wm * WM, wn * WN,
                                                     int(g.m - m0), int(g.n - n0));
}

// Whether the 32-bit offsets of the EDGE kernels reach every row of a tile.
inline bool edge_addressable(const GemmArgs &g, int elem_size) {
  return g.lda * elem_size < EDGE_MAX_ROW_BYTES && g.ldb * elem_size < EDGE_MAX_ROW_BYTES &&
         g.ldc * 4 < EDGE_MAX_ROW_BYTES;
}

template <class T, bool A_UNSIGNED, class TL, bool EDGE, bool B_KMAJOR = false, bool CONV = false>
hipError_t launch(const GemmArgs &g, hipStream_t stream) {
  constexpr auto kern = k_gemm<T, A_UNSIGNED, TL, EDGE, B_KMAJOR, CONV>;
  constexpr int BM = TL::BM, BN = TL::BN;
  constexpr int STAGE = TL::template stage<T>();
  if (EDGE && !edge_addressable(g, T::ES)) return hipErrorInvalidValue;
  static std::atomic<uint64_t> lds_limit_set{0};
  if (!plan::recording()) {
    hipError_t e = raise_lds_limit(lds_limit_set, (const void *)kern, 2 * STAGE);
    if (e != hipSuccess) return e;
  }
  const int tiles_m = int((g.m + BM - 1) / BM), tiles_n = int((g.n + BN - 1) / BN);
  const TileWalk walk = tile_walk(tiles_m, tiles_n);
  {
    const double k_steps = double((g.k * T::ES + TL::BKB - 1) / TL::BKB) * (TL::BKB / T::ES);  // k, padded to steps
    const double mn = double(g.m) * g.n * g.batch;
    plan::work(T::ES == 1 ? plan::UNIT_MFMA_I8 : T::ES == 2 ? plan::UNIT_MFMA_BF16 : plan::UNIT_MFMA_F32,
               2.0 * mn * g.k, (double(g.m) * g.k + double(g.k) * g.n) * g.batch * T::ES + mn * 4 * (g.accum ? 2 : 1),
               2.0 * BM * BN * k_steps,
               // prologue and epilogue, then one barrier-to-barrier trip per step of K, longer for a
               // larger tile (measured 0.4-0.55 us at 64 x 64, 0.6-1.0 at 128 x 128, 1.4-2.0 at 256 x 256)
               // on int8 and bf16, whose steps hold the same MFMA time; an f32 step's MFMAs take
               // longer by the difference of the datasheet rates, and a workgroup alone on its unit
               // does not overlap them with the trip (f32 at 64 x 64: 0.9 us per step)
               500.0 + (100.0 + 3.0 * (BM + BN) +
                        2.0 * BM * BN * ((TL::BKB / T::ES) / plan::nominal_unit_rate(T::ES) - TL::BKB / plan::nominal_unit_rate(1))) *
                           double((g.k * T::ES + TL::BKB - 1) / TL::BKB));
  }
  MRL_LAUNCH((k_gemm<T, A_UNSIGNED, TL, EDGE, B_KMAJOR, CONV>), dim3(tiles_m * tiles_n, g.batch), dim3(TL::NT),
             2 * STAGE, stream, MRL_WALK_ARGS(walk), g);
  return mrl::plan::last_error();
}


}  // namespace gemm
}  // namespace mrl
