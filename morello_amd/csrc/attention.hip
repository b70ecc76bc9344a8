// Fused Matmul -> Softmax -> Matmul for bf16 inputs (the attention-shaped Compose of
// morello/examples/matmul_chain.rs:26-57; semantics morello/src/verification.rs:225-286):
//     S = Q . KT        [m, n2]  f32
//     P = softmax(S)    row-wise over n2, f32
//     out = P . V       [m, n]   f32
// with no scale and no mask, one independent problem per batch entry.
//
// The reference materialises S and P in memory between three loop nests
// (matmul_chain.rs:60-81).  Here a 512-thread workgroup owns 128 query rows of one batch
// entry: four waves take 32 queries each over the first half of the keys, four more take
// the same queries over the second half (the parallel split of
// morello/src/scheduling/parallel_softmax.rs:31-223, with k = n2/2).  Each wave streams
// blocks of 64 keys: S^T = K.Q^T is formed on the bf16 MFMA, folded into a running
// (max, denominator) per query with the online update of morello/src/spec.rs:96-106
// (new = max(old, x); d = d*exp(old-new) + exp(x-new)), and P^T (rounded to bf16, the one
// deviation from the f32 closed form; at most 2^-9 relative per element) feeds the second
// MFMA as O^T += V^T.P^T.  At the end the two halves' (max, denominator, O) triples are
// merged with SoftmaxDenominatorAndMaxFromParts' formula (morello/src/spec.rs:107-132).
// S and P never reach HBM: traffic is Q, K, V once and the output once.
//
// Both products are formed transposed, in 16 x 16 blocks (v_mfma_f32_16x16x32_bf16: on a
// power-limited board this form sustains 12 % more than the 32 x 32 one, an accumulator being
// updated once per 32 multiply-adds instead of once per 16), so that a lane owns query columns
// (two of a wave's 32: l % 16 and 16 + l % 16): the running max, the denominator and the rescale
// factor are per-lane scalars, and a row reduction is 16 in-register values plus two cross-lane
// exchanges.  The k index of an MFMA is a contraction index, so which keys a lane group holds in
// the second product is free as long as both operands agree: lane group g takes keys
// 4 g .. 4 g + 3 of each of two 16-key blocks, exactly the P values its own accumulators of the
// first product hold, and V^T's operand is read from LDS with the same choice of rows.  K and V
// blocks go from global memory straight into LDS (no staging registers; two K tiles and three V
// tiles per key half), the bank-conflict swizzles applied on the source side of those loads.  The
// two key halves run one slot apart (matrix work of one beside vector work of the other), two
// barriers per block.
#include <algorithm>

#include "kernels.h"

namespace mrl {
namespace {

typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v2i __attribute__((ext_vector_type(2)));
typedef short v4s __attribute__((ext_vector_type(4)));
typedef float v4f __attribute__((ext_vector_type(4)));
typedef __bf16 v8bf __attribute__((ext_vector_type(8)));
typedef __attribute__((address_space(3))) v4s lds_v4s;
typedef __attribute__((address_space(3))) void lds_void;
typedef __attribute__((address_space(1))) const void global_cvoid;

constexpr int BKV = 64;       // keys per block
// Sizes that follow from the head dim D (k and n of the Compose; 32, 64 or 128).
template <int D>
struct Dims {
  static constexpr int ROW = D * 2;             // bytes per K or V row
  static constexpr int TILE = BKV * ROW;        // one K or V block (16 KiB at D = 128)
  static constexpr int HALF = 5 * TILE;         // per key half: two K tiles, three V tiles
  static constexpr int CHUNKS = ROW / 16;       // 16-byte chunks per row
  static constexpr int SLOTS = ROW / 32;        // 32-byte slots per row (16 values: a block's share of a V row)
  static constexpr int ROWS_PER_LINE = ROW >= 256 ? 1 : 256 / ROW;  // rows per 256-byte bank line
  static constexpr int ROWS_PER_LOAD = 1024 / ROW;  // rows one direct-to-LDS instruction fills
  static constexpr int MERGE_ROWS = D / 2 + 4;  // a lane's O, two maxima and two denominators
  static constexpr int LDS_BYTES = 2 * HALF > 4 * MERGE_ROWS * 64 * 4 ? 2 * HALF : 4 * MERGE_ROWS * 64 * 4;
  // 16 lanes of a K operand read touch 16 consecutive rows at one chunk index, 32 lanes of a V
  // operand read 8 rows (4 g .. 4 g + 3 of two lane groups) at one slot index; rows lie 256 bytes
  // apart or closer.  XOR-ing the chunk (K) or the slot (V) with the row's bank-line index spreads them.
  __device__ static constexpr int k_swizzle(int row) { return (row / ROWS_PER_LINE) & (CHUNKS - 1); }
  __device__ static constexpr int v_swizzle(int row) { return (row / ROWS_PER_LINE) & (SLOTS - 1); }
};
// KT given row-major: a block is D rows (one per d) of 64 keys, 128 bytes; 32 lanes of a K operand
// read touch rows 8 g .. 8 g + 3 of two lane groups (two rows to a bank line) at one 32-byte slot.
__device__ constexpr int kt_swizzle(int d) { return ((d >> 1) & 1) | (((d >> 3) & 1) << 1); }
// Wave priorities of the two kinds of slot: the matrix slot is the longer one and its MFMAs
// should not queue behind the partner wave's vector instructions (worth ~0.5 % at 16 x 2048 x 128).
constexpr int PRIO_A = 2, PRIO_B = 0;
constexpr float LOG2E = 1.44269504088896340736f;
constexpr float STALE_REFERENCE = 1.0e12f;  // ~2^40: an exponential beyond it moves the reference

// One direct-to-LDS load: 64 lanes x 16 bytes from `base + voff` (voff per lane) to the 1 KiB at
// LDS address `lds_addr` (wave-uniform), lane l to slot l.  Written as assembly so that the
// compiler does not know of it: it would otherwise make every later LDS read wait for all such
// loads in flight (it cannot tell the stages apart), which serialises a block's softmax behind
// the next block's fetch.  The waits that matter are the explicit ones before the barriers.
__device__ inline void dma16(const uint8_t *base, uint32_t voff, uint32_t lds_addr) {
  asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2" : : "s"(lds_addr), "v"(voff), "s"(base));
}
__device__ inline uint32_t lds_address(const void *p) {
  return uint32_t(reinterpret_cast<uintptr_t>((lds_void *)p));
}

__device__ inline v2i read_tr16(const uint8_t *p) {
  const v4s r = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_v4s *)p);
  return __builtin_bit_cast(v2i, r);
}

// RAGGED: m need not be a multiple of 128 nor n2 of 128.  Query rows past m are computed on
// a clamped (valid) row and not stored; the key blocks are dealt ceil/floor to the two halves,
// loads past the end of K / V are clamped to the entry's last 16 bytes (finite data, weighted
// by exp(-inf) = 0), and the scores of keys past n2 are set to -inf before the softmax.
// KT_ROWS: KT is given row-major, [b][k][n2] with n2 fastest (the reference's default layout for
// the Compose's third parameter) instead of k-fastest.  A block of 64 keys is then D rows of 128
// bytes in LDS (one row per d), and the K operand comes out of it through the same transposing
// read that serves V.  n2 must be a multiple of 8.
// QG: query groups of 32 per workgroup (4 or 2): the Compose's tile_out over its rows.  A workgroup
// is 2 * QG waves; with 2 groups the four waves share a compute unit's LDS and matrix cores between
// them alone, which pays when 128-query blocks would leave half of the compute units without work
// or pad a short query dimension.
template <int D, bool RAGGED, bool KT_ROWS, int QG>
__global__ __launch_bounds__(512) void k_attn(const void *q, const void *kt, const void *v, float *out, uint32_t b, uint32_t m,
                                              uint32_t n2, uint32_t n_out, uint32_t key_splits, float *partials) {
  // Scalar arguments (the file is built with kernel-argument preloading): the first fourteen
  // dwords arrive in SGPRs with the wave instead of through a load the prologue would wait for.
  struct {
    const void *q, *kt, *v;
    float *out;
    uint32_t b, m, n2, n_out, key_splits;
    float *partials;
  } const p = {q, kt, v, out, b, m, n2, n_out, key_splits, partials};
  typedef Dims<D> DD;
#ifdef MRL_ATTN_TRACE  // timing build: cycle stamps replace the first floats of a wave's first output row
  const uint64_t t_start = __builtin_amdgcn_s_memtime(), r_start = __builtin_amdgcn_s_memrealtime();
  uint64_t t_wait = 0, t_slot_a = 0, t_slot_b = 0;
#define MRL_ATTN_SYNC() do { const uint64_t t_ = __builtin_amdgcn_s_memtime(); __syncthreads(); t_wait += __builtin_amdgcn_s_memtime() - t_; } while (0)
#define MRL_ATTN_TIMED(acc, stmt) do { const uint64_t t_ = __builtin_amdgcn_s_memtime(); stmt; acc += __builtin_amdgcn_s_memtime() - t_; } while (0)
#else
#define MRL_ATTN_SYNC() __syncthreads()
#define MRL_ATTN_TIMED(acc, stmt) stmt
#endif
  constexpr int ROW = DD::ROW, TILE = DD::TILE, HALF = DD::HALF;
  constexpr int NC = D / 32;   // 32-wide chunks of d: k steps of S = K.Q
  constexpr int NDB = D / 16;  // 16-row blocks of O^T
  constexpr int NKB = BKV / 16, NKC = BKV / 32;  // 16-key blocks of S^T, 32-key k steps of O += V.P
  extern __shared__ __attribute__((aligned(1024))) uint8_t lds[];
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int qg = wave % QG, half = wave / QG;  // query group, key half
  constexpr int BQ = 32 * QG;
  const int lr = lane & 15, lgp = lane >> 4;   // position within a block's 16 rows / columns, lane group
  // Workgroups go to the 8 XCDs round-robin.  All query blocks of a batch entry share its K
  // and V, so a batch entry's blocks are kept on one XCD (one L2) whenever the counts allow:
  // XCD x takes the x-th run of consecutive (entry, block) pairs.
  const uint32_t nqb = (p.m + BQ - 1) / BQ, total = nqb * p.b;
  uint32_t lin = blockIdx.x;
  if (total % 8 == 0) lin = (lin % 8) * (total / 8) + lin / 8;
  const int64_t head = lin / nqb;
  const int q0 = int(lin % nqb) * BQ + qg * 32;
  // Key blocks of this half: [first_block, first_block + nblocks); both halves run `steps`
  // iterations so that they meet at the same barriers.
  const int all_blocks = int((p.n2 + BKV - 1) / BKV);
  // With key_splits > 1 (few queries, many keys: too few workgroups otherwise) blockIdx.y picks
  // a contiguous share of the key blocks; the result is then a partial (max, denominator, O)
  // triple per split, merged by k_attn_merge.
  int split_first = 0, split_end = all_blocks;
  if (p.key_splits > 1) {
    const int per = (all_blocks + int(p.key_splits) - 1) / int(p.key_splits);
    split_first = min(all_blocks, int(blockIdx.y) * per);
    split_end = min(all_blocks, split_first + per);
  }
  const int my_blocks = split_end - split_first;
  const int steps = (my_blocks + 1) / 2;
  const int first_block = split_first + (half ? steps : 0);
  const int nblocks = half ? my_blocks - steps : steps;
  const uint32_t head_bytes = p.n2 * ROW;  // K or V of one batch entry

  const uint8_t *K = (const uint8_t *)p.kt + head * p.n2 * ROW;
  const uint8_t *V = (const uint8_t *)p.v + head * p.n2 * ROW;
  uint8_t *my_lds = lds + half * HALF;

  // Q^T operands: block column qb (queries 16 qb + l % 16 of the wave's 32), chunk c of d:
  // lane (l % 16, l / 16) holds d = 32 c + 8 (l / 16) .. + 7.
  // Only the waves of half 0 load them; their partners of half 1, which own the same queries,
  // get them through LDS at the first barrier (below): the start-up of a workgroup is bound by
  // what it asks of its compute unit's load path, and Q twice was two fifths of that.
  v4i qf[2][NC];
  if (!half) {
#pragma unroll
    for (int qb = 0; qb < 2; qb++) {
      const int q_row = RAGGED ? min(q0 + 16 * qb + lr, int(p.m) - 1) : q0 + 16 * qb + lr;
      const uint8_t *Q = (const uint8_t *)p.q + (head * p.m + q_row) * int64_t(ROW);
#pragma unroll
      for (int c = 0; c < NC; c++) qf[qb][c] = *(const v4i *)(Q + c * 64 + lgp * 16);
    }
  }

  // Block staging.  One direct-to-LDS instruction fills 1 KiB (4 rows at D = 128); lane l lands
  // in 16-byte slot l.  K rows are XOR-swizzled by chunk, V rows by 32-byte slot; each lane
  // fetches the global chunk that belongs in its slot.  The 4 waves of a key half share its
  // instructions: PER_WAVE for K and as many for V per block and wave.
  constexpr int PER_WAVE = TILE / 1024 / QG;
  static_assert(PER_WAVE >= 1 && 16 % PER_WAVE == 0, "the fetches are dealt evenly over the softmax's exponentials");
  const int ld_row = lane / DD::CHUNKS, ld_pc = lane % DD::CHUNKS;
  uint32_t k_src[PER_WAVE], v_src[PER_WAVE];
#pragma unroll
  for (int i = 0; i < PER_WAVE; i++) {
    const int q = qg * PER_WAVE + i, row = q * DD::ROWS_PER_LOAD + ld_row;
    if constexpr (KT_ROWS) {
      // 8 rows (d) of 128 bytes per instruction
      const int krow = q * 8 + (lane >> 3), kpc = lane & 7;
      k_src[i] = krow * (p.n2 * 2) + ((((kpc >> 1) ^ kt_swizzle(krow)) << 5) | ((kpc & 1) << 4));
    } else {
      k_src[i] = row * ROW + ((ld_pc ^ DD::k_swizzle(row)) << 4);
    }
    v_src[i] = row * ROW + ((((ld_pc >> 1) ^ DD::v_swizzle(row)) << 5) | ((ld_pc & 1) << 4));
  }
  // Fetch of this lane's chunk i of K (V) block kb into the KiB at LDS address `dst`.  The block's
  // offset is wave-uniform and goes into the scalar base; only the ragged form, which clamps
  // each lane's address to the entry's last bytes, forms the offset per lane.
  auto fetch_k = [&](int kb, int i, uint32_t dst) {
    const uint32_t block = uint32_t(first_block + kb) * (KT_ROWS ? BKV * 2 : TILE);
    if constexpr (RAGGED) dma16(K, min(block + k_src[i], head_bytes - 16), dst);
    else dma16(K + block, k_src[i], dst);
  };
  auto fetch_v = [&](int kb, int i, uint32_t dst) {
    const uint32_t block = uint32_t(first_block + kb) * TILE;
    if constexpr (RAGGED) dma16(V, min(block + v_src[i], head_bytes - 16), dst);
    else dma16(V + block, v_src[i], dst);
  };
  // O^T: block row db (d = 16 db + 4 (l / 16) + i in register i), block column qb.
  v4f o[NDB][2];
#pragma unroll
  for (int db = 0; db < NDB; db++)
#pragma unroll
    for (int qb = 0; qb < 2; qb++)
#pragma unroll
      for (int r = 0; r < 4; r++) o[db][qb][r] = 0.0f;
  float m_run[2] = {-3.0e38f, -3.0e38f};
  // The denominators come out of the second product too: one more block row of V^T, all ones,
  // sums P over the keys (every register of every lane then holds its query's denominator: the
  // sum of the very values, rounded to bf16, that O is made of).
  v4f den[2];
#pragma unroll
  for (int qb = 0; qb < 2; qb++)
#pragma unroll
    for (int r = 0; r < 4; r++) den[qb][r] = 0.0f;
  const v4i ones = {0x3f803f80, 0x3f803f80, 0x3f803f80, 0x3f803f80};

  // LDS of a key half: K tiles 0 and 1, then V tiles 0, 1 and 2.  K block kb goes to K tile
  // kb & 1, V block kb to V tile kb % 3.  A block index past the half's last block fetches the
  // last block again, into a tile that nobody reads any more, so that every slot issues the same
  // number of loads and the counts given to s_waitcnt below hold.
  auto issue_k = [&](int kb) {
    const int src = min(kb, nblocks - 1);
    const uint32_t dst = lds_address(my_lds + (kb & 1) * TILE);
#pragma unroll
    for (int i = 0; i < PER_WAVE; i++) fetch_k(src, i, dst + (qg * PER_WAVE + i) * 1024);
  };
  auto issue_v = [&](int kb) {
    const int src = min(kb, nblocks - 1);
    const uint32_t dst = lds_address(my_lds + (2 + kb % 3) * TILE);
#pragma unroll
    for (int i = 0; i < PER_WAVE; i++) fetch_v(src, i, dst + (qg * PER_WAVE + i) * 1024);
  };

  // The two key halves of a workgroup run the same program ONE SLOT APART.  A wave's work per
  // block is a slot of matrix-core work (A_j: O += V.P of block j - 1, then S = K.Q of block j)
  // and a slot of vector-unit work (B_j: the online softmax of block j), a barrier after each.
  // Half 1 passes one extra barrier first, so whenever the wave of half 0 on a SIMD is in a matrix
  // slot its partner of half 1 is in a softmax slot and the other way round: measured, one wave
  // issues a vector instruction every 6-7 cycles at best and an MFMA wave beside it keeps its
  // full rate, so the exponentials of one half ride under the MFMAs of the other, where two
  // waves in step would queue for the matrix core and then for the vector unit.
  //   B_j issues the fetches of V(j + 1) (into the tile of V(j - 2), last read in A_(j-1)) and of
  //   K(j + 2) (into the tile of K(j), last read in A_j), one instruction at a time between the
  //   exponentials (the softmax slot is the shorter one; in the matrix slot they cost more), and
  //   ends by waiting for everything but its own fetches: K(j + 1) and V(j), which A_(j+1) reads,
  //   have then landed.
  // S^T: block row kb (key 16 kb + 4 (l / 16) + i in register i), block column qb.
  v4f s[NKB][2];
  // P^T operands of the second product: k step kc covers key blocks 2 kc and 2 kc + 1; lane group g
  // holds keys 4 g .. 4 g + 3 of each, its own eight values of S^T.
  v8bf pb[NKC][2];
  // Lane-dependent, block-independent parts of the operand addresses (the swizzles depend on the
  // lane only: the row offsets that vary per read are multiples of the swizzle periods).
  uint32_t v_lane[NDB], k_lane[KT_ROWS ? NKB : NC];
  {
    const int piece = (lr & 3) * 8;     // a lane's 8 bytes of a transposing read's 32
    const int vrow = 4 * lgp + (lr >> 2);
#pragma unroll
    for (int db = 0; db < NDB; db++) v_lane[db] = vrow * ROW + ((db ^ DD::v_swizzle(vrow)) << 5) + piece;
    if constexpr (KT_ROWS) {
      const int drow = 8 * lgp + (lr >> 2);
#pragma unroll
      for (int kb = 0; kb < NKB; kb++) k_lane[kb] = drow * (BKV * 2) + ((kb ^ kt_swizzle(drow)) << 5) + piece;
    } else {
#pragma unroll
      for (int c = 0; c < NC; c++) k_lane[c] = lr * ROW + (((4 * c + lgp) ^ DD::k_swizzle(lr)) << 4);
    }
  }
  // s_waitcnt vmcnt(n) (six bits: the low four and two at the top), the other counters left alone.
  constexpr int WAIT_BUT_TWO = 0x0F70 | ((2 * PER_WAVE) & 15) | (((2 * PER_WAVE) >> 4) << 14);
  // Start-up.  Everything a workgroup asks for at once goes through its compute unit's vector
  // cache at 64 bytes a clock, so only what the first matrix slot needs is asked for first: Q and
  // half 0's K(0).  Behind the barrier that says they are in go V(0) and K(1), and all of half 1's
  // fetches, which have half 0's first slot to land in.  (The wait is for everything in flight, Q's
  // operand registers included: from there on the only loads in flight are the block fetches,
  // which the compiler does not know of, so it adds no waits of its own for them in the loop.)
  if (nblocks > 0 && !half) issue_k(0);
  __builtin_amdgcn_s_waitcnt(0x0F70);
  {
    // Q's operands from half 0 to half 1, through V tiles 1 and 2 of half 1 (QG * D * 64 bytes: two
    // tiles at most), which no fetch touches before that half's first softmax slot.
    static_assert(QG * D * 64 <= 2 * TILE, "the exchange fits the two tiles");
    v4i *qx = (v4i *)(lds + HALF + 3 * TILE) + qg * (2 * NC * 64) + lane;
    if (!half) {
#pragma unroll
      for (int qb = 0; qb < 2; qb++)
#pragma unroll
        for (int c = 0; c < NC; c++) qx[(qb * NC + c) * 64] = qf[qb][c];
    }
    __syncthreads();
    if (half) {
#pragma unroll
      for (int qb = 0; qb < 2; qb++)
#pragma unroll
        for (int c = 0; c < NC; c++) qf[qb][c] = qx[(qb * NC + c) * 64];
    }
  }
  if (nblocks > 0) {
    if (half) issue_k(0);
    issue_v(0);
    issue_k(1);
  }
  if (half) {
    __builtin_amdgcn_s_waitcnt(WAIT_BUT_TWO);  // K(0)
    __syncthreads();
  }
  // K operand of key block kb, chunk c of d: lane (key 16 kb + l % 16, group g) holds d = 32 c + 8 g .. + 7.
  auto read_k = [&](const uint8_t *lk, int kb, int c) {
    if constexpr (KT_ROWS) {
      const uint8_t *a = lk + k_lane[kb] + c * 32 * (BKV * 2);
      const v2i lo = read_tr16(a), hi = read_tr16(a + 4 * (BKV * 2));
      return v4i{lo[0], lo[1], hi[0], hi[1]};
    } else {
      return *(const v4i *)(lk + k_lane[c] + kb * 16 * ROW);
    }
  };
  // V^T operand of block row db, k step kc: lane (d 16 db + l % 16, group g) holds keys 4 g .. + 3 of
  // key block 2 kc, then of key block 2 kc + 1.
  auto read_v = [&](const uint8_t *lv, int db, int kc) {
    const uint8_t *a = lv + v_lane[db] + kc * 32 * ROW;
    const v2i lo = read_tr16(a), hi = read_tr16(a + 16 * ROW);
    return v4i{lo[0], lo[1], hi[0], hi[1]};
  };
  auto mfma = [](v4i a, auto bop, v4f c) {
    return __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(v8bf, a), __builtin_bit_cast(v8bf, bop), c, 0, 0, 0);
  };
  // A matrix slot is a sequence of steps of two MFMAs on one operand read from LDS (a V operand
  // against the two block columns of P, or a K operand against those of Q); the operand of step
  // t + AHEAD is read behind the MFMAs of step t.  Two steps ahead measured best (16 x 2048 x 128:
  // 33.8 us; 1: 34.1, 3: 33.9, 4: 34.5, 8: 35.6, 12: 36.1, none: 45.4): the reads ahead of a
  // slot's first MFMA are time the matrix core of that SIMD stands still.
  constexpr int PV_ROWS = NDB + 1;   // block rows of the second product: O^T's and the denominators'
  constexpr int PV_STEPS = NKC * PV_ROWS, QK_STEPS = NC * NKB, AHEAD = 2, RING = AHEAD + 1;
  constexpr int K_READS = KT_ROWS ? 2 : 1;   // LDS instructions per K operand (V: always 2)
  v4i ring[RING];
  // steps [first, last) of the sequence PV(0 .. PV_STEPS) then QK(0 .. QK_STEPS)
  auto run_steps = [&](auto first_c, auto last_c, const uint8_t *lv, const uint8_t *lk) {
    constexpr int FIRST = decltype(first_c)::value, LAST = decltype(last_c)::value;
    auto fetch = [&](int t) {
      if (t < PV_STEPS) {
        if (t % PV_ROWS < NDB) ring[t % RING] = read_v(lv, t % PV_ROWS, t / PV_ROWS);
      } else {
        ring[t % RING] = read_k(lk, (t - PV_STEPS) % NKB, (t - PV_STEPS) / NKB);
      }
    };
    auto reads_of = [](int t) { return t < PV_STEPS ? (t % PV_ROWS < NDB ? 2 : 0) : K_READS; };
#pragma unroll
    for (int t = FIRST; t < LAST && t < FIRST + AHEAD; t++) fetch(t);
#pragma unroll
    for (int t = FIRST; t < LAST; t++) {
      if (t + AHEAD < LAST) fetch(t + AHEAD);
      const v4i a = ring[t % RING];
      if (t < PV_STEPS) {
        const int db = t % PV_ROWS, kc = t / PV_ROWS;
        if (db < NDB) {
          o[db][0] = mfma(a, pb[kc][0], o[db][0]);
          o[db][1] = mfma(a, pb[kc][1], o[db][1]);
        } else {
          den[0] = mfma(ones, pb[kc][0], den[0]);
          den[1] = mfma(ones, pb[kc][1], den[1]);
        }
      } else {
        const int kb = (t - PV_STEPS) % NKB, c = (t - PV_STEPS) / NKB;
        s[kb][0] = mfma(a, qf[0][c], s[kb][0]);
        s[kb][1] = mfma(a, qf[1][c], s[kb][1]);
      }
    }
    // The order wanted of the scheduler: the first AHEAD operands' reads, then per step the reads
    // of the operand AHEAD steps on and the step's two MFMAs.
    auto reads_group = [&](int t) {   // the builtin wants literal sizes
      if (reads_of(t) == 2) __builtin_amdgcn_sched_group_barrier(0x100, 2, 0);
      else if (reads_of(t) == 1) __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
    };
#pragma unroll
    for (int t = FIRST; t < LAST && t < FIRST + AHEAD; t++) reads_group(t);
#pragma unroll
    for (int t = FIRST; t < LAST; t++) {
      if (t + AHEAD < LAST) reads_group(t + AHEAD);
      __builtin_amdgcn_sched_group_barrier(0x008, 2, 0);
    }
  };
  auto zero_s = [&]() {
#pragma unroll
    for (int kb = 0; kb < NKB; kb++)
#pragma unroll
      for (int qb = 0; qb < 2; qb++)
#pragma unroll
        for (int r = 0; r < 4; r++) s[kb][qb][r] = 0.0f;
  };
  using std::integral_constant;
  // Slot A of the first block: S = K.Q only.
  auto slot_a_first = [&]() {
    zero_s();
    run_steps(integral_constant<int, PV_STEPS>{}, integral_constant<int, PV_STEPS + QK_STEPS>{}, my_lds, my_lds);
  };
  // Slot A of block j, 1 <= j < nblocks: O += V.P of block j - 1, then S = K.Q of block j.
  auto slot_a = [&](int j, const uint8_t *lv) {
    __builtin_amdgcn_s_setprio(PRIO_A);
    zero_s();
    run_steps(integral_constant<int, 0>{}, integral_constant<int, PV_STEPS + QK_STEPS>{}, lv, my_lds + (j & 1) * TILE);
  };
  // Slot A after the last block: O += V.P of block nblocks - 1.
  auto slot_a_last = [&](const uint8_t *lv) {
    run_steps(integral_constant<int, 0>{}, integral_constant<int, PV_STEPS>{}, lv, my_lds);
  };
  // Slot B of block j: the online softmax of S into P (bf16), the running maxima and denominators.
  auto slot_b = [&](int j) {
    __builtin_amdgcn_s_setprio(PRIO_B);
    if (RAGGED) {
      // Keys past n2 (only ever in the very last block): their scores leave the softmax.
      const int valid = int(p.n2) - (first_block + j) * BKV;
      if (valid < BKV) {
#pragma unroll
        for (int kb = 0; kb < NKB; kb++)
#pragma unroll
          for (int qb = 0; qb < 2; qb++)
#pragma unroll
            for (int r = 0; r < 4; r++)
              if (kb * 16 + 4 * lgp + r >= valid) s[kb][qb][r] = -__builtin_inff();
      }
    }
    // The running reference m_run (exponentials are taken as exp(x - m_run); the final division
    // by the denominator, accumulated against the same reference, cancels it exactly) is set from
    // the first block's maxima and then left alone: a block's maximum is only looked for when its
    // largest exponential shows that some score outgrew the reference by more than 2^40, far
    // inside f32 and bf16 range.  That block's exponentials are then redone against the moved
    // reference, and the accumulators (the denominators' among them) rescaled.  This takes the maximum
    // (a quarter of the softmax's instructions and two cross-lane exchanges) out of almost every block.
    auto move_reference = [&]() {
#pragma unroll
      for (int qb = 0; qb < 2; qb++) {
        float mx = s[0][qb][0];
#pragma unroll
        for (int kb = 0; kb < NKB; kb++)
#pragma unroll
          for (int r = 0; r < 4; r++) mx = fmaxf(mx, s[kb][qb][r]);
        mx = fmaxf(mx, __shfl_xor(mx, 16));
        mx = fmaxf(mx, __shfl_xor(mx, 32));
        const float m_new = fmaxf(m_run[qb], mx);
        const float alpha = __builtin_amdgcn_exp2f((m_run[qb] - m_new) * LOG2E);
        m_run[qb] = m_new;
#pragma unroll
        for (int r = 0; r < 4; r++) den[qb][r] *= alpha;
#pragma unroll
        for (int db = 0; db < NDB; db++)
#pragma unroll
          for (int r = 0; r < 4; r++) o[db][qb][r] *= alpha;
      }
    };
    if (j == 0) move_reference();
    // In base 2: exp(x - m) = 2^(x*log2e - m*log2e).
    const float neg_m2[2] = {-m_run[0] * LOG2E, -m_run[1] * LOG2E};
    float pmax[2] = {0.0f, 0.0f};   // the block's largest exponential per query: what tells a stale reference
    // The fetches of V(j + 1) and K(j + 2) go out one instruction at a time between the exponentials.
    const int ksrc = min(j + 2, nblocks - 1), vsrc = min(j + 1, nblocks - 1);
    const uint32_t kdst = lds_address(my_lds + (j & 1) * TILE), vdst = lds_address(my_lds + (2 + (j + 1) % 3) * TILE);
#pragma unroll
    for (int kb = 0; kb < NKB; kb++)
#pragma unroll
      for (int qb = 0; qb < 2; qb++)
#pragma unroll
        for (int r = 0; r < 4; r++) {
          const float e = __builtin_amdgcn_exp2f(__builtin_fmaf(s[kb][qb][r], LOG2E, neg_m2[qb]));
          pmax[qb] = fmaxf(pmax[qb], e);
          pb[kb / 2][qb][(kb % 2) * 4 + r] = (__bf16)e;
          constexpr int EVERY = 16 / PER_WAVE;
          const int n = (kb * 2 + qb) * 4 + r;   // 0 .. 31
          if (n % EVERY == EVERY - 1) {
            const int i = n / EVERY;
            if (i < PER_WAVE) fetch_v(vsrc, i, vdst + (qg * PER_WAVE + i) * 1024);
            else fetch_k(ksrc, i - PER_WAVE, kdst + (qg * PER_WAVE + i - PER_WAVE) * 1024);
          }
        }
    if (j > 0 && __any(!(pmax[0] < STALE_REFERENCE) || !(pmax[1] < STALE_REFERENCE))) {
      move_reference();
#pragma unroll
      for (int qb = 0; qb < 2; qb++) {
        const float neg2 = -m_run[qb] * LOG2E;
#pragma unroll
        for (int kb = 0; kb < NKB; kb++)
#pragma unroll
          for (int r = 0; r < 4; r++)
            pb[kb / 2][qb][(kb % 2) * 4 + r] = (__bf16)__builtin_amdgcn_exp2f(__builtin_fmaf(s[kb][qb][r], LOG2E, neg2));
      }
    }
    __builtin_amdgcn_s_waitcnt(WAIT_BUT_TWO);
  };

  // Every wave passes steps + 1 pairs of barriers; a half with fewer blocks idles through the rest.
#ifdef MRL_ATTN_TRACE
  const uint64_t t_loop = __builtin_amdgcn_s_memtime();
#endif
  if (nblocks > 0) slot_a_first();
  MRL_ATTN_SYNC();
  if (nblocks > 0) slot_b(0);
  MRL_ATTN_SYNC();
  int vstage = 0;  // V stage of block j - 1
  for (int j = 1; j < nblocks; j++) {
    MRL_ATTN_TIMED(t_slot_a, slot_a(j, my_lds + (2 + vstage) * TILE));
    vstage = vstage == 2 ? 0 : vstage + 1;
    MRL_ATTN_SYNC();
    MRL_ATTN_TIMED(t_slot_b, slot_b(j));
    MRL_ATTN_SYNC();
  }
  if (nblocks > 0) slot_a_last(my_lds + (2 + vstage) * TILE);
#ifdef MRL_ATTN_TRACE
  const uint64_t t_loop_end = __builtin_amdgcn_s_memtime();
#endif
  for (int j = max(nblocks, 1); j <= steps; j++) {
    __syncthreads();
    __syncthreads();
  }
  if (!half) __syncthreads();

  // Merge the two key halves: (m, d, O) of half 1 goes through LDS to the wave of half 0
  // that owns the same queries.  Layout [value][lane] keeps lanes on distinct banks.
  const float l_tot[2] = {den[0][0], den[1][0]};
  __syncthreads();  // all K/V reads are done: the staging area is free
  // [quad of values][lane], 16 bytes per lane: lanes on distinct banks, one instruction per quad.
  constexpr int MQ = DD::MERGE_ROWS / 4;   // a lane's quads: O^T's blocks, then (m, m, l, l)
  v4f *mbuf = (v4f *)lds + qg * (MQ * 64) + lane;
  if (half == 1) {
#pragma unroll
    for (int db = 0; db < NDB; db++)
#pragma unroll
      for (int qb = 0; qb < 2; qb++) mbuf[(db * 2 + qb) * 64] = o[db][qb];
    mbuf[(NDB * 2) * 64] = v4f{m_run[0], m_run[1], l_tot[0], l_tot[1]};
  }
  __syncthreads();
  if (half == 0) {
    const v4f ml = mbuf[(NDB * 2) * 64];
#pragma unroll
    for (int qb = 0; qb < 2; qb++) {
      const float m1 = ml[qb], l1 = ml[2 + qb];
      const float mm = fmaxf(m_run[qb], m1);
      const float a0 = __builtin_amdgcn_exp2f((m_run[qb] - mm) * LOG2E), a1 = __builtin_amdgcn_exp2f((m1 - mm) * LOG2E);
      const int row = q0 + 16 * qb + lr;
      if (p.key_splits > 1) {
        // Partial triple of this split, relative to mm: rows of D + 4 floats (O, then the maximum,
        // then the denominator), [query][split].
        if (row < int(p.m)) {
          float *part = p.partials + ((head * p.m + row) * int64_t(p.key_splits) + blockIdx.y) * (D + 4);
#pragma unroll
          for (int db = 0; db < NDB; db++) {
            const v4f v = o[db][qb] * a0 + mbuf[(db * 2 + qb) * 64] * a1;
            *(float4 *)(part + db * 16 + 4 * lgp) = float4{v[0], v[1], v[2], v[3]};
          }
          if (lgp == 0) part[D] = mm, part[D + 1] = l_tot[qb] * a0 + l1 * a1;
        }
        continue;
      }
      const float inv = 1.0f / (l_tot[qb] * a0 + l1 * a1);
      const float w0 = a0 * inv, w1 = a1 * inv;
      float *orow = p.out + (head * p.m + row) * int64_t(p.n_out);
      const bool whole_rows = p.n_out == D;  // else: padded head dim, columns past n_out are dropped
      if (!RAGGED || row < int(p.m))
#pragma unroll
        for (int db = 0; db < NDB; db++) {
          const v4f v = o[db][qb] * w0 + mbuf[(db * 2 + qb) * 64] * w1;
          const int col = db * 16 + 4 * lgp;
          if (whole_rows) {
            *(float4 *)(orow + col) = float4{v[0], v[1], v[2], v[3]};   // ordinary stores: non-temporal ones measured 33.0 against 32.5 us a launch
          } else {
            if (col + 0 < int(p.n_out)) orow[col + 0] = v[0];
            if (col + 1 < int(p.n_out)) orow[col + 1] = v[1];
            if (col + 2 < int(p.n_out)) orow[col + 2] = v[2];
            if (col + 3 < int(p.n_out)) orow[col + 3] = v[3];
          }
        }
    }
  }
#ifdef MRL_ATTN_TRACE
  {
    const uint64_t t_issued = __builtin_amdgcn_s_memtime();
    __builtin_amdgcn_s_waitcnt(0x0F70);   // the stores have drained
    const uint64_t t_end = __builtin_amdgcn_s_memtime(), r_end = __builtin_amdgcn_s_memrealtime();
    if (lane == 0) {
      uint32_t *stamp = (uint32_t *)(p.out + (head * p.m + q0 + 16 * half) * int64_t(p.n_out));
      stamp[0] = uint32_t(t_loop - t_start), stamp[1] = uint32_t(t_loop_end - t_loop), stamp[2] = uint32_t(t_issued - t_loop_end);
      stamp[3] = uint32_t(t_end - t_issued), stamp[4] = uint32_t(t_wait), stamp[5] = uint32_t(t_slot_a), stamp[6] = uint32_t(t_slot_b);
      stamp[7] = uint32_t(r_end - r_start), stamp[8] = uint32_t(r_start), stamp[9] = uint32_t(r_end);
      stamp[10] = uint32_t(t_end - t_start);
    }
  }
#endif
}

// out[row][0 .. n_out) = sum_s O_s * 2^((m_s - M) log2 e) / sum_s l_s * 2^((m_s - M) log2 e), M = max_s m_s:
// the parts formula of morello/src/spec.rs:107-132 over the splits' triples.  One thread per
// output element; a split that saw no key has l = 0 and the smallest m, so it drops out.
__global__ __launch_bounds__(256) void k_attn_merge(const float *__restrict__ partials, float *__restrict__ out,
                                                    uint64_t rows, uint32_t splits, uint32_t d, uint32_t n_out) {
  const uint64_t i = uint64_t(blockIdx.x) * 256 + threadIdx.x;
  if (i >= rows * n_out) return;
  const uint64_t row = i / n_out;
  const uint32_t col = uint32_t(i % n_out);
  const float *part = partials + row * splits * (d + 4);
  const uint32_t stride = d + 4;
  // Eight splits' loads in flight at a time: the loop is all latency otherwise (35 splits one
  // after another took 20 us).
  constexpr uint32_t U = 8;
  float m = -3.0e38f;
  for (uint32_t s0 = 0; s0 < splits; s0 += U) {
    float ms[U];
#pragma unroll
    for (uint32_t u = 0; u < U; u++) {
      const float v = part[(s0 + u < splits ? s0 + u : 0) * stride + d];  // always a valid address
      ms[u] = s0 + u < splits ? v : -3.0e38f;
    }
#pragma unroll
    for (uint32_t u = 0; u < U; u++) m = fmaxf(m, ms[u]);
  }
  float num = 0.0f, den = 0.0f;
  for (uint32_t s0 = 0; s0 < splits; s0 += U) {
    float ms[U], ls[U], os[U];
#pragma unroll
    for (uint32_t u = 0; u < U; u++) {
      const bool in = s0 + u < splits;
      const float *p = part + (in ? s0 + u : 0) * stride;
      const float mv = p[d], lv = p[d + 1], ov = p[col];
      ms[u] = in ? mv : -3.0e38f, ls[u] = in ? lv : 0.0f, os[u] = in ? ov : 0.0f;
    }
#pragma unroll
    for (uint32_t u = 0; u < U; u++) {
      const float w = __builtin_amdgcn_exp2f((ms[u] - m) * LOG2E);
      num += os[u] * w;
      den += ls[u] * w;
    }
  }
  out[row * n_out + col] = num / den;
}

}  // namespace

// Key splits for a launch: 1 unless the (entry, query block) pairs fill at most half of the
// compute units and there are keys enough to share out (four blocks of 64 per workgroup at
// least, and more time saved than the partial results cost).  The workgroups then number at most one per compute unit: measured on 256 units, 256
// workgroups stream K and V at 4.9-5.6 TB/s where 320 or 512 reach 3.6-4.8.
uint32_t g_compute_units = 256;

uint32_t attn_key_splits(const AttnArgs &a) {
  const uint64_t units = g_compute_units;  // set by mrl_init: planning makes no runtime call
  const uint64_t bq = a.query_block, groups = uint64_t((a.m + bq - 1) / bq) * a.b, blocks = (a.n2 + BKV - 1) / BKV;
  if (groups == 0) return 1;
  const uint64_t splits = std::min<uint64_t>({units / groups, blocks / 4, 256});
  // A workgroup spends ~0.5 us per block; the partial results and their merge cost ~4 us.
  if (splits < 2 || blocks * (splits - 1) <= 8 * splits) return 1;
  return uint32_t(splits);
}
size_t attn_partial_bytes(const AttnArgs &a, uint32_t splits) {
  return splits > 1 ? size_t(a.b) * a.m * splits * (a.k + 4) * sizeof(float) : 0;
}

bool attn_applicable(const AttnArgs &a) {
  auto al16 = [](const void *p) { return (reinterpret_cast<uintptr_t>(p) & 15) == 0; };
  return a.k == a.n && (a.k == 32 || a.k == 64 || a.k == 128) && a.n_out >= 1 && a.n_out <= a.n && a.m && a.n2 && a.b &&
         (!a.kt_rows || a.n2 % 8 == 0) && (a.key_splits <= 1 || (a.partials && a.key_splits <= 65535)) &&
         uint64_t(a.n2) * a.k * 2 < (1ull << 31) && (a.query_block == 64 || a.query_block == 128) &&
         uint64_t((a.m + a.query_block - 1) / a.query_block) * a.b < (1u << 31) &&
         al16(a.q) && al16(a.kt) && al16(a.v) && al16(a.out);
}

namespace {
template <int D, bool RAGGED, bool KT_ROWS, int QG>
hipError_t launch_one(const AttnArgs &a, hipStream_t stream) {
  constexpr int LDS = Dims<D>::LDS_BYTES, BQ = 32 * QG;
  static std::atomic<uint64_t> lds_limit_set{0};
  if (!plan::recording()) {
    hipError_t e = raise_lds_limit(lds_limit_set, (const void *)k_attn<D, RAGGED, KT_ROWS, QG>, LDS);
    if (e != hipSuccess) return e;
  }
  const dim3 grid(((a.m + BQ - 1) / BQ) * a.b, std::max(1u, a.key_splits));
  plan::work(plan::UNIT_MFMA_BF16, 4.0 * a.b * a.m * a.n2 * D,
             double(a.b) * (2.0 * a.m * D + 4.0 * a.n2 * D + 4.0 * a.m * a.n_out) + attn_partial_bytes(a, a.key_splits),
             // the softmax between the two products shares the issue slots and the launch has fixed
             // costs the model does not price: 1.17 x the MFMA time at the model's sustained rate puts
             // 16 x 2048 x 128 at 37 us (measured 33-35 with the launch gap) and head dim 64, half the
             // heads or twice the keys at 0.87-0.9 of their measured times; four waves hide less than
             // eight: 1.2 x that
             (QG == 2 ? 1.2 : 1.0) * 1.17 * 4.0 * BQ * D * (double((a.n2 + BKV - 1) / BKV) * BKV / std::max(1u, a.key_splits)),
             3000.0);
  MRL_LAUNCH((k_attn<D, RAGGED, KT_ROWS, QG>), grid, dim3(128 * QG), LDS, stream, a.q, a.kt, a.v, a.out, a.b, a.m, a.n2, a.n_out,
             a.key_splits, a.partials);
  if (a.key_splits > 1) {
    const uint64_t rows = uint64_t(a.b) * a.m, total = rows * a.n_out;
    plan::work(plan::UNIT_STREAM, 0, double(attn_partial_bytes(a, a.key_splits)) + 4.0 * total);
    MRL_LAUNCH(k_attn_merge, dim3(uint32_t((total + 255) / 256)), dim3(256), 0, stream, a.partials, a.out, rows,
                       a.key_splits, uint32_t(D), a.n_out);
  }
  return mrl::plan::last_error();
}

template <int D, int QG>
hipError_t launch_for(const AttnArgs &a, hipStream_t stream) {
  const bool whole = a.m % (32 * QG) == 0 && a.n2 % (2 * BKV) == 0;
  if (a.kt_rows) return whole ? launch_one<D, false, true, QG>(a, stream) : launch_one<D, true, true, QG>(a, stream);
  return whole ? launch_one<D, false, false, QG>(a, stream) : launch_one<D, true, false, QG>(a, stream);
}
}  // namespace

hipError_t launch_attn(const AttnArgs &a, hipStream_t stream) {
  if (!attn_applicable(a)) return hipErrorInvalidValue;
  if (a.query_block == 64) {
    switch (a.k) {
      case 32: return launch_for<32, 2>(a, stream);
      case 64: return launch_for<64, 2>(a, stream);
      default: return launch_for<128, 2>(a, stream);
    }
  }
  switch (a.k) {
    case 32: return launch_for<32, 4>(a, stream);
    case 64: return launch_for<64, 4>(a, stream);
    default: return launch_for<128, 4>(a, stream);
  }
}

}  // namespace mrl
