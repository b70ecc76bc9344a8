// Host side of the C ABI declared in include/morello_amd.h: Spec validation, layout
// handling and dispatch onto the kernels.  No compute happens on the CPU here; a Spec the
// fast kernels do not cover runs on the generic GPU kernels, and a missing device is an
// error, never a fallback.
#include <hip/hip_runtime.h>

#include <cstdio>
#include <algorithm>
#include <cstring>
#include <map>
#include <memory>
#include <mutex>
#include <string>
#include <vector>

#include "kernels.h"
#include "layout_factor.h"

namespace {

thread_local std::string g_last_error;
int g_device = -1;

int hip_fail(hipError_t e, const char *what) {
  g_last_error = std::string(what) + ": " + hipGetErrorString(e);
  return MRL_ERR_HIP;
}
#define HIP_TRY(expr)                                  \
  do {                                                 \
    hipError_t e_ = (expr);                            \
    if (e_ != hipSuccess) return hip_fail(e_, #expr);  \
  } while (0)

bool valid_dtype(int d) { return d >= MRL_U8 && d <= MRL_BF16; }

uint64_t volume(const uint32_t *s, uint32_t r) {
  uint64_t v = 1;
  for (uint32_t i = 0; i < r; i++) v *= s[i];
  return v;
}

uint32_t expected_params(int kind) {
  switch (kind) {
    case MRL_SPEC_MATMUL: case MRL_SPEC_CONV: return 3;
    case MRL_SPEC_SOFTMAX: case MRL_SPEC_MOVE: return 2;
    case MRL_SPEC_COMPOSE_MSM: return 4;
    case MRL_SPEC_FILL: return 1;
    case MRL_SPEC_MAX: case MRL_SPEC_DIVIDE_VEC: case MRL_SPEC_DIVIDE_VEC_SCALAR:
    case MRL_SPEC_BROADCAST: case MRL_SPEC_ONE_PREFIX: return 2;
    case MRL_SPEC_SOFTMAX_DENOMINATOR: case MRL_SPEC_SOFTMAX_DENOMINATOR_AND_MAX:
    case MRL_SPEC_SOFTMAX_DENOMINATOR_AND_UNSCALED: return 3;
    case MRL_SPEC_SOFTMAX_DENOMINATOR_AND_MAX_FROM_PARTS:
    case MRL_SPEC_SOFTMAX_DENOMINATOR_AND_UNSCALED_FROM_MAX: case MRL_SPEC_SOFTMAX_COMPLETE: return 4;
    default: return 0;
  }
}

// Kinds whose spec_shape is one tensor's shape and which reduce or broadcast over scan_dim.
bool is_parts_kind(int kind) { return kind >= MRL_SPEC_MAX && kind <= MRL_SPEC_DIVIDE_VEC_SCALAR; }

// Bit i set: parameter i has size one on scan_dim (spec.rs:499-583).
uint32_t reduced_mask(int kind) {
  switch (kind) {
    case MRL_SPEC_MAX: return 0b0010;
    case MRL_SPEC_SOFTMAX_DENOMINATOR: case MRL_SPEC_SOFTMAX_DENOMINATOR_AND_MAX: return 0b0110;
    case MRL_SPEC_SOFTMAX_DENOMINATOR_AND_MAX_FROM_PARTS: return 0b1100;
    case MRL_SPEC_SOFTMAX_DENOMINATOR_AND_UNSCALED: return 0b0010;
    case MRL_SPEC_SOFTMAX_DENOMINATOR_AND_UNSCALED_FROM_MAX: case MRL_SPEC_SOFTMAX_COMPLETE: return 0b0110;
    case MRL_SPEC_DIVIDE_VEC_SCALAR: return 0b0010;
    case MRL_SPEC_BROADCAST: return 0b0001;
    default: return 0;
  }
}

uint32_t expected_rank(const mrl_spec &s) {
  switch (s.kind) {
    case MRL_SPEC_MATMUL: return 4;
    case MRL_SPEC_CONV: return 7;
    case MRL_SPEC_SOFTMAX: case MRL_SPEC_MOVE: return s.rank;
    case MRL_SPEC_COMPOSE_MSM: return 5;
    default: return s.kind >= MRL_SPEC_FILL && s.kind <= MRL_SPEC_ONE_PREFIX ? s.rank : 0;
  }
}

// morello/src/spec.rs:467-583
int parameter_shape(const mrl_spec &s, uint32_t idx, uint32_t *shape, uint32_t *rank) {
  const uint32_t *ss = s.spec_shape;
  switch (s.kind) {
    case MRL_SPEC_MATMUL:
      *rank = 3;
      if (idx == 0) shape[0] = ss[0], shape[1] = ss[1], shape[2] = ss[2];
      else if (idx == 1) shape[0] = ss[0], shape[1] = ss[2], shape[2] = ss[3];
      else if (idx == 2) shape[0] = ss[0], shape[1] = ss[1], shape[2] = ss[3];
      else return MRL_ERR_BAD_SPEC;
      return MRL_OK;
    case MRL_SPEC_CONV: {
      const uint32_t b = ss[0], f = ss[1], c = ss[2], oh = ss[3], ow = ss[4], fh = ss[5], fw = ss[6];
      *rank = 4;
      if (idx == 0) shape[0] = b, shape[1] = c, shape[2] = oh + fh - 1, shape[3] = ow + fw - 1;
      else if (idx == 1) shape[0] = f, shape[1] = c, shape[2] = fh, shape[3] = fw;
      else if (idx == 2) shape[0] = b, shape[1] = f, shape[2] = oh, shape[3] = ow;
      else return MRL_ERR_BAD_SPEC;
      return MRL_OK;
    }
    case MRL_SPEC_SOFTMAX:
    case MRL_SPEC_MOVE:
      if (idx > 1 || s.rank > MRL_MAX_RANK) return MRL_ERR_BAD_SPEC;
      *rank = s.rank;
      for (uint32_t d = 0; d < s.rank; d++) shape[d] = ss[d];
      return MRL_OK;
    case MRL_SPEC_COMPOSE_MSM: {
      // spec_shape [b, m, k, n2, n]; parameters V, Q, KT, out (spec.rs:3329-3365).
      const uint32_t b = ss[0], m = ss[1], k = ss[2], n2 = ss[3], n = ss[4];
      *rank = 3;
      if (idx == 0) shape[0] = b, shape[1] = n2, shape[2] = n;
      else if (idx == 1) shape[0] = b, shape[1] = m, shape[2] = k;
      else if (idx == 2) shape[0] = b, shape[1] = k, shape[2] = n2;
      else if (idx == 3) shape[0] = b, shape[1] = m, shape[2] = n;
      else return MRL_ERR_BAD_SPEC;
      return MRL_OK;
    }
    case MRL_SPEC_ONE_PREFIX:
      if (idx > 1 || s.rank + idx > MRL_MAX_RANK) return MRL_ERR_BAD_SPEC;
      *rank = s.rank + idx;
      if (idx == 1) shape[0] = 1;
      for (uint32_t d = 0; d < s.rank; d++) shape[d + idx] = ss[d];
      return MRL_OK;
    default:
      if (s.kind < MRL_SPEC_FILL || s.kind > MRL_SPEC_BROADCAST || idx >= expected_params(s.kind) ||
          s.rank > MRL_MAX_RANK || (s.kind != MRL_SPEC_FILL && s.scan_dim >= s.rank))
        return MRL_ERR_BAD_SPEC;
      *rank = s.rank;
      for (uint32_t d = 0; d < s.rank; d++) shape[d] = ss[d];
      if (s.kind != MRL_SPEC_FILL && ((reduced_mask(s.kind) >> idx) & 1)) shape[s.scan_dim] = 1;
      return MRL_OK;
  }
}

// morello/src/spec.rs:1204-1245.  0 In, 1 Out, 2 InOut.
int parameter_direction(const mrl_spec &s, uint32_t idx) {
  const uint32_t n = expected_params(s.kind);
  if (n == 0 || idx >= n) return -1;
  const int acc = s.accum ? 2 : 1;
  switch (s.kind) {
    case MRL_SPEC_DIVIDE_VEC: case MRL_SPEC_DIVIDE_VEC_SCALAR: return idx == 0 ? 2 : 0;
    case MRL_SPEC_SOFTMAX_DENOMINATOR_AND_MAX: return idx == 0 ? 0 : acc;
    case MRL_SPEC_SOFTMAX_DENOMINATOR_AND_MAX_FROM_PARTS: return idx < 2 ? 0 : acc;
    case MRL_SPEC_SOFTMAX_DENOMINATOR_AND_UNSCALED: return idx == 0 ? 0 : 1;
    case MRL_SPEC_SOFTMAX_DENOMINATOR_AND_UNSCALED_FROM_MAX: return idx < 2 ? 0 : (idx == 2 ? acc : 1);
    case MRL_SPEC_MATMUL: case MRL_SPEC_CONV: case MRL_SPEC_MAX: case MRL_SPEC_SOFTMAX_DENOMINATOR:
      return idx + 1 < n ? 0 : acc;
    default: return idx + 1 < n ? 0 : 1;
  }
}

int check_spec(const mrl_spec *sp) {
  if (!sp) return MRL_ERR_NULL;
  const mrl_spec &s = *sp;
  const uint32_t np = expected_params(s.kind);
  if (np == 0) return MRL_ERR_UNSUPPORTED;
  if (s.n_params != np) return MRL_ERR_BAD_SPEC;
  if (s.rank == 0 || s.rank > MRL_MAX_SPEC_RANK || s.rank != expected_rank(s)) return MRL_ERR_BAD_SPEC;
  if (s.kind == MRL_SPEC_SOFTMAX && (s.rank > MRL_MAX_RANK || s.scan_dim >= s.rank)) return MRL_ERR_BAD_SPEC;
  if (s.kind == MRL_SPEC_MOVE && s.rank > MRL_MAX_RANK) return MRL_ERR_BAD_SPEC;
  if (s.kind >= MRL_SPEC_FILL && s.rank > MRL_MAX_RANK) return MRL_ERR_BAD_SPEC;
  if (s.kind == MRL_SPEC_ONE_PREFIX && s.rank + 1 > MRL_MAX_RANK) return MRL_ERR_BAD_SPEC;
  if ((is_parts_kind(s.kind) && s.kind != MRL_SPEC_DIVIDE_VEC) || s.kind == MRL_SPEC_BROADCAST) {
    if (s.scan_dim >= s.rank) return MRL_ERR_BAD_SPEC;
  }
  if (s.kind == MRL_SPEC_FILL && s.scan_dim > MRL_FILL_MIN) return MRL_ERR_BAD_SPEC;
  for (uint32_t d = 0; d < s.rank; d++)
    if (s.spec_shape[d] == 0) return MRL_ERR_BAD_SPEC;
  for (uint32_t i = 0; i < np; i++) {
    if (!valid_dtype(s.dtypes[i])) return MRL_ERR_BAD_SPEC;
    uint32_t shape[MRL_MAX_RANK], rank;
    if (parameter_shape(s, i, shape, &rank) != MRL_OK) return MRL_ERR_BAD_SPEC;
    // DimSize volume is a u32 in the reference (tensorspec.rs:180-182); buffer indices are i32.
    if (volume(shape, rank) > 0x7fffffffull) return MRL_ERR_TOO_LARGE;
    uint32_t phys[MRL_MAX_PHYS];
    if (!mrl::physical_shape(s.layouts[i], shape, rank, phys)) return MRL_ERR_BAD_LAYOUT;
  }
  switch (s.kind) {
    case MRL_SPEC_MATMUL:
    case MRL_SPEC_CONV:
      break;  // every dtype triple, bf16 outputs included (run_bf16_output)
    case MRL_SPEC_SOFTMAX:
      if (s.dtypes[0] != MRL_F32 || s.dtypes[1] != MRL_F32) return MRL_ERR_UNSUPPORTED;
      break;
    case MRL_SPEC_COMPOSE_MSM:
      if (s.dtypes[3] != MRL_F32) return MRL_ERR_UNSUPPORTED;
      break;
    case MRL_SPEC_FILL:
      // NegInf exists only for floats (verification.rs fill_neg_inf).
      if (s.scan_dim == MRL_FILL_NEG_INF && s.dtypes[0] != MRL_F32 && s.dtypes[0] != MRL_BF16)
        return MRL_ERR_BAD_SPEC;
      break;
    case MRL_SPEC_BROADCAST:
    case MRL_SPEC_ONE_PREFIX:
      if (s.dtypes[0] != s.dtypes[1]) return MRL_ERR_UNSUPPORTED;
      break;
    default:
      if (is_parts_kind(s.kind)) {
        for (uint32_t i = 0; i < np; i++)
          if (s.dtypes[i] != MRL_F32) return MRL_ERR_UNSUPPORTED;
        // The accumulating form of this one is unimplemented in the reference too (spec.rs:688).
        if (s.kind == MRL_SPEC_SOFTMAX_DENOMINATOR_AND_UNSCALED && s.accum) return MRL_ERR_UNSUPPORTED;
      }
      break;
  }
  return MRL_OK;
}

// A parameter prepared for the kernels: either used in place through strides, or staged
// into a dense row-major scratch buffer by the relayout kernel.
struct Prepared {
  mrl::Strided t;
  void *scratch = nullptr;      // non-null when staged
  void *user = nullptr;
  mrl::LayoutEval user_layout;  // valid when staged
  mrl::LayoutEval dense_layout;
  mrl_layout user_desc, dense_desc;  // the same two as descriptors
  uint64_t count = 0;
  uint32_t elem = 0;
};

// Scratch memory of one call.  Requests are carved out of an arena that stays allocated per
// stream (work on a stream runs in order, so the next call may overwrite what this one staged):
// hipMallocAsync / hipFreeAsync cost several microseconds of host time apiece for small blocks
// and hundreds for blocks of 100 MB, more than the kernels of most Specs.  A call holds its
// stream's arena until it returns, so host threads that share a stream take turns.  The arena
// starts at 64 MiB; a call that asks for more gets the excess from the stream-ordered allocator
// and leaves behind an arena large enough for its next run (up to ARENA_MAX_BYTES).
constexpr size_t ARENA_BYTES = size_t(64) << 20, ARENA_MAX_BYTES = size_t(16) << 30;
struct Arena {
  std::mutex in_use;
  void *base = nullptr;
  size_t size = 0;
};
std::mutex g_arenas_mutex;
std::map<hipStream_t, std::unique_ptr<Arena>> g_arenas;

Arena *arena_of(hipStream_t stream) {
  std::lock_guard<std::mutex> lock(g_arenas_mutex);
  std::unique_ptr<Arena> &slot = g_arenas[stream];
  if (!slot) slot.reset(new Arena);
  return slot.get();
}

// Frees the arena of a stream whose work has completed.
void drop_arena(hipStream_t stream) {
  std::unique_ptr<Arena> arena;
  {
    std::lock_guard<std::mutex> lock(g_arenas_mutex);
    auto it = g_arenas.find(stream);
    if (it == g_arenas.end()) return;
    arena = std::move(it->second);
    g_arenas.erase(it);
  }
  std::lock_guard<std::mutex> lock(arena->in_use);
  if (arena->base) (void)hipFree(arena->base);
}

// Scratch for callers that may not allocate (mrl_run_noalloc): one array per GPU, there from the
// moment the library's code is loaded onto it until the process ends.  Host code never uses
// the array's name as an address: mrl_init asks the runtime where the current device holds it
// (hipGetSymbolAddress) and keeps that pointer per device.
constexpr size_t NOALLOC_SCRATCH_BYTES = size_t(MRL_NOALLOC_SCRATCH_BYTES);
static __device__ __align__(256) unsigned char scratch[NOALLOC_SCRATCH_BYTES];
constexpr int MAX_DEVICES = 64;
void *g_scratch_ptr[MAX_DEVICES] = {};

struct Workspace {
  hipStream_t stream;
  std::vector<void *> allocs;
  Arena *arena = nullptr;  // locked while non-null
  size_t arena_used = 0;
  size_t requested = 0;    // everything this call asked for
  uint8_t *fixed = nullptr;  // non-null: requests come out of these fixed_size bytes and nowhere else
  size_t fixed_size = 0;
  bool fixed_overflow = false;
  explicit Workspace(hipStream_t s) : stream(s) {}
  Workspace(hipStream_t s, void *region, size_t bytes) : stream(s), fixed(static_cast<uint8_t *>(region)), fixed_size(bytes) {}
  Workspace(const Workspace &) = delete;
  Workspace &operator=(const Workspace &) = delete;
  hipError_t alloc(void **p, size_t bytes) {
    const size_t rounded = std::max<size_t>(256, (bytes + 255) & ~size_t(255));
    if (mrl::plan::recording()) {
      // Planning: a stand-in address, aligned as the allocator's are, never dereferenced.
      mrl::plan::Recorder *r = mrl::plan::g_recorder;
      *p = reinterpret_cast<void *>((uintptr_t(1) << 44) + r->scratch_bytes);
      r->scratch_bytes += rounded;
      return hipSuccess;
    }
    if (fixed) {
      if (rounded > fixed_size - arena_used) {
        fixed_overflow = true;
        return hipErrorOutOfMemory;
      }
      *p = fixed + arena_used;
      arena_used += rounded;
      return hipSuccess;
    }
    if (!arena) {
      arena = arena_of(stream);
      arena->in_use.lock();
    }
    requested += rounded;
    if (!arena->base && rounded <= ARENA_BYTES && hipMalloc(&arena->base, ARENA_BYTES) == hipSuccess)
      arena->size = ARENA_BYTES;
    if (arena->base && rounded <= arena->size - arena_used) {
      *p = static_cast<uint8_t *>(arena->base) + arena_used;
      arena_used += rounded;
      return hipSuccess;
    }
    hipError_t e = hipMallocAsync(p, rounded, stream);
    if (e == hipSuccess) allocs.push_back(*p);
    return e;
  }
  ~Workspace() {
    for (void *p : allocs) (void)hipFreeAsync(p, stream);
    if (!arena) return;
    if (requested > arena->size && requested <= ARENA_MAX_BYTES) {
      // Once per size: wait for the work that uses the old arena, free it, allocate one that
      // holds this call.
      size_t grown = ARENA_BYTES;
      while (grown < requested) grown *= 2;
      if (hipStreamSynchronize(stream) == hipSuccess) {
        if (arena->base) (void)hipFree(arena->base);
        arena->base = nullptr, arena->size = 0;
        if (hipMalloc(&arena->base, grown) == hipSuccess) arena->size = grown;
        else arena->base = nullptr;
      }
    }
    arena->in_use.unlock();
  }
};

// Same dtype, between the caller's layout of parameter `p` and its dense staging copy (to_dense:
// caller's -> dense): as a strided permutation of the two layouts' common view when they have
// one (Packed and OddEven dims are digits of their logical index), else by index arithmetic
// per element.
int relayout(const void *src, void *dst, bool to_dense, const Prepared &p, Workspace &ws) {
  const mrl_layout &from = to_dense ? p.user_desc : p.dense_desc, &to = to_dense ? p.dense_desc : p.user_desc;
  std::vector<mrl::MoveDim> view;
  if (mrl::common_view(from, to, p.t.shape, p.t.rank, &view)) {
    const hipError_t e = mrl::launch_move_view(src, p.t.dtype, dst, p.t.dtype, view.data(), uint32_t(view.size()), ws.stream);
    if (e == hipSuccess) return MRL_OK;
    if (e != hipErrorInvalidValue) HIP_TRY(e);
  }
  HIP_TRY(mrl::launch_relayout(src, dst, to_dense ? p.user_layout : p.dense_layout,
                               to_dense ? p.dense_layout : p.user_layout, p.elem, p.count, ws.stream));
  return MRL_OK;
}

int prepare(const mrl_spec &s, uint32_t idx, void *ptr, bool needs_read, Workspace &ws, Prepared *out) {
  uint32_t shape[MRL_MAX_RANK], rank;
  parameter_shape(s, idx, shape, &rank);
  out->t.dtype = s.dtypes[idx];
  out->t.rank = rank;
  out->user = ptr;
  out->elem = uint32_t(mrl_dtype_size(s.dtypes[idx]));
  out->count = volume(shape, rank);
  for (uint32_t d = 0; d < MRL_MAX_RANK; d++) out->t.shape[d] = d < rank ? shape[d] : 1;
  if (mrl::layout_strides(s.layouts[idx], shape, rank, out->t.stride)) {
    out->t.ptr = ptr;
    return MRL_OK;
  }
  mrl_layout dense;
  mrl_layout_row_major(shape, rank, &dense);
  // A layout with Packed dims can still be row-major order (layout![0, 1, 1p16], say).
  std::vector<mrl::MoveDim> view;
  if (mrl::common_view(s.layouts[idx], dense, shape, rank, &view) &&
      mrl::same_order(view)) {
    out->t.ptr = ptr;
    mrl::layout_strides(dense, shape, rank, out->t.stride);
    return MRL_OK;
  }
  if (!mrl::make_layout_eval(s.layouts[idx], shape, rank, &out->user_layout) ||
      !mrl::make_layout_eval(dense, shape, rank, &out->dense_layout))
    return MRL_ERR_BAD_LAYOUT;
  HIP_TRY(ws.alloc(&out->scratch, out->count * out->elem));
  out->t.ptr = out->scratch;
  mrl::layout_strides(dense, shape, rank, out->t.stride);
  out->user_desc = s.layouts[idx], out->dense_desc = dense;
  if (needs_read) return relayout(ptr, out->scratch, true, *out, ws);
  return MRL_OK;
}

int finish_output(Prepared &p, Workspace &ws) {
  if (!p.scratch) return MRL_OK;
  return relayout(p.scratch, p.user, false, p, ws);
}

bool dense_row_major(const mrl::Strided &t) {
  int64_t run = 1;
  for (int d = int(t.rank) - 1; d >= 0; d--) {
    if (t.shape[d] == 1) continue;
    if (t.stride[d] != run) return false;
    run *= t.shape[d];
  }
  return true;
}

// Leading dimension / batch stride of a [b, r, c] tensor whose last dim is contiguous.
bool as_rows(const mrl::Strided &t, int64_t *ld, int64_t *batch_stride) {
  if (t.rank != 3) return false;
  if (t.shape[2] != 1 && t.stride[2] != 1) return false;
  // A single row has no stride of its own to go by, unless it is a padded one.
  *ld = (t.shape[1] == 1 && t.stride[1] < int64_t(t.shape[2])) ? int64_t(t.shape[2]) : t.stride[1];
  *batch_stride = t.shape[0] == 1 ? 0 : t.stride[0];
  return *ld >= int64_t(t.shape[2]);
}

int run_matmul(const mrl_spec &s, void *const *params, Workspace &ws,
               const mrl_matmul_schedule *sched = nullptr) {
  Prepared a, b, c;
  int rc;
  if ((rc = prepare(s, 0, params[0], true, ws, &a)) != MRL_OK) return rc;
  if ((rc = prepare(s, 1, params[1], true, ws, &b)) != MRL_OK) return rc;
  if ((rc = prepare(s, 2, params[2], s.accum != 0, ws, &c)) != MRL_OK) return rc;
  int da = s.dtypes[0], db = s.dtypes[1];
  const int dc = s.dtypes[2];
  // f32 output with one bf16 and one f32 input: the reference converts both inputs to the
  // output dtype before multiplying (verification.rs:115-134); widening the bf16 operand
  // (exact) makes it an f32 Matmul, which the matrix cores take.
  if (dc == MRL_F32 && ((da == MRL_BF16 && db == MRL_F32) || (da == MRL_F32 && db == MRL_BF16))) {
    Prepared &narrow = da == MRL_BF16 ? a : b;
    void *wide = nullptr;
    HIP_TRY(ws.alloc(&wide, narrow.count * sizeof(float)));
    HIP_TRY(mrl::launch_widen_bf16(narrow.t.ptr, wide, narrow.count, ws.stream));
    narrow.t.ptr = wide, narrow.t.dtype = MRL_F32, narrow.elem = sizeof(float);
    da = db = MRL_F32;
  }
  mrl::GemmArgs g;
  g.a = a.t.ptr, g.b = b.t.ptr, g.c = c.t.ptr;
  g.batch = s.spec_shape[0], g.m = s.spec_shape[1], g.k = s.spec_shape[2], g.n = s.spec_shape[3];
  g.accum = s.accum;
  // B either with n fastest (row-major) or with k fastest (col-major, layout![0,2,1]).
  bool b_ok = as_rows(b.t, &g.ldb, &g.sb);
  if (!b_ok) {
    mrl::Strided bt = b.t;  // view [b, k, n] as [b, n, k]
    std::swap(bt.shape[1], bt.shape[2]);
    std::swap(bt.stride[1], bt.stride[2]);
    b_ok = g.b_kmajor = as_rows(bt, &g.ldb, &g.sb);
  }
  bool rows = as_rows(a.t, &g.lda, &g.sa) && b_ok && as_rows(c.t, &g.ldc, &g.sc);
  mrl::Strided c_user = c.t;
  bool c_densified = false;
  // -1: no matrix-core kernel for these dtypes.
  const int kind = (da == MRL_I8 && db == MRL_I8 && dc == MRL_I32)       ? 0
                   : (da == MRL_U8 && db == MRL_I8 && dc == MRL_I32)     ? 1
                   : (da == MRL_BF16 && db == MRL_BF16 && dc == MRL_F32) ? 2
                   : (da == MRL_F32 && db == MRL_F32 && dc == MRL_F32)   ? 3
                                                                         : -1;
  // Operands the matrix-core kernels cannot walk in place are copied with the strided Move
  // first when that opens the fast path: A or C stored column-major becomes row-major, and rows
  // that are not whole 16-byte chunks (K or N not a multiple of 16 bytes) are padded with zeros
  // to the next chunk.  Two extra passes over an operand against a generic kernel that is tens
  // of times slower.
  // The generic kernel's threads each walk K on their own: measured ~2.5 us + 40 ns per step of
  // K + 2 ops per 3e6 per us; a copy pass costs ~3 us at these sizes, the matrix-core kernel
  // ~3.5 us + 0.45 us per 128 bytes of K.
  const double macs = double(g.m) * g.n * g.k * g.batch;
  const double generic_us = 2.5 + 0.04 * g.k + 2.0 * macs / 3e6;
  const double copies_us = 6.0 + 3.5 + 0.45 * double((uint64_t(g.k) * a.elem + 127) / 128);
  const bool worth_two_more_passes = macs >= 256.0 * 256 * 256 || generic_us > copies_us;
  if (!sched && kind >= 0 && worth_two_more_passes) {
    const int64_t per16 = 16 / int64_t(a.elem);
    auto walkable = [&](const mrl::Strided &t) {
      int64_t ld, bs;
      return as_rows(t, &ld, &bs) && ld % per16 == 0 && bs % per16 == 0;
    };
    auto densify = [&](Prepared &p, bool read, bool pad) -> int {
      mrl::Strided dense = p.t;
      const int64_t cols = p.t.shape[2], ld = pad ? (cols + per16 - 1) / per16 * per16 : cols;
      dense.stride[2] = 1, dense.stride[1] = ld, dense.stride[0] = int64_t(p.t.shape[1]) * ld;
      const size_t bytes = size_t(p.t.shape[0]) * dense.stride[0] * p.elem;
      HIP_TRY(ws.alloc(&dense.ptr, bytes));
      int64_t old_ld, old_bs;
      if (read && as_rows(p.t, &old_ld, &old_bs)) {  // rows stay rows: one pass, padding included
        HIP_TRY(mrl::launch_pad_rows(p.t, dense.ptr, uint32_t(ld), p.elem, ws.stream));
      } else if (read) {
        if (ld != cols) HIP_TRY(mrl::launch_fill_zero(dense.ptr, bytes, ws.stream));
        HIP_TRY(mrl::launch_move_strided(p.t, dense, ws.stream));
      }
      p.t = dense;
      return MRL_OK;
    };
    bool b_walkable = walkable(b.t);
    if (!b_walkable) {
      mrl::Strided bt = b.t;  // [b, n, k] view: B with k fastest needs whole chunks along K
      std::swap(bt.shape[1], bt.shape[2]);
      std::swap(bt.stride[1], bt.stride[2]);
      b_walkable = walkable(bt);
    }
    int64_t any_ld, any_bs;
    if (!walkable(a.t) && !b_walkable && a.elem == b.elem && as_rows(a.t, &any_ld, &any_bs) && as_rows(b.t, &any_ld, &any_bs)) {
      // Both operands keep their rows and only need them padded: the two copies in one launch.
      Prepared *both[2] = {&a, &b};
      mrl::Strided dense[2];
      for (int i = 0; i < 2; i++) {
        const Prepared &p = *both[i];
        dense[i] = p.t;
        const int64_t cols = p.t.shape[2], ld = (cols + per16 - 1) / per16 * per16;
        dense[i].stride[2] = 1, dense[i].stride[1] = ld, dense[i].stride[0] = int64_t(p.t.shape[1]) * ld;
        HIP_TRY(ws.alloc(&dense[i].ptr, size_t(p.t.shape[0]) * dense[i].stride[0] * p.elem));
      }
      HIP_TRY(mrl::launch_pad_rows_pair(a.t, dense[0].ptr, uint32_t(dense[0].stride[1]), b.t, dense[1].ptr,
                                        uint32_t(dense[1].stride[1]), a.elem, ws.stream));
      a.t = dense[0], b.t = dense[1];
      g.b_kmajor = false;
    } else {
      if (!walkable(a.t) && (rc = densify(a, true, true)) != MRL_OK) return rc;
      if (!b_walkable) {
        if ((rc = densify(b, true, true)) != MRL_OK) return rc;
        g.b_kmajor = false;
      }
    }
    int64_t ld, bs;
    c_densified = !as_rows(c.t, &ld, &bs);
    if (c_densified && (rc = densify(c, s.accum != 0, false)) != MRL_OK) return rc;
    g.a = a.t.ptr, g.b = b.t.ptr, g.c = c.t.ptr;
    b_ok = g.b_kmajor || as_rows(b.t, &g.ldb, &g.sb);
    rows = as_rows(a.t, &g.lda, &g.sa) && b_ok && as_rows(c.t, &g.ldc, &g.sc);
  }
  auto finish = [&]() -> int {
    if (c_densified) HIP_TRY(mrl::launch_move_strided(c.t, c_user, ws.stream));
    if (c_densified) c.t = c_user;
    return finish_output(c, ws);
  };
  if (sched) {
    // A manual schedule is honoured wherever the kernel can run, whatever the size model says.
    if (kind < 0 || !rows || g.b_kmajor || !mrl::gemm_possible(g, kind)) return MRL_ERR_UNSUPPORTED;
    hipError_t e = mrl::launch_gemm_scheduled(g, kind, sched->tile_m, sched->tile_n, sched->split_k, ws.stream, sched->staging);
    if (e == hipErrorInvalidValue) return MRL_ERR_UNSUPPORTED;
    HIP_TRY(e);
    return finish_output(c, ws);
  }
  if (kind >= 0 && rows && mrl::gemm_possible(g, kind) && mrl::gemm_pays(g, kind)) {
    uint32_t left = 0;
    const uint32_t splits = mrl::gemm_k_splits(g, kind, &left);
    if (splits > 1) {
      // Slices of K as batch entries writing dense partial results, summed into C in slice order;
      // what K has behind the equal slices is one more, shorter slice in a launch of its own.
      void *partial = nullptr;
      HIP_TRY(ws.alloc(&partial, size_t(splits + (left ? 1 : 0)) * g.m * g.n * 4));
      mrl::GemmArgs slices = g;
      slices.batch = splits, slices.k = (g.k - left) / splits;
      slices.sa = slices.k, slices.sb = g.b_kmajor ? int64_t(slices.k) : int64_t(slices.k) * g.ldb;
      slices.c = partial, slices.ldc = g.n, slices.sc = int64_t(g.m) * g.n, slices.accum = 0;
      HIP_TRY(mrl::launch_gemm(slices, kind, ws.stream));
      if (left) {
        mrl::GemmArgs rest = slices;
        const size_t elem = kind <= 1 ? 1 : kind == 2 ? 2 : 4;
        rest.batch = 1, rest.k = left;
        rest.a = (const char *)g.a + size_t(g.k - left) * elem;
        rest.b = (const char *)g.b + (g.b_kmajor ? size_t(g.k - left) : size_t(g.k - left) * g.ldb) * elem;
        rest.c = (char *)partial + size_t(splits) * g.m * g.n * 4;
        HIP_TRY(mrl::launch_gemm(rest, kind, ws.stream));
      }
      HIP_TRY(mrl::launch_sum_splits(partial, g.c, splits + (left ? 1 : 0), g.m, g.n, g.ldc, g.accum != 0, kind <= 1, ws.stream));
    } else {
      HIP_TRY(mrl::launch_gemm(g, kind, ws.stream));
    }
  } else
    HIP_TRY(mrl::launch_matmul_generic(a.t, b.t, c.t, s.accum, ws.stream));
  return finish();
}

// A lowering picked from outside (mrl_run_action / mrl_action_plan) instead of by the dispatch
// rules: which of a Conv's or a Compose's paths to take.  Zero everywhere = the rules decide.
struct Forced {
  int conv_path = 0;        // 1 fused kernel, 2 implicit Matmul (tile side conv_tile), 3 unfold + Matmul, 4 generic
  uint32_t conv_tile = 0;
  bool conv_rows = false;   // fused kernel: whole output rows per workgroup, pixels shared through LDS
  int msm_path = 0;         // 1 fused kernel (key_splits workgroups per query block), 2 staged
  uint32_t key_splits = 0;
  uint32_t query_block = 0; // fused kernel: queries per workgroup (64 or 128), 0 = the rule below
};
thread_local const Forced *g_forced = nullptr;

// Where the kernel of conv_small.hip is taken (switches for measurement builds).
// Measured against the implicit Matmul (us, this kernel / the other): int8 32 x (16 -> 16) x 110^2
// 3 x 3 19.5 / 33.8, 16 -> 48 27.3 / 32, 32 -> 32 32.8 / 36, 32 -> 48 39.4 / 36.7; bf16 16 -> 48 38.9 /
// 32.9; 8 x (16 -> 32) x 56^2 5.9 / 5.3, 8 x (32 -> 48) x 56^2 8.3 / 5.9: large images, and filters
// times window bytes within what 32 filters of a 288-byte window make.
#ifndef MRL_CONV_SMALL_MIN_PIXELS
#define MRL_CONV_SMALL_MIN_PIXELS 65536ull
#endif
#ifndef MRL_CONV_SMALL_MAX_BANK
#define MRL_CONV_SMALL_MAX_BANK 9216ull
#endif
#ifndef MRL_CONV_SMALL_MAX_FILTERS
#define MRL_CONV_SMALL_MAX_FILTERS 48u
#endif
#ifndef MRL_CONV_SMALL_MAX_WINDOW
#define MRL_CONV_SMALL_MAX_WINDOW 320ull
#endif

int run_conv(const mrl_spec &s, void *const *params, Workspace &ws) {
  const int forced = g_forced ? g_forced->conv_path : 0;
  Prepared img, filt, out;
  int rc;
  if ((rc = prepare(s, 0, params[0], true, ws, &img)) != MRL_OK) return rc;
  if ((rc = prepare(s, 1, params[1], true, ws, &filt)) != MRL_OK) return rc;
  if ((rc = prepare(s, 2, params[2], s.accum != 0, ws, &out)) != MRL_OK) return rc;
  // NHWC / KRSC: logical [n,c,h,w] with channel fastest, then w, then h.
  auto channels_last = [](const mrl::Strided &t) {
    const int64_t c = t.shape[1], h = t.shape[2], w = t.shape[3];
    (void)h;
    return (c == 1 || t.stride[1] == 1) && (w == 1 || t.stride[3] == c) &&
           (t.shape[2] == 1 || t.stride[2] == c * w) &&
           (t.shape[0] == 1 || t.stride[0] == c * w * int64_t(t.shape[2]));
  };
  mrl::ConvArgs cv;
  cv.image = img.t.ptr, cv.filters = filt.t.ptr, cv.out = out.t.ptr;
  cv.b = s.spec_shape[0], cv.f = s.spec_shape[1], cv.c = s.spec_shape[2], cv.oh = s.spec_shape[3];
  cv.ow = s.spec_shape[4], cv.fh = s.spec_shape[5], cv.fw = s.spec_shape[6];
  cv.accum = s.accum;
  const int di = s.dtypes[0], df = s.dtypes[1], dout = s.dtypes[2];
  const bool fast_types = (di == MRL_U8 || di == MRL_I8) && df == MRL_I8 && dout == MRL_I32;
  const uint32_t slabs = cv.c % 64 == 0 ? cv.fh * cv.fw * (cv.c / 64) : 0;
  const bool fused_shape = fast_types && cv.f % 64 == 0 && cv.f <= 64 * 65535 &&
                           (slabs == 1 || slabs == 2 || slabs == 3 || slabs == 4 || slabs == 6 || slabs == 9);
  // Matmul kind of the same dtypes (-1: none): any other shape runs as unfold + Matmul.
  const int kind = (di == MRL_I8 && df == MRL_I8 && dout == MRL_I32)       ? 0
                   : (di == MRL_U8 && df == MRL_I8 && dout == MRL_I32)     ? 1
                   : (di == MRL_BF16 && df == MRL_BF16 && dout == MRL_F32) ? 2
                   : (di == MRL_F32 && df == MRL_F32 && dout == MRL_F32)   ? 3
                                                                           : -1;
  const uint64_t pixels = uint64_t(cv.oh) * cv.ow, window = uint64_t(cv.fh) * cv.fw * cv.c;
  const int64_t per16 = 16 / int64_t(img.elem);
  const uint64_t row_elems = (window + per16 - 1) / per16 * per16;  // a window, padded to whole chunks
  // Windows of this many images are unfolded at a time.
  constexpr uint64_t UNFOLD_BYTES = uint64_t(1) << 30;
  const uint64_t image_rows_bytes = pixels * row_elems * img.elem;
  // One kernel (windows read in place, or a 1x1 filter) pays from 1e5 multiply-adds on, as a
  // Matmul does; unfolding first (two or three launches) from 1e6.
  const double macs = double(cv.b) * pixels * cv.f * window;
  const bool as_matmul = (!fused_shape || forced == 2 || forced == 3) && forced != 4 && kind >= 0 &&
                         row_elems * img.elem < (1u << 24) && macs >= 1e5;
  const bool can_unfold = image_rows_bytes <= UNFOLD_BYTES &&
                          (macs >= 1e6 || (cv.fh == 1 && cv.fw == 1 && row_elems == window));
  // Tensors in another permutation layout (NCHW, say) are moved to channels-last when a
  // matrix-core path takes the shape: three small extra passes against a generic kernel
  // that is hundreds of times slower.
  const mrl::Strided out_user = out.t;
  bool out_moved = false;
  if (fused_shape || as_matmul) {
    auto to_channels_last = [&](Prepared &p, bool read) -> int {
      if (channels_last(p.t)) return MRL_OK;
      mrl::Strided dense = p.t;
      HIP_TRY(ws.alloc(&dense.ptr, p.count * p.elem));
      const int64_t c = p.t.shape[1], h = p.t.shape[2], w = p.t.shape[3];
      dense.stride[1] = 1, dense.stride[3] = c, dense.stride[2] = c * w, dense.stride[0] = c * w * h;
      if (read) HIP_TRY(mrl::launch_move_strided(p.t, dense, ws.stream));
      p.t = dense;
      return MRL_OK;
    };
    if ((rc = to_channels_last(filt, true)) != MRL_OK) return rc;
    cv.filters = filt.t.ptr;
    // Two kernels take dense row-major (NCHW) tensors as they are, and those stay where they are:
    // the fused kernel writes planes of filters (the Move back would be the largest of the three:
    // 24 MB at the benchmark's shape), the kernel that forms windows in LDS also reads planes of
    // channels.
    const bool plain_choice = forced <= 1 && !(forced == 1 && g_forced->conv_rows);
    const bool img_planes = !channels_last(img.t) && dense_row_major(img.t), out_planes = !channels_last(out.t) && dense_row_major(out.t);
    if (plain_choice && !fused_shape && kind >= 0 && kind <= 3 && as_matmul && channels_last(filt.t) && (img_planes || out_planes)) {
      mrl::ConvArgs as_is = cv;
      as_is.in_planes = img_planes, as_is.out_planes = out_planes;
      if (mrl::conv_windows_applicable(as_is, kind)) cv = as_is;
    }
    if (!cv.in_planes && (rc = to_channels_last(img, true)) != MRL_OK) return rc;
    cv.image = img.t.ptr;
    if (fused_shape && plain_choice && out_planes && mrl::conv_i8_applicable(cv)) cv.out_planes = true;
    out_moved = !channels_last(out.t) && !cv.out_planes;
    if (!cv.out_planes && (rc = to_channels_last(out, s.accum != 0)) != MRL_OK) return rc;
    cv.out = out.t.ptr;
  }
  // The Conv as an implicit Matmul: left operand = the image's windows, B = the KRSC filters.
  mrl::GemmArgs conv_args;
  auto implicit_args = [&](mrl::GemmArgs *g) {
    const uint64_t c_bytes = uint64_t(cv.c) * img.elem, h = cv.oh + cv.fh - 1, w = cv.ow + cv.fw - 1;
    if (c_bytes % 16 != 0 || uint64_t(cv.b) * pixels >= (1ull << 31)) return false;
    g->a = img.t.ptr, g->b = filt.t.ptr, g->c = out.t.ptr;
    g->batch = 1, g->m = uint32_t(cv.b * pixels), g->n = cv.f, g->k = uint32_t(window);
    g->lda = 0, g->ldb = int64_t(window), g->ldc = cv.f;
    g->sa = g->sb = g->sc = 0;
    g->accum = s.accum;
    g->b_kmajor = true;
    g->conv.h = uint32_t(h), g->conv.w = uint32_t(w), g->conv.oh = cv.oh, g->conv.ow = cv.ow, g->conv.fw = cv.fw;
    g->conv.c_bytes = uint32_t(c_bytes);
    g->conv.image_bytes = uint64_t(cv.b) * h * w * c_bytes;
    return true;
  };
  const bool fused_ok = fast_types && channels_last(img.t) && channels_last(filt.t) && (channels_last(out.t) || cv.out_planes) &&
                        mrl::conv_i8_applicable(cv);
  const bool implicit_ok = as_matmul && !(cv.fh == 1 && cv.fw == 1) && implicit_args(&conv_args) &&
                           mrl::conv_gemm_applicable(conv_args, kind);
  const bool unfold_ok = as_matmul && can_unfold && (reinterpret_cast<uintptr_t>(img.t.ptr) & 15) == 0 &&
                         (reinterpret_cast<uintptr_t>(filt.t.ptr) & 15) == 0 && (reinterpret_cast<uintptr_t>(out.t.ptr) & 3) == 0;
  // Few channels per pixel (a first layer): the fused kernel that forms the windows in LDS.
  const bool windows_ok = kind >= 0 && kind <= 3 && as_matmul && (channels_last(img.t) || cv.in_planes) && channels_last(filt.t) &&
                          (channels_last(out.t) || cv.out_planes) && mrl::conv_windows_applicable(cv, kind) &&
                          !(forced == 1 && g_forced->conv_rows);
  // Short windows over pixels of whole chunks and few filters (early layers of 16 or 32 channels):
  // the filters stay in registers and the pixels come straight from memory.  Measured against
  // the implicit Matmul, whose 64-wide tiles are then mostly padding (us, this kernel / implicit):
  // 32 x (32 -> 32) x 112^2 3 x 3 int8 35.6 / 44.3, bf16 16 -> 16 24.7 / 40.1, int8 48 -> 48 2 x 2 at
  // 56^2 11.7 / 13.2; with 64 filters or more, or windows beyond five k steps, it is the slower one
  // (a wave has one tile of 16 pixels in flight: int8 32 -> 64 at 56^2 17.6 / 13.9, 16 -> 32 5 x 5 62.7 /
  // 47.3, bf16 32 -> 32 3 x 3 71.5 / 49.5), so those stay implicit.
  const bool small_ok = kind >= 0 && kind <= 2 && as_matmul && !(cv.fh == 1 && cv.fw == 1) && channels_last(img.t) &&
                        channels_last(filt.t) && channels_last(out.t) && mrl::conv_small_applicable(cv, kind) &&
                        cv.f <= MRL_CONV_SMALL_MAX_FILTERS &&
                        uint64_t(cv.fh) * cv.fw * cv.c * (kind == 2 ? 2 : 1) <= MRL_CONV_SMALL_MAX_WINDOW &&
                        uint64_t(cv.fh) * cv.fw * cv.c * (kind == 2 ? 2 : 1) * cv.f <= MRL_CONV_SMALL_MAX_BANK &&
                        uint64_t(cv.b) * cv.oh * cv.ow >= MRL_CONV_SMALL_MIN_PIXELS;
  if ((forced == 1 && !fused_ok && !windows_ok) || (forced == 2 && !implicit_ok) || (forced == 3 && !unfold_ok)) return MRL_ERR_UNSUPPORTED;
  if (fused_ok && forced <= 1) {
    const bool rows = forced == 1 && g_forced->conv_rows;
    if (rows && !mrl::conv_rows_applicable(cv)) return MRL_ERR_UNSUPPORTED;
    HIP_TRY(mrl::launch_conv_i8(cv, di == MRL_U8, ws.stream, rows));
  } else if (windows_ok && forced <= 1) {
    HIP_TRY(mrl::launch_conv_windows(cv, kind, ws.stream));
  } else if (small_ok && forced == 0) {
    HIP_TRY(mrl::launch_conv_small(cv, kind, ws.stream));
  } else if (implicit_ok && (forced == 0 || forced == 2)) {
    // Channel vectors of whole 16-byte chunks: the windows are read where they lie.  (A 1x1 filter
    // needs no window arithmetic: its image is the left operand of a plain Matmul, below.)
    // Few output tiles and long windows (deep layers on small images): slices of the window as
    // batch entries with partial results, summed in slice order, as for a Matmul.
    const uint32_t splits = forced == 2 ? 1 : mrl::gemm_k_splits(conv_args, kind);
    if (splits > 1) {
      void *partial = nullptr;
      HIP_TRY(ws.alloc(&partial, size_t(splits) * conv_args.m * conv_args.n * 4));
      mrl::GemmArgs slices = conv_args;
      slices.batch = splits, slices.k = conv_args.k / splits;
      slices.sb = int64_t(slices.k), slices.conv.slice_bytes = uint32_t(slices.k * img.elem);
      slices.c = partial, slices.ldc = conv_args.n, slices.sc = int64_t(conv_args.m) * conv_args.n, slices.accum = 0;
      HIP_TRY(mrl::launch_conv_gemm(slices, kind, ws.stream, 64));
      HIP_TRY(mrl::launch_sum_splits(partial, conv_args.c, splits, conv_args.m, conv_args.n, conv_args.ldc,
                                     s.accum != 0, kind <= 1, ws.stream));
    } else {
      HIP_TRY(mrl::launch_conv_gemm(conv_args, kind, ws.stream, forced == 2 ? g_forced->conv_tile : 0));
    }
  } else if (unfold_ok && (forced == 0 || forced == 3)) {
    // Filters in KRSC order are the B operand stored k-fastest; their rows padded like U's.
    const void *weights = filt.t.ptr;
    if (row_elems != window) {
      void *padded = nullptr;
      HIP_TRY(ws.alloc(&padded, size_t(cv.f) * row_elems * filt.elem));
      mrl::Strided flat;
      flat.ptr = filt.t.ptr, flat.dtype = filt.t.dtype, flat.rank = 3;
      flat.shape[0] = 1, flat.shape[1] = cv.f, flat.shape[2] = uint32_t(window);
      flat.stride[0] = 0, flat.stride[1] = int64_t(window), flat.stride[2] = 1;
      HIP_TRY(mrl::launch_pad_rows(flat, padded, uint32_t(row_elems), filt.elem, ws.stream));
      weights = padded;
    }
    // A 1x1 filter over whole chunks of channels: the image is U already.
    const bool in_place = cv.fh == 1 && cv.fw == 1 && row_elems == window;
    const uint32_t per_pass = uint32_t(std::min<uint64_t>(cv.b, std::max<uint64_t>(1, UNFOLD_BYTES / image_rows_bytes)));
    void *rows_buf = nullptr;
    if (!in_place) HIP_TRY(ws.alloc(&rows_buf, size_t(per_pass) * image_rows_bytes));
    const uint64_t image_bytes = uint64_t(cv.oh + cv.fh - 1) * (cv.ow + cv.fw - 1) * cv.c * img.elem;
    for (uint32_t b0 = 0; b0 < cv.b; b0 += per_pass) {
      const uint32_t nb = std::min(per_pass, cv.b - b0);
      const uint8_t *images = static_cast<const uint8_t *>(img.t.ptr) + b0 * image_bytes;
      if (!in_place)
        HIP_TRY(mrl::launch_unfold(images, rows_buf, nb, cv.c, cv.oh, cv.ow, cv.fh, cv.fw, uint32_t(row_elems),
                                   img.elem, ws.stream));
      mrl::GemmArgs g;
      g.a = in_place ? static_cast<const void *>(images) : rows_buf;
      g.b = weights;
      g.c = static_cast<uint8_t *>(out.t.ptr) + uint64_t(b0) * pixels * cv.f * out.elem;
      g.batch = 1, g.m = uint32_t(nb * pixels), g.n = cv.f, g.k = uint32_t(window);
      g.lda = g.ldb = int64_t(row_elems), g.ldc = cv.f;
      g.sa = g.sb = g.sc = 0;
      g.accum = s.accum;
      g.b_kmajor = true;
      if (!mrl::gemm_possible(g, kind)) return MRL_ERR_UNSUPPORTED;  // ruled out by the checks above
      HIP_TRY(mrl::launch_gemm(g, kind, ws.stream));
    }
  } else {
    HIP_TRY(mrl::launch_conv_generic(img.t, filt.t, out.t, s.accum, ws.stream));
  }
  if (out_moved) {
    HIP_TRY(mrl::launch_move_strided(out.t, out_user, ws.stream));
    out.t = out_user;
  }
  return finish_output(out, ws);
}

// A Softmax's two tensors and shape, possibly with the dims renumbered into storage order.
struct Shaped {
  uint32_t rank, scan_dim, shape[MRL_MAX_RANK];
  mrl::Strided in, out;
};

int run_softmax(const mrl_spec &s, void *const *params, Workspace &ws) {
  Prepared in, out;
  int rc;
  if ((rc = prepare(s, 0, params[0], true, ws, &in)) != MRL_OK) return rc;
  if ((rc = prepare(s, 1, params[1], false, ws, &out)) != MRL_OK) return rc;
  // The dims in the order the tensors are stored, when both are stored the same dense way: a
  // column-major tensor scanned along dim 0 is a row-major one scanned along its rows.
  Shaped v;
  v.rank = s.rank, v.scan_dim = s.scan_dim, v.in = in.t, v.out = out.t;
  for (uint32_t d = 0; d < MRL_MAX_RANK; d++) v.shape[d] = d < s.rank ? s.spec_shape[d] : 1;
  if (!dense_row_major(in.t) && s.spec_shape[s.scan_dim] > 1) {
    uint32_t order[MRL_MAX_RANK];
    bool same = true;
    for (uint32_t d = 0; d < s.rank; d++) {
      order[d] = d;
      same = same && (s.spec_shape[d] == 1 || in.t.stride[d] == out.t.stride[d]);
    }
    // size-one dims first (they address nothing), the others by falling stride
    std::stable_sort(order, order + s.rank, [&](uint32_t x, uint32_t y) {
      const bool ux = s.spec_shape[x] == 1, uy = s.spec_shape[y] == 1;
      if (ux != uy) return ux;
      return !ux && in.t.stride[x] > in.t.stride[y];
    });
    Shaped w = v;
    for (uint32_t i = 0; i < s.rank; i++) {
      const uint32_t d = order[i];
      w.shape[i] = s.spec_shape[d];
      w.in.shape[i] = w.out.shape[i] = s.spec_shape[d];
      w.in.stride[i] = in.t.stride[d], w.out.stride[i] = out.t.stride[d];
      if (d == s.scan_dim) w.scan_dim = i;
    }
    if (same && dense_row_major(w.in) && dense_row_major(w.out)) v = w;
  }
  // Trailing size-one dims do not change which dim is innermost.
  uint32_t last = v.rank - 1;
  while (last > v.scan_dim && v.shape[last] == 1) last--;
  if (v.scan_dim == last && dense_row_major(v.in) && dense_row_major(v.out) &&
      (reinterpret_cast<uintptr_t>(v.in.ptr) & 15) == 0 &&
      (reinterpret_cast<uintptr_t>(v.out.ptr) & 15) == 0) {
    const uint32_t cols = v.shape[v.scan_dim];
    void *scratch = nullptr;
    if (const size_t bytes = mrl::softmax_scratch_bytes(in.count / cols, cols)) HIP_TRY(ws.alloc(&scratch, bytes));
    HIP_TRY(mrl::launch_softmax_rows((const float *)v.in.ptr, (float *)v.out.ptr, in.count / cols,
                                     cols, scratch, ws.stream));
  } else if (v.scan_dim < last && dense_row_major(v.in) && dense_row_major(v.out) && in.count < (1ull << 31) &&
             [&] {
               uint64_t after = 1;
               for (uint32_t d = v.scan_dim + 1; d < v.rank; d++) after *= v.shape[d];
               return after >= 16;
             }()) {
    // The tensor as [before][scan][after] with `after` contiguous: the column kernel, 64
    // positions of `after` per workgroup; with few columns the scan dim is shared out as well.
    const uint32_t scan = v.shape[v.scan_dim];
    uint64_t before = 1, after = 1;
    for (uint32_t d = 0; d < v.scan_dim; d++) before *= v.shape[d];
    for (uint32_t d = v.scan_dim + 1; d < v.rank; d++) after *= v.shape[d];
    mrl::Strided vi, vo;
    vi.dtype = vo.dtype = MRL_F32, vi.rank = vo.rank = 3;
    for (uint32_t d = 0; d < MRL_MAX_RANK; d++) vi.shape[d] = vo.shape[d] = 1, vi.stride[d] = vo.stride[d] = 0;
    vi.shape[0] = vo.shape[0] = uint32_t(before), vi.shape[1] = vo.shape[1] = scan, vi.shape[2] = vo.shape[2] = uint32_t(after);
    vi.stride[0] = vo.stride[0] = int64_t(scan) * after, vi.stride[1] = vo.stride[1] = int64_t(after), vi.stride[2] = vo.stride[2] = 1;
    vi.ptr = v.in.ptr, vo.ptr = v.out.ptr;
    void *pairs = nullptr;
    if (const size_t bytes = mrl::softmax_cols_scratch_bytes(before * ((after + 63) / 64), scan)) HIP_TRY(ws.alloc(&pairs, bytes));
    HIP_TRY(mrl::launch_softmax_generic(vi, vo, 1, pairs, ws.stream));
  } else if (v.scan_dim < last && dense_row_major(v.in) && dense_row_major(v.out) && in.count < (1ull << 31) &&
             [&] {
               // Fewer than 16 contiguous elements behind the scan dim: the generic kernel, a
               // wavefront per line with strided accesses, measured 2.5 us + 10 ns per scan step on
               // small tensors; against it three or four launches, ~14 us.
               const double scan = v.shape[v.scan_dim];
               if (in.count <= (1u << 20)) return 2.5 + 0.010 * scan > 15.0;
               return true;
             }()) {
    // Scan dim made innermost by a transposing Move, the row kernels, and a Move back: three
    // passes of tuned kernels ([2149, 172] over dim 0: 57 -> 9 us; [1818, 10]: 23 -> 8 us).
    const uint32_t scan = v.shape[v.scan_dim];
    uint64_t before = 1, after = 1;
    for (uint32_t d = 0; d < v.scan_dim; d++) before *= v.shape[d];
    for (uint32_t d = v.scan_dim + 1; d < v.rank; d++) after *= v.shape[d];
    void *turned = nullptr, *scratch = nullptr;
    HIP_TRY(ws.alloc(&turned, in.count * sizeof(float)));
    mrl::Strided as_given, as_turned;  // both over the index space (before, scan, after)
    as_given.dtype = as_turned.dtype = MRL_F32, as_given.rank = as_turned.rank = 3;
    for (uint32_t d = 0; d < MRL_MAX_RANK; d++) as_given.shape[d] = as_turned.shape[d] = 1, as_given.stride[d] = as_turned.stride[d] = 0;
    as_given.shape[0] = as_turned.shape[0] = uint32_t(before);
    as_given.shape[1] = as_turned.shape[1] = scan;
    as_given.shape[2] = as_turned.shape[2] = uint32_t(after);
    as_given.stride[0] = int64_t(scan) * after, as_given.stride[1] = int64_t(after), as_given.stride[2] = 1;
    as_turned.stride[0] = int64_t(scan) * after, as_turned.stride[1] = 1, as_turned.stride[2] = scan;
    as_given.ptr = v.in.ptr, as_turned.ptr = turned;
    HIP_TRY(mrl::launch_move_strided(as_given, as_turned, ws.stream));
    const uint64_t rows = before * after;
    if (const size_t bytes = mrl::softmax_scratch_bytes(rows, scan)) HIP_TRY(ws.alloc(&scratch, bytes));
    HIP_TRY(mrl::launch_softmax_rows((const float *)turned, (float *)turned, rows, scan, scratch, ws.stream));
    as_given.ptr = v.out.ptr;
    HIP_TRY(mrl::launch_move_strided(as_turned, as_given, ws.stream));
  } else {
    HIP_TRY(mrl::launch_softmax_generic(v.in, v.out, v.scan_dim, nullptr, ws.stream));
  }
  return finish_output(out, ws);
}

int run_compose_msm(const mrl_spec &s, void *const *params, Workspace &ws) {
  const uint32_t b = s.spec_shape[0], m = s.spec_shape[1], k = s.spec_shape[2], n2 = s.spec_shape[3],
                 n = s.spec_shape[4];
  // Fused path: bf16 Q, K, V and an f32 result, head dims up to 128.  The kernel wants Q and V
  // row-major, KT with k fastest (layout![0,2,1]: K row-major) and rows of a head dim it is built
  // for (32, 64, 128).  Parameters that lie so are used in place; others are copied once: to that
  // order through the layouts' common strided view, and / or to rows padded with zeros (zero
  // columns of Q and K add nothing to the scores, zero columns of V give result columns that are
  // not stored).  A result in another layout is formed in scratch memory and moved out.
  const uint32_t widest = std::max(k, n), dp = widest <= 32 ? 32 : widest <= 64 ? 64 : 128;
  const int forced = g_forced ? g_forced->msm_path : 0;
  if (forced != 2 && s.dtypes[0] == MRL_BF16 && s.dtypes[1] == MRL_BF16 && s.dtypes[2] == MRL_BF16 && s.dtypes[3] == MRL_F32 &&
      widest <= 128 && (reinterpret_cast<uintptr_t>(params[3]) & 15) == 0) {
    // Parameter i as `rows` rows of `cols` bf16 per batch entry; wanted: the order of `want`.
    auto operand = [&](uint32_t i, const uint32_t *shape, const mrl_layout &want, uint32_t rows, uint32_t cols,
                       const void **result) -> int {
      const void *dense = params[i];
      std::vector<mrl::MoveDim> view;
      if (!mrl::common_view(s.layouts[i], want, shape, 3, &view)) return MRL_ERR_UNSUPPORTED;
      const bool in_order = mrl::same_order(view);
      if (!in_order) {
        void *buf = nullptr;
        HIP_TRY(ws.alloc(&buf, size_t(b) * rows * cols * 2));
        HIP_TRY(mrl::launch_move_view(params[i], MRL_BF16, buf, MRL_BF16, view.data(), uint32_t(view.size()), ws.stream));
        dense = buf;
      }
      if (cols != dp || (reinterpret_cast<uintptr_t>(dense) & 15) != 0) {
        void *buf = nullptr;
        HIP_TRY(ws.alloc(&buf, size_t(b) * rows * dp * 2));
        mrl::Strided flat;
        flat.ptr = const_cast<void *>(dense), flat.dtype = MRL_BF16, flat.rank = 3;
        flat.shape[0] = 1, flat.shape[1] = b * rows, flat.shape[2] = cols;
        flat.stride[0] = 0, flat.stride[1] = cols, flat.stride[2] = 1;
        HIP_TRY(mrl::launch_pad_rows(flat, buf, dp, 2, ws.stream));
        dense = buf;
      }
      *result = dense;
      return MRL_OK;
    };
    const uint32_t v_shape[3] = {b, n2, n}, q_shape[3] = {b, m, k}, kt_shape[3] = {b, k, n2}, o_shape[3] = {b, m, n};
    mrl_layout rows_v, rows_q, rows_o, k_fastest;
    mrl_layout_row_major(v_shape, 3, &rows_v);
    mrl_layout_row_major(q_shape, 3, &rows_q);
    mrl_layout_row_major(o_shape, 3, &rows_o);
    k_fastest.ndims = 3;
    k_fastest.dims[0] = {0, MRL_DYNAMIC, 0}, k_fastest.dims[1] = {2, MRL_DYNAMIC, 0}, k_fastest.dims[2] = {1, MRL_DYNAMIC, 0};
    mrl::AttnArgs at;
    at.b = b, at.m = m, at.k = at.n = dp, at.n2 = n2, at.n_out = n;
    // KT row-major as the reference lays it out by default ([b, k, n2], n2 fastest) is read in
    // place by the kernel's own build for it; any other order is brought to k-fastest.
    auto kt_operand = [&]() -> int {
      mrl_layout rows_kt;
      mrl_layout_row_major(kt_shape, 3, &rows_kt);
      std::vector<mrl::MoveDim> view;
      if (k == dp && n2 % 8 == 0 && (reinterpret_cast<uintptr_t>(params[2]) & 15) == 0 &&
          mrl::common_view(s.layouts[2], rows_kt, kt_shape, 3, &view) && mrl::same_order(view)) {
        at.kt = params[2], at.kt_rows = true;
        return MRL_OK;
      }
      return operand(2, kt_shape, k_fastest, n2, k, &at.kt);
    };
    std::vector<mrl::MoveDim> out_view;
    int rc = MRL_OK;
    if (mrl::common_view(rows_o, s.layouts[3], o_shape, 3, &out_view) &&
        (rc = operand(0, v_shape, rows_v, n2, n, &at.v)) == MRL_OK &&
        (rc = operand(1, q_shape, rows_q, m, k, &at.q)) == MRL_OK &&
        (rc = kt_operand()) == MRL_OK) {
      const bool out_in_order = mrl::same_order(out_view);
      void *result = params[3];
      if (!out_in_order) HIP_TRY(ws.alloc(&result, size_t(b) * m * n * sizeof(float)));
      at.out = static_cast<float *>(result);
      // Queries per workgroup (tile_out over the Compose's rows): 64 where 128 would leave half of
      // the compute units or more without a workgroup, or pad a query dimension of 64 or less.
      // Unless the keys are many enough to share out instead: 128 queries with the keys in as many
      // parts as fill the chip measured faster once a part holds 4096 keys, or 1024 with at most a
      // quarter of the units taken (2 x 8192 x 8192 keys: 68.8 us against 77.1, 1 x 8192 x 8192 39.9
      // against 49.7, 2 x 4096 x 4096 30.6 against 34.1; 4 x 4096 x 4096 the other way, 47.2 against 42.8).
      const uint64_t groups128 = uint64_t(b) * ((m + 127) / 128), units = mrl::g_compute_units;
      bool few_groups = 2 * groups128 <= units;
      if (few_groups && m > 64) {
        const uint64_t parts = std::min<uint64_t>(units / groups128, ((n2 + 63) / 64) / 4);
        const uint64_t keys = parts >= 2 ? n2 / parts : 0;
        if (keys >= 4096 || (4 * groups128 <= units && keys >= 1024)) few_groups = false;
      }
      at.query_block = forced == 1 && g_forced->query_block ? g_forced->query_block
                       : (m <= 64 || few_groups) && m > 32 ? 64 : 128;
      at.key_splits = forced == 1 && g_forced->key_splits ? g_forced->key_splits : mrl::attn_key_splits(at);
      if (at.key_splits > 1) {
        void *partials = nullptr;
        HIP_TRY(ws.alloc(&partials, mrl::attn_partial_bytes(at, at.key_splits)));
        at.partials = static_cast<float *>(partials);
      }
      if (mrl::attn_applicable(at)) {
        HIP_TRY(mrl::launch_attn(at, ws.stream));
        if (!out_in_order)
          HIP_TRY(mrl::launch_move_view(result, MRL_F32, params[3], MRL_F32, out_view.data(), uint32_t(out_view.size()), ws.stream));
        return MRL_OK;
      }
    } else if (rc != MRL_OK && rc != MRL_ERR_UNSUPPORTED) {
      return rc;
    }
  }
  if (forced == 1) return MRL_ERR_UNSUPPORTED;  // the fused kernel was asked for and does not take this Spec
  // Staged path, as the reference schedules it (examples/matmul_chain.rs:60-81): S and P
  // live in device memory as f32 (verification.rs:239-285); each stage is the Spec it is.
  void *sbuf = nullptr;
  HIP_TRY(ws.alloc(&sbuf, size_t(b) * m * n2 * sizeof(float)));
  mrl_spec st;
  std::memset(&st, 0, sizeof st);
  st.kind = MRL_SPEC_MATMUL, st.rank = 4, st.n_params = 3;
  st.spec_shape[0] = b, st.spec_shape[1] = m, st.spec_shape[2] = k, st.spec_shape[3] = n2;
  st.dtypes[0] = s.dtypes[1], st.dtypes[1] = s.dtypes[2], st.dtypes[2] = MRL_F32;
  st.layouts[0] = s.layouts[1], st.layouts[1] = s.layouts[2];
  const uint32_t s_shape[3] = {b, m, n2};
  mrl_layout_row_major(s_shape, 3, &st.layouts[2]);
  void *p1[3] = {params[1], params[2], sbuf};
  int rc = run_matmul(st, p1, ws);
  if (rc != MRL_OK) return rc;
  // bf16 inputs: P is rounded to bf16 on its way out of the Softmax, as in the fused kernel (the
  // one deviation from the f32 closed form, within the Compose's 1e-2), so that the second
  // product runs at the bf16 rate of the matrix cores instead of the f32 rate.
  const bool p_bf16 = s.dtypes[0] == MRL_BF16 && s.dtypes[1] == MRL_BF16 && s.dtypes[2] == MRL_BF16 &&
                      s.dtypes[3] == MRL_F32;
  void *pbuf = sbuf, *stats = nullptr;
  if (const size_t bytes = mrl::softmax_scratch_bytes(uint64_t(b) * m, n2)) HIP_TRY(ws.alloc(&stats, bytes));
  if (p_bf16) {
    HIP_TRY(ws.alloc(&pbuf, size_t(b) * m * n2 * 2));
    HIP_TRY(mrl::launch_softmax_rows_bf16((const float *)sbuf, pbuf, uint64_t(b) * m, n2, stats, ws.stream));
  } else if ((reinterpret_cast<uintptr_t>(sbuf) & 15) == 0) {
    HIP_TRY(mrl::launch_softmax_rows((const float *)sbuf, (float *)sbuf, uint64_t(b) * m, n2, stats, ws.stream));
  } else {
    mrl::Strided sv;
    sv.ptr = sbuf, sv.dtype = MRL_F32, sv.rank = 3;
    sv.shape[0] = b, sv.shape[1] = m, sv.shape[2] = n2, sv.shape[3] = sv.shape[4] = 1;
    sv.stride[0] = int64_t(m) * n2, sv.stride[1] = n2, sv.stride[2] = 1, sv.stride[3] = sv.stride[4] = 0;
    HIP_TRY(mrl::launch_softmax_generic(sv, sv, 2, nullptr, ws.stream));
  }
  st.spec_shape[2] = n2, st.spec_shape[3] = n;
  st.dtypes[0] = p_bf16 ? MRL_BF16 : MRL_F32, st.dtypes[1] = s.dtypes[0], st.dtypes[2] = s.dtypes[3];
  st.layouts[0] = st.layouts[2];  // P: row-major [b, m, n2]
  st.layouts[1] = s.layouts[0], st.layouts[2] = s.layouts[3];
  void *p2[3] = {pbuf, params[0], params[3]};
  return run_matmul(st, p2, ws);
}

int run_move(const mrl_spec &s, void *const *params, Workspace &ws) {
  uint32_t shape[MRL_MAX_RANK], rank;
  parameter_shape(s, 0, shape, &rank);
  const uint64_t count = volume(shape, rank);
  const mrl_layout &li = s.layouts[0], &lo = s.layouts[1];
  bool same_layout = li.ndims == lo.ndims;
  for (uint32_t i = 0; same_layout && i < li.ndims; i++)
    same_layout = li.dims[i].logical_dim == lo.dims[i].logical_dim && li.dims[i].kind == lo.dims[i].kind &&
                  (li.dims[i].kind == MRL_DYNAMIC || li.dims[i].size == lo.dims[i].size);
  auto al16 = [](const void *p) { return (reinterpret_cast<uintptr_t>(p) & 15) == 0; };
  if (same_layout && s.dtypes[0] == s.dtypes[1] && al16(params[0]) && al16(params[1])) {
    HIP_TRY(mrl::launch_copy(params[0], params[1], count * mrl_dtype_size(s.dtypes[0]), ws.stream));
    return MRL_OK;
  }
  // Layouts with a common strided view (permutations of the logical dims; Packed and OddEven
  // dims whose sizes refine each other): strided kernels, coalesced on both sides.
  std::vector<mrl::MoveDim> view;
  if (mrl::common_view(li, lo, shape, rank, &view)) {
    const hipError_t e = mrl::launch_move_view(params[0], s.dtypes[0], params[1], s.dtypes[1], view.data(),
                                               uint32_t(view.size()), ws.stream);
    if (e == hipSuccess) return MRL_OK;
    if (e != hipErrorInvalidValue) HIP_TRY(e);
  }
  mrl::LayoutEval sl, dl;
  if (!mrl::make_layout_eval(li, shape, rank, &sl) || !mrl::make_layout_eval(lo, shape, rank, &dl))
    return MRL_ERR_BAD_LAYOUT;
  HIP_TRY(mrl::launch_move_generic(params[0], params[1], sl, dl, s.dtypes[0], s.dtypes[1], count, ws.stream));
  return MRL_OK;
}

// Max, the SoftmaxDenominator* family, SoftmaxComplete, DivideVec, DivideVecScalar: one
// wavefront per line along scan_dim over strided f32 tensors.
int run_parts(const mrl_spec &s, void *const *params, Workspace &ws) {
  Prepared pr[4];
  mrl::PartsArgs pa;
  pa.kind = s.kind, pa.accum = s.accum, pa.rank = s.rank, pa.n_params = s.n_params;
  // DivideVec has no dim of its own: walk the innermost one.
  pa.scan_dim = s.kind == MRL_SPEC_DIVIDE_VEC ? s.rank - 1 : s.scan_dim;
  pa.lines = 1;
  for (uint32_t d = 0; d < MRL_MAX_RANK; d++) {
    pa.shape[d] = d < s.rank ? s.spec_shape[d] : 1;
    if (d < s.rank && d != pa.scan_dim) pa.lines *= pa.shape[d];
  }
  for (uint32_t i = 0; i < 4; i++) {
    pa.ptr[i] = nullptr;
    for (uint32_t d = 0; d < MRL_MAX_RANK; d++) pa.stride[i][d] = 0;
  }
  for (uint32_t i = 0; i < s.n_params; i++) {
    const int dir = parameter_direction(s, i);
    int rc = prepare(s, i, params[i], dir != 1, ws, &pr[i]);
    if (rc != MRL_OK) return rc;
    pa.ptr[i] = (float *)pr[i].t.ptr;
    for (uint32_t d = 0; d < s.rank; d++) pa.stride[i][d] = pr[i].t.shape[d] == 1 ? 0 : pr[i].t.stride[d];
  }
  HIP_TRY(mrl::launch_parts(pa, ws.stream));
  for (uint32_t i = 0; i < s.n_params; i++) {
    if (parameter_direction(s, i) == 0) continue;
    int rc = finish_output(pr[i], ws);
    if (rc != MRL_OK) return rc;
  }
  return MRL_OK;
}

int run_fill(const mrl_spec &s, void *const *params, Workspace &ws) {
  // Every element of the buffer is written, so the layout (a bijection onto the buffer)
  // does not matter.
  HIP_TRY(mrl::launch_fill(params[0], s.dtypes[0], int(s.scan_dim), volume(s.spec_shape, s.rank), ws.stream));
  return MRL_OK;
}

int run_broadcast(const mrl_spec &s, void *const *params, Workspace &ws) {
  uint32_t ishape[MRL_MAX_RANK], oshape[MRL_MAX_RANK], rank;
  parameter_shape(s, 0, ishape, &rank);
  parameter_shape(s, 1, oshape, &rank);
  // Both tensors row-major: whole 16-byte pieces, no index arithmetic per element.
  int64_t si[MRL_MAX_RANK], so[MRL_MAX_RANK];
  if (mrl::layout_strides(s.layouts[0], ishape, rank, si) && mrl::layout_strides(s.layouts[1], oshape, rank, so)) {
    bool dense = true;
    int64_t run_i = 1, run_o = 1;
    for (int d = int(rank) - 1; d >= 0; d--) {
      dense = dense && (ishape[d] == 1 || si[d] == run_i) && (oshape[d] == 1 || so[d] == run_o);
      run_i *= ishape[d], run_o *= oshape[d];
    }
    uint64_t before = 1, after = 1;
    for (uint32_t d = 0; d < rank; d++) (d < s.scan_dim ? before : after) *= d == s.scan_dim ? 1 : oshape[d];
    hipError_t err = hipSuccess;
    if (dense && mrl::launch_broadcast_rows(params[0], params[1], before, oshape[s.scan_dim], after,
                                            uint32_t(mrl_dtype_size(s.dtypes[0])), ws.stream, &err)) {
      HIP_TRY(err);
      return MRL_OK;
    }
  }
  mrl::LayoutEval il, ol;
  if (!mrl::make_layout_eval(s.layouts[0], ishape, rank, &il) ||
      !mrl::make_layout_eval(s.layouts[1], oshape, rank, &ol))
    return MRL_ERR_BAD_LAYOUT;
  HIP_TRY(mrl::launch_broadcast(params[0], params[1], il, ol, s.scan_dim, uint32_t(mrl_dtype_size(s.dtypes[0])),
                                volume(oshape, rank), ws.stream));
  return MRL_OK;
}

int run_one_prefix(const mrl_spec &s, void *const *params, Workspace &ws) {
  // The output's leading unit dim takes no part in addressing: restate its layout over the
  // input's shape (drop physical dims of logical dim 0, renumber the rest) and copy.
  uint32_t shape[MRL_MAX_RANK], oshape[MRL_MAX_RANK], rank, orank;
  parameter_shape(s, 0, shape, &rank);
  parameter_shape(s, 1, oshape, &orank);
  uint32_t phys[MRL_MAX_PHYS];
  if (!mrl::physical_shape(s.layouts[1], oshape, orank, phys)) return MRL_ERR_BAD_LAYOUT;
  mrl_layout lo;
  lo.ndims = 0;
  for (uint32_t i = 0; i < s.layouts[1].ndims; i++) {
    mrl_physdim pd = s.layouts[1].dims[i];
    if (pd.logical_dim == 0) continue;
    pd.logical_dim--;
    lo.dims[lo.ndims++] = pd;
  }
  // What is left is a Move over the input's shape: the plain copy when the two orders agree,
  // the strided kernels when they share a view.
  mrl_spec mv;
  std::memset(&mv, 0, sizeof mv);
  mv.kind = MRL_SPEC_MOVE, mv.n_params = 2, mv.rank = rank;
  for (uint32_t d = 0; d < rank; d++) mv.spec_shape[d] = shape[d];
  mv.dtypes[0] = s.dtypes[0], mv.dtypes[1] = s.dtypes[1], mv.layouts[0] = s.layouts[0], mv.layouts[1] = lo;
  return run_move(mv, params, ws);
}

// Matmul / Conv with a bf16 output (a legal dtype triple, spec.rs:3663-3698).  The reference's
// interpreter casts both inputs to the output dtype (verification.rs:629-642) and then works in
// bf16 arithmetic, rounding after every operation; its own comparison for bf16 is `todo!`
// (verification.rs:597).  Here the inputs are cast to bf16 the same way, the products are summed
// in f32 on the matrix cores, and the sum (plus the old output, for an accumulating Spec) is
// rounded to bf16 once: the Spec with an f32 output into scratch, between Moves.
int run_bf16_output(const mrl_spec &s, void *const *params, Workspace &ws) {
  mrl_spec t = s;
  void *p[3] = {params[0], params[1], nullptr};
  auto move = [&](uint32_t idx, int dt_from, const mrl_layout &l_from, const void *from, int dt_to, const mrl_layout &l_to,
                  void *to) -> int {
    mrl_spec mv;
    std::memset(&mv, 0, sizeof mv);
    mv.kind = MRL_SPEC_MOVE, mv.n_params = 2;
    parameter_shape(s, idx, mv.spec_shape, &mv.rank);
    mv.dtypes[0] = dt_from, mv.dtypes[1] = dt_to, mv.layouts[0] = l_from, mv.layouts[1] = l_to;
    void *mp[2] = {const_cast<void *>(from), to};
    return run_move(mv, mp, ws);
  };
  int rc;
  for (uint32_t i = 0; i < 2; i++) {
    if (s.dtypes[i] == MRL_BF16) continue;
    uint32_t shape[MRL_MAX_RANK], rank;
    parameter_shape(s, i, shape, &rank);
    void *buf = nullptr;
    HIP_TRY(ws.alloc(&buf, size_t(volume(shape, rank)) * 2));
    mrl_layout_row_major(shape, rank, &t.layouts[i]);
    if ((rc = move(i, s.dtypes[i], s.layouts[i], params[i], MRL_BF16, t.layouts[i], buf)) != MRL_OK) return rc;
    t.dtypes[i] = MRL_BF16, p[i] = buf;
  }
  uint32_t shape[MRL_MAX_RANK], rank;
  parameter_shape(s, 2, shape, &rank);
  HIP_TRY(ws.alloc(&p[2], size_t(volume(shape, rank)) * 4));
  t.dtypes[2] = MRL_F32;
  mrl_layout_row_major(shape, rank, &t.layouts[2]);
  if (s.accum && (rc = move(2, MRL_BF16, s.layouts[2], params[2], MRL_F32, t.layouts[2], p[2])) != MRL_OK) return rc;
  if ((rc = s.kind == MRL_SPEC_MATMUL ? run_matmul(t, p, ws) : run_conv(t, p, ws)) != MRL_OK) return rc;
  return move(2, MRL_F32, t.layouts[2], p[2], MRL_BF16, s.layouts[2], params[2]);
}

int dispatch(const mrl_spec &spec, void *const *params, Workspace &ws) {
  if ((spec.kind == MRL_SPEC_MATMUL || spec.kind == MRL_SPEC_CONV) && spec.dtypes[2] == MRL_BF16)
    return run_bf16_output(spec, params, ws);
  switch (spec.kind) {
    case MRL_SPEC_MATMUL: return run_matmul(spec, params, ws);
    case MRL_SPEC_CONV: return run_conv(spec, params, ws);
    case MRL_SPEC_SOFTMAX: return run_softmax(spec, params, ws);
    case MRL_SPEC_COMPOSE_MSM: return run_compose_msm(spec, params, ws);
    case MRL_SPEC_MOVE: return run_move(spec, params, ws);
    case MRL_SPEC_FILL: return run_fill(spec, params, ws);
    case MRL_SPEC_BROADCAST: return run_broadcast(spec, params, ws);
    case MRL_SPEC_ONE_PREFIX: return run_one_prefix(spec, params, ws);
    default: return is_parts_kind(spec.kind) ? run_parts(spec, params, ws) : MRL_ERR_UNSUPPORTED;
  }
}

// ---- general Compose (spec.rs:1519-1590, 3329-3365) ----

// A component as a stand-alone Spec with row-major layouts.
int component_spec(const mrl_component &c, mrl_spec *s) {
  std::memset(s, 0, sizeof *s);
  s->kind = c.kind, s->accum = c.accum, s->scan_dim = c.scan_dim, s->rank = c.rank, s->n_params = c.n_params;
  if (c.rank > MRL_MAX_SPEC_RANK || c.n_params > MRL_MAX_PARAMS) return MRL_ERR_BAD_SPEC;
  for (uint32_t d = 0; d < c.rank; d++) s->spec_shape[d] = c.spec_shape[d];
  for (uint32_t i = 0; i < c.n_params; i++) s->dtypes[i] = c.dtypes[i];
  if (c.kind == MRL_SPEC_COMPOSE_MSM || expected_params(c.kind) != c.n_params) return MRL_ERR_BAD_SPEC;
  for (uint32_t i = 0; i < c.n_params; i++) {
    uint32_t shape[MRL_MAX_RANK], rank;
    if (parameter_shape(*s, i, shape, &rank) != MRL_OK) return MRL_ERR_BAD_SPEC;
    mrl_layout_row_major(shape, rank, &s->layouts[i]);
  }
  return MRL_OK;
}

// spec.rs:1270-1278: the index of the only written parameter, or -1.
int unique_output_index(const mrl_spec &s) {
  int found = -1;
  for (uint32_t i = 0; i < s.n_params; i++)
    if (parameter_direction(s, i) != 0) {
      if (found >= 0) return -1;
      found = int(i);
    }
  return found;
}

struct ComposeParam {
  uint32_t component, param;
};

// compose_parameter_visit, spec.rs:3329-3365.
int compose_parameters(const mrl_compose &c, std::vector<ComposeParam> *out, std::vector<mrl_spec> *specs) {
  if (c.n_components < 2 || c.n_components > MRL_MAX_COMPONENTS) return MRL_ERR_BAD_SPEC;
  specs->resize(c.n_components);
  std::vector<int> out_idx(c.n_components);
  for (uint32_t i = 0; i < c.n_components; i++) {
    int rc = component_spec(c.components[i], &(*specs)[i]);
    if (rc != MRL_OK) return rc;
    // Only the head (listed first, run last) may accumulate: a tail component with side effects is
    // CanonicalizeError::SideEffectingComponent (spec.rs:1760-1764); an accumulating head is
    // accepted (spec.rs:3829-3838) and makes the Compose's output parameter read-write.
    if (i > 0 && c.components[i].accum) return MRL_ERR_BAD_SPEC;
    if ((rc = check_spec(&(*specs)[i])) != MRL_OK) return rc;
    if ((out_idx[i] = unique_output_index((*specs)[i])) < 0) return MRL_ERR_BAD_SPEC;
    if (out_idx[i] == 0) return MRL_ERR_BAD_SPEC;  // the first parameter must be an input to chain on
  }
  const uint32_t last = c.n_components - 1;
  for (uint32_t i = 0; i < c.n_components; i++) {
    const uint32_t first = i == last ? 0 : 1;
    for (uint32_t p = first; p < (*specs)[i].n_params; p++)
      if (int(p) != out_idx[i]) out->push_back({i, p});
  }
  out->push_back({0, uint32_t(out_idx[0])});
  if (out->size() > MRL_MAX_COMPOSE_PARAMS) return MRL_ERR_BAD_SPEC;
  // Each component's first input is the next-listed component's output.
  for (uint32_t i = 0; i < last; i++) {
    uint32_t in_shape[MRL_MAX_RANK], in_rank, o_shape[MRL_MAX_RANK], o_rank;
    parameter_shape((*specs)[i], 0, in_shape, &in_rank);
    parameter_shape((*specs)[i + 1], uint32_t(out_idx[i + 1]), o_shape, &o_rank);
    if (in_rank != o_rank) return MRL_ERR_BAD_SPEC;
    for (uint32_t d = 0; d < in_rank; d++)
      if (in_shape[d] != o_shape[d]) return MRL_ERR_BAD_SPEC;
    if ((*specs)[i].dtypes[0] != (*specs)[i + 1].dtypes[out_idx[i + 1]]) return MRL_ERR_BAD_SPEC;
  }
  return MRL_OK;
}

int run_compose_general(const mrl_compose &c, void *const *params, Workspace &ws) {
  std::vector<ComposeParam> ext;
  std::vector<mrl_spec> specs;
  int rc = compose_parameters(c, &ext, &specs);
  if (rc != MRL_OK) return rc;
  if (ext.size() != c.n_params) return MRL_ERR_BAD_SPEC;
  for (size_t i = 0; i < ext.size(); i++) {
    if (!params[i]) return MRL_ERR_NULL;
    mrl_spec &s = specs[ext[i].component];
    uint32_t shape[MRL_MAX_RANK], rank, phys[MRL_MAX_PHYS];
    parameter_shape(s, ext[i].param, shape, &rank);
    if (!mrl::physical_shape(c.layouts[i], shape, rank, phys)) return MRL_ERR_BAD_LAYOUT;
    s.layouts[ext[i].param] = c.layouts[i];
  }
  const uint32_t n = c.n_components;
  // The attention shape: [Matmul[b,m,n2,n], Softmax{2}[b,m,n2], Matmul[b,m,k,n2]] -> the fused path.
  if (c.bufferize_mask >> (n - 1)) return MRL_ERR_BAD_SPEC;  // only boundaries 0 .. n-2 exist
  if (c.bufferize_mask == 0 && n == 3 && specs[0].kind == MRL_SPEC_MATMUL && specs[1].kind == MRL_SPEC_SOFTMAX && specs[1].rank == 3 &&
      specs[1].scan_dim == 2 && specs[2].kind == MRL_SPEC_MATMUL && specs[0].dtypes[2] == MRL_F32 &&
      specs[0].dtypes[0] == MRL_F32 && !specs[0].accum) {
    mrl_spec msm;
    std::memset(&msm, 0, sizeof msm);
    msm.kind = MRL_SPEC_COMPOSE_MSM, msm.rank = 5, msm.n_params = 4;
    msm.spec_shape[0] = specs[2].spec_shape[0], msm.spec_shape[1] = specs[2].spec_shape[1];
    msm.spec_shape[2] = specs[2].spec_shape[2], msm.spec_shape[3] = specs[2].spec_shape[3];
    msm.spec_shape[4] = specs[0].spec_shape[3];
    msm.dtypes[0] = specs[0].dtypes[1], msm.dtypes[1] = specs[2].dtypes[0], msm.dtypes[2] = specs[2].dtypes[1];
    msm.dtypes[3] = MRL_F32;
    for (uint32_t i = 0; i < 4; i++) msm.layouts[i] = c.layouts[i];
    if (check_spec(&msm) == MRL_OK) return run_compose_msm(msm, params, ws);
  }
  // Component by component, last-listed first.
  void *carried = nullptr;  // the previous component's output
  for (int i = int(n) - 1; i >= 0; i--) {
    const mrl_spec &s = specs[i];
    const int out_idx = unique_output_index(s);
    void *cp[MRL_MAX_PARAMS] = {nullptr, nullptr, nullptr, nullptr};
    for (size_t e = 0; e < ext.size(); e++)
      if (ext[e].component == uint32_t(i)) cp[ext[e].param] = params[e];
    if (i < int(n) - 1) cp[0] = carried;
    if (i > 0) {
      uint32_t shape[MRL_MAX_RANK], rank;
      parameter_shape(s, uint32_t(out_idx), shape, &rank);
      HIP_TRY(ws.alloc(&cp[out_idx], size_t(volume(shape, rank)) * mrl_dtype_size(s.dtypes[out_idx])));
      carried = cp[out_idx];
    }
    if ((rc = dispatch(s, cp, ws)) != MRL_OK) return rc;
  }
  return MRL_OK;
}

int run_async_impl(const mrl_spec *spec, void *const *params, hipStream_t stream) {
  if (g_device < 0) {
    int rc = mrl_init(0);
    if (rc != MRL_OK) return rc;
  }
  int rc = check_spec(spec);
  if (rc != MRL_OK) return rc;
  if (!params) return MRL_ERR_NULL;
  for (uint32_t i = 0; i < spec->n_params; i++)
    if (!params[i]) return MRL_ERR_NULL;
  Workspace ws(stream);
  return dispatch(*spec, params, ws);
}

// Runs `body` (a dispatch) with a Recorder installed on this thread and stand-in parameter
// addresses, then writes the recorded launches out.
template <class Body>
int plan_with(uint32_t n_params, mrl_plan *plan, mrl_plan_step *steps, uint32_t cap, Body body) {
  if (!plan || (cap && !steps)) return MRL_ERR_NULL;
  void *params[64];
  if (n_params > 64) return MRL_ERR_BAD_SPEC;
  for (uint32_t i = 0; i < n_params; i++) params[i] = reinterpret_cast<void *>((uintptr_t(1) << 40) + (uintptr_t(i) << 36));
  mrl::plan::Recorder recorder;
  int rc;
  {
    mrl::plan::g_recorder = &recorder;
    Workspace ws(nullptr);
    rc = body(params, ws);
    mrl::plan::g_recorder = nullptr;
  }
  if (rc != MRL_OK) return rc;
  int units = 256;
  if (g_device >= 0) (void)hipDeviceGetAttribute(&units, hipDeviceAttributeMultiprocessorCount, g_device);
  plan->n_steps = uint32_t(recorder.steps.size());
  plan->scratch_bytes = recorder.scratch_bytes;
  plan->cost_ns = 0;
  for (uint32_t i = 0; i < plan->n_steps; i++) {
    const mrl::plan::Step &from = recorder.steps[i];
    const double ns = mrl::plan::step_ns(from, uint32_t(units));
    plan->cost_ns += ns;
    if (i >= cap) continue;
    mrl_plan_step &to = steps[i];
    std::snprintf(to.kernel, sizeof to.kernel, "%s", from.kernel.c_str());
    for (int d = 0; d < 3; d++) to.grid[d] = from.grid[d], to.block[d] = from.block[d];
    to.lds_bytes = from.lds_bytes, to.unit = from.unit, to.ops = from.ops, to.bytes = from.bytes, to.cost_ns = ns;
  }
  return MRL_OK;
}

void set_conv_default_layouts(mrl_spec *s) {
  for (uint32_t i = 0; i < 3; i++) {
    uint32_t shape[MRL_MAX_RANK], rank;
    parameter_shape(*s, i, shape, &rank);
    mrl_layout_nhwc(shape, rank, &s->layouts[i]);
  }
}

}  // namespace

extern "C" {

int mrl_init(int device) {
  int count = 0;
  hipError_t e = hipGetDeviceCount(&count);
  if (e != hipSuccess || count <= 0) {
    g_last_error = e != hipSuccess ? hipGetErrorString(e) : "no HIP device";
    return MRL_ERR_NO_DEVICE;
  }
  if (device < 0 || device >= count) return MRL_ERR_NO_DEVICE;
  hipDeviceProp_t prop;
  HIP_TRY(hipGetDeviceProperties(&prop, device));
  if (std::strncmp(prop.gcnArchName, "gfx950", 6) != 0) {
    g_last_error = std::string("device is ") + prop.gcnArchName + ", kernels are built for gfx950";
    return MRL_ERR_NO_DEVICE;
  }
  HIP_TRY(hipSetDevice(device));
  if (device < MAX_DEVICES && !g_scratch_ptr[device]) {
    // This device's copy of the array.  A failure here only takes mrl_run_noalloc away (it finds
    // no pointer and says so): every other entry point allocates what it needs.
    void *ptr = nullptr;
    if (hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch)) == hipSuccess) g_scratch_ptr[device] = ptr;
    else (void)hipGetLastError();
  }
  g_device = device;
  mrl::g_compute_units = prop.multiProcessorCount > 0 ? uint32_t(prop.multiProcessorCount) : 256u;
  return MRL_OK;
}

const char *mrl_status_string(int status) {
  switch (status) {
    case MRL_OK: return "ok";
    case MRL_ERR_UNSUPPORTED: return "unsupported Spec";
    case MRL_ERR_BAD_LAYOUT: return "layout does not apply to the parameter shape";
    case MRL_ERR_BAD_SPEC: return "malformed Spec descriptor";
    case MRL_ERR_HIP: return "HIP runtime error";
    case MRL_ERR_NO_DEVICE: return "no gfx950 device";
    case MRL_ERR_NULL: return "null pointer";
    case MRL_ERR_TOO_LARGE: return "tensor too large";
    default: return "unknown status";
  }
}

const char *mrl_last_error(void) { return g_last_error.c_str(); }
const char *mrl_version(void) { return "0.1.0"; }

uint32_t mrl_abi_version(void) { return MRL_ABI_VERSION; }

size_t mrl_dtype_size(int dtype) {
  switch (dtype) {
    case MRL_U8: case MRL_I8: return 1;
    case MRL_U16: case MRL_I16: case MRL_BF16: return 2;
    case MRL_U32: case MRL_I32: case MRL_F32: return 4;
    default: return 0;
  }
}

const char *mrl_dtype_name(int dtype) {
  static const char *names[] = {"u8", "i8", "u16", "i16", "u32", "i32", "f32", "bf16"};
  return valid_dtype(dtype) ? names[dtype] : "?";
}

int mrl_layout_row_major(const uint32_t *shape, uint32_t rank, mrl_layout *out) {
  if (!shape || !out) return MRL_ERR_NULL;
  if (rank > MRL_MAX_RANK) return MRL_ERR_BAD_SPEC;
  out->ndims = 0;
  for (uint32_t d = 0; d < rank; d++) {
    if (shape[d] == 1) continue;  // layout.rs:1234-1247 drops size-one dims
    out->dims[out->ndims++] = mrl_physdim{uint8_t(d), MRL_DYNAMIC, 0};
  }
  return MRL_OK;
}

int mrl_layout_col_major(const uint32_t *shape, uint32_t rank, mrl_layout *out) {
  int rc = mrl_layout_row_major(shape, rank, out);
  if (rc != MRL_OK) return rc;
  for (uint32_t i = 0; i < out->ndims / 2; i++) {
    mrl_physdim t = out->dims[i];
    out->dims[i] = out->dims[out->ndims - 1 - i];
    out->dims[out->ndims - 1 - i] = t;
  }
  return MRL_OK;
}

int mrl_layout_batched_col_major(const uint32_t *shape, uint32_t rank, mrl_layout *out) {
  if (!shape || !out) return MRL_ERR_NULL;
  if (rank == 0) {
    out->ndims = 0;
    return MRL_OK;
  }
  mrl_layout inner;
  int rc = mrl_layout_col_major(shape + 1, rank - 1, &inner);
  if (rc != MRL_OK) return rc;
  out->ndims = 0;
  if (shape[0] != 1) out->dims[out->ndims++] = mrl_physdim{0, MRL_DYNAMIC, 0};
  for (uint32_t i = 0; i < inner.ndims; i++) {
    mrl_physdim d = inner.dims[i];
    d.logical_dim = uint8_t(d.logical_dim + 1);
    out->dims[out->ndims++] = d;
  }
  return MRL_OK;
}

int mrl_layout_nhwc(const uint32_t *shape, uint32_t rank, mrl_layout *out) {
  if (!shape || !out) return MRL_ERR_NULL;
  if (rank != 4) return MRL_ERR_BAD_SPEC;
  static const uint8_t order[4] = {0, 2, 3, 1};
  out->ndims = 0;
  for (int i = 0; i < 4; i++)
    if (shape[order[i]] != 1) out->dims[out->ndims++] = mrl_physdim{order[i], MRL_DYNAMIC, 0};
  return MRL_OK;
}

int mrl_layout_physical_shape(const mrl_layout *layout, const uint32_t *shape, uint32_t rank,
                              uint32_t *phys_shape) {
  if (!layout || !shape || !phys_shape) return MRL_ERR_NULL;
  return mrl::physical_shape(*layout, shape, rank, phys_shape) ? MRL_OK : MRL_ERR_BAD_LAYOUT;
}

int64_t mrl_layout_buffer_index(const mrl_layout *layout, const uint32_t *shape, uint32_t rank,
                                const uint32_t *point) {
  if (!layout || !shape || !point) return -1;
  mrl::LayoutEval ev;
  if (!mrl::make_layout_eval(*layout, shape, rank, &ev)) return -1;
  return mrl::layout_offset(ev, point);
}

int mrl_spec_parameter_shape(const mrl_spec *spec, uint32_t idx, uint32_t *shape, uint32_t *rank) {
  if (!spec || !shape || !rank) return MRL_ERR_NULL;
  if (expected_params(spec->kind) == 0 || spec->rank != expected_rank(*spec)) return MRL_ERR_BAD_SPEC;
  return parameter_shape(*spec, idx, shape, rank);
}

int mrl_spec_parameter_direction(const mrl_spec *spec, uint32_t idx) {
  return spec ? parameter_direction(*spec, idx) : -1;
}

size_t mrl_spec_parameter_bytes(const mrl_spec *spec, uint32_t idx) {
  uint32_t shape[MRL_MAX_RANK], rank;
  if (mrl_spec_parameter_shape(spec, idx, shape, &rank) != MRL_OK) return 0;
  return size_t(volume(shape, rank)) * mrl_dtype_size(spec->dtypes[idx]);
}

uint64_t mrl_spec_ops(const mrl_spec *spec) {
  if (!spec) return 0;
  const uint32_t *s = spec->spec_shape;
  switch (spec->kind) {
    case MRL_SPEC_MATMUL: return 2ull * s[0] * s[1] * s[2] * s[3];
    case MRL_SPEC_CONV: return 2ull * s[0] * s[1] * s[2] * s[3] * s[4] * s[5] * s[6];
    case MRL_SPEC_SOFTMAX: return 5ull * volume(s, spec->rank);
    case MRL_SPEC_MOVE: return 0;
    case MRL_SPEC_COMPOSE_MSM:
      return 2ull * s[0] * s[1] * s[2] * s[3] + 5ull * s[0] * s[1] * s[3] + 2ull * s[0] * s[1] * s[3] * s[4];
    default: return 0;
  }
}

int mrl_spec_check(const mrl_spec *spec) { return check_spec(spec); }

size_t mrl_spec_workspace_bytes(const mrl_spec *spec) {
  if (check_spec(spec) != MRL_OK) return 0;
  // These run on the parameters' own layouts and stage nothing.
  if (spec->kind == MRL_SPEC_MOVE || spec->kind == MRL_SPEC_FILL || spec->kind == MRL_SPEC_BROADCAST ||
      spec->kind == MRL_SPEC_ONE_PREFIX)
    return 0;
  size_t total = 0;
  for (uint32_t i = 0; i < spec->n_params; i++) {
    uint32_t shape[MRL_MAX_RANK], rank;
    int64_t strides[MRL_MAX_RANK];
    parameter_shape(*spec, i, shape, &rank);
    if (mrl::layout_strides(spec->layouts[i], shape, rank, strides)) continue;
    mrl_layout dense;
    mrl_layout_row_major(shape, rank, &dense);
    std::vector<mrl::MoveDim> view;
    if (mrl::common_view(spec->layouts[i], dense, shape, rank, &view) && mrl::same_order(view))
      continue;  // Packed dims in row-major order
    total += size_t(volume(shape, rank)) * mrl_dtype_size(spec->dtypes[i]);
  }
  return total;
}

uint64_t mrl_launch_count(void) { return mrl::plan::g_launches; }

const char *mrl_target_id(void) { return "Gfx950"; }
uint32_t mrl_target_line_size(void) { return 128; }
uint32_t mrl_target_processors(void) { return mrl::g_compute_units; }

uint32_t mrl_target_memories(mrl_target_memory *out, uint32_t cap) {
  // Fastest first, as CpuMemory's order (target/cpu.rs:2536-2560).  ACC: the MFMA accumulators
  // (a wavefront's share of the unified 512-register file the kernels give them); VGPR: the
  // rest of the register file, whose 4 / 8 / 16-byte forms are what loads and stores move per
  // lane; LDS: 160 KiB per compute unit, addressed by the kernels (unlike the reference's L1);
  // HBM: 288 GB, the only level a grid can tile in parallel.  Hit costs follow the reference's
  // scale of 1 for registers (target/cpu.rs cache_hit_cost) by latency ratio.
  static const mrl_target_memory levels[4] = {
      {"ACC", 1, 0, 1, 0, {0, 0, 0, 0}, 256, 0},
      {"VGPR", 1, 0, 1, 1, {4, 8, 16, 0}, 256, 0},
      {"LDS", 1, 0, 0, 1, {0, 0, 0, 0}, 160 * 1024, 8},
      {"HBM", 1, 1, 0, 1, {0, 0, 0, 0}, 288ull << 30, 100},
  };
  for (uint32_t i = 0; i < 4 && i < cap && out; i++) out[i] = levels[i];
  return 4;
}

uint32_t mrl_target_default_memory(void) { return 3; }

uint32_t mrl_target_destination_memories(uint32_t slower, uint32_t *out, uint32_t cap) {
  // HBM feeds LDS (global_load ... lds) and registers directly; LDS feeds registers; the MFMA
  // accumulators are initialised from and drained to VGPRs.
  static const uint32_t table[4][3] = {{0, 0, 0}, {1, 0, 0}, {2, 1, 0}, {3, 2, 1}};
  static const uint32_t counts[4] = {1, 2, 2, 3};
  if (slower > 3) return 0;
  for (uint32_t i = 0; i < counts[slower] && i < cap && out; i++) out[i] = table[slower][i];
  return counts[slower];
}

uint32_t mrl_target_layouts_for_shape(const uint32_t *shape, uint32_t rank, int dtype, mrl_layout *out, uint32_t cap) {
  if (!shape || rank == 0 || rank > MRL_MAX_RANK || mrl_dtype_size(dtype) == 0) return 0;
  const uint32_t es = uint32_t(mrl_dtype_size(dtype));
  std::vector<mrl_layout> base(1), result;
  mrl_layout_row_major(shape, rank, &base[0]);
  bool only_ones = true;
  for (uint32_t d = 0; d < rank; d++) only_ones = only_ones && shape[d] == 1;
  auto same = [](const mrl_layout &a, const mrl_layout &b) {
    if (a.ndims != b.ndims) return false;
    for (uint32_t i = 0; i < a.ndims; i++)
      if (a.dims[i].logical_dim != b.dims[i].logical_dim || a.dims[i].kind != b.dims[i].kind ||
          a.dims[i].size != b.dims[i].size)
        return false;
    return true;
  };
  if (!only_ones && (rank == 2 || rank == 3 || rank == 4)) {
    mrl_layout other;
    const int rc = rank == 2   ? mrl_layout_col_major(shape, rank, &other)
                   : rank == 3 ? mrl_layout_batched_col_major(shape, rank, &other)
                               : mrl_layout_nhwc(shape, rank, &other);
    if (rc == MRL_OK && !same(other, base[0])) base.push_back(other);
  }
  result = base;
  // Vector widths of the register file in elements, and 2 (pack_sizes_all, target/cpu.rs:2894-2906);
  // twice the widths for OddEven (oddeven_sizes_all, target/cpu.rs:2935-2947).
  std::vector<uint32_t> pack{2}, oddeven;
  for (uint32_t bytes : {4u, 8u, 16u}) {
    if (bytes % es == 0 && bytes / es > 1 && std::find(pack.begin(), pack.end(), bytes / es) == pack.end())
      pack.push_back(bytes / es);
    if ((2 * bytes) % es == 0 && 2 * bytes / es > 1 &&
        std::find(oddeven.begin(), oddeven.end(), 2 * bytes / es) == oddeven.end())
      oddeven.push_back(2 * bytes / es);
  }
  auto extend = [&](const mrl_layout &from, uint32_t dim, uint8_t kind, uint32_t size) {
    if (from.ndims >= MRL_MAX_PHYS) return;
    mrl_layout l = from;
    l.dims[l.ndims].logical_dim = uint8_t(dim), l.dims[l.ndims].kind = kind, l.dims[l.ndims].size = size;
    l.ndims++;
    uint32_t phys[MRL_MAX_PHYS];
    if (!mrl::physical_shape(l, shape, rank, phys)) return;  // does not apply to this shape
    for (const mrl_layout &have : result)
      if (same(have, l)) return;
    result.push_back(l);
  };
  for (const mrl_layout &b : base) {
    std::vector<uint32_t> dims;
    for (uint32_t i = 0; i < b.ndims; i++)
      if (std::find(dims.begin(), dims.end(), b.dims[i].logical_dim) == dims.end()) dims.push_back(b.dims[i].logical_dim);
    const uint32_t innermost = b.dims[b.ndims - 1].logical_dim;
    for (uint32_t d : dims)
      for (uint32_t size : pack)
        if (d != innermost && shape[d] % size == 0) extend(b, d, MRL_PACKED, size);
  }
  for (const mrl_layout &b : base) {
    std::vector<uint32_t> dims;
    for (uint32_t i = 0; i < b.ndims; i++)
      if (std::find(dims.begin(), dims.end(), b.dims[i].logical_dim) == dims.end()) dims.push_back(b.dims[i].logical_dim);
    for (uint32_t d : dims)
      for (uint32_t size : oddeven)
        if (shape[d] % size == 0) extend(b, d, MRL_ODDEVEN, size);
  }
  for (uint32_t i = 0; i < result.size() && i < cap && out; i++) out[i] = result[i];
  return uint32_t(result.size());
}

uint32_t mrl_target_kernels(const char **names, uint32_t cap) {
  static const char *const families[] = {
      "k_gemm", "k_gemm_big", "k_gemm_wide", "k_gemv", "k_matmul_generic", "k_sum_splits", "k_conv_i8", "k_conv_rows_i8", "k_conv_windows", "k_conv_small", "k_conv_generic", "k_conv_generic_wave", "k_unfold",
      "k_unfold_gather", "k_attn", "k_attn_merge", "k_softmax_regs", "k_softmax_regs1", "k_softmax_short", "k_softmax_block", "k_softmax_chunk_stats", "k_softmax_chunk_write",
      "k_softmax_cols",
      "k_softmax_generic", "k_softmax_cols_short", "k_parts", "k_parts_block", "k_parts_rows", "k_parts_cols", "k_broadcast", "k_broadcast_rows", "k_broadcast_fill_rows", "k_fill", "k_fill16", "k_fill_zero", "k_move_rows", "k_move_rows16",
      "k_move_tiled", "k_move_tiled_as", "k_move_tiled8v", "k_move_tiled16", "k_move_tiled16v", "k_move_tiled32", "k_move_gather", "k_move_generic", "k_relayout", "k_convert4", "k_copy1",
      "k_copy16", "k_pad_rows", "k_pad_rows_pair", "k_pad_rows16", "k_widen_bf16"};
  const uint32_t n = sizeof families / sizeof families[0];
  for (uint32_t i = 0; i < n && i < cap && names; i++) names[i] = families[i];
  return n;
}

int mrl_spec_plan(const mrl_spec *spec, mrl_plan *plan, mrl_plan_step *steps, uint32_t cap) {
  int rc = check_spec(spec);
  if (rc != MRL_OK) return rc;
  return plan_with(spec->n_params, plan, steps, cap,
                   [&](void *const *params, Workspace &ws) { return dispatch(*spec, params, ws); });
}

int mrl_compose_plan(const mrl_compose *c, mrl_plan *plan, mrl_plan_step *steps, uint32_t cap) {
  if (!c) return MRL_ERR_NULL;
  std::vector<ComposeParam> ext;
  std::vector<mrl_spec> specs;
  int rc = compose_parameters(*c, &ext, &specs);
  if (rc != MRL_OK) return rc;
  return plan_with(uint32_t(ext.size()), plan, steps, cap,
                   [&](void *const *params, Workspace &ws) { return run_compose_general(*c, params, ws); });
}

int mrl_run_async(const mrl_spec *spec, void *const *params, void *stream) {
  return run_async_impl(spec, params, (hipStream_t)stream);
}

int mrl_run_noalloc(const mrl_spec *spec, void *const *params, void *stream) {
  if (g_device < 0 || g_device >= MAX_DEVICES || !g_scratch_ptr[g_device]) {
    g_last_error = "mrl_run_noalloc: call mrl_init first (it looks up the device's scratch array)";
    return MRL_ERR_NO_DEVICE;
  }
  // The array belongs to the device mrl_init chose: a thread that has made another one current
  // would hand its kernels a pointer of the wrong GPU.
  int current = -1;
  HIP_TRY(hipGetDevice(&current));
  if (current != g_device) {
    g_last_error = "mrl_run_noalloc: the calling thread's current device is " + std::to_string(current) +
                   ", the library was initialised for device " + std::to_string(g_device);
    return MRL_ERR_NO_DEVICE;
  }
  int rc = check_spec(spec);
  if (rc != MRL_OK) return rc;
  if (!params) return MRL_ERR_NULL;
  for (uint32_t i = 0; i < spec->n_params; i++) {
    if (!params[i]) return MRL_ERR_NULL;
    // The plan below assumes parameters aligned as device allocations are; others could take a
    // path with a larger scratch need, found only after kernels have written to the outputs.
    if (reinterpret_cast<uintptr_t>(params[i]) & 255) {
      g_last_error = "mrl_run_noalloc: parameter " + std::to_string(i) + " is not 256-byte aligned";
      return MRL_ERR_UNSUPPORTED;
    }
  }
  // What the call would take, from the plan (host arithmetic only), so that a Spec that does not
  // fit is turned down before anything is launched.
  mrl_plan plan;
  if ((rc = mrl_spec_plan(spec, &plan, nullptr, 0)) != MRL_OK) return rc;
  const std::string too_large = "mrl_run_noalloc: the Spec needs " + std::to_string(plan.scratch_bytes) +
                                " bytes of scratch, the fixed array holds " + std::to_string(NOALLOC_SCRATCH_BYTES);
  if (plan.scratch_bytes > NOALLOC_SCRATCH_BYTES) {
    g_last_error = too_large;
    return MRL_ERR_TOO_LARGE;
  }
  Workspace ws((hipStream_t)stream, g_scratch_ptr[g_device], NOALLOC_SCRATCH_BYTES);
  rc = dispatch(*spec, params, ws);
  if (ws.fixed_overflow) {  // parameters aligned otherwise than the plan assumes can take another path
    g_last_error = too_large + " (exceeded during the run: parameters not 256-byte aligned?)";
    return MRL_ERR_TOO_LARGE;
  }
  return rc;
}

int mrl_run(const mrl_spec *spec, void *const *params) {
  int rc = run_async_impl(spec, params, nullptr);
  if (rc != MRL_OK) return rc;
  HIP_TRY(hipStreamSynchronize(nullptr));
  return MRL_OK;
}

int mrl_run_host(const mrl_spec *spec, void *const *params) {
  int rc = check_spec(spec);
  if (rc != MRL_OK) return rc;
  if (!params) return MRL_ERR_NULL;
  if (g_device < 0 && (rc = mrl_init(0)) != MRL_OK) return rc;
  void *dev[MRL_MAX_PARAMS] = {nullptr, nullptr, nullptr, nullptr};
  auto cleanup = [&]() {
    for (void *p : dev)
      if (p) (void)hipFree(p);
  };
  for (uint32_t i = 0; i < spec->n_params; i++) {
    if (!params[i]) {
      cleanup();
      return MRL_ERR_NULL;
    }
    const size_t bytes = mrl_spec_parameter_bytes(spec, i);
    hipError_t e = hipMalloc(&dev[i], bytes ? bytes : 4);
    if (e == hipSuccess && parameter_direction(*spec, i) != 1)
      e = hipMemcpy(dev[i], params[i], bytes, hipMemcpyHostToDevice);
    if (e != hipSuccess) {
      cleanup();
      return hip_fail(e, "staging parameter to device");
    }
  }
  rc = mrl_run(spec, dev);
  if (rc == MRL_OK) {
    for (uint32_t i = 0; i < spec->n_params; i++) {
      if (parameter_direction(*spec, i) == 0) continue;
      hipError_t e = hipMemcpy(params[i], dev[i], mrl_spec_parameter_bytes(spec, i), hipMemcpyDeviceToHost);
      if (e != hipSuccess) {
        cleanup();
        return hip_fail(e, "copying output to host");
      }
    }
  }
  cleanup();
  return rc;
}

int mrl_matmul(uint32_t b, uint32_t m, uint32_t k, uint32_t n, int dt_a, int dt_b, int dt_c, int accum,
               const void *a, const void *bmat, void *c, void *stream) {
  mrl_spec s;
  std::memset(&s, 0, sizeof s);
  s.kind = MRL_SPEC_MATMUL, s.accum = accum, s.rank = 4, s.n_params = 3;
  s.spec_shape[0] = b, s.spec_shape[1] = m, s.spec_shape[2] = k, s.spec_shape[3] = n;
  s.dtypes[0] = dt_a, s.dtypes[1] = dt_b, s.dtypes[2] = dt_c;
  for (uint32_t i = 0; i < 3; i++) {
    uint32_t shape[MRL_MAX_RANK], rank;
    parameter_shape(s, i, shape, &rank);
    mrl_layout_row_major(shape, rank, &s.layouts[i]);
  }
  void *params[3] = {const_cast<void *>(a), const_cast<void *>(bmat), c};
  return mrl_run_async(&s, params, stream);
}

int mrl_conv(uint32_t b, uint32_t f, uint32_t c, uint32_t oh, uint32_t ow, uint32_t fh, uint32_t fw,
             int dt_img, int dt_filt, int dt_out, int accum, const void *image, const void *filters,
             void *out, void *stream) {
  mrl_spec s;
  std::memset(&s, 0, sizeof s);
  s.kind = MRL_SPEC_CONV, s.accum = accum, s.rank = 7, s.n_params = 3;
  const uint32_t ss[7] = {b, f, c, oh, ow, fh, fw};
  for (int i = 0; i < 7; i++) {
    if (ss[i] == 0) return MRL_ERR_BAD_SPEC;
    s.spec_shape[i] = ss[i];
  }
  s.dtypes[0] = dt_img, s.dtypes[1] = dt_filt, s.dtypes[2] = dt_out;
  set_conv_default_layouts(&s);
  void *params[3] = {const_cast<void *>(image), const_cast<void *>(filters), out};
  return mrl_run_async(&s, params, stream);
}

int mrl_softmax(const uint32_t *shape, uint32_t rank, uint32_t scan_dim, const void *in, void *out,
                void *stream) {
  if (!shape) return MRL_ERR_NULL;
  if (rank == 0 || rank > MRL_MAX_RANK) return MRL_ERR_BAD_SPEC;
  mrl_spec s;
  std::memset(&s, 0, sizeof s);
  s.kind = MRL_SPEC_SOFTMAX, s.scan_dim = scan_dim, s.rank = rank, s.n_params = 2;
  for (uint32_t d = 0; d < rank; d++) s.spec_shape[d] = shape[d];
  s.dtypes[0] = s.dtypes[1] = MRL_F32;
  mrl_layout_row_major(shape, rank, &s.layouts[0]);
  s.layouts[1] = s.layouts[0];
  void *params[2] = {const_cast<void *>(in), out};
  return mrl_run_async(&s, params, stream);
}

int mrl_move(const uint32_t *shape, uint32_t rank, int dtype, const void *in, void *out, void *stream) {
  if (!shape) return MRL_ERR_NULL;
  if (rank == 0 || rank > MRL_MAX_RANK) return MRL_ERR_BAD_SPEC;
  mrl_spec s;
  std::memset(&s, 0, sizeof s);
  s.kind = MRL_SPEC_MOVE, s.rank = rank, s.n_params = 2;
  for (uint32_t d = 0; d < rank; d++) s.spec_shape[d] = shape[d];
  s.dtypes[0] = s.dtypes[1] = dtype;
  mrl_layout_row_major(shape, rank, &s.layouts[0]);
  s.layouts[1] = s.layouts[0];
  void *params[2] = {const_cast<void *>(in), out};
  return mrl_run_async(&s, params, stream);
}

int mrl_compose_msm(uint32_t b, uint32_t m, uint32_t k, uint32_t n2, uint32_t n, int dt_v, int dt_q,
                    int dt_kt, int kt_col_major, const void *v, const void *q, const void *kt,
                    void *out, void *stream) {
  mrl_spec s;
  std::memset(&s, 0, sizeof s);
  s.kind = MRL_SPEC_COMPOSE_MSM, s.rank = 5, s.n_params = 4;
  s.spec_shape[0] = b, s.spec_shape[1] = m, s.spec_shape[2] = k, s.spec_shape[3] = n2, s.spec_shape[4] = n;
  s.dtypes[0] = dt_v, s.dtypes[1] = dt_q, s.dtypes[2] = dt_kt, s.dtypes[3] = MRL_F32;
  for (uint32_t i = 0; i < 4; i++) {
    uint32_t shape[MRL_MAX_RANK], rank;
    if (parameter_shape(s, i, shape, &rank) != MRL_OK) return MRL_ERR_BAD_SPEC;
    if (i == 2 && kt_col_major) mrl_layout_batched_col_major(shape, rank, &s.layouts[i]);
    else mrl_layout_row_major(shape, rank, &s.layouts[i]);
  }
  void *params[4] = {const_cast<void *>(v), const_cast<void *>(q), const_cast<void *>(kt), out};
  return mrl_run_async(&s, params, stream);
}

uint32_t mrl_matmul_schedules(const mrl_spec *spec, mrl_matmul_schedule *out, uint32_t cap) {
  if (!spec || spec->kind != MRL_SPEC_MATMUL || check_spec(spec) != MRL_OK) return 0;
  const int da = spec->dtypes[0], db = spec->dtypes[1], dc = spec->dtypes[2];
  int es = 0;
  if ((da == MRL_U8 || da == MRL_I8) && db == MRL_I8 && dc == MRL_I32) es = 1;
  if (da == MRL_BF16 && db == MRL_BF16 && dc == MRL_F32) es = 2;
  if (da == MRL_F32 && db == MRL_F32 && dc == MRL_F32) es = 4;
  if (!es) return 0;
  const uint32_t n = mrl::gemm_schedule_count();
  for (uint32_t i = 0; i < n && out && i < cap; i++)
    mrl::gemm_schedule_at(i, es, &out[i].tile_m, &out[i].tile_n, &out[i].split_k, &out[i].staging);
  return n;
}

int mrl_run_matmul_scheduled(const mrl_spec *spec, void *const *params,
                             const mrl_matmul_schedule *schedule, void *stream) {
  if (!schedule || !params) return MRL_ERR_NULL;
  int rc;
  if (g_device < 0 && (rc = mrl_init(0)) != MRL_OK) return rc;
  if ((rc = check_spec(spec)) != MRL_OK) return rc;
  if (spec->kind != MRL_SPEC_MATMUL) return MRL_ERR_UNSUPPORTED;
  for (uint32_t i = 0; i < spec->n_params; i++)
    if (!params[i]) return MRL_ERR_NULL;
  Workspace ws((hipStream_t)stream);
  return run_matmul(*spec, params, ws, schedule);
}

int mrl_matmul_scheduled_plan(const mrl_spec *spec, const mrl_matmul_schedule *schedule, mrl_plan *plan,
                              mrl_plan_step *steps, uint32_t cap) {
  if (!schedule) return MRL_ERR_NULL;
  int rc = check_spec(spec);
  if (rc != MRL_OK) return rc;
  if (spec->kind != MRL_SPEC_MATMUL) return MRL_ERR_UNSUPPORTED;
  return plan_with(spec->n_params, plan, steps, cap,
                   [&](void *const *params, Workspace &ws) { return run_matmul(*spec, params, ws, schedule); });
}

int mrl_matmul_search_schedule(const mrl_spec *spec, mrl_matmul_schedule *best, double *cost_ns) {
  if (!best) return MRL_ERR_NULL;
  mrl_matmul_schedule all[16];
  const uint32_t n = mrl_matmul_schedules(spec, all, 16);
  if (n == 0) return MRL_ERR_UNSUPPORTED;
  double lowest = 0;
  bool found = false;
  for (uint32_t i = 0; i < n && i < 16; i++) {
    mrl_plan plan;
    if (mrl_matmul_scheduled_plan(spec, &all[i], &plan, nullptr, 0) != MRL_OK) continue;  // not for this shape
    if (!found || plan.cost_ns < lowest) lowest = plan.cost_ns, *best = all[i], found = true;
  }
  if (!found) return MRL_ERR_UNSUPPORTED;
  if (cost_ns) *cost_ns = lowest;
  return MRL_OK;
}

// ---- actions: the lowerings a search may choose among (Target::actions, target/mod.rs:69) ----

namespace {
// A primitive of the Softmax decomposition as a stand-alone Spec over row-major tensors.
int part_spec(int kind, const uint32_t *shape, uint32_t rank, uint32_t scan_dim, mrl_spec *s) {
  std::memset(s, 0, sizeof *s);
  s->kind = kind, s->scan_dim = scan_dim, s->rank = rank, s->n_params = expected_params(kind);
  for (uint32_t d = 0; d < rank; d++) s->spec_shape[d] = shape[d];
  for (uint32_t i = 0; i < s->n_params; i++) {
    s->dtypes[i] = MRL_F32;
    uint32_t pshape[MRL_MAX_RANK], prank;
    if (parameter_shape(*s, i, pshape, &prank) != MRL_OK) return MRL_ERR_BAD_SPEC;
    mrl_layout_row_major(pshape, prank, &s->layouts[i]);
  }
  return check_spec(s);
}

// A Softmax Spec through one of the reference's rewrites instead of the fused kernels, each stage
// a primitive Spec of its own (parts.hip), the tensors between the stages in intermediate buffers:
//   TO_SOFTMAX_PARTS            SoftmaxDenominatorAndUnscaled, then DivideVecScalar on the output
//                               (scheduling/to_softmax_parts.rs:33-108)
//   TO_SOFTMAX_PARTS_RECOMPUTE  SoftmaxDenominatorAndMax, then SoftmaxComplete, which forms the
//                               exponentials a second time (to_softmax_parts.rs:110-181)
//   PARALLEL_SOFTMAX            the same with the first stage split along the scan dim in `parts`
//                               tiles (scheduling/parallel_softmax.rs:24-223): a (max, denominator)
//                               pair per tile, merged by SoftmaxDenominatorAndMaxFromParts
// Written once, as the list of sub-Specs with their parameter sources (mrl_rewrite): what
// mrl_action_apply hands out is what run_rewrite runs.
int softmax_rewrite(const mrl_spec &s, const mrl_action &a, mrl_rewrite *rw) {
  if (s.kind != MRL_SPEC_SOFTMAX || s.dtypes[0] != MRL_F32 || s.dtypes[1] != MRL_F32) return MRL_ERR_UNSUPPORTED;
  std::memset(rw, 0, sizeof *rw);
  const uint32_t scan = s.spec_shape[s.scan_dim];
  uint64_t lines = 1;
  for (uint32_t d = 0; d < s.rank; d++)
    if (d != s.scan_dim) lines *= s.spec_shape[d];
  int rc;
  auto child = [&](int kind, const uint32_t *shape, uint32_t rank, uint32_t scan_dim, std::initializer_list<int32_t> sources) -> mrl_spec * {
    mrl_subspec &c = rw->subspecs[rw->n_subspecs++];
    rc = part_spec(kind, shape, rank, scan_dim, &c.spec);
    uint32_t i = 0;
    for (int32_t src : sources) c.source[i++] = src;
    return &c.spec;
  };
  auto intermediate = [&](uint64_t bytes) { rw->intermediate_bytes[rw->n_intermediates] = bytes; return -1 - int32_t(rw->n_intermediates++); };
  if (a.kind == MRL_ACTION_TO_SOFTMAX_PARTS) {
    const int32_t denom = intermediate(lines * sizeof(float));
    mrl_spec *st = child(MRL_SPEC_SOFTMAX_DENOMINATOR_AND_UNSCALED, s.spec_shape, s.rank, s.scan_dim, {0, denom, 1});
    if (rc != MRL_OK) return rc;
    st->layouts[0] = s.layouts[0], st->layouts[2] = s.layouts[1];
    st = child(MRL_SPEC_DIVIDE_VEC_SCALAR, s.spec_shape, s.rank, s.scan_dim, {1, denom});
    if (rc != MRL_OK) return rc;
    st->layouts[0] = s.layouts[1];
    return MRL_OK;
  }
  const int32_t mx = intermediate(lines * sizeof(float)), denom = intermediate(lines * sizeof(float));
  if (a.kind == MRL_ACTION_TO_SOFTMAX_PARTS_RECOMPUTE) {
    mrl_spec *st = child(MRL_SPEC_SOFTMAX_DENOMINATOR_AND_MAX, s.spec_shape, s.rank, s.scan_dim, {0, mx, denom});
    if (rc != MRL_OK) return rc;
    st->layouts[0] = s.layouts[0];
  } else if (a.kind == MRL_ACTION_PARALLEL_SOFTMAX) {
    // The tiles are a dim of their own: [.., scan, ..] read as [.., parts, scan / parts, ..], which
    // is the same buffer when the input is row-major and the tiles are equal.
    const uint32_t parts = a.parts;
    int64_t strides[MRL_MAX_RANK], running = 1;
    bool dense = mrl::layout_strides(s.layouts[0], s.spec_shape, s.rank, strides);
    for (int d = int(s.rank) - 1; dense && d >= 0; d--) {
      dense = s.spec_shape[d] == 1 || strides[d] == running;
      running *= s.spec_shape[d];
    }
    if (parts < 2 || scan % parts != 0 || s.rank + 1 > MRL_MAX_RANK || !dense) return MRL_ERR_UNSUPPORTED;
    uint32_t split[MRL_MAX_RANK], tiles[MRL_MAX_RANK];
    for (uint32_t d = 0, o = 0; d < s.rank; d++) {
      tiles[d] = d == s.scan_dim ? parts : s.spec_shape[d];
      if (d == s.scan_dim) split[o++] = parts, split[o++] = scan / parts;
      else split[o++] = s.spec_shape[d];
    }
    const int32_t tile_max = intermediate(lines * parts * sizeof(float)), tile_denom = intermediate(lines * parts * sizeof(float));
    child(MRL_SPEC_SOFTMAX_DENOMINATOR_AND_MAX, split, s.rank + 1, s.scan_dim + 1, {0, tile_max, tile_denom});
    if (rc != MRL_OK) return rc;
    child(MRL_SPEC_SOFTMAX_DENOMINATOR_AND_MAX_FROM_PARTS, tiles, s.rank, s.scan_dim, {tile_max, tile_denom, mx, denom});
    if (rc != MRL_OK) return rc;
  } else {
    return MRL_ERR_UNSUPPORTED;
  }
  mrl_spec *st = child(MRL_SPEC_SOFTMAX_COMPLETE, s.spec_shape, s.rank, s.scan_dim, {0, mx, denom, 1});
  if (rc != MRL_OK) return rc;
  st->layouts[0] = s.layouts[0], st->layouts[3] = s.layouts[1];
  return MRL_OK;
}

// The attention-shaped Compose with both tensors between its components in buffers
// (scheduling/bufferize.rs:24-116): S = Q . KT and P = softmax(S) as f32 tensors, row-major.
int compose_msm_rewrite(const mrl_spec &s, mrl_rewrite *rw) {
  if (s.kind != MRL_SPEC_COMPOSE_MSM) return MRL_ERR_UNSUPPORTED;
  std::memset(rw, 0, sizeof *rw);
  const uint32_t b = s.spec_shape[0], m = s.spec_shape[1], k = s.spec_shape[2], n2 = s.spec_shape[3], n = s.spec_shape[4];
  const uint64_t scores = uint64_t(b) * m * n2 * sizeof(float);
  rw->n_intermediates = 2, rw->intermediate_bytes[0] = rw->intermediate_bytes[1] = scores;
  rw->n_subspecs = 3;
  auto fill = [&](mrl_subspec &c, int kind, std::initializer_list<uint32_t> shape, uint32_t scan_dim, std::initializer_list<int32_t> dtypes,
                  std::initializer_list<int32_t> sources) {
    std::memset(&c, 0, sizeof c);
    c.spec.kind = kind, c.spec.scan_dim = scan_dim, c.spec.rank = uint32_t(shape.size()), c.spec.n_params = uint32_t(dtypes.size());
    uint32_t i = 0;
    for (uint32_t d : shape) c.spec.spec_shape[i++] = d;
    i = 0;
    for (int32_t dt : dtypes) c.spec.dtypes[i++] = dt;
    i = 0;
    for (int32_t src : sources) c.source[i++] = src;
    for (i = 0; i < c.spec.n_params; i++) {
      uint32_t pshape[MRL_MAX_RANK], prank;
      if (c.source[i] >= 0) c.spec.layouts[i] = s.layouts[c.source[i]];
      else if (parameter_shape(c.spec, i, pshape, &prank) == MRL_OK) mrl_layout_row_major(pshape, prank, &c.spec.layouts[i]);
    }
    return check_spec(&c.spec);
  };
  // Parameters of the Compose: V [b, n2, n], Q [b, m, k], KT [b, k, n2], out [b, m, n].
  int rc;
  if ((rc = fill(rw->subspecs[0], MRL_SPEC_MATMUL, {b, m, k, n2}, 0, {s.dtypes[1], s.dtypes[2], MRL_F32}, {1, 2, -1})) != MRL_OK) return rc;
  if ((rc = fill(rw->subspecs[1], MRL_SPEC_SOFTMAX, {b, m, n2}, 2, {MRL_F32, MRL_F32}, {-1, -2})) != MRL_OK) return rc;
  return fill(rw->subspecs[2], MRL_SPEC_MATMUL, {b, m, n2, n}, 0, {MRL_F32, s.dtypes[0], s.dtypes[3]}, {-2, 0, 3});
}

// The rewrites that apply to any Spec with an output parameter last:
//   TO_ACCUM       Fill{Zero} on the output, then the accumulating Spec (scheduling/to_accum.rs:12-60)
//   MOVE_RELAYOUT  a parameter through a row-major copy, CAST an input through a copy of the
//                  output's dtype: prologue Move when the parameter is read, the Spec on the copy,
//                  epilogue Move when it is written (scheduling/moves.rs:49-130)
int general_rewrite(const mrl_spec &s, const mrl_action &a, mrl_rewrite *rw) {
  std::memset(rw, 0, sizeof *rw);
  if (s.kind == MRL_SPEC_COMPOSE_MSM || s.n_params < 2) return MRL_ERR_UNSUPPORTED;
  const uint32_t out = s.n_params - 1;
  auto move_spec = [&](mrl_subspec &c, uint32_t i, int dt_from, const mrl_layout &l_from, int dt_to, const mrl_layout &l_to,
                       int32_t src_from, int32_t src_to) -> int {
    std::memset(&c, 0, sizeof c);
    c.spec.kind = MRL_SPEC_MOVE, c.spec.n_params = 2;
    if (parameter_shape(s, i, c.spec.spec_shape, &c.spec.rank) != MRL_OK) return MRL_ERR_BAD_SPEC;
    c.spec.dtypes[0] = dt_from, c.spec.dtypes[1] = dt_to;
    c.spec.layouts[0] = l_from, c.spec.layouts[1] = l_to;
    c.source[0] = src_from, c.source[1] = src_to;
    return check_spec(&c.spec);
  };
  int rc;
  if (a.kind == MRL_ACTION_TO_ACCUM) {
    if ((s.kind != MRL_SPEC_MATMUL && s.kind != MRL_SPEC_CONV) || s.accum) return MRL_ERR_UNSUPPORTED;
    mrl_subspec &zero = rw->subspecs[0];
    zero.spec.kind = MRL_SPEC_FILL, zero.spec.scan_dim = MRL_FILL_ZERO, zero.spec.n_params = 1;
    if (parameter_shape(s, out, zero.spec.spec_shape, &zero.spec.rank) != MRL_OK) return MRL_ERR_BAD_SPEC;
    zero.spec.dtypes[0] = s.dtypes[out], zero.spec.layouts[0] = s.layouts[out], zero.source[0] = int32_t(out);
    if ((rc = check_spec(&zero.spec)) != MRL_OK) return rc;
    mrl_subspec &body = rw->subspecs[1];
    body.spec = s, body.spec.accum = 1;
    for (uint32_t i = 0; i < s.n_params; i++) body.source[i] = int32_t(i);
    rw->n_subspecs = 2;
    return check_spec(&body.spec);
  }
  const uint32_t i = a.tile_m;
  if (i >= s.n_params) return MRL_ERR_UNSUPPORTED;
  uint32_t pshape[MRL_MAX_RANK], prank;
  if (parameter_shape(s, i, pshape, &prank) != MRL_OK) return MRL_ERR_BAD_SPEC;
  mrl_layout to_layout = s.layouts[i];
  int to_dtype = s.dtypes[i];
  if (a.kind == MRL_ACTION_MOVE_RELAYOUT) {
    mrl_layout_row_major(pshape, prank, &to_layout);
    int64_t now[MRL_MAX_RANK], rm[MRL_MAX_RANK];
    const bool strided = mrl::layout_strides(s.layouts[i], pshape, prank, now) && mrl::layout_strides(to_layout, pshape, prank, rm);
    bool same = strided;
    for (uint32_t d = 0; same && d < prank; d++) same = pshape[d] == 1 || now[d] == rm[d];
    if (same) return MRL_ERR_UNSUPPORTED;   // row-major already: nothing to move
  } else if (a.kind == MRL_ACTION_CAST) {
    if ((s.kind != MRL_SPEC_MATMUL && s.kind != MRL_SPEC_CONV) || i >= out || int(a.tile_n) != s.dtypes[out] ||
        s.dtypes[i] == s.dtypes[out])
      return MRL_ERR_UNSUPPORTED;
    to_dtype = s.dtypes[out];
  } else {
    return MRL_ERR_UNSUPPORTED;
  }
  uint64_t count = 1;
  for (uint32_t d = 0; d < prank; d++) count *= pshape[d];
  rw->n_intermediates = 1, rw->intermediate_bytes[0] = count * mrl_dtype_size(to_dtype);
  const bool written = i == out, read = !written || s.accum;
  if (read && (rc = move_spec(rw->subspecs[rw->n_subspecs++], i, s.dtypes[i], s.layouts[i], to_dtype, to_layout, int32_t(i), -1)) != MRL_OK)
    return rc;
  mrl_subspec &body = rw->subspecs[rw->n_subspecs++];
  body.spec = s, body.spec.dtypes[i] = to_dtype, body.spec.layouts[i] = to_layout;
  for (uint32_t j = 0; j < s.n_params; j++) body.source[j] = j == i ? -1 : int32_t(j);
  if ((rc = check_spec(&body.spec)) != MRL_OK) return rc;
  if (written && (rc = move_spec(rw->subspecs[rw->n_subspecs++], i, to_dtype, to_layout, s.dtypes[i], s.layouts[i], -1, int32_t(i))) != MRL_OK)
    return rc;
  return MRL_OK;
}

// The rewrites of the Softmax primitives, each two stages on f32 tensors:
//   TO_MAX_AND_DENOMINATOR  SoftmaxDenominatorAndMax -> Max, SoftmaxDenominator (to_max_and_denom.rs:13-72)
//   TO_MAX_AND_UNSCALED     SoftmaxDenominatorAndUnscaled -> Max into a buffer,
//                           SoftmaxDenominatorAndUnscaledFromMax (to_max_and_unscaled.rs:30-110)
//   BROADCAST_FIRST         DivideVecScalar -> Broadcast of the denominators, DivideVec (broadcast_first.rs:24-130)
int primitive_rewrite(const mrl_spec &s, const mrl_action &a, mrl_rewrite *rw) {
  std::memset(rw, 0, sizeof *rw);
  for (uint32_t i = 0; i < s.n_params; i++)
    if (s.dtypes[i] != MRL_F32) return MRL_ERR_UNSUPPORTED;
  int rc = MRL_OK;
  auto child = [&](int kind, std::initializer_list<int32_t> sources) {
    mrl_subspec &c = rw->subspecs[rw->n_subspecs++];
    if ((rc = part_spec(kind, s.spec_shape, s.rank, s.scan_dim, &c.spec)) != MRL_OK) return;
    uint32_t i = 0;
    for (int32_t src : sources) {
      if (src >= 0) c.spec.layouts[i] = s.layouts[src];
      c.source[i++] = src;
    }
    rc = check_spec(&c.spec);
  };
  uint64_t count = 1, lines = 1;
  for (uint32_t d = 0; d < s.rank; d++) count *= s.spec_shape[d], lines *= d == s.scan_dim ? 1 : s.spec_shape[d];
  if (a.kind == MRL_ACTION_TO_MAX_AND_DENOMINATOR) {
    if (s.kind != MRL_SPEC_SOFTMAX_DENOMINATOR_AND_MAX || s.accum) return MRL_ERR_UNSUPPORTED;
    child(MRL_SPEC_MAX, {0, 1});
    if (rc == MRL_OK) child(MRL_SPEC_SOFTMAX_DENOMINATOR, {0, 1, 2});
  } else if (a.kind == MRL_ACTION_TO_MAX_AND_UNSCALED) {
    if (s.kind != MRL_SPEC_SOFTMAX_DENOMINATOR_AND_UNSCALED || s.accum) return MRL_ERR_UNSUPPORTED;
    rw->n_intermediates = 1, rw->intermediate_bytes[0] = lines * sizeof(float);
    child(MRL_SPEC_MAX, {0, -1});
    if (rc == MRL_OK) child(MRL_SPEC_SOFTMAX_DENOMINATOR_AND_UNSCALED_FROM_MAX, {0, -1, 1, 2});
  } else if (a.kind == MRL_ACTION_BROADCAST_FIRST) {
    if (s.kind != MRL_SPEC_DIVIDE_VEC_SCALAR) return MRL_ERR_UNSUPPORTED;
    rw->n_intermediates = 1, rw->intermediate_bytes[0] = count * sizeof(float);
    child(MRL_SPEC_BROADCAST, {1, -1});
    if (rc == MRL_OK) child(MRL_SPEC_DIVIDE_VEC, {0, -1});
  } else {
    return MRL_ERR_UNSUPPORTED;
  }
  return rc;
}

int rewrite_of(const mrl_spec &s, const mrl_action &a, mrl_rewrite *rw) {
  switch (a.kind) {
    case MRL_ACTION_TO_SOFTMAX_PARTS:
    case MRL_ACTION_TO_SOFTMAX_PARTS_RECOMPUTE:
    case MRL_ACTION_PARALLEL_SOFTMAX: return softmax_rewrite(s, a, rw);
    case MRL_ACTION_TO_ACCUM:
    case MRL_ACTION_MOVE_RELAYOUT:
    case MRL_ACTION_CAST: return general_rewrite(s, a, rw);
    case MRL_ACTION_TO_MAX_AND_DENOMINATOR:
    case MRL_ACTION_TO_MAX_AND_UNSCALED:
    case MRL_ACTION_BROADCAST_FIRST: return primitive_rewrite(s, a, rw);
    default: return MRL_ERR_UNSUPPORTED;
  }
}

// A rewrite run as what it is: its sub-Specs one after the other, the buffers between them in scratch.
int run_rewrite(const mrl_spec &s, void *const *params, Workspace &ws, const mrl_action &a) {
  mrl_rewrite rw;
  int rc;
  if ((rc = rewrite_of(s, a, &rw)) != MRL_OK) return rc;
  void *between[MRL_MAX_SUBSPECS] = {};
  for (uint32_t j = 0; j < rw.n_intermediates; j++) HIP_TRY(ws.alloc(&between[j], rw.intermediate_bytes[j]));
  for (uint32_t c = 0; c < rw.n_subspecs; c++) {
    void *p[MRL_MAX_PARAMS];
    for (uint32_t i = 0; i < rw.subspecs[c].spec.n_params; i++) {
      const int32_t src = rw.subspecs[c].source[i];
      p[i] = src >= 0 ? params[src] : between[-1 - src];
    }
    if ((rc = dispatch(rw.subspecs[c].spec, p, ws)) != MRL_OK) return rc;
  }
  return MRL_OK;
}

// Runs `spec` under `action` through `ws` (a recording Workspace when planning).
int dispatch_action(const mrl_spec &spec, void *const *params, Workspace &ws, const mrl_action &a) {
  Forced f;
  switch (a.kind) {
    case MRL_ACTION_SELECT: return dispatch(spec, params, ws);
    case MRL_ACTION_TO_SOFTMAX_PARTS:
    case MRL_ACTION_TO_SOFTMAX_PARTS_RECOMPUTE:
    case MRL_ACTION_PARALLEL_SOFTMAX:
    case MRL_ACTION_TO_ACCUM:
    case MRL_ACTION_MOVE_RELAYOUT:
    case MRL_ACTION_CAST:
    case MRL_ACTION_TO_MAX_AND_DENOMINATOR:
    case MRL_ACTION_TO_MAX_AND_UNSCALED:
    case MRL_ACTION_BROADCAST_FIRST: return run_rewrite(spec, params, ws, a);
    case MRL_ACTION_TILE_OUT_SPLIT: {
      if (spec.kind != MRL_SPEC_MATMUL) return MRL_ERR_UNSUPPORTED;
      const mrl_matmul_schedule sched = {a.tile_m, a.tile_n, a.split_k, a.staging};
      return run_matmul(spec, params, ws, &sched);
    }
    case MRL_ACTION_SPATIAL_SPLIT: f.conv_path = 2, f.conv_tile = a.tile_m; break;
    case MRL_ACTION_UNFOLD: f.conv_path = 3; break;
    case MRL_ACTION_GENERIC: f.conv_path = 4; break;
    case MRL_ACTION_FUSED:
      f.conv_path = 1, f.msm_path = 1, f.key_splits = a.parts ? a.parts : 1, f.query_block = a.tile_m;
      f.conv_rows = spec.kind == MRL_SPEC_CONV && a.tile_m != 0;   // tile_out over whole output rows
      break;
    case MRL_ACTION_BUFFERIZE: f.msm_path = 2; break;
    default: return MRL_ERR_BAD_SPEC;
  }
  // A Compose's key shares: what mrl_target_actions lists, one share or at least two blocks of 64 keys each.
  if (a.kind == MRL_ACTION_FUSED && spec.kind == MRL_SPEC_COMPOSE_MSM && a.parts > 1 &&
      (a.parts > 64 || 2 * uint64_t(a.parts) > (uint64_t(spec.spec_shape[3]) + 63) / 64))
    return MRL_ERR_UNSUPPORTED;
  const bool conv_action = a.kind == MRL_ACTION_SPATIAL_SPLIT || a.kind == MRL_ACTION_UNFOLD || a.kind == MRL_ACTION_GENERIC;
  if ((conv_action && spec.kind != MRL_SPEC_CONV) || (a.kind == MRL_ACTION_BUFFERIZE && spec.kind != MRL_SPEC_COMPOSE_MSM) ||
      (a.kind == MRL_ACTION_FUSED && spec.kind != MRL_SPEC_CONV && spec.kind != MRL_SPEC_COMPOSE_MSM) ||
      (a.kind == MRL_ACTION_SPATIAL_SPLIT && (a.tile_m != a.tile_n || (a.tile_m != 64 && a.tile_m != 128 && a.tile_m != 256))))
    return MRL_ERR_UNSUPPORTED;
  g_forced = &f;
  const int rc = dispatch(spec, params, ws);
  g_forced = nullptr;
  return rc;
}
}  // namespace

int mrl_action_apply(const mrl_spec *spec, const mrl_action *action, mrl_rewrite *out) {
  if (!action || !out) return MRL_ERR_NULL;
  int rc = check_spec(spec);
  if (rc != MRL_OK) return rc;
  switch (action->kind) {
    case MRL_ACTION_TO_SOFTMAX_PARTS:
    case MRL_ACTION_TO_SOFTMAX_PARTS_RECOMPUTE:
    case MRL_ACTION_PARALLEL_SOFTMAX:
    case MRL_ACTION_TO_ACCUM:
    case MRL_ACTION_MOVE_RELAYOUT:
    case MRL_ACTION_CAST:
    case MRL_ACTION_TO_MAX_AND_DENOMINATOR:
    case MRL_ACTION_TO_MAX_AND_UNSCALED:
    case MRL_ACTION_BROADCAST_FIRST: return rewrite_of(*spec, *action, out);
    case MRL_ACTION_BUFFERIZE: return compose_msm_rewrite(*spec, out);
    default: break;
  }
  // A leaf: the action must at least apply to the Spec.
  mrl_plan plan;
  if ((rc = mrl_action_plan(spec, action, &plan, nullptr, 0)) != MRL_OK) return rc;
  std::memset(out, 0, sizeof *out);
  return MRL_OK;
}

int mrl_action_plan(const mrl_spec *spec, const mrl_action *action, mrl_plan *plan, mrl_plan_step *steps, uint32_t cap) {
  if (!action) return MRL_ERR_NULL;
  int rc = check_spec(spec);
  if (rc != MRL_OK) return rc;
  return plan_with(spec->n_params, plan, steps, cap,
                   [&](void *const *params, Workspace &ws) { return dispatch_action(*spec, params, ws, *action); });
}

int mrl_run_action(const mrl_spec *spec, void *const *params, const mrl_action *action, void *stream) {
  if (!action || !params) return MRL_ERR_NULL;
  int rc;
  if (g_device < 0 && (rc = mrl_init(0)) != MRL_OK) return rc;
  if ((rc = check_spec(spec)) != MRL_OK) return rc;
  for (uint32_t i = 0; i < spec->n_params; i++)
    if (!params[i]) return MRL_ERR_NULL;
  Workspace ws((hipStream_t)stream);
  return dispatch_action(*spec, params, ws, *action);
}

uint32_t mrl_target_actions(const mrl_spec *spec, mrl_action *out, uint32_t cap) {
  if (check_spec(spec) != MRL_OK) return 0;
  std::vector<mrl_action> candidates;
  auto candidate = [&](int kind, uint32_t tm = 0, uint32_t tn = 0, uint32_t sk = 0, uint32_t parts = 0) {
    mrl_action a;
    std::memset(&a, 0, sizeof a);
    a.kind = kind, a.tile_m = tm, a.tile_n = tn, a.split_k = sk, a.parts = parts;
    candidates.push_back(a);
  };
  candidate(MRL_ACTION_SELECT);
  if (spec->kind == MRL_SPEC_MATMUL) {
    mrl_matmul_schedule all[16];
    const uint32_t n = std::min<uint32_t>(16, mrl_matmul_schedules(spec, all, 16));
    for (uint32_t i = 0; i < n; i++) {
      candidate(MRL_ACTION_TILE_OUT_SPLIT, all[i].tile_m, all[i].tile_n, all[i].split_k);
      candidates.back().staging = all[i].staging;
    }
  } else if (spec->kind == MRL_SPEC_CONV) {
    candidate(MRL_ACTION_FUSED);
    candidate(MRL_ACTION_FUSED, spec->spec_shape[4]);   // tile_out over whole output rows (tile_m = ow)
    for (uint32_t side : {64u, 128u, 256u}) candidate(MRL_ACTION_SPATIAL_SPLIT, side, side, 0);
    candidate(MRL_ACTION_UNFOLD);
    candidate(MRL_ACTION_GENERIC);
  } else if (spec->kind == MRL_SPEC_COMPOSE_MSM) {
    // parallel_softmax.rs:31-223: the keys in `parts` shares, each at least two blocks of 64.
    const uint32_t blocks = (spec->spec_shape[3] + 63) / 64;
    for (uint32_t parts = 1; parts <= 64 && (parts == 1 || 2 * parts <= blocks); parts *= 2)
      for (uint32_t rows : {128u, 64u}) candidate(MRL_ACTION_FUSED, rows, 0, 0, parts);
    candidate(MRL_ACTION_BUFFERIZE);
  } else if (spec->kind == MRL_SPEC_SOFTMAX) {
    candidate(MRL_ACTION_TO_SOFTMAX_PARTS);
    candidate(MRL_ACTION_TO_SOFTMAX_PARTS_RECOMPUTE);
    // parallel_softmax.rs:60-66: a tile shorter than the scan dim; here equal tiles of 64 elements or more
    const uint32_t scan = spec->spec_shape[spec->scan_dim];
    for (uint32_t parts = 2; parts <= 64 && scan / parts >= 64; parts *= 2)
      if (scan % parts == 0) candidate(MRL_ACTION_PARALLEL_SOFTMAX, 0, 0, 0, parts);
  }
  if (spec->kind == MRL_SPEC_SOFTMAX_DENOMINATOR_AND_MAX) candidate(MRL_ACTION_TO_MAX_AND_DENOMINATOR);
  if (spec->kind == MRL_SPEC_SOFTMAX_DENOMINATOR_AND_UNSCALED) candidate(MRL_ACTION_TO_MAX_AND_UNSCALED);
  if (spec->kind == MRL_SPEC_DIVIDE_VEC_SCALAR) candidate(MRL_ACTION_BROADCAST_FIRST);
  // The rewrites any Spec may take, last in the list: to_accum, and per parameter a row-major
  // copy (move_relayout) or a copy in the output's dtype (cast); those that do not apply drop out below.
  if (spec->kind != MRL_SPEC_COMPOSE_MSM) {
    candidate(MRL_ACTION_TO_ACCUM);
    for (uint32_t i = 0; i < spec->n_params; i++) candidate(MRL_ACTION_MOVE_RELAYOUT, i);
    for (uint32_t i = 0; i + 1 < spec->n_params; i++) candidate(MRL_ACTION_CAST, i, uint32_t(spec->dtypes[spec->n_params - 1]));
  }
  uint32_t n = 0;
  for (mrl_action &a : candidates) {
    mrl_plan plan;
    if (mrl_action_plan(spec, &a, &plan, nullptr, 0) != MRL_OK) continue;   // not for this Spec
    a.n_steps = plan.n_steps, a.scratch_bytes = plan.scratch_bytes, a.cost_ns = plan.cost_ns;
    if (out && n < cap) out[n] = a;
    n++;
  }
  return n;
}

int mrl_bench(const mrl_spec *spec, void *const *params, uint32_t iters, uint32_t repeats,
              double *best_ns_per_iter, double *mean_ns_per_iter) {
  if (!best_ns_per_iter || !mean_ns_per_iter) return MRL_ERR_NULL;
  if (iters == 0 || repeats == 0) return MRL_ERR_BAD_SPEC;
  int rc = mrl_run(spec, params);  // warm-up, as the emitted benchmark main does
  if (rc != MRL_OK) return rc;
  hipEvent_t t0, t1;
  HIP_TRY(hipEventCreate(&t0));
  HIP_TRY(hipEventCreate(&t1));
  double best = 1e300, total = 0.0;
  for (uint32_t r = 0; r < repeats && rc == MRL_OK; r++) {
    (void)hipEventRecord(t0, nullptr);
    for (uint32_t i = 0; i < iters && rc == MRL_OK; i++) rc = run_async_impl(spec, params, nullptr);
    (void)hipEventRecord(t1, nullptr);
    hipError_t e = hipEventSynchronize(t1);
    if (e != hipSuccess) rc = hip_fail(e, "hipEventSynchronize");
    float ms = 0.0f;
    (void)hipEventElapsedTime(&ms, t0, t1);
    const double ns = double(ms) * 1e6 / iters;
    if (ns < best) best = ns;
    total += ns;
  }
  (void)hipEventDestroy(t0);
  (void)hipEventDestroy(t1);
  *best_ns_per_iter = best;
  *mean_ns_per_iter = total / repeats;
  return rc;
}

int mrl_run_timed(const mrl_spec *spec, void *const *params, uint32_t steps,
                  double *device_ms_total) {
  if (!device_ms_total) return MRL_ERR_NULL;
  if (steps == 0) return MRL_ERR_BAD_SPEC;
  int rc = check_spec(spec);
  if (rc != MRL_OK) return rc;
  hipEvent_t t0, t1;
  HIP_TRY(hipEventCreate(&t0));
  HIP_TRY(hipEventCreate(&t1));
  (void)hipEventRecord(t0, nullptr);
  for (uint32_t i = 0; i < steps && rc == MRL_OK; i++) rc = run_async_impl(spec, params, nullptr);
  (void)hipEventRecord(t1, nullptr);
  hipError_t e = hipEventSynchronize(t1);
  float ms = 0.0f;
  if (e == hipSuccess) e = hipEventElapsedTime(&ms, t0, t1);
  (void)hipEventDestroy(t0);
  (void)hipEventDestroy(t1);
  if (rc != MRL_OK) return rc;
  if (e != hipSuccess) return hip_fail(e, "event timing");
  *device_ms_total = double(ms);
  return MRL_OK;
}

int mrl_run_action_timed(const mrl_spec *spec, void *const *params, const mrl_action *action, uint32_t steps,
                         double *device_ms_total) {
  if (!device_ms_total || !action) return MRL_ERR_NULL;
  if (steps == 0) return MRL_ERR_BAD_SPEC;
  hipEvent_t t0, t1;
  HIP_TRY(hipEventCreate(&t0));
  HIP_TRY(hipEventCreate(&t1));
  (void)hipEventRecord(t0, nullptr);
  int rc = MRL_OK;
  for (uint32_t i = 0; i < steps && rc == MRL_OK; i++) rc = mrl_run_action(spec, params, action, nullptr);
  (void)hipEventRecord(t1, nullptr);
  hipError_t e = hipEventSynchronize(t1);
  float ms = 0.0f;
  if (e == hipSuccess) e = hipEventElapsedTime(&ms, t0, t1);
  (void)hipEventDestroy(t0);
  (void)hipEventDestroy(t1);
  if (rc != MRL_OK) return rc;
  if (e != hipSuccess) return hip_fail(e, "event timing");
  *device_ms_total = double(ms);
  return MRL_OK;
}

int mrl_compose_init(mrl_compose *c) {
  if (!c) return MRL_ERR_NULL;
  std::vector<ComposeParam> ext;
  std::vector<mrl_spec> specs;
  int rc = compose_parameters(*c, &ext, &specs);
  if (rc != MRL_OK) return rc;
  c->n_params = uint32_t(ext.size());
  c->bufferize_mask = 0;
  for (size_t i = 0; i < ext.size(); i++) c->layouts[i] = specs[ext[i].component].layouts[ext[i].param];
  return MRL_OK;
}

int mrl_compose_parameter(const mrl_compose *c, uint32_t idx, uint32_t *component, uint32_t *param) {
  if (!c || !component || !param) return MRL_ERR_NULL;
  std::vector<ComposeParam> ext;
  std::vector<mrl_spec> specs;
  int rc = compose_parameters(*c, &ext, &specs);
  if (rc != MRL_OK) return rc;
  if (idx >= ext.size()) return MRL_ERR_BAD_SPEC;
  *component = ext[idx].component, *param = ext[idx].param;
  return MRL_OK;
}

int mrl_compose_parameter_shape(const mrl_compose *c, uint32_t idx, uint32_t *shape, uint32_t *rank) {
  if (!c || !shape || !rank) return MRL_ERR_NULL;
  std::vector<ComposeParam> ext;
  std::vector<mrl_spec> specs;
  int rc = compose_parameters(*c, &ext, &specs);
  if (rc != MRL_OK) return rc;
  if (idx >= ext.size()) return MRL_ERR_BAD_SPEC;
  return parameter_shape(specs[ext[idx].component], ext[idx].param, shape, rank);
}

int mrl_compose_parameter_dtype(const mrl_compose *c, uint32_t idx) {
  if (!c) return -1;
  std::vector<ComposeParam> ext;
  std::vector<mrl_spec> specs;
  if (compose_parameters(*c, &ext, &specs) != MRL_OK || idx >= ext.size()) return -1;
  return specs[ext[idx].component].dtypes[ext[idx].param];
}

int mrl_run_compose(const mrl_compose *c, void *const *params, void *stream) {
  if (!c || !params) return MRL_ERR_NULL;
  int rc;
  if (g_device < 0 && (rc = mrl_init(0)) != MRL_OK) return rc;
  Workspace ws(static_cast<hipStream_t>(stream));
  return run_compose_general(*c, params, ws);
}

int mrl_measure_mfma_rate(int kind, int random_operands, uint32_t iters, double *ops_per_second) {
  if (!ops_per_second) return MRL_ERR_NULL;
  if ((kind != 0 && kind != 1) || iters == 0) return MRL_ERR_BAD_SPEC;
  int rc;
  if (g_device < 0 && (rc = mrl_init(0)) != MRL_OK) return rc;
  HIP_TRY(mrl::measure_mfma_rate(kind, random_operands != 0, iters, nullptr, ops_per_second));
  return MRL_OK;
}

int mrl_device_malloc(void **ptr, size_t bytes) {
  if (!ptr) return MRL_ERR_NULL;
  int rc;
  if (g_device < 0 && (rc = mrl_init(0)) != MRL_OK) return rc;
  HIP_TRY(hipMalloc(ptr, bytes ? bytes : 4));
  return MRL_OK;
}
int mrl_device_free(void *ptr) {
  HIP_TRY(hipFree(ptr));
  return MRL_OK;
}
int mrl_memcpy_h2d(void *dst, const void *src, size_t bytes) {
  HIP_TRY(hipMemcpy(dst, src, bytes, hipMemcpyHostToDevice));
  return MRL_OK;
}
int mrl_memcpy_d2h(void *dst, const void *src, size_t bytes) {
  HIP_TRY(hipMemcpy(dst, src, bytes, hipMemcpyDeviceToHost));
  return MRL_OK;
}
int mrl_memset(void *dst, int value, size_t bytes) {
  HIP_TRY(hipMemset(dst, value, bytes));
  return MRL_OK;
}
int mrl_stream_create(void **stream) {
  if (!stream) return MRL_ERR_NULL;
  int rc;
  if (g_device < 0 && (rc = mrl_init(0)) != MRL_OK) return rc;
  hipStream_t st = nullptr;
  HIP_TRY(hipStreamCreate(&st));
  *stream = st;
  return MRL_OK;
}

int mrl_stream_synchronize(void *stream) {
  HIP_TRY(hipStreamSynchronize(static_cast<hipStream_t>(stream)));
  return MRL_OK;
}

int mrl_stream_release(void *stream) {
  HIP_TRY(hipStreamSynchronize(static_cast<hipStream_t>(stream)));
  drop_arena(static_cast<hipStream_t>(stream));
  return MRL_OK;
}

int mrl_stream_destroy(void *stream) {
  if (!stream) return MRL_ERR_NULL;
  HIP_TRY(hipStreamSynchronize(static_cast<hipStream_t>(stream)));
  drop_arena(static_cast<hipStream_t>(stream));
  HIP_TRY(hipStreamDestroy(static_cast<hipStream_t>(stream)));
  return MRL_OK;
}

int mrl_device_mem_free(size_t *free_bytes) {
  if (!free_bytes) return MRL_ERR_NULL;
  size_t total = 0;
  HIP_TRY(hipMemGetInfo(free_bytes, &total));
  return MRL_OK;
}

int mrl_device_synchronize(void) {
  HIP_TRY(hipDeviceSynchronize());
  return MRL_OK;
}
int mrl_device_info(char *name, size_t name_len, int *compute_units, int *clock_khz,
                    size_t *total_mem_bytes) {
  int rc;
  if (g_device < 0 && (rc = mrl_init(0)) != MRL_OK) return rc;
  hipDeviceProp_t prop;
  HIP_TRY(hipGetDeviceProperties(&prop, g_device));
  if (name && name_len) std::snprintf(name, name_len, "%s (%s)", prop.name, prop.gcnArchName);
  if (compute_units) *compute_units = prop.multiProcessorCount;
  if (clock_khz) *clock_khz = prop.clockRate;
  if (total_mem_bytes) *total_mem_bytes = prop.totalGlobalMem;
  return MRL_OK;
}

}  // extern "C"
