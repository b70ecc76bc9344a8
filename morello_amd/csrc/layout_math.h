// Layout index arithmetic shared by host code and device kernels.
//
// A Morello layout is a list of physical dims, slowest to fastest, each naming a logical
// dim and being Dynamic, Packed(n) or OddEven(n) (morello/src/layout.rs:67-81).  The flat
// buffer offset of a logical point is defined by buffer_indexing_expr
// (layout.rs:221-272) over the physical shape from expand_physical_shape
// (layout.rs:769-810).  LayoutEval is that expression with all shape-dependent constants
// folded, in a plain struct that can be passed to a kernel by value.
#pragma once
#include <stdint.h>

#include "../../include/morello_amd.h"

#if defined(__HIPCC__)
#define MRL_HD __host__ __device__
#else
#define MRL_HD
#endif

namespace mrl {

struct LayoutEval {
  uint32_t rank;
  uint32_t ndims;
  uint32_t shape[MRL_MAX_RANK];
  uint8_t ld[MRL_MAX_PHYS];      // logical dim of each physical dim
  uint8_t oddeven[MRL_MAX_PHYS]; // 1 if OddEven
  uint8_t divide[MRL_MAX_PHYS];  // 1 if the term is divided by `next`
  uint32_t psize[MRL_MAX_PHYS];  // physical size
  uint32_t mod[MRL_MAX_PHYS];    // 0 = no modulo, else term %= mod
  uint32_t next[MRL_MAX_PHYS];   // remaining volume of the logical dim after this dim
  uint32_t strip[MRL_MAX_PHYS];  // OddEven strip size
};

// layout.rs:769-810.  Returns false when the layout does not apply to the shape.
inline bool physical_shape(const mrl_layout &l, const uint32_t *shape, uint32_t rank,
                           uint32_t *phys) {
  if (rank > MRL_MAX_RANK || l.ndims > MRL_MAX_PHYS) return false;
  uint32_t remaining[MRL_MAX_RANK];
  bool tiled[MRL_MAX_RANK];
  for (uint32_t d = 0; d < rank; d++) {
    if (shape[d] == 0) return false;
    remaining[d] = shape[d];
    tiled[d] = false;
  }
  for (int i = int(l.ndims) - 1; i >= 0; i--) {
    const mrl_physdim &pd = l.dims[i];
    if (pd.logical_dim >= rank) return false;
    uint32_t &rem = remaining[pd.logical_dim];
    if (rem == 0) return false;  // a Dynamic dim already consumed this logical dim
    if (pd.kind == MRL_DYNAMIC) {
      phys[i] = rem;
      rem = 0;
    } else if (pd.kind == MRL_PACKED || pd.kind == MRL_ODDEVEN) {
      if (pd.size == 0) return false;
      if (pd.kind == MRL_ODDEVEN && (pd.size & 1u)) return false;
      if (rem < pd.size) {
        const bool smaller_ok = pd.kind == MRL_PACKED || rem == 1;
        if (!smaller_ok || tiled[pd.logical_dim]) return false;
        phys[i] = rem;
        rem = 1;
        tiled[pd.logical_dim] = true;
      } else if (rem % pd.size != 0) {
        return false;
      } else {
        phys[i] = pd.size;
        rem /= pd.size;
      }
    } else {
      return false;
    }
  }
  for (uint32_t d = 0; d < rank; d++)
    if (remaining[d] > 1) return false;
  return true;
}

// Folds layout.rs:221-272 for a concrete shape.
inline bool make_layout_eval(const mrl_layout &l, const uint32_t *shape, uint32_t rank,
                             LayoutEval *ev) {
  uint32_t phys[MRL_MAX_PHYS];
  if (!physical_shape(l, shape, rank, phys)) return false;
  ev->rank = rank;
  ev->ndims = l.ndims;
  uint32_t remaining[MRL_MAX_RANK];
  for (uint32_t d = 0; d < MRL_MAX_RANK; d++) ev->shape[d] = d < rank ? shape[d] : 1;
  for (uint32_t d = 0; d < rank; d++) remaining[d] = shape[d];
  for (uint32_t i = 0; i < l.ndims; i++) {
    const uint32_t ld = l.dims[i].logical_dim;
    const uint32_t prev = remaining[ld];
    const uint32_t next = prev / phys[i];
    remaining[ld] = next;
    ev->ld[i] = uint8_t(ld);
    ev->psize[i] = phys[i];
    ev->mod[i] = prev != shape[ld] ? prev : 0;
    ev->next[i] = next;
    ev->oddeven[i] = l.dims[i].kind == MRL_ODDEVEN;
    ev->strip[i] = l.dims[i].size;
    ev->divide[i] = ev->oddeven[i] || shape[ld] != phys[i];
  }
  return true;
}

MRL_HD inline int64_t layout_offset(const LayoutEval &ev, const uint32_t *pt) {
  int64_t working = 0;
  for (uint32_t i = 0; i < ev.ndims; i++) {
    uint32_t term = pt[ev.ld[i]];
    if (ev.mod[i]) term %= ev.mod[i];
    if (ev.oddeven[i]) {
      const uint32_t in_strip = term % ev.strip[i];
      term = in_strip / 2 + (in_strip % 2) * (ev.strip[i] / 2);
    }
    if (ev.divide[i]) term /= ev.next[i];
    working = working * int64_t(ev.psize[i]) + int64_t(term);
  }
  return working;
}

// A layout whose physical dims are all Dynamic is a pure permutation of the logical dims:
// element (p0..pr) lives at sum(stride[d] * pd).  Fills strides (0 for size-one dims that
// the layout omits) and returns true in that case.
inline bool layout_strides(const mrl_layout &l, const uint32_t *shape, uint32_t rank,
                           int64_t *strides) {
  uint32_t phys[MRL_MAX_PHYS];
  if (!physical_shape(l, shape, rank, phys)) return false;
  for (uint32_t d = 0; d < rank; d++) strides[d] = 0;
  int64_t running = 1;
  for (int i = int(l.ndims) - 1; i >= 0; i--) {
    if (l.dims[i].kind != MRL_DYNAMIC) {
      // A Packed/OddEven dim that covers its whole logical dim once is still strided only
      // if it is Packed and is the sole physical dim of that logical dim.
      const uint32_t ld = l.dims[i].logical_dim;
      uint32_t uses = 0;
      for (uint32_t j = 0; j < l.ndims; j++) uses += l.dims[j].logical_dim == ld;
      if (l.dims[i].kind != MRL_PACKED || uses != 1 || phys[i] != shape[ld]) return false;
    }
    strides[l.dims[i].logical_dim] = running;
    running *= phys[i];
  }
  return true;
}

}  // namespace mrl
