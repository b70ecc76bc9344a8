// Two layouts of one logical shape as a common strided view (host code).
//
// A Packed(n) physical dim splits its logical dim into "which group of n" and "which of the n";
// an OddEven(n) dim splits a strip of n into "which pair" and "odd or even" and stores the
// parity outermost (morello/src/layout.rs:221-272).  Either way a layout is a mixed-radix
// decomposition of each logical index, one stride per digit.  Two layouts of the same shape can
// be given the same digits whenever their radices refine each other (8 and 16 do, 6 and 4 do
// not); the Move between them is then a plain permutation of a higher-rank tensor, which the
// strided Move kernels take.  Where they do not, the caller falls back to index arithmetic per
// element.
#pragma once
#include <algorithm>
#include <vector>

#include "layout_math.h"

namespace mrl {

constexpr uint32_t MOVE_MAX_RANK = 12;

// One digit of the common view: `size` values, `ss` / `ds` elements apart on the two sides.
struct MoveDim {
  uint32_t size;
  int64_t ss, ds;
};

namespace detail {

struct Digit {
  uint32_t size;
  int64_t stride;
};

// Digits of each logical dim, most significant first.  False for a layout this view cannot
// express (an OddEven dim that is not the innermost dim of its logical dim).
inline bool digits_of(const mrl_layout &l, const uint32_t *shape, uint32_t rank,
                      std::vector<Digit> (&out)[MRL_MAX_RANK]) {
  uint32_t phys[MRL_MAX_PHYS];
  if (!physical_shape(l, shape, rank, phys)) return false;
  int64_t stride[MRL_MAX_PHYS], running = 1;
  for (int i = int(l.ndims) - 1; i >= 0; i--) stride[i] = running, running *= phys[i];
  uint32_t remaining[MRL_MAX_RANK];
  for (uint32_t d = 0; d < rank; d++) remaining[d] = shape[d];
  for (uint32_t i = 0; i < l.ndims; i++) {
    const uint32_t ld = l.dims[i].logical_dim;
    remaining[ld] /= phys[i];
    if (phys[i] == 1) continue;
    if (l.dims[i].kind == MRL_ODDEVEN) {
      if (remaining[ld] != 1 || phys[i] != l.dims[i].size) return false;
      // index within the strip e = 2 * pair + parity lives at parity * (n / 2) + pair
      out[ld].push_back({phys[i] / 2, stride[i]});
      out[ld].push_back({2, stride[i] * (phys[i] / 2)});
    } else {
      out[ld].push_back({phys[i], stride[i]});
    }
  }
  for (uint32_t d = 0; d < rank; d++)
    if (remaining[d] != 1) return false;
  return true;
}

}  // namespace detail

// The common view of `src` and `dst` layouts over `shape`, digits with contiguous neighbours
// on both sides merged, size-one digits dropped.  False when there is none (or it has more
// than MOVE_MAX_RANK digits).
inline bool common_view(const mrl_layout &src, const mrl_layout &dst, const uint32_t *shape, uint32_t rank,
                        std::vector<MoveDim> *view) {
  std::vector<detail::Digit> a[MRL_MAX_RANK], b[MRL_MAX_RANK];
  if (!detail::digits_of(src, shape, rank, a) || !detail::digits_of(dst, shape, rank, b)) return false;
  std::vector<MoveDim> dims;
  for (uint32_t d = 0; d < rank; d++) {
    // Least significant digits first; the larger of the two current digits is split.
    int ia = int(a[d].size()) - 1, ib = int(b[d].size()) - 1;
    detail::Digit ra{1, 0}, rb{1, 0};
    if (ia >= 0) ra = a[d][ia];
    if (ib >= 0) rb = b[d][ib];
    while (ia >= 0 && ib >= 0) {
      const uint32_t take = std::min(ra.size, rb.size);
      if (ra.size % take != 0 || rb.size % take != 0) return false;
      dims.push_back({take, ra.stride, rb.stride});
      ra.size /= take, ra.stride *= take;
      rb.size /= take, rb.stride *= take;
      if (ra.size == 1 && --ia >= 0) ra = a[d][ia];
      if (rb.size == 1 && --ib >= 0) rb = b[d][ib];
    }
    if (ia >= 0 || ib >= 0) return false;  // the two products differ: not the same shape
  }
  // Slowest to fastest on the destination side, then merge digits that continue each other.
  std::stable_sort(dims.begin(), dims.end(), [](const MoveDim &x, const MoveDim &y) { return x.ds > y.ds; });
  view->clear();
  for (const MoveDim &m : dims) {
    if (m.size == 1) continue;
    if (!view->empty()) {
      MoveDim &last = view->back();
      if (last.ss == m.ss * int64_t(m.size) && last.ds == m.ds * int64_t(m.size)) {
        last.size *= m.size, last.ss = m.ss, last.ds = m.ds;
        continue;
      }
    }
    view->push_back(m);
  }
  return view->size() <= MOVE_MAX_RANK;
}

// Whether a common view says that both sides store the elements in the same order.
inline bool same_order(const std::vector<MoveDim> &view) {
  return view.empty() || (view.size() == 1 && view[0].ss == 1 && view[0].ds == 1);
}

}  // namespace mrl
