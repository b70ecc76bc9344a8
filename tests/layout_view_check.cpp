// Host check of morello_amd/csrc/layout_factor.h: for pairs of layouts, the common strided view
// must send every source offset to the destination offset that the layouts' index expressions
// (layout_math.h, after morello/src/layout.rs:221-272) give for the same logical point.
#include <cstdio>
#include <cstdlib>
#include <vector>

#include "../morello_amd/csrc/layout_factor.h"

using namespace mrl;

static mrl_layout make(std::initializer_list<mrl_physdim> dims) {
  mrl_layout l{};
  l.ndims = 0;
  for (const auto &d : dims) l.dims[l.ndims++] = d;
  return l;
}
static mrl_physdim dim(uint32_t d, int kind, uint32_t n) {
  mrl_physdim p{};
  p.logical_dim = decltype(p.logical_dim)(d), p.kind = decltype(p.kind)(kind), p.size = n;
  return p;
}
static mrl_physdim dyn(uint32_t d) { return dim(d, MRL_DYNAMIC, 0); }
static mrl_physdim packed(uint32_t d, uint32_t n) { return dim(d, MRL_PACKED, n); }
static mrl_physdim oddeven(uint32_t d, uint32_t n) { return dim(d, MRL_ODDEVEN, n); }

// 1: view exists and is right; 0: no view (allowed only if `may_fail`); exits on a wrong view.
static int check(const char *name, const mrl_layout &a, const mrl_layout &b, std::vector<uint32_t> shape,
                 bool expect_view) {
  const uint32_t rank = uint32_t(shape.size());
  LayoutEval ea, eb;
  if (!make_layout_eval(a, shape.data(), rank, &ea) || !make_layout_eval(b, shape.data(), rank, &eb)) {
    std::printf("%s: layout does not apply\n", name);
    std::exit(1);
  }
  uint64_t count = 1;
  for (uint32_t s : shape) count *= s;
  std::vector<int64_t> want(count, -1), got(count, -1);
  std::vector<uint32_t> pt(MRL_MAX_RANK, 0);
  for (uint64_t i = 0; i < count; i++) {
    uint64_t rem = i;
    for (int d = int(rank) - 1; d >= 0; d--) pt[d] = uint32_t(rem % shape[d]), rem /= shape[d];
    want[layout_offset(ea, pt.data())] = layout_offset(eb, pt.data());
  }
  std::vector<MoveDim> view;
  const bool has = common_view(a, b, shape.data(), rank, &view);
  if (has != expect_view) {
    std::printf("%s: view %s\n", name, has ? "unexpectedly exists" : "missing");
    std::exit(1);
  }
  if (!has) return 0;
  uint64_t vcount = 1;
  for (const MoveDim &m : view) vcount *= m.size;
  if (vcount != count) {
    std::printf("%s: view covers %llu of %llu elements\n", name, (unsigned long long)vcount, (unsigned long long)count);
    std::exit(1);
  }
  for (uint64_t i = 0; i < count; i++) {
    uint64_t rem = i;
    int64_t so = 0, d_o = 0;
    for (int d = int(view.size()) - 1; d >= 0; d--) {
      const uint64_t c = rem % view[d].size;
      rem /= view[d].size;
      so += int64_t(c) * view[d].ss, d_o += int64_t(c) * view[d].ds;
    }
    if (so < 0 || uint64_t(so) >= count || got[so] != -1) {
      std::printf("%s: source offset %lld out of range or repeated\n", name, (long long)so);
      std::exit(1);
    }
    got[so] = d_o;
  }
  for (uint64_t i = 0; i < count; i++)
    if (got[i] != want[i]) {
      std::printf("%s: source offset %llu goes to %lld, expected %lld\n", name, (unsigned long long)i,
                  (long long)got[i], (long long)want[i]);
      std::exit(1);
    }
  std::printf("%s: ok, rank %zu\n", name, view.size());
  return 1;
}

int main() {
  const mrl_layout rm2 = make({dyn(0), dyn(1)}), cm2 = make({dyn(1), dyn(0)});
  check("rm -> cm", rm2, cm2, {12, 20}, true);
  check("rm -> [0,1,1p4] (same order)", rm2, make({dyn(0), dyn(1), packed(1, 4)}), {6, 16}, true);
  check("rm -> [0,1,0p8]", rm2, make({dyn(0), dyn(1), packed(0, 8)}), {16, 10}, true);
  check("[0,1,0p8] -> rm", make({dyn(0), dyn(1), packed(0, 8)}), rm2, {16, 10}, true);
  check("[0,1,1p16] -> [0,1,1p8]", make({dyn(0), dyn(1), packed(1, 16)}), make({dyn(0), dyn(1), packed(1, 8)}), {3, 32}, true);
  check("[0,1,0p4] -> [1,0,1p8]", make({dyn(0), dyn(1), packed(0, 4)}), make({dyn(1), dyn(0), packed(1, 8)}), {8, 16}, true);
  check("rm -> [0,1,1o8]", rm2, make({dyn(0), dyn(1), oddeven(1, 8)}), {5, 24}, true);
  check("[0,1,1o8] -> [0,1,1p4]", make({dyn(0), dyn(1), oddeven(1, 8)}), make({dyn(0), dyn(1), packed(1, 4)}), {5, 24}, true);
  check("[0,1,1o8] -> cm", make({dyn(0), dyn(1), oddeven(1, 8)}), cm2, {4, 16}, true);
  check("[0,1,1p6] -> [0,1,1p4] (6 and 4 do not refine)", make({dyn(0), dyn(1), packed(1, 6)}),
        make({dyn(0), dyn(1), packed(1, 4)}), {2, 12}, false);
  check("[0,1,1o6] -> [0,1,1p3]", make({dyn(0), dyn(1), oddeven(1, 6)}), make({dyn(0), dyn(1), packed(1, 3)}), {2, 12}, false);
  check("layout.rs:1537 shape -> rm", make({dyn(1), dyn(0), packed(1, 4), packed(0, 2), packed(1, 4)}), rm2, {10, 8}, true);
  check("packed larger than the dim", make({dyn(0), dyn(1), packed(0, 4)}), rm2, {2, 64}, true);
  const mrl_layout nchw = make({dyn(0), dyn(1), dyn(2), dyn(3)}), nhwc = make({dyn(0), dyn(2), dyn(3), dyn(1)});
  check("nchw -> nhwc", nchw, nhwc, {2, 6, 5, 4}, true);
  check("nchw -> nchw c-packed", nchw, make({dyn(0), dyn(1), dyn(2), dyn(3), packed(1, 4)}), {2, 8, 3, 5}, true);
  check("nhwc -> [0,1,2,3,1p8,3o2]", nhwc, make({dyn(0), dyn(1), dyn(2), dyn(3), packed(1, 8), oddeven(3, 2)}), {2, 16, 3, 6}, true);
  // Seeded random pairs over a shape with many divisors.
  uint32_t state = 12345;
  auto rnd = [&](uint32_t n) { state = state * 1664525u + 1013904223u; return (state >> 8) % n; };
  int with_view = 0;
  for (int t = 0; t < 300; t++) {
    const std::vector<uint32_t> shape = {24, 16, 12};
    mrl_layout l[2];
    for (mrl_layout &x : l) {
      uint32_t perm[3] = {0, 1, 2};
      for (int i = 2; i > 0; i--) std::swap(perm[i], perm[rnd(i + 1)]);
      x = make({dyn(perm[0]), dyn(perm[1]), dyn(perm[2])});
      const uint32_t extra = rnd(3);
      const uint32_t sizes[] = {2, 3, 4, 6, 8};
      for (uint32_t e = 0; e < extra; e++) {
        const uint32_t d = rnd(3), n = sizes[rnd(5)];
        x.dims[x.ndims++] = rnd(4) == 0 && n % 2 == 0 ? oddeven(d, n) : packed(d, n);
      }
    }
    uint32_t phys[MRL_MAX_PHYS];
    if (!physical_shape(l[0], shape.data(), 3, phys) || !physical_shape(l[1], shape.data(), 3, phys)) continue;
    std::vector<MoveDim> probe;
    const bool has = common_view(l[0], l[1], shape.data(), 3, &probe);
    char name[64];
    std::snprintf(name, sizeof name, "random pair %d", t);
    with_view += check(name, l[0], l[1], shape, has);
  }
  std::printf("random pairs with a view: %d\n", with_view);
  if (with_view < 50) return 1;
  std::printf("layout view ok\n");
  return 0;
}
