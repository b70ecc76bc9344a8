// C++ view of the MI355X backend with Morello's own vocabulary.
//
// Morello's host side is Rust; this header is its C++ mirror over the C ABI in
// morello_amd.h, so that code written against the reference's Spec surface reads the same:
//
//   reference (Rust)                                   here (C++)
//   ------------------------------------------------   ---------------------------------
//   Dtype::{Uint8, .., Bfloat16}      common.rs:15-24   morello::Dtype
//   PhysDim::{Dynamic, Packed, OddEven} layout.rs:74-81 morello::PhysDim
//   Layout, row_major, col_major, nhwc layout.rs:67-70,  morello::Layout, row_major(), ...
//     batched_col_major, layout!       1234-1302
//   TensorSpec{shape,dtype,aux}     tensorspec.rs:19-32 morello::TensorSpec
//   PrimitiveSpecType::{Matmul,Conv,Softmax,Move}       morello::SpecType
//   LogicalSpec / Spec, lspec!/spec!   spec.rs:33-162   morello::Spec, Spec::matmul(...), ...
//   parameter_shape / parameters     spec.rs:467-583    Spec::parameter_shape / parameters
//   OperandDirection              spec.rs:1091-1095     morello::OperandDirection
//   BuiltArtifact::run / bench  codegen/mod.rs:269-341  Spec::run / Spec::run_host / Spec::bench
//   RunError / BuildError        codegen/mod.rs:66-91   morello::Error (carries the status code)
//
// Header-only; link with -lmorello_amd.
#pragma once
#include <initializer_list>
#include <stdexcept>
#include <string>
#include <utility>
#include <vector>

#include "morello_amd.h"

namespace morello {

class Error : public std::runtime_error {
 public:
  Error(int status, const std::string &where)
      : std::runtime_error(where + ": " + mrl_status_string(status) +
                           (status == MRL_ERR_HIP ? std::string(" (") + mrl_last_error() + ")" : "")),
        status_(status) {}
  int status() const { return status_; }

 private:
  int status_;
};

inline void check(int status, const char *where) {
  if (status != MRL_OK) throw Error(status, where);
}

enum class Dtype : int { Uint8 = 0, Sint8, Uint16, Sint16, Uint32, Sint32, Float32, Bfloat16 };
inline size_t size_of(Dtype d) { return mrl_dtype_size(int(d)); }
inline const char *to_string(Dtype d) { return mrl_dtype_name(int(d)); }

enum class OperandDirection : int { In = 0, Out = 1, InOut = 2 };

struct PhysDim {
  enum Kind : uint8_t { Dynamic = 0, Packed = 1, OddEven = 2 } kind = Dynamic;
  uint32_t size = 0;
  static PhysDim dynamic() { return {}; }
  static PhysDim packed(uint32_t n) { return {Packed, n}; }
  static PhysDim odd_even(uint32_t n) { return {OddEven, n}; }
};

using Shape = std::vector<uint32_t>;

class Layout {
 public:
  Layout() { c_.ndims = 0; }
  // `layout![...]`: physical dims slowest to fastest.
  Layout(std::initializer_list<std::pair<uint8_t, PhysDim>> dims) {
    if (dims.size() > MRL_MAX_PHYS) throw Error(MRL_ERR_BAD_LAYOUT, "Layout");
    c_.ndims = 0;
    for (const auto &d : dims) c_.dims[c_.ndims++] = mrl_physdim{d.first, uint8_t(d.second.kind), d.second.size};
  }
  explicit Layout(const mrl_layout &c) : c_(c) {}
  const mrl_layout &c() const { return c_; }
  size_t len() const { return c_.ndims; }

  // expand_physical_shape (layout.rs:769-810)
  Shape physical_shape(const Shape &shape) const {
    Shape out(c_.ndims);
    check(mrl_layout_physical_shape(&c_, shape.data(), uint32_t(shape.size()), out.data()), "physical_shape");
    return out;
  }
  bool applies_to_shape(const Shape &shape) const {
    Shape out(MRL_MAX_PHYS);
    return mrl_layout_physical_shape(&c_, shape.data(), uint32_t(shape.size()), out.data()) == MRL_OK;
  }
  // buffer_indexing_expr (layout.rs:221-272) at a concrete point.
  int64_t buffer_index(const Shape &shape, const Shape &point) const {
    const int64_t i = mrl_layout_buffer_index(&c_, shape.data(), uint32_t(shape.size()), point.data());
    if (i < 0) throw Error(MRL_ERR_BAD_LAYOUT, "buffer_index");
    return i;
  }

 private:
  mrl_layout c_;
};

inline Layout row_major(const Shape &s) {
  mrl_layout l;
  check(mrl_layout_row_major(s.data(), uint32_t(s.size()), &l), "row_major");
  return Layout(l);
}
inline Layout col_major(const Shape &s) {
  mrl_layout l;
  check(mrl_layout_col_major(s.data(), uint32_t(s.size()), &l), "col_major");
  return Layout(l);
}
inline Layout batched_col_major(const Shape &s) {
  mrl_layout l;
  check(mrl_layout_batched_col_major(s.data(), uint32_t(s.size()), &l), "batched_col_major");
  return Layout(l);
}
inline Layout nhwc(const Shape &s) {
  mrl_layout l;
  check(mrl_layout_nhwc(s.data(), uint32_t(s.size()), &l), "nhwc");
  return Layout(l);
}

// One parameter's type: tensorspec.rs:19-32 without the memory level (every parameter of a
// top-level Spec lives in GL, which is HBM here).
struct TensorSpec {
  Shape shape;
  Dtype dtype;
  Layout layout;
  size_t volume() const {
    size_t v = 1;
    for (uint32_t d : shape) v *= d;
    return v;
  }
  size_t bytes_used() const { return volume() * size_of(dtype); }
};

enum class SpecType : int {
  Matmul = 0, Conv = 1, Softmax = 2, ComposeMatmulSoftmaxMatmul = 3, Move = 4,
  // The primitives Softmax decomposes into (spec.rs:57-162).
  Fill = 5, Max = 6, SoftmaxDenominator = 7, SoftmaxDenominatorAndMax = 8,
  SoftmaxDenominatorAndMaxFromParts = 9, SoftmaxDenominatorAndUnscaled = 10,
  SoftmaxDenominatorAndUnscaledFromMax = 11, SoftmaxComplete = 12, DivideVec = 13,
  DivideVecScalar = 14, Broadcast = 15, OnePrefix = 16
};
// spec.rs:165-170
enum class FillValue : uint32_t { Zero = 0, NegInf = 1, Min = 2 };

// What a run of a Spec would launch and what the cost model expects of it: the backend's answer
// to Kernel::applies_to_logical_spec / main_cost / memory_allocated (target/mod.rs:103-109).
struct Plan {
  std::vector<mrl_plan_step> steps;
  double cost_ns = 0;
  uint64_t scratch_bytes = 0;
};

class Spec {
 public:
  // Matmul{accum} over [b, m, k, n] (spec.rs:480-485).  Layouts default to row-major.
  static Spec matmul(const Shape &bmkn, Dtype a, Dtype b, Dtype c, bool accum = false) {
    return make(SpecType::Matmul, bmkn, {a, b, c}, accum, 0, false);
  }
  // Conv{accum} over [b, f, c, oh, ow, fh, fw] (spec.rs:486-498).  Layouts default to NHWC /
  // KRSC (layout![0,2,3,1]).
  static Spec conv(const Shape &s, Dtype image, Dtype filters, Dtype out, bool accum = false) {
    return make(SpecType::Conv, s, {image, filters, out}, accum, 0, true);
  }
  static Spec softmax(const Shape &shape, uint32_t scan_dim) {
    return make(SpecType::Softmax, shape, {Dtype::Float32, Dtype::Float32}, false, scan_dim, false);
  }
  static Spec move(const Shape &shape, Dtype from, Dtype to) {
    return make(SpecType::Move, shape, {from, to}, false, 0, false);
  }
  // Compose [Matmul, Softmax{2}, Matmul] over [b, m, k, n2, n]; parameters V, Q, KT, out
  // (spec.rs:3329-3365).
  static Spec compose_msm(const Shape &bmkn2n, Dtype v, Dtype q, Dtype kt) {
    return make(SpecType::ComposeMatmulSoftmaxMatmul, bmkn2n, {v, q, kt, Dtype::Float32}, false, 0, false);
  }

  // The remaining primitives, f32 (spec.rs:57-162; parameter lists spec.rs:499-583).
  // `n_params` f32 parameters of kind `t` over `shape`, reducing over `dim`.
  static Spec softmax_part(SpecType t, const Shape &shape, uint32_t dim, bool accum = false) {
    static const uint8_t count[] = {1, 2, 3, 3, 4, 3, 4, 4, 2, 2, 2, 2};
    const int k = int(t);
    if (k < int(SpecType::Max) || k > int(SpecType::DivideVecScalar)) throw Error(MRL_ERR_BAD_SPEC, "softmax_part");
    const Dtype f = Dtype::Float32;
    switch (count[k - int(SpecType::Fill)]) {
      case 2: return make(t, shape, {f, f}, accum, dim, false);
      case 3: return make(t, shape, {f, f, f}, accum, dim, false);
      default: return make(t, shape, {f, f, f, f}, accum, dim, false);
    }
  }
  static Spec fill(const Shape &shape, Dtype dt, FillValue v) {
    return make(SpecType::Fill, shape, {dt}, false, uint32_t(v), false);
  }
  static Spec broadcast(const Shape &shape, uint32_t dim, Dtype dt) {
    return make(SpecType::Broadcast, shape, {dt, dt}, false, dim, false);
  }
  static Spec one_prefix(const Shape &shape, Dtype dt) {
    return make(SpecType::OnePrefix, shape, {dt, dt}, false, 0, false);
  }

  Spec &with_layout(uint32_t param, const Layout &l) {
    if (param >= c_.n_params) throw Error(MRL_ERR_BAD_SPEC, "with_layout");
    c_.layouts[param] = l.c();
    return *this;
  }

  size_t parameter_count() const { return c_.n_params; }
  Shape parameter_shape(uint32_t idx) const {
    uint32_t shape[MRL_MAX_RANK], rank = 0;
    check(mrl_spec_parameter_shape(&c_, idx, shape, &rank), "parameter_shape");
    return Shape(shape, shape + rank);
  }
  std::vector<TensorSpec> parameters() const {
    std::vector<TensorSpec> out;
    for (uint32_t i = 0; i < c_.n_params; i++)
      out.push_back(TensorSpec{parameter_shape(i), Dtype(c_.dtypes[i]), Layout(c_.layouts[i])});
    return out;
  }
  OperandDirection parameter_direction(uint32_t idx) const {
    const int d = mrl_spec_parameter_direction(&c_, idx);
    if (d < 0) throw Error(MRL_ERR_BAD_SPEC, "parameter_direction");
    return OperandDirection(d);
  }
  uint64_t flops() const { return mrl_spec_ops(&c_); }
  bool is_supported() const { return mrl_spec_check(&c_) == MRL_OK; }
  // The manual Matmul schedule the cost model predicts cheapest, as {tile_m, tile_n, split_k}
  // (scheduling_sugar.rs:37-132: what `tile_out([1, m, n])` and `split(k)` would be called with).
  mrl_matmul_schedule search_schedule() const {
    mrl_matmul_schedule best{};
    check(mrl_matmul_search_schedule(&c_, &best, nullptr), "search_schedule");
    return best;
  }
  // Target::actions (target/mod.rs:69): the lowerings the backend can run for this Spec, priced.
  std::vector<mrl_action> actions() const {
    std::vector<mrl_action> out(mrl_target_actions(&c_, nullptr, 0));
    if (!out.empty()) out.resize(mrl_target_actions(&c_, out.data(), uint32_t(out.size())));
    return out;
  }
  // ActionT::apply (scheduling/mod.rs:40-63): the sub-Specs a rewrite turns this Spec into, with
  // their parameter sources and the buffers between them; n_subspecs == 0 for a leaf.
  mrl_rewrite apply(const mrl_action &action) const {
    mrl_rewrite out{};
    check(mrl_action_apply(&c_, &action, &out), "action_apply");
    return out;
  }
  // Runs the Spec under one of its actions: `params` are device pointers in parameter order.
  void run(const mrl_action &action, void *const *params, void *stream = nullptr) const {
    check(mrl_run_action(&c_, params, &action, stream), "run_action");
  }
  // Host-only: needs no GPU.
  Plan plan() const {
    mrl_plan head{};
    Plan out;
    out.steps.resize(64);
    check(mrl_spec_plan(&c_, &head, out.steps.data(), 64), "plan");
    out.steps.resize(head.n_steps < 64 ? head.n_steps : 64);
    out.cost_ns = head.cost_ns, out.scratch_bytes = head.scratch_bytes;
    return out;
  }
  const mrl_spec &c() const { return c_; }

  // Where `kernel(p0, .., pk)` is called: device pointers in parameter order.
  void run(const std::vector<void *> &device_params) const {
    if (device_params.size() != c_.n_params) throw Error(MRL_ERR_BAD_SPEC, "run");
    check(mrl_run(&c_, device_params.data()), "run");
  }
  void run_async(const std::vector<void *> &device_params, void *stream) const {
    if (device_params.size() != c_.n_params) throw Error(MRL_ERR_BAD_SPEC, "run_async");
    check(mrl_run_async(&c_, device_params.data(), stream), "run_async");
  }
  // BuiltArtifact::run_with_input_data without the files: host buffers laid out by each
  // parameter's layout; written parameters are copied back.
  void run_host(const std::vector<void *> &host_params) const {
    if (host_params.size() != c_.n_params) throw Error(MRL_ERR_BAD_SPEC, "run_host");
    check(mrl_run_host(&c_, host_params.data()), "run_host");
  }
  // CodeGen::bench: best inner-loop runtime in nanoseconds over `repeats` trials.
  double bench(const std::vector<void *> &device_params, uint32_t iters, uint32_t repeats = 10) const {
    double best = 0, mean = 0;
    check(mrl_bench(&c_, device_params.data(), iters, repeats, &best, &mean), "bench");
    return best;
  }

 private:
  static Spec make(SpecType t, const Shape &shape, std::initializer_list<Dtype> dts, bool accum,
                   uint32_t scan_dim, bool channels_last) {
    Spec s;
    s.c_ = mrl_spec{};
    if (shape.size() > MRL_MAX_SPEC_RANK || dts.size() > MRL_MAX_PARAMS) throw Error(MRL_ERR_BAD_SPEC, "Spec");
    s.c_.kind = int(t), s.c_.accum = accum, s.c_.scan_dim = scan_dim, s.c_.rank = uint32_t(shape.size());
    for (size_t i = 0; i < shape.size(); i++) s.c_.spec_shape[i] = shape[i];
    s.c_.n_params = uint32_t(dts.size());
    uint32_t i = 0;
    for (Dtype d : dts) s.c_.dtypes[i++] = int(d);
    for (i = 0; i < s.c_.n_params; i++) {
      const Shape ps = s.parameter_shape(i);
      s.c_.layouts[i] = (channels_last ? nhwc(ps) : row_major(ps)).c();
    }
    return s;
  }
  mrl_spec c_;
};

// LogicalSpec::Compose (spec.rs:39-45, 1519-1590): components listed last-executed first; the
// external parameters follow compose_parameter_visit (spec.rs:3329-3365).
class Compose {
 public:
  explicit Compose(const std::vector<Spec> &components) {
    c_ = mrl_compose{};
    if (components.size() > MRL_MAX_COMPONENTS) throw Error(MRL_ERR_BAD_SPEC, "Compose");
    c_.n_components = uint32_t(components.size());
    for (size_t i = 0; i < components.size(); i++) {
      const mrl_spec &s = components[i].c();
      mrl_component &d = c_.components[i];
      d.kind = s.kind, d.accum = s.accum, d.scan_dim = s.scan_dim, d.rank = s.rank, d.n_params = s.n_params;
      for (uint32_t k = 0; k < s.rank; k++) d.spec_shape[k] = s.spec_shape[k];
      for (uint32_t k = 0; k < s.n_params; k++) d.dtypes[k] = s.dtypes[k];
    }
    check(mrl_compose_init(&c_), "Compose");
  }
  Compose &with_layout(uint32_t param, const Layout &l) {
    if (param >= c_.n_params) throw Error(MRL_ERR_BAD_SPEC, "with_layout");
    c_.layouts[param] = l.c();
    return *this;
  }
  // scheduling/bufferize.rs:24-116 with memory GL and a row-major layout.
  Compose &bufferize(uint32_t index) {
    if (index + 1 >= c_.n_components) throw Error(MRL_ERR_BAD_SPEC, "bufferize");
    c_.bufferize_mask |= 1u << index;
    return *this;
  }
  size_t parameter_count() const { return c_.n_params; }
  std::vector<TensorSpec> parameters() const {
    std::vector<TensorSpec> out;
    for (uint32_t i = 0; i < c_.n_params; i++) {
      uint32_t shape[MRL_MAX_RANK], rank = 0;
      check(mrl_compose_parameter_shape(&c_, i, shape, &rank), "parameters");
      out.push_back(TensorSpec{Shape(shape, shape + rank), Dtype(mrl_compose_parameter_dtype(&c_, i)),
                               Layout(c_.layouts[i])});
    }
    return out;
  }
  void run(const std::vector<void *> &device_params, void *stream = nullptr) const {
    if (device_params.size() != c_.n_params) throw Error(MRL_ERR_BAD_SPEC, "run");
    check(mrl_run_compose(&c_, device_params.data(), stream), "run");
  }
  const mrl_compose &c() const { return c_; }

 private:
  mrl_compose c_;
};

inline void init(int device = 0) { check(mrl_init(device), "init"); }

}  // namespace morello
