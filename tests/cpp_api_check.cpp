// Host-only exercise of include/morello_amd.hpp (no device needed): the same expectations
// the Python tests assert, through the C++ view.  Built and run by tests/test_cpp_api.py.
#include <cstdio>
#include <string>

#include "morello_amd.hpp"

#define EXPECT(c)                                            \
  do {                                                       \
    if (!(c)) {                                              \
      std::printf("FAILED: %s (line %d)\n", #c, __LINE__);   \
      return 1;                                              \
    }                                                        \
  } while (0)

int main() {
  using namespace morello;
  EXPECT(size_of(Dtype::Bfloat16) == 2 && std::string(to_string(Dtype::Sint8)) == "i8");
  // layout.rs:2391-2433 and book/src/data_layouts.md:59-99
  EXPECT(row_major({16, 4}).buffer_index({16, 4}, {3, 2}) == 14);
  Layout oe{{0, PhysDim::odd_even(8)}};
  EXPECT(oe.buffer_index({8}, {3}) == 5);
  Layout packed{{1, PhysDim::dynamic()}, {0, PhysDim::dynamic()}, {1, PhysDim::packed(4)}};
  EXPECT(packed.buffer_index({6, 8}, {2, 5}) == 24 * (5 / 4) + 4 * 2 + 5 % 4);
  EXPECT((packed.physical_shape({6, 8}) == Shape{2, 6, 4}));
  Layout bad{{0, PhysDim::packed(4)}, {1, PhysDim::dynamic()}};
  EXPECT(bad.applies_to_shape({1, 64}) && !bad.applies_to_shape({8, 64}));  // layout.rs:1470-1527
  EXPECT(batched_col_major({2, 2, 2, 2}).len() == 4);
  // spec.rs:480-498, 3329-3365
  Spec mm = Spec::matmul({32, 2, 3, 3}, Dtype::Uint8, Dtype::Sint8, Dtype::Uint16, true);
  EXPECT((mm.parameter_shape(1) == Shape{32, 3, 3}));
  EXPECT(mm.parameter_direction(2) == OperandDirection::InOut);
  Spec cv = Spec::conv({1, 2, 3, 4, 5, 2, 2}, Dtype::Uint8, Dtype::Sint8, Dtype::Sint32);
  EXPECT((cv.parameter_shape(0) == Shape{1, 3, 5, 6}) && (cv.parameter_shape(2) == Shape{1, 2, 4, 5}));
  EXPECT(cv.parameters()[1].bytes_used() == 2 * 3 * 2 * 2);
  Spec msm = Spec::compose_msm({16, 2048, 128, 2048, 128}, Dtype::Bfloat16, Dtype::Bfloat16, Dtype::Bfloat16)
                 .with_layout(2, Layout{{0, PhysDim::dynamic()}, {2, PhysDim::dynamic()}, {1, PhysDim::dynamic()}});
  EXPECT(msm.is_supported() && msm.flops() == 34359738368ull + 335544320ull);
  EXPECT((msm.parameter_shape(2) == Shape{16, 128, 2048}));
  EXPECT(Spec::matmul({1, 4096, 4096, 4096}, Dtype::Uint8, Dtype::Sint8, Dtype::Sint32).flops() == 137438953472ull);
  EXPECT(Spec::matmul({1, 4, 4, 4}, Dtype::Float32, Dtype::Float32, Dtype::Bfloat16).is_supported());  // bf16 output: a legal triple
  // The primitives of the Softmax decomposition and a general Compose (spec.rs:3733-3785).
  Spec sdm = Spec::softmax_part(SpecType::SoftmaxDenominatorAndMax, {4, 6, 8}, 1, true);
  EXPECT(sdm.parameter_count() == 3 && (sdm.parameter_shape(2) == Shape{4, 1, 8}));
  EXPECT(sdm.parameter_direction(1) == OperandDirection::InOut);
  EXPECT(Spec::fill({3, 3}, Dtype::Sint32, FillValue::Min).parameter_direction(0) == OperandDirection::Out);
  EXPECT((Spec::one_prefix({6, 8}, Dtype::Float32).parameter_shape(1) == Shape{1, 6, 8}));
  Compose chain({Spec::matmul({16, 128, 128, 128}, Dtype::Uint8, Dtype::Uint16, Dtype::Uint32),
                 Spec::matmul({16, 128, 128, 128}, Dtype::Uint32, Dtype::Uint16, Dtype::Uint8),
                 Spec::matmul({16, 128, 128, 128}, Dtype::Uint8, Dtype::Uint8, Dtype::Uint32)});
  EXPECT(chain.parameter_count() == 5);
  EXPECT(chain.parameters()[0].dtype == Dtype::Uint16 && chain.parameters()[2].dtype == Dtype::Uint8 &&
         chain.parameters()[4].dtype == Dtype::Uint32);
  try {
    Compose bad_chain({Spec::matmul({1, 4, 8, 4}, Dtype::Float32, Dtype::Float32, Dtype::Float32),
                       Spec::matmul({1, 4, 4, 4}, Dtype::Float32, Dtype::Float32, Dtype::Float32)});
    EXPECT(false);
  } catch (const Error &e) {
    EXPECT(e.status() == MRL_ERR_BAD_SPEC);
  }
  // error behaviour: exceptions carry the status code
  try {
    Spec::softmax({4, 4}, 1).parameter_shape(5);
    EXPECT(false);
  } catch (const Error &e) {
    EXPECT(e.status() == MRL_ERR_BAD_SPEC);
  }
  // The plan of a Spec (host only): benchmark configuration 2 is one launch of the int8 256-tile.
  {
    const Plan p = Spec::matmul({1, 4096, 4096, 4096}, Dtype::Uint8, Dtype::Sint8, Dtype::Sint32).plan();
    EXPECT(p.steps.size() == 1 && p.scratch_bytes == 0 && p.cost_ns > 20e3 && p.cost_ns < 500e3);
    EXPECT(std::string(p.steps[0].kernel).find("k_gemm_wide [T = I8, A_UNSIGNED = true") == 0);
    EXPECT(std::string(mrl_target_id()) == "Gfx950" && mrl_target_memories(nullptr, 0) == 4);
    const std::vector<mrl_action> acts = Spec::matmul({1, 4096, 4096, 4096}, Dtype::Uint8, Dtype::Sint8, Dtype::Sint32).actions();
    EXPECT(acts.size() == 15 && acts[12].kind == MRL_ACTION_TO_ACCUM && acts[14].kind == MRL_ACTION_CAST && acts[11].staging == MRL_STAGING_DIRECT_B_WIDE && acts[0].kind == MRL_ACTION_SELECT && acts[1].kind == MRL_ACTION_TILE_OUT_SPLIT &&
           acts[1].tile_m == 256 && acts[0].cost_ns > 20e3);
    const mrl_matmul_schedule best =
        Spec::matmul({1, 4096, 4096, 4096}, Dtype::Uint8, Dtype::Sint8, Dtype::Sint32).search_schedule();
    EXPECT(best.tile_m == 256 && best.tile_n == 256);
    // A leaf has no children; the Softmax rewrite to_softmax_parts has two, with one buffer between them.
    const Spec mm = Spec::matmul({1, 4096, 4096, 4096}, Dtype::Uint8, Dtype::Sint8, Dtype::Sint32);
    EXPECT(mm.apply(acts[1]).n_subspecs == 0);
    const uint32_t rows[3] = {16, 2048, 2048};
    mrl_spec sm{};
    sm.kind = MRL_SPEC_SOFTMAX, sm.scan_dim = 2, sm.rank = 3, sm.n_params = 2;
    for (int d = 0; d < 3; d++) sm.spec_shape[d] = rows[d];
    for (int i = 0; i < 2; i++) sm.dtypes[i] = MRL_F32, mrl_layout_row_major(rows, 3, &sm.layouts[i]);
    mrl_action parts{};
    parts.kind = MRL_ACTION_TO_SOFTMAX_PARTS;
    mrl_rewrite rw{};
    EXPECT(mrl_action_apply(&sm, &parts, &rw) == MRL_OK && rw.n_subspecs == 2 && rw.n_intermediates == 1);
    EXPECT(rw.subspecs[0].spec.kind == MRL_SPEC_SOFTMAX_DENOMINATOR_AND_UNSCALED && rw.subspecs[0].source[1] == -1 &&
           rw.subspecs[1].spec.kind == MRL_SPEC_DIVIDE_VEC_SCALAR && rw.intermediate_bytes[0] == 16 * 2048 * 4);
  }
  std::printf("cpp api ok\n");
  return 0;
}
