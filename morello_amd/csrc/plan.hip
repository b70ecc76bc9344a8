// Recorder of planned launches and the cost model over them (host code only).
#include "plan.h"

#include <algorithm>
#include <cmath>
#include <cstring>

namespace mrl {
namespace plan {

thread_local Recorder *g_recorder = nullptr;
thread_local uint64_t g_launches = 0;

// "(k_attn<D, RAGGED, KT_ROWS>)" within "hipError_t mrl::(anonymous namespace)::launch_one(...)
// [D = 128, RAGGED = false, KT_ROWS = false]" -> "k_attn [D = 128, RAGGED = false, KT_ROWS = false]".
static std::string kernel_name(const char *kernel_text, const char *launcher) {
  std::string family(kernel_text);
  family.erase(0, family.find_first_not_of("( "));
  family = family.substr(0, family.find_first_of("<) "));
  std::string args(launcher);
  const size_t at = args.rfind(" [");
  if (at == std::string::npos || !std::strchr(kernel_text, '<')) return family;  // not a template kernel
  args = args.substr(at);
  for (const char *drop : {"mrl::", "gemm::", "(anonymous namespace)::", "plan::"}) {
    const size_t n = std::strlen(drop);
    for (size_t i = args.find(drop); i != std::string::npos; i = args.find(drop, i)) args.erase(i, n);
  }
  return family + args;
}

void note(const char *kernel_text, const char *launcher, dim3 grid, dim3 block, size_t lds_bytes) {
  Recorder *r = g_recorder;
  if (!r) return;
  Step step;
  step.kernel = kernel_name(kernel_text, launcher);
  step.grid[0] = grid.x, step.grid[1] = grid.y, step.grid[2] = grid.z;
  step.block[0] = block.x, step.block[1] = block.y, step.block[2] = block.z;
  step.lds_bytes = uint32_t(lds_bytes);
  step.unit = r->unit, step.ops = r->ops, step.bytes = r->bytes, step.tile_ops = r->tile_ops;
  step.serial_ns = r->serial_ns, step.rate_scale = r->rate_scale;
  r->steps.push_back(step);
  r->unit = UNIT_STREAM, r->ops = r->bytes = r->tile_ops = r->serial_ns = 0, r->rate_scale = 1;
}

// Nanoseconds of one planned launch on an MI355X, launches queued back to back on one stream.
// Constants are fits to launches measured through the timed-run entry point (benchmark
// configurations and the size sweeps the tests cover): the model is
//     launch gap + max(traffic / streaming rate, arithmetic / sustained rate),
// the arithmetic of a matrix-core kernel being its workgroups' padded tiles taken in rounds over
// the compute units.
double step_ns(const Step &s, uint32_t compute_units) {
  constexpr double LAUNCH_NS = 2200.0;        // gap between dependent launches on a stream
  constexpr double STREAM_BYTES_PER_NS = 5500.0;  // 5.5 TB/s: what copy / softmax / GEMV kernels sustain
  // Sustained whole-chip rates under the board's power limit, ops per ns.
  // `nominal`: the datasheet rate, the ceiling of what a compute unit does when few of them are
  // busy and the board's power is not the limit.
  double rate = 0, nominal = 0;
  switch (s.unit) {
    case UNIT_MFMA_I8: rate = 1440e3, nominal = 5033e3; break;
    case UNIT_MFMA_BF16: rate = 1150e3, nominal = 2516e3; break;
    case UNIT_MFMA_F32: rate = 125e3, nominal = 157e3; break;   // 4096^3: 143 TFLOPS, 2048^3 on 64 x 64 tiles: 115-120
    case UNIT_VALU: rate = 3e3; break;   // the generic kernels: dtype switches and index arithmetic per term
    default: break;
  }
  rate *= s.rate_scale;
  const double workgroups = double(s.grid[0]) * s.grid[1] * s.grid[2];
  double bytes = s.bytes;
  if (bytes == 0 && s.ops == 0) bytes = workgroups * s.block[0] * s.block[1] * s.block[2] * 16.0;  // undeclared: a guess
  double compute = 0;
  if (rate > 0) {
    if (s.tile_ops > 0) {
      // A compute unit takes its share of the workgroups one after another or several at a time
      // (they then share its matrix pipes): either way its time is its tiles' arithmetic, the
      // last, partly filled round counting as a whole one (f32 3072^3 as 2304 tiles of 64 x 64,
      // nine per unit: 466 us measured, 464 from this).
      const double per_unit = std::ceil(workgroups / compute_units);
      const double active = std::min(workgroups, double(compute_units));
      // Measured: with a quarter of the units busy each runs ~1.4x its share of the sustained rate.
      const double unit_rate =
          std::min(0.8 * nominal, rate * (1.0 + 0.5 * (1.0 - active / compute_units))) / compute_units;
      compute = per_unit * s.tile_ops / unit_rate;
    } else {
      compute = s.ops / rate;
    }
  }
  return LAUNCH_NS + std::max({bytes / STREAM_BYTES_PER_NS, compute, s.serial_ns});
}

}  // namespace plan
}  // namespace mrl
