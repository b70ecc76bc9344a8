// mrl_harness: the process-level stand-in for a program Morello emits, builds and runs.
//
// Morello's generated `main` (morello/src/codegen/cpu.rs:284-409) takes one file per Spec
// parameter, output included, each holding raw little-endian values in logical row-major
// order (morello/src/verification.rs:957-1001, loader cpu.rs:221-270), calls the kernel,
// and prints the output parameter (every written parameter, for Specs with several): a
// line with its shape `AxBxC`, then every element in logical row-major order, space separated, one newline at the end of every loop level but
// the outermost (cpu.rs:570-618), integers in decimal and floats as %.10f
// (codegen/c_utils.rs:334-344).  With no files the buffers are zero-filled (cpu.rs:320).
// Exit status 1 = wrong argument count, 2 = an input could not be loaded (cpu.rs:344-364).
// The benchmarking build prints `cpu: <s>s <ns>ns` for `iters` calls after one warm-up
// call (cpu.rs:516-568).
//
// An emitted program has its Spec baked in; this one takes it as the first argument:
//
//   mrl_harness <spec> [file_0 ... file_k]          check mode
//   mrl_harness <spec> --bench <iters>              benchmark mode
//
//   <spec> = kind:shape:dtypes[:flag]...
//     kind   matmul | conv | softmax | msm | move | fill | max | softmaxdenominator |
//            softmaxdenominatorandmax | softmaxdenominatorandmaxfromparts |
//            softmaxdenominatorandunscaled | softmaxdenominatorandunscaledfrommax |
//            softmaxcomplete | dividevec | dividevecscalar | broadcast | oneprefix
//            (these take the tensor shape; scan=d names the dim, for fill the value 0/1/2)
//     shape  the Spec shape, `x` separated (matmul b x m x k x n; conv b x f x c x oh x ow x fh x fw;
//            softmax/move the tensor shape; msm b x m x k x n2 x n)
//     dtypes one per parameter, comma separated: u8 i8 u16 i16 u32 i32 f32 bf16
//     flags  accum | scan=<dim> | layouts=<l0,l1,..> with each l one of rm cm bcm nhwc
//            (row-major, col-major, batched col-major, NHWC; default rm, conv default nhwc)
//            or a layout! spelled with dots: 0.2.1.2p16 = layout![0, 2, 1, 2 p(16)], 1o8 = OddEven
//
// Unlike the reference's loader, which refuses non-row-major top-level tensors
// (cpu.rs:226-231), files are always logical row-major and parameters with another layout
// are brought to it on the device with the Move Spec.
#include <cinttypes>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <string>
#include <vector>

#include "../../include/morello_amd.h"

namespace {

int parse_dtype(const std::string &s) {
  static const char *names[] = {"u8", "i8", "u16", "i16", "u32", "i32", "f32", "bf16"};
  for (int i = 0; i < 8; i++)
    if (s == names[i]) return i;
  return -1;
}

std::vector<std::string> split(const std::string &s, char sep) {
  std::vector<std::string> out;
  size_t start = 0;
  while (true) {
    size_t pos = s.find(sep, start);
    out.push_back(s.substr(start, pos == std::string::npos ? pos : pos - start));
    if (pos == std::string::npos) break;
    start = pos + 1;
  }
  return out;
}

// The `layout!` macro as text: physical dims slowest to fastest separated by dots, each a
// logical dim index, optionally followed by p<n> (Packed) or o<n> (OddEven): "0.2.1.2p16" is
// layout![0, 2, 1, 2 p(16)] (examples/matmul_x86.rs:34-53).
bool parse_layout(const std::string &text, mrl_layout *out) {
  const auto dims = split(text, '.');
  if (dims.empty() || dims.size() > MRL_MAX_PHYS) return false;
  out->ndims = 0;
  for (const std::string &d : dims) {
    char *end = nullptr;
    const unsigned long dim = std::strtoul(d.c_str(), &end, 10);
    if (end == d.c_str() || dim >= MRL_MAX_RANK) return false;
    mrl_physdim pd = {uint8_t(dim), MRL_DYNAMIC, 0};
    if (*end == 'p' || *end == 'o') {
      pd.kind = *end == 'p' ? MRL_PACKED : MRL_ODDEVEN;
      char *end2 = nullptr;
      const unsigned long n = std::strtoul(end + 1, &end2, 10);
      if (end2 == end + 1 || *end2 || n == 0 || n > 0xffffffffull) return false;
      pd.size = uint32_t(n);
    } else if (*end) {
      return false;
    }
    out->dims[out->ndims++] = pd;
  }
  return true;
}

bool parse_spec(const std::string &text, mrl_spec *spec, std::string *err) {
  std::memset(spec, 0, sizeof *spec);
  const auto parts = split(text, ':');
  if (parts.size() < 3) return *err = "spec needs kind:shape:dtypes", false;
  const std::string &kind = parts[0];
  if (kind == "matmul") spec->kind = MRL_SPEC_MATMUL, spec->n_params = 3;
  else if (kind == "conv") spec->kind = MRL_SPEC_CONV, spec->n_params = 3;
  else if (kind == "softmax") spec->kind = MRL_SPEC_SOFTMAX, spec->n_params = 2;
  else if (kind == "msm") spec->kind = MRL_SPEC_COMPOSE_MSM, spec->n_params = 4;
  else if (kind == "move") spec->kind = MRL_SPEC_MOVE, spec->n_params = 2;
  else {
    // The primitives Softmax decomposes into, by their reference names in lower case.
    static const struct { const char *name; int kind; uint32_t n; } parts[] = {
        {"fill", MRL_SPEC_FILL, 1}, {"max", MRL_SPEC_MAX, 2},
        {"softmaxdenominator", MRL_SPEC_SOFTMAX_DENOMINATOR, 3},
        {"softmaxdenominatorandmax", MRL_SPEC_SOFTMAX_DENOMINATOR_AND_MAX, 3},
        {"softmaxdenominatorandmaxfromparts", MRL_SPEC_SOFTMAX_DENOMINATOR_AND_MAX_FROM_PARTS, 4},
        {"softmaxdenominatorandunscaled", MRL_SPEC_SOFTMAX_DENOMINATOR_AND_UNSCALED, 3},
        {"softmaxdenominatorandunscaledfrommax", MRL_SPEC_SOFTMAX_DENOMINATOR_AND_UNSCALED_FROM_MAX, 4},
        {"softmaxcomplete", MRL_SPEC_SOFTMAX_COMPLETE, 4}, {"dividevec", MRL_SPEC_DIVIDE_VEC, 2},
        {"dividevecscalar", MRL_SPEC_DIVIDE_VEC_SCALAR, 2}, {"broadcast", MRL_SPEC_BROADCAST, 2},
        {"oneprefix", MRL_SPEC_ONE_PREFIX, 2}};
    bool found = false;
    for (const auto &p : parts)
      if (kind == p.name) spec->kind = p.kind, spec->n_params = p.n, found = true;
    if (!found) return *err = "unknown kind " + kind, false;
  }
  const auto dims = split(parts[1], 'x');
  if (dims.empty() || dims.size() > MRL_MAX_SPEC_RANK) return *err = "bad shape", false;
  spec->rank = uint32_t(dims.size());
  for (size_t i = 0; i < dims.size(); i++) {
    char *end = nullptr;
    const unsigned long v = std::strtoul(dims[i].c_str(), &end, 10);
    if (!end || *end || v == 0 || v > 0xffffffffull) return *err = "bad dim " + dims[i], false;
    spec->spec_shape[i] = uint32_t(v);
  }
  const auto dts = split(parts[2], ',');
  if (dts.size() != spec->n_params) return *err = "need one dtype per parameter", false;
  for (size_t i = 0; i < dts.size(); i++)
    if ((spec->dtypes[i] = parse_dtype(dts[i])) < 0) return *err = "bad dtype " + dts[i], false;
  std::vector<std::string> layouts(spec->n_params, spec->kind == MRL_SPEC_CONV ? "nhwc" : "rm");
  for (size_t i = 3; i < parts.size(); i++) {
    if (parts[i] == "accum") spec->accum = 1;
    else if (parts[i].rfind("scan=", 0) == 0) spec->scan_dim = uint32_t(std::atoi(parts[i].c_str() + 5));
    else if (parts[i].rfind("layouts=", 0) == 0) {
      const auto ls = split(parts[i].substr(8), ',');
      if (ls.size() != spec->n_params) return *err = "need one layout per parameter", false;
      layouts = ls;
    } else return *err = "unknown flag " + parts[i], false;
  }
  for (uint32_t i = 0; i < spec->n_params; i++) {
    uint32_t shape[MRL_MAX_RANK], rank;
    if (mrl_spec_parameter_shape(spec, i, shape, &rank) != MRL_OK) return *err = "bad spec shape", false;
    int rc;
    if (layouts[i] == "rm") rc = mrl_layout_row_major(shape, rank, &spec->layouts[i]);
    else if (layouts[i] == "cm") rc = mrl_layout_col_major(shape, rank, &spec->layouts[i]);
    else if (layouts[i] == "bcm") rc = mrl_layout_batched_col_major(shape, rank, &spec->layouts[i]);
    else if (layouts[i] == "nhwc") rc = mrl_layout_nhwc(shape, rank, &spec->layouts[i]);
    else if (parse_layout(layouts[i], &spec->layouts[i])) rc = MRL_OK;
    else return *err = "unknown layout " + layouts[i], false;
    if (rc == MRL_OK) {
      uint32_t phys[MRL_MAX_PHYS];
      rc = mrl_layout_physical_shape(&spec->layouts[i], shape, rank, phys);
    }
    if (rc != MRL_OK) return *err = "layout " + layouts[i] + " does not fit parameter", false;
  }
  return true;
}

uint64_t volume(const uint32_t *s, uint32_t r) {
  uint64_t v = 1;
  for (uint32_t i = 0; i < r; i++) v *= s[i];
  return v;
}

bool read_file(const char *path, void *dst, size_t bytes) {
  FILE *f = std::fopen(path, "rb");
  if (!f) return false;
  const size_t got = std::fread(dst, 1, bytes, f);
  // A longer file is as wrong as a shorter one: the emitted loader maps exactly `bytes`.
  const bool exact = got == bytes && std::fgetc(f) == EOF;
  std::fclose(f);
  return exact;
}

float bf16_to_f32(uint16_t v) {
  uint32_t bits = uint32_t(v) << 16;
  float f;
  std::memcpy(&f, &bits, 4);
  return f;
}

void print_element(int dtype, const void *buf, size_t i) {
  switch (dtype) {
    case MRL_U8: std::printf("%" PRIu8 " ", ((const uint8_t *)buf)[i]); break;
    case MRL_I8: std::printf("%" PRIi8 " ", ((const int8_t *)buf)[i]); break;
    case MRL_U16: std::printf("%" PRIu16 " ", ((const uint16_t *)buf)[i]); break;
    case MRL_I16: std::printf("%" PRIi16 " ", ((const int16_t *)buf)[i]); break;
    case MRL_U32: std::printf("%" PRIu32 " ", ((const uint32_t *)buf)[i]); break;
    case MRL_I32: std::printf("%" PRIi32 " ", ((const int32_t *)buf)[i]); break;
    case MRL_F32: std::printf("%.10f ", ((const float *)buf)[i]); break;
    default: std::printf("%.10f ", bf16_to_f32(((const uint16_t *)buf)[i])); break;
  }
}

// cpu.rs:570-618: nested loops, a newline after every loop level except the outermost.
void print_tensor(int dtype, const void *buf, const uint32_t *shape, uint32_t rank) {
  for (uint32_t d = 0; d < rank; d++) std::printf(d ? "x%u" : "%u", shape[d]);
  std::printf("\n");
  const uint64_t n = volume(shape, rank);
  for (uint64_t i = 0; i < n; i++) {
    print_element(dtype, buf, i);
    uint64_t idx = i + 1;
    for (int d = int(rank) - 1; d >= 1; d--) {
      if (idx % shape[d] != 0) break;
      std::printf("\n");
      idx /= shape[d];
    }
  }
}

#define DIE(code, ...)                 \
  do {                                 \
    std::fprintf(stderr, __VA_ARGS__); \
    std::fprintf(stderr, "\n");        \
    return code;                       \
  } while (0)

// Brings a logical row-major device buffer to `layout` (or back) with the Move Spec.
int relayout(const mrl_spec &spec, uint32_t idx, void *src, void *dst, bool to_layout) {
  mrl_spec mv;
  std::memset(&mv, 0, sizeof mv);
  uint32_t shape[MRL_MAX_RANK], rank;
  mrl_spec_parameter_shape(&spec, idx, shape, &rank);
  mv.kind = MRL_SPEC_MOVE, mv.rank = rank, mv.n_params = 2;
  for (uint32_t d = 0; d < rank; d++) mv.spec_shape[d] = shape[d];
  mv.dtypes[0] = mv.dtypes[1] = spec.dtypes[idx];
  mrl_layout rm;
  mrl_layout_row_major(shape, rank, &rm);
  mv.layouts[0] = to_layout ? rm : spec.layouts[idx];
  mv.layouts[1] = to_layout ? spec.layouts[idx] : rm;
  void *params[2] = {src, dst};
  return mrl_run(&mv, params);
}

}  // namespace

int main(int argc, char *argv[]) {
  if (argc < 2) DIE(1, "usage: %s <spec> [file...] | <spec> --bench <iters>", argv[0]);
  mrl_spec spec;
  std::string err;
  if (!parse_spec(argv[1], &spec, &err)) DIE(1, "Bad Spec: %s", err.c_str());
  const bool bench = argc == 4 && std::string(argv[2]) == "--bench";
  const int nfiles = bench ? 0 : argc - 2;
  if (!bench && nfiles != 0 && nfiles != int(spec.n_params)) DIE(1, "Unexpected number of arguments.");
  int rc = mrl_spec_check(&spec);
  if (rc != MRL_OK) DIE(1, "Spec rejected: %s", mrl_status_string(rc));

  // Host buffers in logical row-major order, zero-filled unless files are given.
  std::vector<std::vector<uint8_t>> host(spec.n_params);
  std::vector<size_t> bytes(spec.n_params);
  for (uint32_t i = 0; i < spec.n_params; i++) {
    bytes[i] = mrl_spec_parameter_bytes(&spec, i);
    host[i].assign(bytes[i], 0);
    if (nfiles && !read_file(argv[2 + i], host[i].data(), bytes[i])) DIE(2, "Error loading input tensors.");
  }
  if (bench) {
    // c_utils.rs:193-252: random fill; ints take rand() truncated, floats land in [1, 2).
    std::srand(1);
    for (uint32_t i = 0; i < spec.n_params; i++) {
      const int dt = spec.dtypes[i];
      const size_t es = mrl_dtype_size(dt), n = bytes[i] / es;
      for (size_t j = 0; j < n; j++) {
        const uint32_t r = uint32_t(std::rand());
        if (dt == MRL_F32) ((uint32_t *)host[i].data())[j] = 0x3f800000u | (r & 0x7fffffu);
        else if (dt == MRL_BF16) ((uint16_t *)host[i].data())[j] = uint16_t(0x3f80u | (r & 0x7fu));
        else std::memcpy(host[i].data() + j * es, &r, es);
      }
    }
  }

  if ((rc = mrl_init(0)) != MRL_OK) DIE(3, "No device: %s (%s)", mrl_status_string(rc), mrl_last_error());
  std::vector<void *> dev(spec.n_params, nullptr), staged(spec.n_params, nullptr);
  for (uint32_t i = 0; i < spec.n_params; i++) {
    if (mrl_device_malloc(&dev[i], bytes[i]) != MRL_OK || mrl_device_malloc(&staged[i], bytes[i]) != MRL_OK ||
        mrl_memcpy_h2d(staged[i], host[i].data(), bytes[i]) != MRL_OK ||
        relayout(spec, i, staged[i], dev[i], true) != MRL_OK)
      DIE(3, "Device staging failed: %s", mrl_last_error());
  }

  if (bench) {
    const uint32_t iters = uint32_t(std::strtoul(argv[3], nullptr, 10));
    if (iters == 0) DIE(1, "Unexpected number of arguments.");
    double best = 0, mean = 0;
    rc = mrl_bench(&spec, dev.data(), iters, 1, &best, &mean);
    if (rc != MRL_OK) DIE(3, "Run failed: %s (%s)", mrl_status_string(rc), mrl_last_error());
    const double total_ns = mean * iters;
    std::printf("cpu: %llus %lluns\n", (unsigned long long)(total_ns / 1e9),
                (unsigned long long)(total_ns - double((unsigned long long)(total_ns / 1e9)) * 1e9));
  } else {
    rc = mrl_run(&spec, dev.data());
    if (rc != MRL_OK) DIE(3, "Run failed: %s (%s)", mrl_status_string(rc), mrl_last_error());
    // Every parameter the Spec writes, in parameter order (one for Matmul, Conv, Softmax, Move
    // and the Compose: the last, as the reference's emitted main prints).
    for (uint32_t o = 0; o < spec.n_params; o++) {
      if (mrl_spec_parameter_direction(&spec, o) == 0) continue;
      if (relayout(spec, o, dev[o], staged[o], false) != MRL_OK ||
          mrl_memcpy_d2h(host[o].data(), staged[o], bytes[o]) != MRL_OK)
        DIE(3, "Reading the output failed: %s", mrl_last_error());
      uint32_t shape[MRL_MAX_RANK], rank;
      mrl_spec_parameter_shape(&spec, o, shape, &rank);
      print_tensor(spec.dtypes[o], host[o].data(), shape, rank);
    }
  }
  for (uint32_t i = 0; i < spec.n_params; i++) {
    mrl_device_free(dev[i]);
    mrl_device_free(staged[i]);
  }
  return 0;
}
