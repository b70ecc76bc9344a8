#include "kernels.h"
namespace mrl {
bool attn_applicable(const AttnArgs &) { return false; }
hipError_t launch_attn(const AttnArgs &, hipStream_t) { return hipErrorNotSupported; }
}  // namespace mrl
