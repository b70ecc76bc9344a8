#include "kernels.h"
namespace mrl {
bool conv_i8_applicable(const ConvArgs &) { return false; }
hipError_t launch_conv_i8(const ConvArgs &, bool, hipStream_t) { return hipErrorNotSupported; }
}  // namespace mrl
