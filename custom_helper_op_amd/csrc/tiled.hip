// double has no tiled kernels: the registered float64 ops run on the general kernels.
#include "internal.h"

namespace chop {
template <>
bool tiled_forward_supported<double>(const Args<double> &) { return false; }
template <>
bool tiled_backward_supported<double>(const Args<double> &) { return false; }
template <>
hipError_t launch_tiled_forward<double>(const Args<double> &, hipStream_t) { return hipErrorNotSupported; }
template <>
hipError_t launch_tiled_backward<double>(const Args<double> &, hipStream_t) { return hipErrorNotSupported; }
}  // namespace chop
