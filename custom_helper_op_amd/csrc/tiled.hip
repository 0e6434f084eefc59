// Tiled kernels (placeholder while the general path is brought up).
#include "internal.h"

namespace chop {
template <typename S> bool tiled_forward_supported(const Args<S> &) { return false; }
template <typename S> hipError_t launch_tiled_forward(const Args<S> &, hipStream_t) { return hipErrorNotSupported; }
template <typename S> bool tiled_backward_supported(const Args<S> &) { return false; }
template <typename S> hipError_t launch_tiled_backward(const Args<S> &, hipStream_t) { return hipErrorNotSupported; }
#define CHOP_INSTANTIATE(S)                                                      \
  template bool tiled_forward_supported<S>(const Args<S> &);                     \
  template hipError_t launch_tiled_forward<S>(const Args<S> &, hipStream_t);     \
  template bool tiled_backward_supported<S>(const Args<S> &);                    \
  template hipError_t launch_tiled_backward<S>(const Args<S> &, hipStream_t);
CHOP_INSTANTIATE(float)
CHOP_INSTANTIATE(double)
CHOP_INSTANTIATE(__half)
CHOP_INSTANTIATE(bf16_t)
}  // namespace chop
