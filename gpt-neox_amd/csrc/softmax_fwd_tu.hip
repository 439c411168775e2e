// Forward softmax kernels of one feature set, and their launcher.  Compiled once per feature set:
// NEOX_TU_FLAGS is a combination of kAlibi (4), kDropout (8), kBias (16) and kRagged (32).
#include "softmax_dispatch.hpp"

#ifndef NEOX_TU_FLAGS
#error "compile with -DNEOX_TU_FLAGS=<feature set>"
#endif

namespace neox {

template <>
hipError_t launch_softmax_fwd_flags<NEOX_TU_FLAGS>(const SoftmaxArgs& a, Mask mask, int dtype, bool vec_ok,
                                                   hipStream_t stream) {
    return dispatch_softmax<false, NEOX_TU_FLAGS>(a, mask, dtype, vec_ok, stream);
}

}  // namespace neox
