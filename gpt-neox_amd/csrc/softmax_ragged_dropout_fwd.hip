// Forward softmax kernels with attention dropout for rows at any alignment, and their launcher.
#include "softmax_dispatch.hpp"

namespace neox {

hipError_t launch_softmax_ragged_dropout_fwd(const SoftmaxArgs& a, Mask mask, int dtype, bool vec_ok, hipStream_t stream) {
    return dispatch_softmax<false, kRagged | kDropout>(a, mask, dtype, vec_ok, stream);
}

}  // namespace neox
