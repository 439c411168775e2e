// Forward softmax kernels that add a bias tensor to the scores, and their launcher.
#include "softmax_dispatch.hpp"

namespace neox {

hipError_t launch_softmax_bias_fwd(const SoftmaxArgs& a, Mask mask, int dtype, bool vec_ok,
                                   hipStream_t stream) {
    return dispatch_softmax<false, kBias>(a, mask, dtype, vec_ok, stream);
}

}  // namespace neox
