// Backward softmax kernels (causal and full-row) and their launcher.
#include "softmax_dispatch.hpp"

namespace neox {

hipError_t launch_softmax_bwd(const SoftmaxArgs& a, Mask mask, int dtype, bool vec_ok,
                              hipStream_t stream) {
    return dispatch_softmax<true>(a, mask, dtype, vec_ok, stream);
}

}  // namespace neox
