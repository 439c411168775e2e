// Sliding-window causal softmax kernels (forward and backward), and their launchers.
#include "softmax_dispatch.hpp"

namespace neox {

hipError_t launch_softmax_band_fwd(const SoftmaxArgs& a, int dtype, bool vec_ok, hipStream_t stream) {
    return dispatch_band<false>(a, dtype, vec_ok, stream);
}

hipError_t launch_softmax_band_bwd(const SoftmaxArgs& a, int dtype, bool vec_ok, hipStream_t stream) {
    return dispatch_band<true>(a, dtype, vec_ok, stream);
}

}  // namespace neox
