// Forward softmax kernels for rows at any alignment (sk % 8 != 0, pointers not 16-byte
// aligned), and their launcher.
#include "softmax_dispatch.hpp"

namespace neox {

hipError_t launch_softmax_ragged_fwd(const SoftmaxArgs& a, Mask mask, int dtype, bool vec_ok, hipStream_t stream) {
    return dispatch_softmax<false, kRagged>(a, mask, dtype, vec_ok, stream);
}

}  // namespace neox
