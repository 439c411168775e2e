// Host-side plumbing shared by the translation units of libneox_fused.so.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "../../include/neox_fused.h"
#include "rope_kernels.hpp"
#include "softmax_kernels.hpp"

namespace neox {

// Records a message for neox_fused_last_error() on this thread and returns `status`.
int fail(int status, const char* fmt, ...) __attribute__((format(printf, 2, 3)));

// Launchers: pick the kernel shape for the row length and launch on `stream`.
// `vec_ok` says that every row starts on a 16-byte boundary (sk % 8 == 0, pointers 16-byte
// aligned); without it these launchers use their element-wise kernels.
hipError_t launch_softmax_fwd(const SoftmaxArgs& a, Mask mask, int dtype, bool vec_ok,
                              hipStream_t stream);
hipError_t launch_softmax_bwd(const SoftmaxArgs& a, Mask mask, int dtype, bool vec_ok,
                              hipStream_t stream);
// The same with attention dropout fused in (a.drop, and a.out2 for the forward pass).
hipError_t launch_softmax_dropout_fwd(const SoftmaxArgs& a, Mask mask, int dtype, bool vec_ok,
                                      hipStream_t stream);
hipError_t launch_softmax_dropout_bwd(const SoftmaxArgs& a, Mask mask, int dtype, bool vec_ok,
                                      hipStream_t stream);
// Forward with an additive bias tensor (a.bias, a.bias_rows, a.bias_bytes).
hipError_t launch_softmax_bias_fwd(const SoftmaxArgs& a, Mask mask, int dtype, bool vec_ok,
                                   hipStream_t stream);
// Rows at any 2-byte alignment with 8 <= sk <= kMaxRegisterRow (a.bias optional in the forward
// passes), without and with attention dropout; `vec_ok` is ignored.
hipError_t launch_softmax_ragged_fwd(const SoftmaxArgs& a, Mask mask, int dtype, bool vec_ok,
                                     hipStream_t stream);
hipError_t launch_softmax_ragged_bwd(const SoftmaxArgs& a, Mask mask, int dtype, bool vec_ok,
                                     hipStream_t stream);
hipError_t launch_softmax_ragged_dropout_fwd(const SoftmaxArgs& a, Mask mask, int dtype, bool vec_ok,
                                             hipStream_t stream);
hipError_t launch_softmax_ragged_dropout_bwd(const SoftmaxArgs& a, Mask mask, int dtype, bool vec_ok,
                                             hipStream_t stream);
// cs_dtype: NEOX_F32 or the dtype of q for cos/sin tables, kRopeAngles for fp32 angles in a.cos
constexpr int kRopeAngles = -1;
hipError_t launch_rope(const RopeArgs& a, int s, int n_outer, int w, int dtype, int cs_dtype,
                       bool backward, hipStream_t stream);

// Longest row the register-resident kernels take (16 waves x 4 chunks x 512 columns).
constexpr int kMaxRegisterRow = 16 * 4 * kChunk;

}  // namespace neox
