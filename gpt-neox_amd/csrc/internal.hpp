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
// aligned); without it the launchers of a feature set without kRagged use their element-wise
// kernels, and those with kRagged (8 <= sk < kMaxStagedRow) ignore it.
// One specialisation per feature set, each in a translation unit of its own: FLAGS combines
// kAlibi (a.slopes, a.np), kBias (a.bias, a.bias_rows, a.bias_bytes), kDropout (a.drop, and a.out2
// in the forward pass) and kRagged for the forward pass, kDropout and kRagged for the backward pass.
template <int FLAGS>
hipError_t launch_softmax_fwd_flags(const SoftmaxArgs& a, Mask mask, int dtype, bool vec_ok, hipStream_t stream);
template <int FLAGS>
hipError_t launch_softmax_bwd_flags(const SoftmaxArgs& a, Mask mask, int dtype, bool vec_ok, hipStream_t stream);
// the feature sets that are built (the Makefile's FWD_SETS and BWD_SETS)
#define NEOX_FWD_FEATURE_SETS(X) X(0) X(4) X(16) X(20) X(8) X(12) X(24) X(28) X(32) X(36) X(48) X(52) X(40) X(44) X(56) X(60)
#define NEOX_BWD_FEATURE_SETS(X) X(0) X(8) X(32) X(40)
#define NEOX_DECLARE_FWD(F) \
    template <>             \
    hipError_t launch_softmax_fwd_flags<F>(const SoftmaxArgs&, Mask, int, bool, hipStream_t);
#define NEOX_DECLARE_BWD(F) \
    template <>             \
    hipError_t launch_softmax_bwd_flags<F>(const SoftmaxArgs&, Mask, int, bool, hipStream_t);
NEOX_FWD_FEATURE_SETS(NEOX_DECLARE_FWD)
NEOX_BWD_FEATURE_SETS(NEOX_DECLARE_BWD)
#undef NEOX_DECLARE_FWD
#undef NEOX_DECLARE_BWD
// The same by a run-time feature set (hipErrorInvalidValue for a set no unit was built for).
hipError_t launch_softmax_fwd(int flags, const SoftmaxArgs& a, Mask mask, int dtype, bool vec_ok, hipStream_t stream);
hipError_t launch_softmax_bwd(int flags, const SoftmaxArgs& a, Mask mask, int dtype, bool vec_ok, hipStream_t stream);
// Sliding-window causal rows (a.window): aligned rows of 513 .. kMaxRegisterRow columns only.
hipError_t launch_softmax_band_fwd(const SoftmaxArgs& a, int dtype, bool vec_ok, hipStream_t stream);
hipError_t launch_softmax_band_bwd(const SoftmaxArgs& a, int dtype, bool vec_ok, hipStream_t stream);
// Folds a mask [rows / sq, 1, sq, sk] into the record described in mask_classify.hip: four words, or
// eight together with the rows' visible ends (row_end, [rows]) when that pointer is given.
hipError_t launch_mask_classify(int32_t* record, int32_t* row_end, const uint8_t* mask, uint32_t rows, int sq, int sk,
                                hipStream_t stream);
// cs_dtype: NEOX_F32 or the dtype of q for cos/sin tables, kRopeAngles for fp32 angles in a.cos
constexpr int kRopeAngles = -1;
hipError_t launch_rope(const RopeArgs& a, int s, int n_outer, int w, int dtype, int cs_dtype,
                       bool backward, hipStream_t stream);

// Longest row the register-resident kernels take (16 waves x 4 chunks x 512 columns).
constexpr int kMaxRegisterRow = 16 * 4 * kChunk;
// Longest row the LDS-staged kernels take (159 KiB of 16-bit values); a ragged row must be shorter.
constexpr int kMaxStagedRow = 159 * 1024 / 2;

}  // namespace neox
