// Kernel-shape selection for the softmax kernels.
//
// chunks = ceil(sk / 512) decides how a row is laid over waves:
//   chunks <= 4            one wave per row, 4 rows per 256-thread block
//   chunks <= 8            2 waves per row
//   chunks <= 16           4 waves per row          (sk <= 8192)
//   chunks <= 32 / <= 64   8 / 16 waves per row     (sk <= 32768)
// so that no wave holds more than 4 chunks (32 fp32 values per lane) and the
// occupancy stays at 8 waves per SIMD for every row length.
#pragma once

#include "internal.hpp"

namespace neox {

template <typename T, Mask M, bool BWD, int NCH, int WPR, int RPB>
static hipError_t launch_shape(const SoftmaxArgs& a, hipStream_t st) {
    const dim3 grid((a.rows + RPB - 1) / RPB);
    const dim3 block(kWave * WPR * RPB);
    if constexpr (BWD) {
        hipLaunchKernelGGL((softmax_bwd_kernel<T, NCH, WPR, RPB, M>), grid, block, 0, st, a);
    } else {
        hipLaunchKernelGGL((softmax_fwd_kernel<T, NCH, WPR, RPB, M>), grid, block, 0, st, a);
    }
    return hipGetLastError();
}

template <typename T, Mask M, bool BWD>
static hipError_t launch_generic(const SoftmaxArgs& a, hipStream_t st) {
    const dim3 grid(a.rows);
    const dim3 block(kGenericThreads);
    if constexpr (BWD) {
        hipLaunchKernelGGL((softmax_bwd_generic_kernel<T, M>), grid, block, 0, st, a);
    } else {
        hipLaunchKernelGGL((softmax_fwd_generic_kernel<T, M>), grid, block, 0, st, a);
    }
    return hipGetLastError();
}

template <typename T, Mask M, bool BWD, int WPR, int RPB>
static hipError_t launch_split(const SoftmaxArgs& a, int chunks, hipStream_t st) {
    // chunks in (2*WPR, 4*WPR]
    if (chunks <= 3 * WPR) return launch_shape<T, M, BWD, 3, WPR, RPB>(a, st);
    return launch_shape<T, M, BWD, 4, WPR, RPB>(a, st);
}

template <typename T, Mask M, bool BWD>
static hipError_t dispatch_rows(const SoftmaxArgs& a, bool vec_ok, hipStream_t st) {
    const int chunks = (a.sk + kChunk - 1) / kChunk;
    if (!vec_ok || a.sk > kMaxRegisterRow) return launch_generic<T, M, BWD>(a, st);
    switch (chunks) {
        case 1: return launch_shape<T, M, BWD, 1, 1, 4>(a, st);
        case 2: return launch_shape<T, M, BWD, 2, 1, 4>(a, st);
        case 3: return launch_shape<T, M, BWD, 3, 1, 4>(a, st);
        case 4: return launch_shape<T, M, BWD, 4, 1, 4>(a, st);
        default: break;
    }
    if (chunks <= 8) return launch_split<T, M, BWD, 2, 2>(a, chunks, st);
    if (chunks <= 16) return launch_split<T, M, BWD, 4, 1>(a, chunks, st);
    if (chunks <= 32) return launch_split<T, M, BWD, 8, 1>(a, chunks, st);
    return launch_split<T, M, BWD, 16, 1>(a, chunks, st);
}

template <bool BWD>
static hipError_t dispatch_softmax(const SoftmaxArgs& a, Mask mask, int dtype, bool vec_ok,
                                   hipStream_t st) {
    const bool f16 = (dtype == NEOX_F16);
    switch (mask) {
        case Mask::Causal:
            return f16 ? dispatch_rows<F16, Mask::Causal, BWD>(a, vec_ok, st)
                       : dispatch_rows<BF16, Mask::Causal, BWD>(a, vec_ok, st);
        case Mask::Bytes:
            if constexpr (!BWD) {
                return f16 ? dispatch_rows<F16, Mask::Bytes, BWD>(a, vec_ok, st)
                           : dispatch_rows<BF16, Mask::Bytes, BWD>(a, vec_ok, st);
            }
            [[fallthrough]];  // the backward pass needs no mask: masked probabilities are 0
        case Mask::None:
            if constexpr (BWD) {
                return f16 ? dispatch_rows<F16, Mask::None, BWD>(a, vec_ok, st)
                           : dispatch_rows<BF16, Mask::None, BWD>(a, vec_ok, st);
            }
            break;
    }
    return hipErrorInvalidValue;
}

}  // namespace neox
