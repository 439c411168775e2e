// libneox_probes.so: two measurement aids for the benchmark.  Not part of the product library --
// nothing here replaces a reference interface, only bench.py --studies loads it, and the default
// make target does not build it (`make probes` does).
//
// * neox_probe_copy   plain copy with the access shape of the product kernels (128-bit non-temporal
//                     accesses, one 16-byte slot per lane, consecutive lanes on consecutive slots):
//                     what this HBM sustains for one read + one write stream, and the known-size
//                     kernel the rocprofv3 FETCH_SIZE / WRITE_SIZE counters are calibrated against;
// * neox_probe_empty  an empty kernel (launch cost).
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "wave.hpp"

using namespace neox;

namespace {

__global__ __launch_bounds__(256) void copy_kernel(u32x4* dst, const u32x4* src, size_t n16) {
    size_t idx = (size_t)blockIdx.x * 1024 + threadIdx.x;
    u32x4 r[4];
#pragma unroll
    for (int k = 0; k < 4; ++k)
        if (idx + k * 256 < n16) r[k] = ld128(src + idx + k * 256);
#pragma unroll
    for (int k = 0; k < 4; ++k)
        if (idx + k * 256 < n16) st128(dst + idx + k * 256, r[k]);
}

__global__ void empty_kernel() {}

inline bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

}  // namespace

#pragma GCC visibility push(default)
extern "C" {

// 0 on success, -1 null pointer, -3 bad size, -5 misaligned, -6 launch failure
int neox_probe_copy(void* dst, const void* src, int64_t nbytes, void* stream) {
    if (!dst || !src) return -1;
    if (nbytes < 16 || nbytes % 16) return -3;
    if (!aligned16(dst) || !aligned16(src)) return -5;
    const size_t n16 = (size_t)nbytes / 16;
    const size_t blocks = (n16 + 1023) / 1024;
    if (blocks > 0x7fffffffULL) return -3;
    hipLaunchKernelGGL(copy_kernel, dim3((unsigned)blocks), dim3(256), 0, (hipStream_t)stream,
                       static_cast<u32x4*>(dst), static_cast<const u32x4*>(src), n16);
    return hipGetLastError() == hipSuccess ? 0 : -6;
}

// A kernel that does nothing: back-to-back launches of it show the launch cost every kernel pays.
int neox_probe_empty(void* stream) {
    hipLaunchKernelGGL(empty_kernel, dim3(1), dim3(64), 0, (hipStream_t)stream);
    return hipGetLastError() == hipSuccess ? 0 : -6;
}

}  // extern "C"
#pragma GCC visibility pop
