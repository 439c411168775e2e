// libneox_probes.so: memory-system probes for the benchmark.  Not part of the product library --
// nothing here replaces a reference interface, and only bench.py and the test of these probes
// load it.  Two kernels with the access shape of the product kernels (128-bit non-temporal
// accesses, one 16-byte slot per lane, consecutive lanes on consecutive slots):
//
// * neox_probe_copy     plain copy: what this HBM sustains for one read + one write stream, and
//                       the known-size kernel the rocprofv3 FETCH_SIZE / WRITE_SIZE counters are
//                       calibrated against;
// * neox_probe_strided  touches the start of every `stride_bytes` of a buffer: loads the first
//                       `load_bytes`, stores the first `store_bytes` back unchanged.  With
//                       load = store = 64 of every 256 bytes this is the memory pattern of an
//                       in-place partial rotary (rotary_pct 0.25 of 128-dim heads) without tables,
//                       index arithmetic or rotation; load only / store only separate the two
//                       streams; load 128 / store 64 asks for whole 128-byte lines; the block size
//                       and the number of accesses a lane keeps in flight are arguments, so that the
//                       ceiling of the pattern is not tied to one launch shape;
// * neox_probe_empty    an empty kernel (launch cost).
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

// slot g of the launch = slot (g % sps) of span (g / sps); sps = max(load, store) slots per span.
// A lane loads its slot if it lies in the first `ld_slots` of the span and stores it back if it
// lies in the first `st_slots`.
template <int THREADS, int K>
__global__ __launch_bounds__(THREADS) void strided_kernel(char* buf, uint64_t slots, uint32_t sps,
                                                          uint32_t ld_slots, uint32_t st_slots,
                                                          uint64_t stride_bytes, uint32_t flip) {
    const uint64_t g0 = (uint64_t)blockIdx.x * (THREADS * K) + threadIdx.x;
    char* p[K];
    u32x4 v[K];
    bool ld[K], st[K];
#pragma unroll
    for (int k = 0; k < K; ++k) {
        const uint64_t g = g0 + (uint64_t)k * THREADS;
        const uint64_t span = g / sps;
        const uint32_t slot = (uint32_t)(g - span * sps);
        p[k] = buf + span * stride_bytes + slot * 16u;
        ld[k] = g < slots && slot < ld_slots;
        st[k] = g < slots && slot < st_slots;
        v[k] = u32x4{flip, flip, flip, flip};
        if (ld[k]) v[k] = ld128(p[k]);
    }
    uint32_t seen = 0;
#pragma unroll
    for (int k = 0; k < K; ++k) {
        v[k].x ^= flip;  // 0 at run time: the compiler cannot drop the store of an unchanged value
        seen |= v[k].x & v[k].y & v[k].z & v[k].w;
        if (st[k]) st128(p[k], v[k]);
    }
    // load-only launches: the loaded values must be used; this store never happens (flip == 0)
    if (st_slots == 0 && flip != 0 && seen == 0x12345678u) *reinterpret_cast<uint32_t*>(buf) = seen;
}

template <int THREADS, int K>
int launch_strided(char* buf, uint64_t slots, uint32_t sps, uint32_t ld_slots, uint32_t st_slots,
                   uint64_t stride_bytes, hipStream_t st) {
    const uint64_t per_block = (uint64_t)THREADS * K;
    const uint64_t blocks = (slots + per_block - 1) / per_block;
    if (blocks > 0x7fffffffULL) return -3;
    hipLaunchKernelGGL((strided_kernel<THREADS, K>), dim3((unsigned)blocks), dim3(THREADS), 0, st, buf,
                       slots, sps, ld_slots, st_slots, stride_bytes, 0u);
    return hipGetLastError() == hipSuccess ? 0 : -6;
}

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

// load_bytes, store_bytes: multiples of 16, at most stride_bytes, not both 0.  threads: 256 or
// 1024 per block; in_flight: 4 or 8 accesses per lane.  The buffer must hold
// (n_spans - 1) * stride_bytes + max(load_bytes, store_bytes) bytes.
int neox_probe_strided(void* buf, int64_t n_spans, int32_t load_bytes, int32_t store_bytes,
                       int64_t stride_bytes, int32_t threads, int32_t in_flight, void* stream) {
    if (!buf) return -1;
    const int32_t widest = load_bytes > store_bytes ? load_bytes : store_bytes;
    if (n_spans < 1 || load_bytes < 0 || store_bytes < 0 || widest < 16 || load_bytes % 16 ||
        store_bytes % 16 || stride_bytes < widest || stride_bytes % 16)
        return -3;
    if (!aligned16(buf)) return -5;
    const uint32_t sps = (uint32_t)widest / 16u;
    const uint64_t slots = (uint64_t)n_spans * sps;
    char* p = static_cast<char*>(buf);
    const uint32_t ld = (uint32_t)load_bytes / 16u, sv = (uint32_t)store_bytes / 16u;
    hipStream_t st = (hipStream_t)stream;
    if (threads == 256 && in_flight == 4) return launch_strided<256, 4>(p, slots, sps, ld, sv, (uint64_t)stride_bytes, st);
    if (threads == 256 && in_flight == 8) return launch_strided<256, 8>(p, slots, sps, ld, sv, (uint64_t)stride_bytes, st);
    if (threads == 1024 && in_flight == 4) return launch_strided<1024, 4>(p, slots, sps, ld, sv, (uint64_t)stride_bytes, st);
    if (threads == 1024 && in_flight == 8) return launch_strided<1024, 8>(p, slots, sps, ld, sv, (uint64_t)stride_bytes, st);
    return -3;
}

}  // extern "C"
#pragma GCC visibility pop
