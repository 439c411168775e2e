// libneox_probes.so: memory-system probes for the benchmark.  Not part of the product library --
// nothing here replaces a reference interface, and only bench.py and the test of these probes
// load it.  Two kernels with the access shape of the product kernels (128-bit non-temporal
// accesses, one 16-byte slot per lane, consecutive lanes on consecutive slots):
//
// * neox_probe_copy     plain copy: what this HBM sustains for one read + one write stream, and
//                       the known-size kernel the rocprofv3 FETCH_SIZE / WRITE_SIZE counters are
//                       calibrated against;
// * neox_probe_strided  touches the start of every `stride_bytes` of a buffer: loads the first
//                       `load_bytes`, stores the first `store_bytes` back unchanged (zeros if nothing
//                       was loaded).  With
//                       load = store = 64 of every 256 bytes this is the memory pattern of an
//                       in-place partial rotary (rotary_pct 0.25 of 128-dim heads) without tables,
//                       index arithmetic or rotation; load only / store only separate the two
//                       streams; load 128 / store 64 asks for whole 128-byte lines; the block size
//                       and the number of accesses a lane keeps in flight are arguments, so that the
//                       ceiling of the pattern is not tied to one launch shape;
// * neox_probe_empty    an empty kernel (launch cost);
// * neox_probe_pieces   a write, read or copy stream in 4 KiB pieces with a chosen block -> piece
//                       order: workgroups go to the 8 XCDs of the chip in turn, and a store stream
//                       runs fastest when every XCD keeps to its own pieces (piece = XCD mod 8);
// * neox_probe_strided_pieces  the partial-rotary pattern (first 64 of every 256 bytes, in place)
//                       with one 4 KiB piece per wave access and the same choice of order.
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

// Block b moves P pieces of 4 KiB (256 threads, one 16-byte access per thread and piece).
// ORDER 0: consecutive pieces b*P .. b*P+P-1.  1: the blocks of a group of 8 share 8*P pieces so
// that block x takes the pieces x, x + 8, ... (one residue mod 8 per block).  2: as 0 with the
// pieces of every group of 8 blocks rotated by the group index (every XCD walks through all residues).
template <int ORDER>
__device__ __forceinline__ uint64_t piece_index(uint64_t b, uint32_t j, uint32_t P) {
    if (ORDER == 1) return (b >> 3) * 8 * P + (uint64_t)j * 8 + (b & 7);
    if (ORDER == 2) { const uint64_t g = (b * P + j) >> 3; return (g << 3) + ((b * P + j + g) & 7); }
    return b * P + j;
}
// OP 0: write, 1: read, 2: copy src -> dst
template <int ORDER, int OP, int P>
__global__ __launch_bounds__(256) void pieces_kernel(char* dst, const char* src, uint64_t pieces, uint32_t flip) {
    u32x4 v[P];
    uint32_t seen = 0;
#pragma unroll
    for (int j = 0; j < P; ++j) {
        const uint64_t pc = piece_index<ORDER>(blockIdx.x, j, P);
        v[j] = u32x4{threadIdx.x, flip, 2, 3};
        if (OP != 0 && pc < pieces) v[j] = ld128(src + pc * 4096 + threadIdx.x * 16);
    }
#pragma unroll
    for (int j = 0; j < P; ++j) {
        const uint64_t pc = piece_index<ORDER>(blockIdx.x, j, P);
        seen |= v[j].x & v[j].y & v[j].z & v[j].w;
        if (OP != 1 && pc < pieces) st128(dst + pc * 4096 + threadIdx.x * 16, v[j]);
    }
    if (OP == 1 && flip != 0 && seen == 0x12345678u) *reinterpret_cast<uint32_t*>(dst) = seen;
}

template <int ORDER, int OP>
int launch_pieces(char* dst, const char* src, uint64_t pieces, int per_block, hipStream_t st) {
    uint64_t blocks = (pieces + per_block - 1) / per_block;
    if (ORDER == 1) blocks = (blocks + 7) & ~7ull;  // whole groups of 8 blocks cover every piece
    if (blocks > 0x7fffffffULL) return -3;
    const dim3 grid((unsigned)blocks), block(256);
    switch (per_block) {
        case 1: hipLaunchKernelGGL((pieces_kernel<ORDER, OP, 1>), grid, block, 0, st, dst, src, pieces, 0u); break;
        case 2: hipLaunchKernelGGL((pieces_kernel<ORDER, OP, 2>), grid, block, 0, st, dst, src, pieces, 0u); break;
        case 4: hipLaunchKernelGGL((pieces_kernel<ORDER, OP, 4>), grid, block, 0, st, dst, src, pieces, 0u); break;
        default: return -3;
    }
    return hipGetLastError() == hipSuccess ? 0 : -6;
}

// The partial-rotary pattern by pieces: a wave access covers the 16 spans (first 64 of every 256
// bytes) of one 4 KiB piece; a block of 4 waves handles 4*K pieces, consecutive (ORDER 0) or 8 apart
// with the residue of the block index (ORDER 1).  OP 0: load + store back, 1: load only, 2: store only.
template <int ORDER, int K, int OP>
__global__ __launch_bounds__(256) void strided_pieces_kernel(char* buf, uint64_t pieces, uint32_t flip) {
    const uint32_t lane = threadIdx.x & 63, w = threadIdx.x >> 6;
    u32x4 v[K];
    char* p[K];
    bool live[K];
    uint32_t seen = 0;
#pragma unroll
    for (int j = 0; j < K; ++j) {
        const uint64_t pc = piece_index<ORDER>(blockIdx.x, w * K + j, 4 * K);
        live[j] = pc < pieces;
        p[j] = buf + pc * 4096 + (lane >> 2) * 256 + (lane & 3) * 16;
        v[j] = u32x4{flip, flip, flip, flip};
        if (OP != 2 && live[j]) v[j] = ld128(p[j]);
    }
#pragma unroll
    for (int j = 0; j < K; ++j) {
        v[j].x ^= flip;
        seen |= v[j].x & v[j].y;
        if (OP != 1 && live[j]) st128(p[j], v[j]);
    }
    if (OP == 1 && flip != 0 && seen == 0x12345678u) *reinterpret_cast<uint32_t*>(buf) = seen;
}

template <int ORDER, int OP>
int launch_strided_pieces(char* buf, uint64_t pieces, int per_wave, hipStream_t st) {
    const uint64_t per_block = 4ull * per_wave;
    uint64_t blocks = (pieces + per_block - 1) / per_block;
    if (ORDER == 1) blocks = (blocks + 7) & ~7ull;
    if (blocks > 0x7fffffffULL) return -3;
    const dim3 grid((unsigned)blocks), block(256);
    switch (per_wave) {
        case 1: hipLaunchKernelGGL((strided_pieces_kernel<ORDER, 1, OP>), grid, block, 0, st, buf, pieces, 0u); break;
        case 2: hipLaunchKernelGGL((strided_pieces_kernel<ORDER, 2, OP>), grid, block, 0, st, buf, pieces, 0u); break;
        case 4: hipLaunchKernelGGL((strided_pieces_kernel<ORDER, 4, OP>), grid, block, 0, st, buf, pieces, 0u); break;
        default: return -3;
    }
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

// nbytes: a multiple of 4096 (of 32768 for order 2).  op: 0 write dst, 1 read src, 2 copy src -> dst.  per_block: 1, 2 or 4
// pieces per 256-thread block.  order: 0 consecutive, 1 eight apart (XCD-aware), 2 rotating.
int neox_probe_pieces(void* dst, const void* src, int64_t nbytes, int32_t op, int32_t per_block, int32_t order,
                      void* stream) {
    if (!dst || !src) return -1;
    if (nbytes < 4096 || nbytes % 4096 || op < 0 || op > 2 || order < 0 || order > 2) return -3;
    if (order == 2 && nbytes % 32768) return -3;  // the rotation permutes whole groups of 8 pieces
    if ((reinterpret_cast<uintptr_t>(dst) | reinterpret_cast<uintptr_t>(src)) & 4095u) return -5;
    char* d = static_cast<char*>(dst);
    const char* s = static_cast<const char*>(src);
    const uint64_t pieces = (uint64_t)nbytes / 4096;
    hipStream_t st = (hipStream_t)stream;
#define NEOX_PROBE_PIECES(ORDER)                                                     \
    (op == 0   ? launch_pieces<ORDER, 0>(d, s, pieces, per_block, st)                \
     : op == 1 ? launch_pieces<ORDER, 1>(d, s, pieces, per_block, st)                \
               : launch_pieces<ORDER, 2>(d, s, pieces, per_block, st))
    return order == 0 ? NEOX_PROBE_PIECES(0) : order == 1 ? NEOX_PROBE_PIECES(1) : NEOX_PROBE_PIECES(2);
#undef NEOX_PROBE_PIECES
}

// buf: nbytes (a multiple of 4096) whose first 64 of every 256 bytes are touched in place.  op: 0 load +
// store back, 1 load only, 2 store only (zeros).  per_wave: 1, 2 or 4 pieces per wave.  order: 0 or 1.
int neox_probe_strided_pieces(void* buf, int64_t nbytes, int32_t op, int32_t per_wave, int32_t order, void* stream) {
    if (!buf) return -1;
    if (nbytes < 4096 || nbytes % 4096 || op < 0 || op > 2 || order < 0 || order > 1) return -3;
    if (reinterpret_cast<uintptr_t>(buf) & 4095u) return -5;
    char* p = static_cast<char*>(buf);
    const uint64_t pieces = (uint64_t)nbytes / 4096;
    hipStream_t st = (hipStream_t)stream;
    if (order == 0) {
        return op == 0 ? launch_strided_pieces<0, 0>(p, pieces, per_wave, st)
               : op == 1 ? launch_strided_pieces<0, 1>(p, pieces, per_wave, st)
                         : launch_strided_pieces<0, 2>(p, pieces, per_wave, st);
    }
    return op == 0 ? launch_strided_pieces<1, 0>(p, pieces, per_wave, st)
           : op == 1 ? launch_strided_pieces<1, 1>(p, pieces, per_wave, st)
                     : launch_strided_pieces<1, 2>(p, pieces, per_wave, st);
}

}  // extern "C"
#pragma GCC visibility pop
