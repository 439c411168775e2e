// Recognises causal attention masks on the device, so that a caller holding only the mask tensor can
// choose the kernel that never reads it.  The masks in question are the ones
// megatron/utils.py:67-80 (get_attn_mask) builds: row i hides every key j > i and, with a sliding
// window of width w, every key j < i - w as well.
//
// One wave per mask row finds the number of visible keys, the first and the last one.  The row fits
// the pattern if the visible keys are the contiguous run [lo, i]; the rows then have to agree on one
// w with lo = max(0, i - w): a row with lo > 0 fixes w = i - lo, a row with lo = 0 only says w >= i.
// What the rows say is folded into the record the host reads afterwards.
//
// The same pass can note where every row's visible keys end (row_end[row] = last visible key + 1, 0
// for a row without one): the mask-tensor forward kernels take that array as a hint and fetch neither
// the scores nor the mask bytes of a row's hidden tail -- the padding of a batch of sequences of
// different lengths, or the upper triangle of a causal mask that a caller combines with something
// else.  The record then also holds the number of keys the hint saves, so that the caller can tell
// whether it is worth passing on.
#include <limits.h>

#include "internal.hpp"

namespace neox {

// record[0]: 1 if some row does not fit the pattern (always, if the mask is not square); [1], [2]:
// smallest and largest i - lo over the rows with lo > 0 (INT_MAX and -1 without such a row); [3]:
// largest i over the rows with lo = 0 (-1 if none).  `words` = 8: [4], [5] the low and high half of the
// 64-bit number of hidden keys behind the rows' last visible ones, [6], [7] zero.
__global__ void mask_classify_init_kernel(int32_t* record, int words, int square) {
    if (threadIdx.x == 0) {
        record[0] = square ? 0 : 1;
        record[1] = INT_MAX;
        record[2] = -1;
        record[3] = -1;
        for (int k = 4; k < words; ++k) record[k] = 0;
    }
}

constexpr int kScanWaves = 16;  // waves per block

// One wave per mask row, the rows dealt to the waves of the grid in turn; every wave keeps what its
// rows say in registers, the waves of a block combine that through LDS, and one thread per block
// folds the block's part into the record: a few hundred atomic operations on the same few words
// instead of several per row (which cost more than reading the mask: about 12 ns each).
template <bool WIDE>
__global__ __launch_bounds__(kScanWaves * kWave) void mask_classify_kernel(int32_t* record, int32_t* row_end,
                                                                           const uint8_t* mask, uint32_t rows, int sq, int sk) {
    __shared__ int s_bad[kScanWaves], s_min[kScanWaves], s_max[kScanWaves], s_top[kScanWaves];
    __shared__ unsigned long long s_tail[kScanWaves];
    const int lane = threadIdx.x & (kWave - 1);
    const int wib = threadIdx.x >> 6;
    const uint32_t waves = gridDim.x * kScanWaves;
    int bad = 0, wmin = INT_MAX, wmax = -1, top = -1;  // wave-uniform, as in the record
    unsigned long long tail = 0;
    for (uint32_t row = blockIdx.x * kScanWaves + wib; row < rows; row += waves) {
        const int i = (int)(row % (uint32_t)sq);
        const uint8_t* m = mask + (size_t)row * sk;
        int count = 0, first = INT_MAX, last = -1;
        if constexpr (WIDE) {  // sk % 8 == 0 and the tensor 8-byte aligned: 8 bytes per lane, 4 loads in flight
            constexpr int U = 4;
            for (int c0 = lane * 8; c0 < sk; c0 += U * kWave * 8) {
                uint64_t v[U];
#pragma unroll
                for (int u = 0; u < U; ++u) {
                    const int c = c0 + u * kWave * 8;
                    v[u] = c < sk ? *reinterpret_cast<const uint64_t*>(m + c) : ~0ull;  // past the row: hidden
                }
#pragma unroll
                for (int u = 0; u < U; ++u) {
                    const int c = c0 + u * kWave * 8;
                    if (v[u] == 0) {
                        count += 8;
                        first = min(first, c);
                        last = c + 7;
                    } else if (c < sk) {
#pragma unroll
                        for (int k = 0; k < 8; ++k) {
                            if (((v[u] >> (8 * k)) & 0xffu) == 0) {
                                ++count;
                                first = min(first, c + k);
                                last = c + k;
                            }
                        }
                    }
                }
            }
        } else {
            for (int c = lane; c < sk; c += kWave) {
                if (m[c] == 0) {
                    ++count;
                    first = min(first, c);
                    last = c;
                }
            }
        }
#pragma unroll
        for (int step = 1; step < kWave; step <<= 1) {
            count += __shfl_xor(count, step);
            first = min(first, __shfl_xor(first, step));
            last = max(last, __shfl_xor(last, step));
        }
        if (row_end != nullptr) {
            if (lane == 0) row_end[row] = last + 1;
            if (count != 0 && last + 1 < sk) tail += (unsigned long long)(sk - (last + 1));
        }
        if (sq != sk) continue;  // record[0] says so already
        if (count == 0 || last != i || count != last - first + 1) {
            bad = 1;
        } else if (first > 0) {
            wmin = min(wmin, i - first);
            wmax = max(wmax, i - first);
        } else {
            top = max(top, i);
        }
    }
    if (lane == 0) {
        s_bad[wib] = bad;
        s_min[wib] = wmin;
        s_max[wib] = wmax;
        s_top[wib] = top;
        s_tail[wib] = tail;
    }
    __syncthreads();
    if (threadIdx.x != 0) return;
    for (int w = 1; w < kScanWaves; ++w) {
        bad |= s_bad[w];
        wmin = min(wmin, s_min[w]);
        wmax = max(wmax, s_max[w]);
        top = max(top, s_top[w]);
        tail += s_tail[w];
    }
    if (bad) atomicOr(record, 1);
    if (wmin != INT_MAX) atomicMin(record + 1, wmin);
    if (wmax >= 0) atomicMax(record + 2, wmax);
    if (top >= 0) atomicMax(record + 3, top);
    if (tail != 0) atomicAdd(reinterpret_cast<unsigned long long*>(record + 4), tail);
}

hipError_t launch_mask_classify(int32_t* record, int32_t* row_end, const uint8_t* mask, uint32_t rows, int sq, int sk,
                                hipStream_t st) {
    hipLaunchKernelGGL(mask_classify_init_kernel, dim3(1), dim3(64), 0, st, record, row_end ? 8 : 4, sq == sk ? 1 : 0);
    // two blocks per CU at most: the record takes a handful of atomic operations per block
    const uint32_t blocks = (rows + kScanWaves - 1) / kScanWaves;
    const dim3 grid(blocks < 512u ? blocks : 512u), block(kScanWaves * kWave);
    const bool wide = sk % 8 == 0 && (reinterpret_cast<uintptr_t>(mask) & 7u) == 0;
    if (wide) hipLaunchKernelGGL((mask_classify_kernel<true>), grid, block, 0, st, record, row_end, mask, rows, sq, sk);
    else hipLaunchKernelGGL((mask_classify_kernel<false>), grid, block, 0, st, record, row_end, mask, rows, sq, sk);
    return hipGetLastError();
}

}  // namespace neox
