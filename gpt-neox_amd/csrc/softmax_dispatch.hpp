// Kernel-shape selection for the softmax kernels.
//
// chunks = ceil(sk / 512) decides how a row is laid over waves.  Measured on MI355X, a
// wave that holds 2 chunks (1024 columns) is the sweet spot at every row length -- 4 chunks
// per wave cost 3-5 % of bandwidth, 1 chunk per wave 10-20 % -- so a row gets
// ceil(chunks / 2) waves:
//   chunks == 1    several rows per wave (packed kernels)            (sk <= 512)
//   chunks <= 4    full-row backward only: packed kernel, one wave per row, R x C = 4
//   chunks == 2    1 wave per row, 4 rows per 256-thread block      (sk <= 1024)
//   chunks <= 4    2 waves per row, 2 rows per block (4 rows at 4 chunks: 2-3 % faster in an
//                  interleaved comparison; at 3 chunks 2 rows are)   (sk <= 2048)
//   chunks <= 8    4 waves per row                                   (sk <= 4096)
//   chunks <= 16   8 waves per row, 512-thread block                 (sk <= 8192)
//   chunks <= 32   16 waves per row, 1024-thread block               (sk <= 16384)
//                  forward, in the lower 3/4 of each of these three ranges (7/8 of the last):
//                  half as many waves with 3 (4) chunks each; causal backward likewise at
//                  8193-12288 columns; mask-tensor forward at 513-2048 columns (unless the call
//                  knows where its rows end) and causal forward at 1025-1408: packed kernel, two
//                  rows of two chunks or one row of three or four chunks per wave
//   chunks <= 64   16 waves per row with 3 or 4 chunks per wave      (sk <= 32768)
//   longer rows    staged in LDS, one 1024-thread block per row: in half of a CU's LDS, two
//                  blocks per CU (sk <= 40448), or in all of it       (sk <= 81408)
//   ragged rows    (sk % 8 != 0 or pointers not 16-byte aligned; 8 <= sk < 81408)
//                  the same packed, one- to sixteen-wave row and LDS-staged kernels with the kRagged flag
//   sliding window (kBand) the one- to sixteen-wave row kernels, aligned rows of 513-32768 columns
//   anything else  element-wise kernels (rows shorter than 8 columns or beyond 81408)
#pragma once

#include <optional>
#include <type_traits>

#include "internal.hpp"

namespace neox {

// EXTRA is the feature set of a translation unit -- any combination of kAlibi, kBias, kDropout and
// kRagged for the forward pass, of kDropout and kRagged for the backward pass, or kBand alone -- and
// every kernel of the unit is compiled for exactly that set: the caller picks the unit by what the
// call brings along (slopes, a bias tensor, a dropout probability, unaligned rows).

// Switches the XCD-aware block -> unit mapping on (see xcd_slot) when the work units of a block
// -- `units` of them, `unit_bytes` each, consecutive in memory -- tile 4 KiB pieces exactly and
// the output starts on a 4 KiB boundary.
static SoftmaxArgs with_xcd_mapping(const SoftmaxArgs& a, uint64_t unit_bytes, uint32_t units, uint32_t blocks) {
    SoftmaxArgs b = a;
    b.units_per_piece = 0;
    b.affine_blocks = 0;
    const bool aligned = (reinterpret_cast<uintptr_t>(a.out) & 4095u) == 0 &&
                         (a.out2 == nullptr || (reinterpret_cast<uintptr_t>(a.out2) & 4095u) == 0);
    if (aligned && unit_bytes > 0 && unit_bytes <= 4096 && 4096 % unit_bytes == 0 && blocks >= 8) {
        const uint32_t upp = (uint32_t)(4096 / unit_bytes);
        if (units % upp == 0 && units / upp >= 1) {
            b.units_per_piece = upp;
            b.affine_blocks = blocks & ~7u;
        }
    }
    return b;
}

template <typename T, Mask M, bool BWD, int EXTRA, int NCH, int WPR, int RPB>
static hipError_t launch_shape(const SoftmaxArgs& a0, hipStream_t st) {
    const dim3 grid((a0.rows + RPB - 1) / RPB);
    const dim3 block(kWave * WPR * RPB);
    const SoftmaxArgs a = with_xcd_mapping(a0, (uint64_t)a0.sk * 2, RPB, grid.x);
    constexpr int FLAGS = kDefaultFlags | EXTRA;
    if constexpr (BWD) {
        hipLaunchKernelGGL((softmax_bwd_kernel<T, NCH, WPR, RPB, M, FLAGS>), grid, block, 0, st, a);
    } else {
        hipLaunchKernelGGL((softmax_fwd_kernel<T, NCH, WPR, RPB, M, FLAGS>), grid, block, 0, st, a);
    }
    return hipGetLastError();
}

template <typename T, Mask M, bool BWD, int EXTRA>
static hipError_t launch_generic(const SoftmaxArgs& a, hipStream_t st) {
    const dim3 grid(a.rows);
    const dim3 block(kGenericThreads);
    if constexpr (BWD) {
        hipLaunchKernelGGL((softmax_bwd_generic_kernel<T, M, EXTRA>), grid, block, 0, st, a);
    } else {
        hipLaunchKernelGGL((softmax_fwd_generic_kernel<T, M, EXTRA>), grid, block, 0, st, a);
    }
    return hipGetLastError();
}

template <typename T, Mask M, bool BWD, int EXTRA, int G, int R, int C>
static hipError_t launch_packed_shape(const SoftmaxArgs& a0, hipStream_t st) {
    const uint32_t per_block = Packed<G, R>::kRowsPerBlock;
    const dim3 grid((a0.rows + per_block - 1) / per_block);
    // the unit is a wave's run of rows: 4 waves per block.  Not for the full-row backward with
    // several chunks per lane group: two loads per store, and the order measured 0-2 % slower there.
    const uint64_t unit_bytes = (BWD && C > 1) ? 0 : (uint64_t)Packed<G, R>::kRowsPerWave * a0.sk * 2;
    const SoftmaxArgs a = with_xcd_mapping(a0, unit_bytes, 4, grid.x);
    constexpr int FLAGS = kDefaultFlags | EXTRA;
    if constexpr (BWD) {
        hipLaunchKernelGGL((softmax_bwd_packed_kernel<T, G, M, FLAGS, R, C>), grid, dim3(256), 0, st, a);
    } else {
        hipLaunchKernelGGL((softmax_fwd_packed_kernel<T, G, M, FLAGS, R, C>), grid, dim3(256), 0, st, a);
    }
    return hipGetLastError();
}

template <typename T, Mask M, bool BWD, int EXTRA, int G>
static hipError_t launch_packed(const SoftmaxArgs& a, hipStream_t st) {
    // passes per wave: 4, except for lane groups of 32 and 64 lanes in the causal kernels and the
    // full-row backward, which run faster with 2 when the rows fill their lane groups (causal forward
    // 15 %, causal backward up to 11 % at 512 columns, full-row backward 0-4 %).  With a quarter or
    // more of the lanes idle (129-192 and 257-384 columns) 4 passes are 4-12 % faster there too.
    constexpr int R = (M != Mask::Bytes && G >= 32) ? 2 : kPackedPasses;
    if constexpr (R != kPackedPasses) {
        const int lanes = (a.sk + kVec - 1) / kVec;
        if (lanes * 4 <= G * 3) return launch_packed_shape<T, M, BWD, EXTRA, G, kPackedPasses, 1>(a, st);
    }
    return launch_packed_shape<T, M, BWD, EXTRA, G, R, 1>(a, st);
}

// sk <= 512: lane groups of G = pow2 >= sk/8 lanes per row
template <typename T, Mask M, bool BWD, int EXTRA>
static hipError_t dispatch_packed(const SoftmaxArgs& a, hipStream_t st) {
    const int lanes = (a.sk + kVec - 1) / kVec;
    if (lanes <= 1) return launch_packed<T, M, BWD, EXTRA, 1>(a, st);
    if (lanes <= 2) return launch_packed<T, M, BWD, EXTRA, 2>(a, st);
    if (lanes <= 4) return launch_packed<T, M, BWD, EXTRA, 4>(a, st);
    if (lanes <= 8) return launch_packed<T, M, BWD, EXTRA, 8>(a, st);
    if (lanes <= 16) return launch_packed<T, M, BWD, EXTRA, 16>(a, st);
    if (lanes <= 32) return launch_packed<T, M, BWD, EXTRA, 32>(a, st);
    return launch_packed<T, M, BWD, EXTRA, 64>(a, st);
}

// sk <= 512.  The packed forward kernels address the mask and the bias tensor through one buffer
// each; a call whose mask or bias tensor is beyond the 32-bit range of a buffer goes to the row
// kernel, which forms a 64-bit address per row.  (The backward pass reads neither.)
template <typename T, Mask M, bool BWD, int EXTRA>
static hipError_t dispatch_short_rows(const SoftmaxArgs& a, hipStream_t st) {
    constexpr bool side_tensor = !BWD && (M == Mask::Bytes || (EXTRA & kBias) != 0);
    if constexpr (side_tensor) {
        const bool fits32 = (M != Mask::Bytes || a.mask_bytes != 0) && (a.bias == nullptr || a.bias_bytes != 0);
        if (!fits32) return launch_shape<T, M, BWD, EXTRA, 1, 1, 4>(a, st);
    }
    return dispatch_packed<T, M, BWD, EXTRA>(a, st);
}

// Rows beyond the register budget, staged in LDS: in half of a CU's LDS when the row fits there,
// two blocks per CU, else in all of it.  Ragged rows need room for one position more.
static_assert(kMaxStagedRow == kMaxLdsRow, "the range the callers check is the range of the kernels");
template <typename T, Mask M, bool BWD, int EXTRA>
static hipError_t launch_lds(const SoftmaxArgs& a, hipStream_t st) {
    const int positions = a.sk + ((EXTRA & kRagged) != 0 ? 1 : 0);
    if (positions > kMaxLdsRow) return hipErrorInvalidValue;  // the caller checks
    const bool half = positions <= kMaxLdsHalfRow;
    const dim3 grid(a.rows), block(kLdsThreads);
    if constexpr (BWD) {
        // ragged rows with dropout need more than the 64 registers per lane that two blocks on a CU
        // leave each: all of the LDS, one block per CU, at any length
        constexpr bool half_fits = EXTRA != (kRagged | kDropout);
        if constexpr (half_fits) {
            if (half) {
                hipLaunchKernelGGL((softmax_bwd_lds_kernel<T, M, 5, kLdsHalf, EXTRA>), grid, block, 0, st, a);
                return hipGetLastError();
            }
        }
        hipLaunchKernelGGL((softmax_bwd_lds_kernel<T, M, 10, kLdsBytes, EXTRA>), grid, block, 0, st, a);
    } else {
        if (half) hipLaunchKernelGGL((softmax_fwd_lds_kernel<T, M, kLdsHalf, EXTRA>), grid, block, 0, st, a);
        else hipLaunchKernelGGL((softmax_fwd_lds_kernel<T, M, kLdsBytes, EXTRA>), grid, block, 0, st, a);
    }
    return hipGetLastError();
}

// The shapes that need 16-byte aligned rows: element-wise kernels when they are not, LDS-staged
// and packed kernels.  No value: none of them applies, the row kernels take the call.
template <typename T, Mask M, bool BWD, int EXTRA>
static std::optional<hipError_t> dispatch_aligned(const SoftmaxArgs& a, bool vec_ok, int chunks, hipStream_t st) {
    if (!vec_ok) return launch_generic<T, M, BWD, EXTRA>(a, st);
    if (a.sk > kMaxRegisterRow) {
        // beyond the register budget: the row is staged in LDS while it fits there
        if (a.sk <= kMaxLdsRow) return launch_lds<T, M, BWD, EXTRA>(a, st);
        return launch_generic<T, M, BWD, EXTRA>(a, st);
    }
    if (chunks == 1) return dispatch_short_rows<T, M, BWD, EXTRA>(a, st);
    if constexpr (!BWD && M == Mask::Bytes) {
        // mask-tensor forward, 513-2048 columns: the packed kernel -- two rows of two chunks, or one row of
        // three or four chunks per wave -- keeps four accesses per tensor in flight and fetches no score of
        // a lane whose keys are all hidden.  Against the row kernels (two waves with four chunk slots from
        // 1025 columns on): -17 % at 520-640 columns, -8 % at 768, -9 % at 1032 and 1152, -5 % at 1280, -1 %
        // at 1536 whatever the mask; at 769-1024 and 1537-2048 columns -5...-19 % under padding and causal
        // masks and +0...3 % under masks that hide nothing or hide at random.  With dropout folded in
        // the steps up to 1536 columns gain 4-11 %.  A call that knows where its rows end
        // (SoftmaxArgs::row_end, which the packed kernels do not look at) takes the row kernel at two
        // chunks, which ends the row there without waiting for the mask bytes and sums in the same order
        // (-16 % at 640 columns, -3...-7 % at 1024 against the packed kernel); at three and four chunks it
        // measured -3...+9 % and would sum in another order, so those stay with the packed kernel.
        const bool fits32 = a.mask_bytes != 0 && (a.bias == nullptr || a.bias_bytes != 0);
        if (fits32) {
            if (chunks == 2 && a.row_end == nullptr) return launch_packed_shape<T, M, BWD, EXTRA, kWave, 2, 2>(a, st);
            if (chunks == 3) return launch_packed_shape<T, M, BWD, EXTRA, kWave, 1, 3>(a, st);
            if (chunks == 4) return launch_packed_shape<T, M, BWD, EXTRA, kWave, 1, 4>(a, st);
        }
    }
    if constexpr (!BWD && M == Mask::Causal) {
        // causal forward, 1025-1408 columns: one row of three chunks per wave instead of two waves with
        // four slots (-11 % at 1032 and 1152 columns, -5 % at 1280, +1 % at 1536).  At two and at four
        // chunks, and in the causal backward at any, the packed kernel measured 2-16 % slower.  The
        // dropout variant follows (it loses 1-8 % here): its undropped output stays bit-equal to the
        // plain kernel's, which needs the same order of summation.
        const bool fits32 = a.bias == nullptr || a.bias_bytes != 0;
        if (chunks == 3 && a.sk <= 1408 && fits32) return launch_packed_shape<T, M, BWD, EXTRA, kWave, 1, 3>(a, st);
    }
    if constexpr (BWD && M == Mask::None) {
        // full rows up to 2048 columns: straight-line packed kernel, R x C = 4 accesses per tensor
        if (chunks == 2) return launch_packed_shape<T, M, BWD, EXTRA, kWave, 2, 2>(a, st);
        if (chunks == 3) return launch_packed_shape<T, M, BWD, EXTRA, kWave, 1, 3>(a, st);
        if (chunks == 4) return launch_packed_shape<T, M, BWD, EXTRA, kWave, 1, 4>(a, st);
    }
    return std::nullopt;
}

template <typename T, Mask M, bool BWD, int EXTRA>
static hipError_t dispatch_rows(const SoftmaxArgs& a, bool vec_ok, hipStream_t st) {
    int chunks = (a.sk + kChunk - 1) / kChunk;
    if constexpr ((EXTRA & kBand) != 0) {
        // sliding-window rows: the row kernels below only (aligned rows of two chunks or more), and the
        // kernel shape goes by the chunks a band can touch -- w + 1 keys lie in at most w / 512 + 2
        // chunks -- not by the row length: the waves hold the band, the rest of the row is zeros
        if (!vec_ok || chunks < 2 || a.sk > kMaxRegisterRow) return hipErrorInvalidValue;  // the caller checks
        const int band_chunks = a.window / kChunk + 2;
        if (band_chunks < chunks) chunks = band_chunks;
    } else if constexpr ((EXTRA & kRagged) != 0) {
        // rows at any alignment: the packed kernels up to 512 columns, the row kernels below beyond
        if (a.sk < kVec || a.sk >= kMaxLdsRow) return hipErrorInvalidValue;  // the caller checks
        if (a.sk >= kMaxRegisterRow) return launch_lds<T, M, BWD, EXTRA>(a, st);
        if (chunks > 1) {
            // rows of odd length: the row kernels lay those that start on an odd element one
            // position later on their lanes
            chunks = (a.sk + (a.sk & 1) + kChunk - 1) / kChunk;
        }
        if (chunks == 1) return dispatch_short_rows<T, M, BWD, EXTRA>(a, st);
    } else {
        if (const auto done = dispatch_aligned<T, M, BWD, EXTRA>(a, vec_ok, chunks, st)) return *done;
    }
    // (the aligned full-row backward has taken 2 to 4 chunks with its packed kernel above)
    if constexpr (!(BWD && M == Mask::None && (EXTRA & kRagged) == 0)) {
        if (chunks == 2) return launch_shape<T, M, BWD, EXTRA, 2, 1, 4>(a, st);
        if (chunks == 3) return launch_shape<T, M, BWD, EXTRA, 2, 2, 2>(a, st);
        if (chunks == 4) {
            // the causal forward with two output streams (dropout) measured 3 % faster with 2 rows
            if constexpr (!BWD && M == Mask::Causal && (EXTRA & kDropout) != 0)
                return launch_shape<T, M, BWD, EXTRA, 2, 2, 2>(a, st);
            return launch_shape<T, M, BWD, EXTRA, 2, 2, 4>(a, st);
        }
    }
    if constexpr (!BWD && (EXTRA & kBand) == 0) {
        // Forward, rows that would leave a quarter or more of the 2-chunk shape's slots empty:
        // half as many waves with 3 or 4 chunks each.  Measured in an interleaved comparison:
        // +20-50 % just above a power of two (2056, 4104, 8200 columns), +4-15 % up to 3/4 (7/8 with
        // 4 chunks) of the range, while full rows lose 2-3 % with 4 chunks per wave and the
        // backward pass gains nothing.
        if (chunks <= 6) return launch_shape<T, M, BWD, EXTRA, 3, 2, 2>(a, st);
        if (chunks > 8 && chunks <= 12) return launch_shape<T, M, BWD, EXTRA, 3, 4, 1>(a, st);
        if (chunks > 16 && chunks <= 24) return launch_shape<T, M, BWD, EXTRA, 3, 8, 1>(a, st);
        if (chunks > 24 && chunks <= 28) return launch_shape<T, M, BWD, EXTRA, 4, 8, 1>(a, st);
    }
    if constexpr (BWD && M == Mask::Causal) {
        // Causal backward just above 8192 columns: 8 waves with 3 chunks each instead of 16 with 2, of
        // which up to half would hold nothing (-13 % at 8200 columns, -8 % at 10240, -4 % at 12288).  The
        // same step at the shorter ranges and for the full-row backward measured -3...+5 %: not taken.
        if (chunks > 16 && chunks <= 24) return launch_shape<T, M, BWD, EXTRA, 3, 8, 1>(a, st);
    }
    if (chunks <= 8) return launch_shape<T, M, BWD, EXTRA, 2, 4, 1>(a, st);
    if (chunks <= 16) return launch_shape<T, M, BWD, EXTRA, 2, 8, 1>(a, st);
    if (chunks <= 32) return launch_shape<T, M, BWD, EXTRA, 2, 16, 1>(a, st);
    if (chunks <= 48) return launch_shape<T, M, BWD, EXTRA, 3, 16, 1>(a, st);
    return launch_shape<T, M, BWD, EXTRA, 4, 16, 1>(a, st);
}

// Sliding-window causal softmax (EXTRA = kBand): causal rows only.
template <bool BWD>
static hipError_t dispatch_band(const SoftmaxArgs& a, int dtype, bool vec_ok, hipStream_t st) {
    return dtype == NEOX_F16 ? dispatch_rows<F16, Mask::Causal, BWD, kBand>(a, vec_ok, st)
                             : dispatch_rows<BF16, Mask::Causal, BWD, kBand>(a, vec_ok, st);
}

template <bool BWD, int EXTRA = 0>
static hipError_t dispatch_softmax(const SoftmaxArgs& a, Mask mask, int dtype, bool vec_ok,
                                   hipStream_t st) {
    const bool f16 = (dtype == NEOX_F16);
    switch (mask) {
        case Mask::Causal:
            return f16 ? dispatch_rows<F16, Mask::Causal, BWD, EXTRA>(a, vec_ok, st)
                       : dispatch_rows<BF16, Mask::Causal, BWD, EXTRA>(a, vec_ok, st);
        case Mask::Bytes:
            if constexpr (!BWD) {
                return f16 ? dispatch_rows<F16, Mask::Bytes, BWD, EXTRA>(a, vec_ok, st)
                           : dispatch_rows<BF16, Mask::Bytes, BWD, EXTRA>(a, vec_ok, st);
            }
            [[fallthrough]];  // the backward pass needs no mask: masked probabilities are 0
        case Mask::None:
            if constexpr (BWD) {
                return f16 ? dispatch_rows<F16, Mask::None, BWD, EXTRA>(a, vec_ok, st)
                           : dispatch_rows<BF16, Mask::None, BWD, EXTRA>(a, vec_ok, st);
            }
            break;
    }
    return hipErrorInvalidValue;
}

}  // namespace neox
