// Scaled masked softmax kernels for gfx950, forward and backward.
//
// Work decomposition: a row of the score matrix is owned by WPR wave64s (1 for rows up
// to 1024 columns, 2 up to 2048, ... 16 beyond 8192).  Each wave keeps its share of the
// row in VGPRs as fp32 -- NCH "chunks" of 512 columns, lane l owning columns 8l..8l+7 of
// a chunk, so every load/store is one 128-bit access per lane and 1 KiB contiguous per
// wave.  With WPR > 1 the chunks of a row are dealt round-robin to its waves (balanced
// under the causal mask) and the row maximum and sum are combined through a few floats
// of LDS.
//
// Causal rows read only the columns j <= i: the row is described to the hardware as a
// buffer of i+1 elements, so lanes past the diagonal fetch nothing, and chunks entirely
// above the diagonal are not computed (wave-uniform branch); the zeros of the upper
// triangle are still stored because the consumer reads the matrix densely.
//
// Arithmetic: fp32, exp(x*scale - max) evaluated as exp2(x*(scale*log2e) - max'),
// one reciprocal per row, one rounding to the storage type on store.
#pragma once

#include <type_traits>

#include "philox.hpp"
#include "wave.hpp"

namespace neox {

struct SoftmaxArgs {
    void* out;            // y (forward) or dx (backward)
    const void* in0;      // x (forward) or dy (backward)
    const void* in1;      // unused (forward) or y (backward)
    const uint8_t* mask;  // masked forward only
    float scale;          // forward: scale*log2(e); backward: scale
    uint32_t rows;        // total number of rows (batches*sq)
    int32_t sq;
    int32_t sk;
    uint32_t rows_per_mask_batch;  // np*sq: rows sharing one mask sample
    int32_t mask_bcast;            // mask batch dim is 1
    uint32_t mask_bytes;           // size of the mask tensor, 0 if it does not fit 32 bits
    const float* slopes;           // ALiBi (kAlibi kernels): one slope per head, fp32 [np]
    uint32_t np;                   // heads per sample (kAlibi kernels)
    void* out2;                    // kDropout forward: the probabilities after dropout
    DropoutArgs drop;              // kDropout kernels
    const void* bias;              // kBias forward: additive bias [1 or b, np, sq, sk], dtype of x
    uint32_t bias_rows;            // np*sq if the bias is shared by all samples, else 0
    uint32_t bias_bytes;           // size of the bias tensor, 0 if it does not fit 32 bits
    // Block -> memory mapping that keeps every XCD on its own 4 KiB pieces (see xcd_slot), filled in
    // by the launchers: work units (rows, or the rows of a wave) per 4 KiB piece, 0 = units in order
    uint32_t units_per_piece;
    uint32_t affine_blocks;        // leading blocks that take part: a multiple of 8
    int32_t window;                // kBand kernels: row i sees the keys max(0, i - window) .. i
    // Mask-tensor forward and full-row backward, optional: per mask row [mask_b * sq], the number of
    // leading keys that can be visible -- the caller's promise that the mask hides every key from
    // there on (backward: that its probability is zero), which a kernel may use or not; 0 = the
    // whole row.  Needs sq, rows_per_mask_batch and mask_bcast.
    const int32_t* row_end;
};

enum class Mask { Causal, Bytes, None };


// Compile-time switches of the kernels (FLAGS): two memory hints and three optional features.
constexpr int kNtLoad = 1;   // non-temporal hint on the streaming loads
constexpr int kNtStore = 2;  // non-temporal hint on the streaming stores
// Forward adds the ALiBi bias slope[head] * min(j - i', 0) to the scores, i' = i + sk - sq the key
// position of query row i (the last row of a decode step sees itself: the reference's AliBi module,
// megatron/model/positional_embeddings.py:210-257, has sq == sk or sq == 1).  Under the causal mask
// only j <= i is evaluated, where the minimum is the difference itself.
constexpr int kAlibi = 4;
// Attention dropout fused in.  Forward: besides y (kept for the backward pass) the kernel
// stores dropout(y) = keep ? round(y)*1/(1-p) : 0 to out2.  Backward: the incoming gradient is
// the gradient of dropout(y); the kernel regenerates the keep pattern and uses
// dy*keep/(1-p) in fp32 where the plain kernel uses dy.
constexpr int kDropout = 8;
// Forward adds a bias tensor to the scores before the scale: softmax(scale * (x + bias)), the sum
// taken in fp32 (the unfused path rounds x + bias to half precision first).
constexpr int kBias = 16;
// Ragged rows: the tensors start at any 2-byte boundary and sk is any number >= 8, so a row
// starts wherever the previous one ends.  128-bit buffer accesses work at any alignment on
// gfx950 and their range check acts per dword: against a buffer of exactly the row's bytes,
// every dword inside the row is transferred and only a dword that crosses the row end is
// dropped.  For 16-bit data that is one element, which these kernels move by a 16-bit access of
// its own; for the mask bytes it is up to three, fetched again by a dword load that ends with the
// row.  Accesses that are not even dword-aligned cost 10-20 % of the bandwidth, though, so a row
// that starts on an odd element is laid over the lanes one element later (sh = 1): lane l of a
// chunk then holds the columns 8l - 1 .. 8l + 6 and all its accesses are dword-aligned; only the
// first lane of the row, whose access would begin in front of the row, takes its seven columns by
// a 16-bit and a 96-bit access.  "Positions" below are columns + sh: the row occupies the
// positions [sh, len + sh).  With kDropout a lane's 8 columns straddle two Philox groups (the
// pattern is a function of the row-major element index).
constexpr int kRagged = 32;
// Sliding-window causal rows (Mask::Causal row kernels only): row i sees the keys lo .. i with
// lo = max(0, i - window) -- the mask megatron/utils.py:67-80 builds for sliding_window_width.  The
// row's buffer starts at the 128-bit access that holds key lo, accesses in front of it are given an
// out-of-range offset, and chunks that lie wholly in front of the band are neither read nor
// computed (wave-uniform branch), like those above the diagonal; their zeros are still stored.
constexpr int kBand = 64;
constexpr int kDefaultFlags = kNtLoad | kNtStore;
constexpr uint32_t kOutOfRange = 0xFFFFFFFFu;  // a byte offset no buffer contains

// kRagged: 1 if the row starts on an odd element (2 mod 4 bytes) of the tensor at `base` and sk is
// odd, so that rows alternate between the two alignments.  (With an even sk every row has the
// alignment of the tensor; moving them all would only cost a chunk.)  Row-uniform.
__device__ __forceinline__ int ragged_shift(const void* base, uint32_t row, int sk) {
    if ((sk & 1) == 0) return 0;
    return (int)(((reinterpret_cast<uintptr_t>(base) >> 1) + row) & 1u);  // row * sk has the parity of row
}
// kRagged: the last element of a row of `len` columns when the dword that holds it crosses the
// row end (len + sh odd), fetched by every lane of the wave in one broadcast access.
__device__ __forceinline__ uint32_t ragged_tail16(rsrc_t r, int len, int sh) {
    return buf_ld16(r, ((len + sh) & 1) ? (uint32_t)(len - 1) * 2u : kOutOfRange);
}
// kRagged: the lane whose 8 positions (from `pos0`) hold the last one, plen - 1, puts `tail`
// where the range check left a zero dword (plen = len + sh, odd).
__device__ __forceinline__ void ragged_patch16(u32x4& raw, int pos0, int plen, uint32_t tail) {
    const int e = plen - 1 - pos0;  // even: plen is odd, pos0 a multiple of 8
    if ((plen & 1) && e >= 0 && e < 8) {
        raw.x = (e == 0) ? tail : raw.x;
        raw.y = (e == 2) ? tail : raw.y;
        raw.z = (e == 4) ? tail : raw.z;
        raw.w = (e == 6) ? tail : raw.w;
    }
}
// kRagged: the last (len + sh) % 4 mask bytes of a row (len >= 4), in the low bytes of the result:
// the bytes of the dword that crosses the row end.
__device__ __forceinline__ uint32_t ragged_tail_mask(rsrc_t rm, int len, int sh) {
    const int n = (len + sh) & 3;
    const uint32_t last4 = buf_ld32(rm, n ? (uint32_t)(len - 4) : kOutOfRange);
    return n ? last4 >> (8 * (4 - n)) : 0u;
}
__device__ __forceinline__ void ragged_patch_mask(u32x2& mk, int pos0, int plen, uint32_t tail) {
    const int e = (plen & ~3) - pos0;  // first dropped byte, relative to the lane's 8 bytes
    if ((plen & 3) && e >= 0 && e < 8) {
        mk.x = (e == 0) ? tail : mk.x;
        mk.y = (e == 4) ? tail : mk.y;
    }
}
// kRagged: 16-bit store of the last element of a row (byte offset `last_off`) from the packed
// vector that holds its position plen - 1, when its dword crosses the row end (plen odd).
__device__ __forceinline__ void ragged_store16(rsrc_t r, const u32x4& o, int pos0, int plen, uint32_t last_off) {
    const int e = plen - 1 - pos0;
    const bool own = (plen & 1) && e >= 0 && e < 8;
    const uint32_t v = (e == 0) ? o.x : (e == 2) ? o.y : (e == 4) ? o.z : o.w;
    buf_st16(r, v, own ? last_off : kOutOfRange);
}
// kRagged, sh = 1: the first lane of a row holds the columns 0 .. 6 in its positions 1 .. 7.
__device__ __forceinline__ u32x4 ragged_head_load(rsrc_t r, bool first_lane) {
    const uint32_t h = buf_ld16(r, first_lane ? 0u : kOutOfRange);
    const u32x3 t = buf_ld96(r, first_lane ? 2u : kOutOfRange);
    return u32x4{h << 16, t.x, t.y, t.z};
}
__device__ __forceinline__ void ragged_head_store(rsrc_t r, const u32x4& o, bool first_lane) {
    buf_st16(r, o.x >> 16, first_lane ? 0u : kOutOfRange);
    buf_st96(r, u32x3{o.y, o.z, o.w}, first_lane ? 2u : kOutOfRange);
}
// kRagged, sh = 1: the first lane's mask bytes for the columns 0 .. 6, in the bytes 1 .. 7.
__device__ __forceinline__ u32x2 ragged_head_mask(rsrc_t rm, bool first_lane) {
    const u32x2 m = buf_ld64(rm, first_lane ? 0u : kOutOfRange, 0);
    return u32x2{m.x << 8, (m.y << 8) | (m.x >> 24)};
}

// ALiBi: distance term of key `j` for the query at key position `ipos`, as a float.  Under the causal
// mask only j <= ipos is ever used.
template <Mask MASK>
__device__ __forceinline__ float alibi_distance(int j, int ipos) {
    return (float)((MASK == Mask::Causal) ? j - ipos : min(j - ipos, 0));
}
// Key position of query row i: the causal kernels align the triangle at the top left (j <= i).
template <Mask MASK>
__device__ __forceinline__ int alibi_row_position(uint32_t i, const SoftmaxArgs& a) {
    return (MASK == Mask::Causal) ? (int)i : (int)i + a.sk - a.sq;
}

// Hidden keys need no score and zero probabilities no gradient.  A lane whose 8 keys are all hidden
// (forward, from the mask bytes) or whose 8 probabilities are all zero (full-row backward) gets an
// out-of-range offset for its other loads: a padding mask that hides the tail of every row, or the
// upper triangle of a causal mask given as a tensor, then costs no traffic for the hidden part.  The
// price is that those loads wait for the mask bytes / the probabilities.  Measured against a build
// without it (NEOX_SKIP_HIDDEN=0), padding and causal masks at 512-8192 columns: the full-row
// backward kernels gain 6-35 % and lose nothing on masks that hide little; the several-rows-per-wave
// forward kernels gain 10-15 % (0-1 % lost on dense masks); the forward row kernels, whose waves meet
// at barriers, lose 3-16 % to the added latency whatever the mask -- they fetch every score.
#ifndef NEOX_SKIP_HIDDEN
#define NEOX_SKIP_HIDDEN 1
#endif
constexpr bool kSkipHidden = NEOX_SKIP_HIDDEN != 0;
// all 8 mask bytes of a lane are non-zero
__device__ __forceinline__ bool all_hidden(const u32x2& mk) {
    const uint32_t zx = (mk.x - 0x01010101u) & ~mk.x & 0x80808080u;  // a bit per zero byte
    const uint32_t zy = (mk.y - 0x01010101u) & ~mk.y & 0x80808080u;
    return (zx | zy) == 0u;
}
// all 8 packed 16-bit values of a lane are +0
__device__ __forceinline__ bool all_zero(const u32x4& w) { return (w.x | w.y | w.z | w.w) == 0u; }

// Row of the bias tensor that belongs to score row `row`
__device__ __forceinline__ uint32_t bias_row(uint32_t row, const SoftmaxArgs& a) {
    return a.bias_rows ? row % a.bias_rows : row;
}

// Philox group (8 consecutive elements) of column `col` (a multiple of 8) of row `row`
__device__ __forceinline__ uint64_t drop_group(uint32_t row, int sk, int col) {
    return (uint64_t)row * (uint32_t)(sk >> 3) + (uint32_t)(col >> 3);
}

// Keep bits of the 8 columns from `col` (a multiple of 8) of row `row`.  Aligned rows: one Philox
// group.  Ragged rows (RAG): the 8 elements straddle two groups unless the row happens to start
// on a group boundary, which is the same for every lane of a wave.
template <bool RAG>
__device__ __forceinline__ uint32_t keep_bits_row8(const DropoutArgs& d, uint32_t row, int sk, int col) {
    if constexpr (!RAG) {
        return keep_bits8(d, drop_group(row, sk, col));
    } else {
        // col may be -1 (the position in front of a row that starts on an odd element)
        const int64_t e = (int64_t)row * sk + col;
        const uint32_t shift = (uint32_t)e & 7u;
        const uint64_t group = (uint64_t)(e >> 3);  // arithmetic shift: -1 for e = -1, whose bits nobody uses
        uint32_t bits = keep_bits8(d, group) >> shift;
        if (shift != 0) bits |= keep_bits8(d, group + 1) << (8u - shift);
        return bits & 0xffu;
    }
}

// Which work unit a block processes.  Workgroups are handed to the 8 XCDs of the chip in turn
// (block b runs on XCD b % 8), and the memory system sustains a write stream best when every XCD
// keeps to its own 4 KiB pieces of the address space, piece index = XCD (mod 8): a plain store
// kernel measured 83 % of the HBM peak with that mapping against 70-75 % when a block stores
// several consecutive pieces or the pieces rotate over the XCDs (loads do not care).  So where the
// units of a block (U of them: rows, or the row groups of its waves) tile 4 KiB pieces exactly,
// `upp` units per piece, the blocks of a group of 8 share the 8 * U units of the group like this:
// block x of the group takes the pieces x, x + 8, x + 16, ... instead of U / upp consecutive ones.
// Returns the unit index for unit l of block b; the identity for the last, incomplete group.
__device__ __forceinline__ uint32_t xcd_slot(uint32_t b, uint32_t l, uint32_t U, const SoftmaxArgs& a) {
    const uint32_t upp = a.units_per_piece;
    if (upp == 0 || b >= a.affine_blocks) return b * U + l;
    const uint32_t g = b >> 3, x = b & 7u;
    const uint32_t j = l / upp, t = l - j * upp;  // piece of the block, unit inside the piece
    return (g * 8u * (U / upp) + j * 8u + x) * upp + t;
}

// Where a wave works: the row, its position i inside its [sq, sk] matrix, the number of
// columns that take part, and whether the result is stored (surplus waves of the last
// block recompute the last row and store nothing, so that every wave of a block reaches
// the barriers).  All fields are wave-uniform.
struct RowPos {
    uint32_t row;
    uint32_t i;
    int len;
    bool store;
};

template <Mask MASK>
__device__ __forceinline__ RowPos locate(uint32_t row, const SoftmaxArgs& a) {
    RowPos p;
    p.store = row < a.rows;
    p.row = p.store ? row : a.rows - 1;
    p.i = p.row % (uint32_t)a.sq;
    p.len = (MASK == Mask::Causal) ? min((int)p.i + 1, a.sk) : a.sk;
    if constexpr (MASK != Mask::Causal) {
        // a row whose tail is known to be hidden ends there, like a causal row on its diagonal: the
        // tail's scores and mask bytes (backward: its probabilities, all zero, and its gradient) are
        // never fetched (one scalar load, the address is row-uniform)
        if (a.row_end != nullptr) {
            const uint32_t mb = a.mask_bcast ? 0u : p.row / a.rows_per_mask_batch;
            const int end = a.row_end[(size_t)mb * a.sq + p.i];
            if (end > 0 && end < a.sk) p.len = end;
        }
    }
    return p;
}

// Combine a per-wave partial across the WPR waves of a row.
template <typename Op, int WPR, int RPB>
__device__ __forceinline__ float row_combine(float v, float* red, int wib, int rib, int lane) {
    if constexpr (WPR == 1) {
        return v;
    } else {
        if (lane == 0) red[wib] = v;
        __syncthreads();
        typename Op::type r = Op::enc(red[rib * WPR]);
#pragma unroll
        for (int w = 1; w < WPR; ++w) r = Op::f(r, Op::enc(red[rib * WPR + w]));
        return Op::dec(r);
    }
}

// kBand: the waves of a row hold the NCH * WPR chunks from the band's first chunk on; the chunks of
// the row in front of those and behind them hold nothing but zeros, which the waves store here,
// dealt round-robin.  `first` = the band's first chunk (wave-uniform).
template <bool NT, int NCH, int WPR>
__device__ __forceinline__ void band_zero_fill(rsrc_t out, int first, int sk, int wir, int lane) {
    const int all = (sk + kChunk - 1) / kChunk;
    for (int g = wir; g < all; g += WPR) {
        if (g < first || g >= first + NCH * WPR) buf_st128<NT>(out, u32x4{0, 0, 0, 0}, g * kChunk * 2 + lane * 16, 0);
    }
}

// ---------------------------------------------------------------------------------
// forward
//
// One launch covers all rows: block b owns rows b*RPB .. b*RPB+RPB-1 and retires when they
// are done; the hardware dispatcher keeps every CU supplied with fresh blocks, which
// measured faster on MI355X than a persistent grid that prefetches its next row.
// Loads and stores are range-checked buffer accesses against the row's valid length:
// lanes past the causal diagonal (or the row end) fetch nothing, and no branch surrounds
// a memory instruction, so the waits are exact.
// ---------------------------------------------------------------------------------
template <typename T, int NCH, int WPR, int RPB, Mask MASK, int FLAGS = kDefaultFlags>
__global__ __launch_bounds__(kWave* WPR* RPB) void softmax_fwd_kernel(SoftmaxArgs a) {
    __shared__ float red_max[WPR * RPB];
    __shared__ float red_sum[WPR * RPB];
    constexpr bool kLdNt = (FLAGS & kNtLoad) != 0, kStNt = (FLAGS & kNtStore) != 0;
    constexpr bool kRag = (FLAGS & kRagged) != 0;
    constexpr bool kBnd = (FLAGS & kBand) != 0;
    static_assert(!kBnd || (MASK == Mask::Causal && (FLAGS & (kRagged | kAlibi | kBias | kDropout)) == 0),
                  "the sliding window comes with the plain causal row kernels only");

    const int lane = threadIdx.x & (kWave - 1);
    const int wib = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);  // wave in block
    const int rib = wib / WPR;                                         // row in block
    const int wir = wib % WPR;                                         // wave in row
    const int sk = a.sk;
    const float ninf = -__builtin_inff();
    // byte offset of the lane inside the row, first chunk of its wave.  Everything goes into
    // the per-lane offset: the hardware's range check does not see the scalar offset operand.
    const RowPos pos = locate<MASK>(xcd_slot(blockIdx.x, rib, RPB, a), a);
    // kRagged: the row lies one position later on the lanes when it starts on an odd element
    int sh = 0;
    if constexpr (kRag) sh = ragged_shift(a.in0, pos.row, sk);
    // kBand: first visible key of the row, and the start of the 128-bit access that holds it.  The
    // waves' chunks are counted from the chunk that holds that key (wch instead of wir), so that a
    // row needs only as many chunk slots as its band is long; see band_zero_fill for the rest.
    int lo = 0;
    if constexpr (kBnd) lo = max((int)pos.i - a.window, 0);
    const int lo8 = lo & ~(kVec - 1);
    const int wch = wir + lo / kChunk;  // the wave's first chunk of the row (wir without a window)
    const int voff = lane * 16 + wch * kChunk * 2 - 2 * sh;
    const bool head = kRag && sh != 0 && wir == 0;  // wave-uniform: this wave holds the row start
    const bool first_lane = head && lane == 0;      // its first access would begin in front of the row
    DropoutArgs drop = a.drop;
    if constexpr ((FLAGS & kDropout) != 0) drop = resolve(drop);
    // ALiBi: scale*(x + slope*(j - i')) = x*scale + slope2*(j - i'), slope2 wave-uniform
    float slope2 = 0.f;
    if constexpr ((FLAGS & kAlibi) != 0) slope2 = a.slopes[(pos.row / (uint32_t)a.sq) % a.np] * a.scale;
    const int ipos = alibi_row_position<MASK>(pos.i, a);
    u32x4 raw[NCH];
    u32x4 rawb[NCH];  // kBias
    u32x2 mk[NCH];
    uint32_t tail_x = 0, tail_b = 0, tail_m = 0;  // kRagged: what the range check drops at the row end
    {
        // ---- issue every load of the row before the first use
        const char* x = static_cast<const char*>(a.in0) + (size_t)pos.row * sk * 2;
        // whole 128-bit accesses up to the valid length; a ragged row ends where the next one begins
        const uint32_t row_bytes = (uint32_t)(kRag ? pos.len : (pos.len + kVec - 1) & ~(kVec - 1)) * 2u;
        const rsrc_t rx = make_rsrc(x, row_bytes);
        if constexpr (MASK == Mask::Bytes) {
            const uint32_t mb = a.mask_bcast ? 0u : pos.row / a.rows_per_mask_batch;
            // (whole 64-bit accesses up to a row end that a hint has moved in front of sk, like the scores)
            const rsrc_t rm = make_rsrc(a.mask + ((size_t)mb * a.sq + pos.i) * sk,
                                        (uint32_t)(kRag ? pos.len : (pos.len + kVec - 1) & ~(kVec - 1)));
#pragma unroll
            for (int c = 0; c < NCH; ++c)
                mk[c] = buf_ld64(rm, (c == 0 && first_lane) ? kOutOfRange : lane * 8 + (wir + c * WPR) * kChunk - sh, 0);
            if constexpr (kRag) {
                tail_m = ragged_tail_mask(rm, pos.len, sh);
                if (head) {
                    const u32x2 hm = ragged_head_mask(rm, first_lane);
                    mk[0].x |= hm.x;
                    mk[0].y |= hm.y;
                }
            }
        }
#pragma unroll
        for (int c = 0; c < NCH; ++c) {
            uint32_t off = (c == 0 && first_lane) ? kOutOfRange : voff + c * WPR * kChunk * 2;
            if constexpr (kBnd) off = ((int)off < lo8 * 2) ? kOutOfRange : off;  // in front of the band: nothing fetched
            raw[c] = buf_ld128<kLdNt>(rx, off, 0);
        }
        if constexpr (kRag) {
            tail_x = ragged_tail16(rx, pos.len, sh);
            if (head) raw[0] |= ragged_head_load(rx, first_lane);
        }
        if constexpr ((FLAGS & kBias) != 0) {
            const rsrc_t rb = make_rsrc(static_cast<const char*>(a.bias) + (size_t)bias_row(pos.row, a) * sk * 2, row_bytes);
#pragma unroll
            for (int c = 0; c < NCH; ++c) {
                const uint32_t off = (c == 0 && first_lane) ? kOutOfRange : voff + c * WPR * kChunk * 2;
                rawb[c] = buf_ld128<false>(rb, off, 0);
            }
            if constexpr (kRag) {
                tail_b = ragged_tail16(rb, pos.len, sh);
                if (head) rawb[0] |= ragged_head_load(rb, first_lane);
            }
        }
    }
    if constexpr (kBnd) {
        // while the loads are in flight: the zeros of the chunks that no wave holds
        const rsrc_t rz = make_rsrc(static_cast<char*>(a.out) + (size_t)pos.row * sk * 2, pos.store ? (uint32_t)sk * 2u : 0u);
        band_zero_fill<kStNt, NCH, WPR>(rz, lo / kChunk, sk, wir, lane);
    }
    {
        const int len = pos.len;
        const int plen = len + sh;  // the row's columns lie at the positions [sh, plen)
        float v[NCH][8];

        // ---- scale, mask, running maximum
        float mx = ninf;
#pragma unroll
        for (int c = 0; c < NCH; ++c) {
            const int c0 = (wch + WPR * c) * kChunk;  // first position of the chunk (wave-uniform)
            if (c0 < plen && (!kBnd || c0 + kChunk > lo)) {
                const int col = c0 + lane * kVec - sh;  // first column of the lane, -1 in front of the row
                if constexpr (kRag) {
                    if (c0 + kChunk >= plen) {  // the chunk that holds the row end
                        ragged_patch16(raw[c], c0 + lane * kVec, plen, tail_x);
                        if constexpr ((FLAGS & kBias) != 0) ragged_patch16(rawb[c], c0 + lane * kVec, plen, tail_b);
                        if constexpr (MASK == Mask::Bytes) ragged_patch_mask(mk[c], c0 + lane * kVec, plen, tail_m);
                    }
                }
                unpack8<T>(raw[c], v[c]);
                if constexpr ((FLAGS & kBias) != 0) {
                    float bv[8];
                    unpack8<T>(rawb[c], bv);
#pragma unroll
                    for (int k = 0; k < 8; ++k) v[c][k] += bv[k];
                }
                // no lane of the wave crosses the row end (or holds the position in front of the row)
                bool plain = (c0 + kChunk <= plen) && !(head && c == 0);
                if constexpr (kBnd) plain = plain && c0 >= lo;
                if constexpr (MASK == Mask::Bytes) {
                    plain = plain && (__builtin_amdgcn_ballot_w64((mk[c].x | mk[c].y) != 0) == 0);
                }
                float bias[8];
#pragma unroll
                for (int k = 0; k < 8; ++k) {
                    bias[k] = 0.f;
                    if constexpr ((FLAGS & kAlibi) != 0) bias[k] = slope2 * alibi_distance<MASK>(col + k, ipos);
                }
                if (plain) {
#pragma unroll
                    for (int k = 0; k < 8; ++k) {
                        v[c][k] = fmaf(v[c][k], a.scale, bias[k]);  // bias 0: the plain product
                        mx = fmaxf(mx, v[c][k]);
                    }
                } else {
#pragma unroll
                    for (int k = 0; k < 8; ++k) {
                        bool keep = (col + k) < len;
                        if constexpr (kRag) keep = keep && (col + k) >= 0;
                        if constexpr (kBnd) keep = keep && (col + k) >= lo;
                        if constexpr (MASK == Mask::Bytes) {
                            const uint32_t w = (k < 4) ? mk[c].x : mk[c].y;
                            keep = keep && (((w >> (8 * (k & 3))) & 0xffu) == 0);
                        }
                        v[c][k] = keep ? fmaf(v[c][k], a.scale, bias[k]) : ninf;
                        mx = fmaxf(mx, v[c][k]);
                    }
                }
            }
        }
        mx = wave_reduce<OpMax>(mx);
        mx = row_combine<OpMax, WPR, RPB>(mx, red_max, wib, rib, lane);

        // ---- exponentials and their sum
        float sum = 0.f;
#pragma unroll
        for (int c = 0; c < NCH; ++c) {
            const int c0 = (wch + WPR * c) * kChunk;
            if (c0 < plen && (!kBnd || c0 + kChunk > lo)) {
#pragma unroll
                for (int k = 0; k < 8; ++k) {
                    v[c][k] = fast_exp2(v[c][k] - mx);
                    sum += v[c][k];
                }
            }
        }
        if constexpr (MASK == Mask::Bytes) {
            // A row whose every key is masked (row-uniform, rare): the unfused path fills all
            // scores with the same value, so the result is uniform over the sk columns.
            if (mx == ninf) {
                sum = 0.f;
#pragma unroll
                for (int c = 0; c < NCH; ++c) {
                    const int col = (wch + WPR * c) * kChunk + lane * kVec - sh;
#pragma unroll
                    for (int k = 0; k < 8; ++k) {
                        v[c][k] = ((col + k) < len && (col + k) >= 0) ? 1.f : 0.f;
                        sum += v[c][k];
                    }
                }
            }
        }
        sum = wave_reduce<OpSum>(sum);
        sum = row_combine<OpSum, WPR, RPB>(sum, red_sum, wib, rib, lane);
        const float inv = 1.0f / sum;

        // ---- normalise and store; chunks above the diagonal store zeros
        char* y = static_cast<char*>(a.out) + (size_t)pos.row * sk * 2;
        const rsrc_t ry = make_rsrc(y, pos.store ? (uint32_t)sk * 2u : 0u);
        rsrc_t ry2 = ry;
        if constexpr ((FLAGS & kDropout) != 0) {
            ry2 = make_rsrc(static_cast<char*>(a.out2) + (size_t)pos.row * sk * 2, pos.store ? (uint32_t)sk * 2u : 0u);
        }
        u32x4 o[NCH];
#pragma unroll
        for (int c = 0; c < NCH; ++c) {
            const int c0 = (wch + WPR * c) * kChunk;
            o[c] = u32x4{0, 0, 0, 0};
            if (c0 < plen && (!kBnd || c0 + kChunk > lo)) {
#pragma unroll
                for (int k = 0; k < 8; ++k) v[c][k] *= inv;
                o[c] = pack8<T>(v[c]);
            }
            buf_st128<kStNt>(ry, o[c], (c == 0 && first_lane) ? kOutOfRange : voff + c * WPR * kChunk * 2, 0);
            if constexpr (kRag) {
                if (c == 0 && head) ragged_head_store(ry, o[c], first_lane);
                if (c0 < sk + sh && c0 + kChunk >= sk + sh)
                    ragged_store16(ry, o[c], c0 + lane * kVec, sk + sh, (uint32_t)(sk - 1) * 2u);
            }
        }
        if constexpr ((FLAGS & kDropout) != 0) {
            // second output after the first: each stream is written in runs of whole rows
#pragma unroll
            for (int c = 0; c < NCH; ++c) {
                const int c0 = (wch + WPR * c) * kChunk;
                u32x4 o2 = u32x4{0, 0, 0, 0};
                if (c0 < plen) {
                    const uint32_t bits = keep_bits_row8<kRag>(drop, pos.row, sk, c0 + lane * kVec - sh);
                    o2 = dropout8<T>(o[c], bits, drop.scale);
                }
                buf_st128<kStNt>(ry2, o2, (c == 0 && first_lane) ? kOutOfRange : voff + c * WPR * kChunk * 2, 0);
                if constexpr (kRag) {
                    if (c == 0 && head) ragged_head_store(ry2, o2, first_lane);
                    if (c0 < sk + sh && c0 + kChunk >= sk + sh)
                        ragged_store16(ry2, o2, c0 + lane * kVec, sk + sh, (uint32_t)(sk - 1) * 2u);
                }
            }
        }
    }
}

// ---------------------------------------------------------------------------------
// backward:  dx = scale * y * (dy - sum_j dy_j*y_j)
// ---------------------------------------------------------------------------------
template <typename T, int NCH, int WPR, int RPB, Mask MASK, int FLAGS = kDefaultFlags>
__global__ __launch_bounds__(kWave* WPR* RPB) void softmax_bwd_kernel(SoftmaxArgs a) {
    __shared__ float red_sum[WPR * RPB];
    constexpr bool kLdNt = (FLAGS & kNtLoad) != 0, kStNt = (FLAGS & kNtStore) != 0;
    constexpr bool kRag = (FLAGS & kRagged) != 0;
    constexpr bool kBnd = (FLAGS & kBand) != 0;
    static_assert(!kBnd || (MASK == Mask::Causal && (FLAGS & (kRagged | kDropout)) == 0),
                  "the sliding window comes with the plain causal row kernels only");

    const int lane = threadIdx.x & (kWave - 1);
    const int wib = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int rib = wib / WPR;
    const int wir = wib % WPR;
    const int sk = a.sk;
    const RowPos pos = locate<MASK>(xcd_slot(blockIdx.x, rib, RPB, a), a);
    // kBand: first visible key of the row, the start of the 128-bit access that holds it, and the
    // wave's first chunk of the row counted from the chunk that holds that key (see the forward kernel)
    int lo = 0;
    if constexpr (kBnd) lo = max((int)pos.i - a.window, 0);
    const int lo8 = lo & ~(kVec - 1);
    const int wch = wir + lo / kChunk;
    // kRagged: the row lies one position later on the lanes when it starts on an odd element; the
    // position in front of it stays zero in both tensors and is never stored
    int sh = 0;
    if constexpr (kRag) sh = ragged_shift(a.in0, pos.row, sk);
    const int voff = lane * 16 + wch * kChunk * 2 - 2 * sh;  // the range check ignores a scalar offset
    const bool head = kRag && sh != 0 && wir == 0;  // wave-uniform: this wave holds the row start
    const bool first_lane = head && lane == 0;      // its first access would begin in front of the row
    DropoutArgs drop = a.drop;
    if constexpr ((FLAGS & kDropout) != 0) drop = resolve(drop);
    u32x4 rg[NCH], rp[NCH];
    uint32_t tail_g = 0, tail_p = 0;  // kRagged: what the range check drops at the row end
    {
        const uint32_t bytes = (uint32_t)(kRag ? pos.len : (pos.len + kVec - 1) & ~(kVec - 1)) * 2u;
        const rsrc_t bg = make_rsrc(static_cast<const char*>(a.in0) + (size_t)pos.row * sk * 2, bytes);
        const rsrc_t by = make_rsrc(static_cast<const char*>(a.in1) + (size_t)pos.row * sk * 2, bytes);
        // full rows (after a mask-tensor forward): the probabilities first, and no gradient for a lane
        // whose 8 probabilities are all zero -- hidden keys
        constexpr bool kSkip = kSkipHidden && MASK == Mask::None && !kRag;
#pragma unroll
        for (int c = 0; c < NCH; ++c) {
            uint32_t off = (c == 0 && first_lane) ? kOutOfRange : voff + c * WPR * kChunk * 2;
            if constexpr (kBnd) off = ((int)off < lo8 * 2) ? kOutOfRange : off;  // in front of the band: nothing fetched
            rp[c] = buf_ld128<kLdNt>(by, off, 0);
            if constexpr (!kSkip) rg[c] = buf_ld128<kLdNt>(bg, off, 0);
        }
        if constexpr (kSkip) {
#pragma unroll
            for (int c = 0; c < NCH; ++c)
                rg[c] = buf_ld128<kLdNt>(bg, all_zero(rp[c]) ? kOutOfRange : voff + c * WPR * kChunk * 2, 0);
        }
        if constexpr (kRag) {
            tail_g = ragged_tail16(bg, pos.len, sh);
            tail_p = ragged_tail16(by, pos.len, sh);
            if (head) {
                rg[0] |= ragged_head_load(bg, first_lane);
                rp[0] |= ragged_head_load(by, first_lane);
            }
        }
    }
    if constexpr (kBnd) {
        // the zeros of the chunks that no wave holds.  dx may alias dy: those chunks lie outside the
        // band, where nothing is read
        const rsrc_t rz = make_rsrc(static_cast<char*>(a.out) + (size_t)pos.row * sk * 2, pos.store ? (uint32_t)sk * 2u : 0u);
        band_zero_fill<kStNt, NCH, WPR>(rz, lo / kChunk, sk, wir, lane);
    }
    {
        // dx may alias dy: a row is read and written by the same waves only, reads first
        const int len = pos.len;
        const int plen = len + sh;  // the row's columns lie at the positions [sh, plen)

        // the row stays packed; it is unpacked once for the dot product and once for dx
        float dot = 0.f;
        uint32_t kb[NCH];  // keep bits of the lane's 8 columns per chunk (kDropout)
#pragma unroll
        for (int c = 0; c < NCH; ++c) {
            const int c0 = (wch + WPR * c) * kChunk;
            kb[c] = 0xffu;
            if (c0 < plen && (!kBnd || c0 + kChunk > lo)) {
                const int col = c0 + lane * kVec - sh;  // first column of the lane
                if constexpr (kRag) {
                    if (c0 + kChunk >= plen) {  // the chunk that holds the row end
                        ragged_patch16(rg[c], c0 + lane * kVec, plen, tail_g);
                        ragged_patch16(rp[c], c0 + lane * kVec, plen, tail_p);
                    }
                }
                float gv[8], pv[8];
                unpack8<T>(rg[c], gv);
                unpack8<T>(rp[c], pv);
                if constexpr ((FLAGS & kDropout) != 0) {
                    kb[c] = keep_bits_row8<kRag>(drop, pos.row, sk, col);
#pragma unroll
                    for (int k = 0; k < 8; ++k) gv[k] = ((kb[c] >> k) & 1u) ? gv[k] * drop.scale : 0.f;
                }
                if (c0 + kChunk > plen) {
                    // the lane holding the diagonal may have loaded columns past it
#pragma unroll
                    for (int k = 0; k < 8; ++k)
                        if ((col + k) >= len) gv[k] = pv[k] = 0.f;
                }
                if constexpr (kBnd) {
                    if (c0 < lo) {  // the lane holding the first visible key has loaded the columns in front of it
#pragma unroll
                        for (int k = 0; k < 8; ++k)
                            if ((col + k) < lo) gv[k] = pv[k] = 0.f;
                    }
                }
#pragma unroll
                for (int k = 0; k < 8; ++k) dot = fmaf(gv[k], pv[k], dot);
            }
        }
        dot = wave_reduce<OpSum>(dot);
        dot = row_combine<OpSum, WPR, RPB>(dot, red_sum, wib, rib, lane);

        char* dx = static_cast<char*>(a.out) + (size_t)pos.row * sk * 2;
        const rsrc_t rdx = make_rsrc(dx, pos.store ? (uint32_t)sk * 2u : 0u);
#pragma unroll
        for (int c = 0; c < NCH; ++c) {
            const int c0 = (wch + WPR * c) * kChunk;
            u32x4 o = u32x4{0, 0, 0, 0};
            if (c0 < plen && (!kBnd || c0 + kChunk > lo)) {
                float gv[8], pv[8];
                unpack8<T>(rg[c], gv);
                unpack8<T>(rp[c], pv);
                const int col = c0 + lane * kVec - sh;
#pragma unroll
                for (int k = 0; k < 8; ++k) {
                    if constexpr ((FLAGS & kDropout) != 0) gv[k] = ((kb[c] >> k) & 1u) ? gv[k] * drop.scale : 0.f;
                    gv[k] = a.scale * (pv[k] * (gv[k] - dot));
                    if ((c0 + kChunk > plen) && (col + k) >= len) gv[k] = 0.f;
                    if constexpr (kBnd) {
                        if (c0 < lo && (col + k) < lo) gv[k] = 0.f;
                    }
                }
                o = pack8<T>(gv);
            }
            buf_st128<kStNt>(rdx, o, (c == 0 && first_lane) ? kOutOfRange : voff + c * WPR * kChunk * 2, 0);
            if constexpr (kRag) {
                if (c == 0 && head) ragged_head_store(rdx, o, first_lane);
                if (c0 < sk + sh && c0 + kChunk >= sk + sh)
                    ragged_store16(rdx, o, c0 + lane * kVec, sk + sh, (uint32_t)(sk - 1) * 2u);
            }
        }
    }
}

// ---------------------------------------------------------------------------------
// Packed kernels: several rows per wave, no LDS, no barriers.
//
// Short rows (sk <= 512): a row is owned by an aligned group of G consecutive lanes
// (G = 64 for sk in (256, 512], 32 for (128, 256], ... 1 for sk = 8), each lane holding
// 8 columns; a wave covers 64/G rows per pass and makes R passes, so it always has a
// few KiB in flight however short the rows are (one row per wave caps out at ~3.6 G
// rows/s).  With G = 64 a lane may also hold C chunks of 512 columns of its row, which
// covers full-row (mask-free) work on rows up to 2048 columns with straight-line code:
// R x C = 4 accesses per tensor in flight per wave measured best (83 % of peak on the
// backward pass against 80 % for the one-row-per-wave kernel).
// Rows of a wave are consecutive in memory; its loads and stores go through one buffer
// resource spanning just those rows, with out-of-range offsets for the lanes that have
// nothing to fetch.  Reductions stay inside the lane group.
// ---------------------------------------------------------------------------------
constexpr int kPackedPasses = 4;  // default number of passes R

// (i0 + lr) mod sq for lr below the rows of a wave: one conditional subtraction when a
// matrix has at least that many rows, a division only for tiny matrices.
__device__ __forceinline__ uint32_t wrap_row(uint32_t i, uint32_t sq) {
    if (sq >= 256u) return i >= sq ? i - sq : i;  // wave-uniform branch; rows per wave <= 256
    return i % sq;
}

// kRagged in the packed kernels.  A wave's rows lie back to back behind one buffer, so the lane
// that holds the end of a row -- rem = sk % 8 columns of it -- must not touch the columns that
// follow: they belong to the next row.  That lane moves its access back by 8 - rem columns
// instead (`back`), so that it ends with the row: it then holds the last 8 columns of the row,
// of which the first 8 - rem are also held by the lane before it.  Both lanes compute the same
// values for those columns from the same inputs and store the same bits; only the row's sums
// count them once (the lane that is moved back leaves its first `back` columns out).  Every
// lane so makes exactly one 128-bit access per tensor, at a 2-byte alignment.
//
// 128-bit access of the packed kernels: nothing for an inactive lane.  `off`: byte offset of the
// lane's first column.
template <bool NT>
__device__ __forceinline__ u32x4 packed_ld(rsrc_t r, uint32_t off, bool active) {
    return buf_ld128<NT>(r, active ? off : kOutOfRange, 0);
}
template <bool NT>
__device__ __forceinline__ void packed_st(rsrc_t r, const u32x4& v, uint32_t off, bool active) {
    buf_st128<NT>(r, v, active ? off : kOutOfRange, 0);
}
// The lane's 8 mask bytes, likewise.
__device__ __forceinline__ u32x2 packed_ld_mask(rsrc_t r, uint32_t off, bool active) {
    return buf_ld64(r, active ? off : kOutOfRange, 0);
}
// Columns by which the lane that holds a ragged row end is moved back (0 for every other lane).
template <bool RAG>
__device__ __forceinline__ int ragged_back(int col0, int sk) {
    if constexpr (!RAG) return 0;
    const int rem = sk & (kVec - 1);
    return (rem != 0 && col0 < sk && col0 + kVec > sk) ? kVec - rem : 0;
}

template <int G, int R = kPackedPasses>
struct Packed {
    static constexpr int kRowsPerPass = kWave / G;
    static constexpr int kRowsPerWave = kRowsPerPass * R;
    static constexpr int kRowsPerBlock = kRowsPerWave * 4;  // 256-thread blocks
};

template <typename T, int G, Mask MASK, int FLAGS = kDefaultFlags, int R = kPackedPasses, int C = 1>
__global__ __launch_bounds__(256) void softmax_fwd_packed_kernel(SoftmaxArgs a) {
    static_assert(C == 1 || G == kWave, "several chunks per row need a whole wave per row");
    constexpr int RPP = Packed<G, R>::kRowsPerPass, RPW = Packed<G, R>::kRowsPerWave;
    constexpr bool kLdNt = (FLAGS & kNtLoad) != 0, kStNt = (FLAGS & kNtStore) != 0;
    constexpr bool kRag = (FLAGS & kRagged) != 0;
    static_assert(!kRag || C == 1, "ragged rows: one chunk per lane group");
    const int lane = threadIdx.x & (kWave - 1);
    const uint32_t wave = xcd_slot(blockIdx.x, __builtin_amdgcn_readfirstlane(threadIdx.x >> 6), 4, a);
    const uint32_t row0 = wave * RPW;  // first row of this wave
    if (row0 >= a.rows) return;
    const uint32_t rows_here = min((uint32_t)RPW, a.rows - row0);
    const int sk = a.sk;
    const int grp = lane / G;
    const int back = ragged_back<kRag>((lane % G) * kVec, sk);  // kRagged: see ragged_back
    const int col0 = (lane % G) * kVec - back;                  // first column of the lane's accesses
    DropoutArgs drop = a.drop;
    if constexpr ((FLAGS & kDropout) != 0) drop = resolve(drop);
    const float ninf = -__builtin_inff();

    const rsrc_t rx = make_rsrc(static_cast<const char*>(a.in0) + (size_t)row0 * sk * 2, rows_here * sk * 2);
    const rsrc_t ry = make_rsrc(static_cast<char*>(a.out) + (size_t)row0 * sk * 2, rows_here * sk * 2);
    const rsrc_t rm = make_rsrc(a.mask, a.mask_bytes);
    rsrc_t ry2 = ry;
    if constexpr ((FLAGS & kDropout) != 0) {
        ry2 = make_rsrc(static_cast<char*>(a.out2) + (size_t)row0 * sk * 2, rows_here * sk * 2);
    }
    const rsrc_t rb = make_rsrc(a.bias, a.bias_bytes);  // kBias: the whole bias tensor

    u32x4 raw[R][C];
    u32x4 rawb[R][C];
    u32x2 mk[R][C];
    int len[R];
    int ipos[R];       // row position inside its matrix (ALiBi)
    float slope2[R];   // slope[head] * scale of the lane's row (ALiBi)
    const uint32_t i0 = row0 % (uint32_t)a.sq;  // wave-uniform
#pragma unroll
    for (int p = 0; p < R; ++p) {
        const uint32_t lr = p * RPP + grp;  // row of this lane group inside the wave
        const uint32_t row = row0 + lr;
        const uint32_t i = wrap_row(i0 + lr, (uint32_t)a.sq);
        len[p] = (MASK == Mask::Causal) ? min((int)i + 1, sk) : sk;
        if (lr >= rows_here) len[p] = 0;
        ipos[p] = alibi_row_position<MASK>(i, a);
        slope2[p] = 0.f;
        if constexpr ((FLAGS & kAlibi) != 0) {
            const uint32_t safe_row = lr < rows_here ? row : row0;
            slope2[p] = a.slopes[(safe_row / (uint32_t)a.sq) % a.np] * a.scale;
        }
        if constexpr (MASK == Mask::Bytes) {
#pragma unroll
            for (int c = 0; c < C; ++c) {
                const int col = col0 + c * kChunk;
                const uint32_t mb = a.mask_bcast ? 0u : row / a.rows_per_mask_batch;
                const uint32_t moff = (mb * (uint32_t)a.sq + i) * sk + col;
                mk[p][c] = packed_ld_mask(rm, moff, col < len[p]);
            }
        }
    }
    // the scores (and the bias) after the mask bytes: a lane whose 8 keys are all hidden fetches neither
#pragma unroll
    for (int p = 0; p < R; ++p) {
        const uint32_t lr = p * RPP + grp;
#pragma unroll
        for (int c = 0; c < C; ++c) {
            const int col = col0 + c * kChunk;
            bool active = col < len[p];
            // (SoftmaxArgs::row_end is not looked at here: it spared nothing more and cost a load per row)
            if constexpr (MASK == Mask::Bytes && kSkipHidden && !kRag) active = active && !all_hidden(mk[p][c]);
            raw[p][c] = packed_ld<kLdNt>(rx, (lr * sk + col) * 2u, active);
            if constexpr ((FLAGS & kBias) != 0) {
                const uint32_t boff = (bias_row(row0 + lr, a) * (uint32_t)sk + col) * 2u;
                rawb[p][c] = packed_ld<false>(rb, boff, active);
            }
        }
    }

#pragma unroll
    for (int p = 0; p < R; ++p) {
        float v[C][8];
        float mx = ninf;
#pragma unroll
        for (int c = 0; c < C; ++c) {
            const int col = col0 + c * kChunk;
            unpack8<T>(raw[p][c], v[c]);
            if constexpr ((FLAGS & kBias) != 0) {
                float bv[8];
                unpack8<T>(rawb[p][c], bv);
#pragma unroll
                for (int k = 0; k < 8; ++k) v[c][k] += bv[k];
            }
#pragma unroll
            for (int k = 0; k < 8; ++k) {
                bool keep = (col + k) < len[p];
                if constexpr (MASK == Mask::Bytes) {
                    const uint32_t w = (k < 4) ? mk[p][c].x : mk[p][c].y;
                    keep = keep && (((w >> (8 * (k & 3))) & 0xffu) == 0);
                }
                float bias = 0.f;
                if constexpr ((FLAGS & kAlibi) != 0) bias = slope2[p] * alibi_distance<MASK>(col + k, ipos[p]);
                v[c][k] = keep ? fmaf(v[c][k], a.scale, bias) : ninf;
                mx = fmaxf(mx, v[c][k]);
            }
        }
        mx = group_reduce<OpMax, G>(mx);
        float sum = 0.f;
#pragma unroll
        for (int c = 0; c < C; ++c)
#pragma unroll
            for (int k = 0; k < 8; ++k) {
                v[c][k] = fast_exp2(v[c][k] - mx);
                sum += (kRag && k < back) ? 0.f : v[c][k];  // columns the lane before counts
            }
        if constexpr (MASK == Mask::Bytes) {
            // rows with every key hidden (rare): uniform over the sk columns
            const bool all_masked = (mx == ninf) && len[p] > 0;
            if (__builtin_amdgcn_ballot_w64(all_masked) != 0) {
                if (all_masked) {
                    sum = 0.f;
#pragma unroll
                    for (int c = 0; c < C; ++c)
#pragma unroll
                        for (int k = 0; k < 8; ++k) {
                            v[c][k] = ((col0 + c * kChunk + k) < len[p]) ? 1.f : 0.f;
                            sum += (kRag && k < back) ? 0.f : v[c][k];
                        }
                }
            }
        }
        sum = group_reduce<OpSum, G>(sum);
        const float inv = 1.0f / sum;
        const uint32_t lr = p * RPP + grp;
#pragma unroll
        for (int c = 0; c < C; ++c) {
            const int col = col0 + c * kChunk;
#pragma unroll
            for (int k = 0; k < 8; ++k) v[c][k] *= inv;  // lanes of absent rows hold NaN and store nothing
            const bool st = lr < rows_here && col < sk;
            const u32x4 o = pack8<T>(v[c]);
            packed_st<kStNt>(ry, o, (lr * sk + col) * 2u, st);
            if constexpr ((FLAGS & kDropout) != 0) {
                const uint32_t bits = keep_bits_row8<kRag>(drop, row0 + lr, sk, col);
                packed_st<kStNt>(ry2, dropout8<T>(o, bits, drop.scale), (lr * sk + col) * 2u, st);
            }
        }
    }
}

template <typename T, int G, Mask MASK, int FLAGS = kDefaultFlags, int R = kPackedPasses, int C = 1>
__global__ __launch_bounds__(256) void softmax_bwd_packed_kernel(SoftmaxArgs a) {
    static_assert(C == 1 || G == kWave, "several chunks per row need a whole wave per row");
    constexpr int RPP = Packed<G, R>::kRowsPerPass, RPW = Packed<G, R>::kRowsPerWave;
    constexpr bool kLdNt = (FLAGS & kNtLoad) != 0, kStNt = (FLAGS & kNtStore) != 0;
    constexpr bool kRag = (FLAGS & kRagged) != 0;
    static_assert(!kRag || C == 1, "ragged rows: one chunk per lane group");
    const int lane = threadIdx.x & (kWave - 1);
    const uint32_t wave = xcd_slot(blockIdx.x, __builtin_amdgcn_readfirstlane(threadIdx.x >> 6), 4, a);
    const uint32_t row0 = wave * RPW;
    if (row0 >= a.rows) return;
    const uint32_t rows_here = min((uint32_t)RPW, a.rows - row0);
    const int sk = a.sk;
    const int grp = lane / G;
    const int back = ragged_back<kRag>((lane % G) * kVec, sk);  // kRagged: see ragged_back
    const int col0 = (lane % G) * kVec - back;                  // first column of the lane's accesses
    DropoutArgs drop = a.drop;
    if constexpr ((FLAGS & kDropout) != 0) drop = resolve(drop);

    const rsrc_t bg = make_rsrc(static_cast<const char*>(a.in0) + (size_t)row0 * sk * 2, rows_here * sk * 2);
    const rsrc_t by = make_rsrc(static_cast<const char*>(a.in1) + (size_t)row0 * sk * 2, rows_here * sk * 2);
    const rsrc_t bo = make_rsrc(static_cast<char*>(a.out) + (size_t)row0 * sk * 2, rows_here * sk * 2);

    u32x4 rg[R][C], rp[R][C];
    int len[R];
    constexpr bool kSkip = kSkipHidden && MASK == Mask::None && !kRag;
    const bool hinted = MASK == Mask::None && a.row_end != nullptr;  // uniform over the launch
    const uint32_t i0 = row0 % (uint32_t)a.sq;  // wave-uniform
#pragma unroll
    for (int p = 0; p < R; ++p) {
        const uint32_t lr = p * RPP + grp;
        const uint32_t i = wrap_row(i0 + lr, (uint32_t)a.sq);
        len[p] = (MASK == Mask::Causal) ? min((int)i + 1, sk) : sk;
        if (lr >= rows_here) len[p] = 0;
        if constexpr (MASK == Mask::None) {
            // the row is known to end early (see SoftmaxArgs::row_end): neither tensor is fetched behind that
            if (hinted && lr < rows_here) {
                const uint32_t row = row0 + lr;
                const uint32_t mb = a.mask_bcast ? 0u : row / a.rows_per_mask_batch;
                const int end = a.row_end[(size_t)mb * a.sq + i];
                if (end > 0 && end < sk) len[p] = end;
            }
        }
#pragma unroll
        for (int c = 0; c < C; ++c) {
            const int col = col0 + c * kChunk;
            rp[p][c] = packed_ld<kLdNt>(by, (lr * sk + col) * 2u, col < len[p]);
            if constexpr (!kSkip) rg[p][c] = packed_ld<kLdNt>(bg, (lr * sk + col) * 2u, col < len[p]);
            else if (hinted) rg[p][c] = packed_ld<kLdNt>(bg, (lr * sk + col) * 2u, col < len[p]);
        }
    }
    if (kSkip && !hinted) {
        // full rows (after a mask-tensor forward): no gradient for a lane whose 8 probabilities are all
        // zero -- unless the rows' ends are known, which spares both tensors without making one load
        // wait for the other
#pragma unroll
        for (int p = 0; p < R; ++p) {
            const uint32_t lr = p * RPP + grp;
#pragma unroll
            for (int c = 0; c < C; ++c) {
                const int col = col0 + c * kChunk;
                rg[p][c] = packed_ld<kLdNt>(bg, (lr * sk + col) * 2u, col < len[p] && !all_zero(rp[p][c]));
            }
        }
    }
#pragma unroll
    for (int p = 0; p < R; ++p) {
        // the row stays packed; it is unpacked once for the dot product and once for dx
        float dot = 0.f;
        uint32_t kb[C];  // keep bits of the lane's 8 columns per chunk (kDropout)
        const uint32_t lr = p * RPP + grp;
#pragma unroll
        for (int c = 0; c < C; ++c) {
            float gv[8], pv[8];
            unpack8<T>(rg[p][c], gv);
            unpack8<T>(rp[p][c], pv);
            kb[c] = 0xffu;
            if constexpr ((FLAGS & kDropout) != 0) kb[c] = keep_bits_row8<kRag>(drop, row0 + lr, sk, col0 + c * kChunk);
#pragma unroll
            for (int k = 0; k < 8; ++k) {
                if constexpr ((FLAGS & kDropout) != 0) gv[k] = ((kb[c] >> k) & 1u) ? gv[k] * drop.scale : 0.f;
                if ((col0 + c * kChunk + k) >= len[p]) gv[k] = pv[k] = 0.f;  // past the diagonal / row end
                if (kRag && k < back) gv[k] = 0.f;  // columns the lane before counts
                dot = fmaf(gv[k], pv[k], dot);
            }
        }
        dot = group_reduce<OpSum, G>(dot);
#pragma unroll
        for (int c = 0; c < C; ++c) {
            const int col = col0 + c * kChunk;
            float gv[8], pv[8];
            unpack8<T>(rg[p][c], gv);
            unpack8<T>(rp[p][c], pv);
#pragma unroll
            for (int k = 0; k < 8; ++k) {
                if constexpr ((FLAGS & kDropout) != 0) gv[k] = ((kb[c] >> k) & 1u) ? gv[k] * drop.scale : 0.f;
                gv[k] = a.scale * (pv[k] * (gv[k] - dot));
                if ((col + k) >= len[p]) gv[k] = 0.f;
            }
            const bool st = lr < rows_here && col < sk;
            packed_st<kStNt>(bo, pack8<T>(gv), (lr * sk + col) * 2u, st);
        }
    }
}

// ---------------------------------------------------------------------------------
// LDS-staged kernels: rows beyond the register budget (sk > 32768).
//
// One 1024-thread block per row.  The row is read from HBM once and the later passes run
// from LDS, where it is kept as raw 16-bit values: a gfx950 workgroup may use the whole
// 160 KiB of its CU, which holds 81408 columns.  Rows of at most 40448 columns take half of
// it, so that two blocks share a CU and one loads while the other stores.  The forward pass
// stages the scores, with masked and out-of-row elements replaced by -inf, which the later
// passes recognise and turn into exact zeros without looking at the mask again.  The
// backward pass stages the probabilities and keeps the gradient packed in registers.  Each
// wave stages and re-reads its own chunks only, so the only barriers are those of the
// reductions.
//
// Features (FLAGS): the ALiBi term is a function of the column and is formed again in every
// pass; a bias tensor is not staged -- the staging area holds one 16-bit value per column --
// but read again by the second pass, from the caches when the row is still there;
// dropout regenerates its keep bits where they are used.  Ragged rows (kRagged) are staged by
// position, columns + sh, like the row kernels lay them over their lanes, with the same
// fix-ups at the two ends of the row; the staging area then needs room for sk + 1 values.
// ---------------------------------------------------------------------------------
constexpr int kLdsWaves = 16;
constexpr int kLdsThreads = kLdsWaves * kWave;
constexpr int kLdsBytes = 159 * 1024;        // one block per CU; the last KiB of the CU's 160 is left to the reductions
constexpr int kLdsHalf = 79 * 1024;          // two blocks per CU
constexpr int kMaxLdsRow = kLdsBytes / 2;    // 81408 columns (159 chunks)
constexpr int kMaxLdsHalfRow = kLdsHalf / 2; // 40448 columns (79 chunks)
constexpr int kLdsUnroll = 4;                // chunks of a wave whose loads are in flight together
// Forward: a chunk whose keys are all hidden is staged and stored without per-element work.
#ifndef NEOX_LDS_BLANK_CHUNKS
#define NEOX_LDS_BLANK_CHUNKS 1
#endif
constexpr bool kLdsBlankChunks = NEOX_LDS_BLANK_CHUNKS != 0;

// Waves per SIMD a kernel with a staging area of `bytes` is compiled for: the register budget
// that lets as many blocks share a CU as its LDS allows.
constexpr int lds_waves_per_simd(int bytes) { return (bytes <= kLdsHalf ? 2 : 1) * kLdsWaves / 4; }

template <typename T>
struct NegInf16;  // -inf of the storage type, as bits
template <>
struct NegInf16<F16> { static constexpr uint32_t bits = 0xFC00u; };
template <>
struct NegInf16<BF16> { static constexpr uint32_t bits = 0xFF80u; };

// Replaces the elements whose keep bit is clear by -inf (8 packed elements, bit k = element k).
template <typename T>
__device__ __forceinline__ u32x4 stage_masked(const u32x4& raw, uint32_t keep) {
    constexpr uint32_t ninf = NegInf16<T>::bits;
    const uint32_t w[4] = {raw.x, raw.y, raw.z, raw.w};
    uint32_t o[4];
#pragma unroll
    for (int k = 0; k < 4; ++k) {
        const uint32_t lo = ((keep >> (2 * k)) & 1u) ? (w[k] & 0xffffu) : ninf;
        const uint32_t hi = ((keep >> (2 * k + 1)) & 1u) ? (w[k] & 0xffff0000u) : (ninf << 16);
        o[k] = lo | hi;
    }
    return u32x4{o[0], o[1], o[2], o[3]};
}

// What the LDS-staged kernels share: where the block's row lies and how its two ends are handled.
// Chunk c of the row holds the positions c * 512 .. c * 512 + 511, position = column + sh.
struct LdsRow {
    int lane, wib;     // lane of the wave, wave of the block
    int sh;            // kRagged: 1 if the row lies one position later (it starts on an odd element)
    int plen;          // the row's columns that take part lie at the positions [sh, plen)
    bool head;         // wave-uniform: sh != 0 and this wave holds chunk 0
    bool first_lane;   // the lane whose access to chunk 0 would begin in front of the row

    // byte offset of the lane's 128-bit access to chunk c of a 16-bit row, of its 64-bit access to the mask bytes
    __device__ __forceinline__ uint32_t off16(int c) const {
        return (c == 0 && first_lane) ? kOutOfRange : (uint32_t)(c * kChunk * 2 + lane * 16 - 2 * sh);
    }
    __device__ __forceinline__ uint32_t off8(int c) const {
        return (c == 0 && first_lane) ? kOutOfRange : (uint32_t)(c * kChunk + lane * kVec - sh);
    }
    __device__ __forceinline__ int pos0(int c) const { return c * kChunk + lane * kVec; }  // the lane's first position
    // kRagged: what a 128-bit load of chunk c could not fetch -- the columns 0 .. 6 of a row that
    // lies one position later, and the last element when its dword crosses the row end
    __device__ __forceinline__ void fix16(u32x4& raw, int c, rsrc_t r, uint32_t tail) const {
        if (head && c == 0) raw |= ragged_head_load(r, first_lane);
        if ((c + 1) * kChunk >= plen) ragged_patch16(raw, pos0(c), plen, tail);
    }
    // 128-bit store of chunk c of an output row of sk columns, with the same two fix-ups
    template <bool RAG>
    __device__ __forceinline__ void store(rsrc_t r, const u32x4& o, int c, int sk) const {
        buf_st128<true>(r, o, off16(c), 0);
        if constexpr (RAG) {
            if (c == 0 && head) ragged_head_store(r, o, first_lane);
            if (c * kChunk < sk + sh && (c + 1) * kChunk >= sk + sh)
                ragged_store16(r, o, pos0(c), sk + sh, (uint32_t)(sk - 1) * 2u);
        }
    }
};

template <bool RAG>
__device__ __forceinline__ LdsRow lds_row(const void* base, const RowPos& pos, int sk) {
    LdsRow r;
    r.lane = threadIdx.x & (kWave - 1);
    r.wib = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    r.sh = 0;
    if constexpr (RAG) r.sh = ragged_shift(base, pos.row, sk);
    r.plen = pos.len + r.sh;
    r.head = RAG && r.sh != 0 && r.wib == 0;
    r.first_lane = r.head && r.lane == 0;
    return r;
}

// BYTES: size of the staging area, at least 2 * sk (2 * (sk + 1) with kRagged).
template <typename T, Mask MASK, int BYTES, int FLAGS = 0>
__global__ __launch_bounds__(kLdsThreads, lds_waves_per_simd(BYTES)) void softmax_fwd_lds_kernel(SoftmaxArgs a) {
    constexpr bool kRag = (FLAGS & kRagged) != 0, kAli = (FLAGS & kAlibi) != 0;
    constexpr bool kBia = (FLAGS & kBias) != 0, kDrp = (FLAGS & kDropout) != 0;
    static_assert((FLAGS & ~(kRagged | kAlibi | kBias | kDropout)) == 0, "features only: the memory hints are fixed here");
    // chunks of a wave whose loads are in flight together, by the registers they take: a block that
    // has a CU to itself has 128 per lane, two that share one have 64 each -- enough for the 5 chunks
    // a wave holds of the rows staged in half of the LDS, unless mask bytes, the ALiBi term or the
    // fix-ups of ragged rows need some too --, and a bias tensor doubles the registers per chunk
    constexpr bool kMsk = MASK == Mask::Bytes;
    constexpr int kHalfUn = kBia ? (kRag && kAli ? 1 : 2) : kRag ? (kMsk || kAli ? 3 : 4) : kMsk ? (kAli ? 3 : 4) : 5;
    constexpr int UN = BYTES <= kLdsHalf ? kHalfUn : (kBia ? 4 : 8);
    constexpr int UB = kBia ? UN : 1;  // the same for the pass that fetches nothing but the bias
    __shared__ __align__(16) char staged[BYTES];
    __shared__ float red_max[kLdsWaves];
    __shared__ float red_sum[kLdsWaves];
    const int sk = a.sk;
    const float ninf = -__builtin_inff();
    const RowPos pos = locate<MASK>(blockIdx.x, a);
    const LdsRow lr = lds_row<kRag>(a.in0, pos, sk);
    const int lane = lr.lane, wib = lr.wib, sh = lr.sh;
    const int len = pos.len, plen = lr.plen;
    const int data_chunks = (plen + kChunk - 1) / kChunk;  // chunks that hold columns of the row
    const int all_chunks = (sk + sh + kChunk - 1) / kChunk;

    // whole 128-bit accesses up to the valid length; a ragged row ends where the next one begins
    const uint32_t row_bytes = (uint32_t)(kRag ? len : (len + kVec - 1) & ~(kVec - 1)) * 2u;
    const rsrc_t rx = make_rsrc(static_cast<const char*>(a.in0) + (size_t)pos.row * sk * 2, row_bytes);
    rsrc_t rm = rx, rb = rx;
    if constexpr (MASK == Mask::Bytes) {
        const uint32_t mb = a.mask_bcast ? 0u : pos.row / a.rows_per_mask_batch;
        rm = make_rsrc(a.mask + ((size_t)mb * a.sq + pos.i) * sk, (uint32_t)(kRag ? len : (len + kVec - 1) & ~(kVec - 1)));
    }
    if constexpr (kBia) rb = make_rsrc(static_cast<const char*>(a.bias) + (size_t)bias_row(pos.row, a) * sk * 2, row_bytes);
    uint32_t tail_x = 0, tail_b = 0, tail_m = 0;  // kRagged: what the range check drops at the row end
    if constexpr (kRag) {
        tail_x = ragged_tail16(rx, len, sh);
        if constexpr (kBia) tail_b = ragged_tail16(rb, len, sh);
        if constexpr (MASK == Mask::Bytes) tail_m = ragged_tail_mask(rm, len, sh);
    }
    DropoutArgs drop = a.drop;
    if constexpr (kDrp) drop = resolve(drop);
    // ALiBi: scale*(x + slope*(j - i')) = x*scale + slope2*(j - i'), slope2 row-uniform
    float slope2 = 0.f;
    if constexpr (kAli) slope2 = a.slopes[(pos.row / (uint32_t)a.sq) % a.np] * a.scale;
    const int ipos = alibi_row_position<MASK>(pos.i, a);
    // the scaled scores of a lane's 8 columns from `col` on, from the raw scores and the raw bias
    auto scores = [&](const float (&xv)[8], const u32x4& braw, int col, float (&t)[8]) {
        float bv[8];
        if constexpr (kBia) unpack8<T>(braw, bv);
#pragma unroll
        for (int k = 0; k < 8; ++k) {
            float x = xv[k];
            if constexpr (kBia) x += bv[k];
            if constexpr (kAli) t[k] = fmaf(x, a.scale, slope2 * alibi_distance<MASK>(col + k, ipos));
            else t[k] = x * a.scale;
        }
    };

    // ---- pass 1: HBM -> LDS; every lane keeps the running maximum mx of its scaled scores and the
    // sum of exp2(score - mx), rescaled whenever a chunk raises the maximum, so that the exponentials
    // are taken while the next loads are under way and no second pass over the row is needed
    float mx = ninf, sum = 0.f;
    // the reference point of the exponentials for a maximum m: m, or 0 while nothing is visible yet
    auto ref_of = [&](float m) { return m == ninf ? 0.f : m; };
    bool hidden = false;  // wave-uniform: this wave staged a -inf in place of a masked or out-of-row element
    uint32_t blank = 0;   // wave-uniform: bit j set = chunk wib + 16 j has no visible key at all
    for (int c0 = wib; c0 < data_chunks; c0 += kLdsWaves * UN) {
        u32x4 raw[UN], rawb[UN];
        u32x2 mk[UN];
#pragma unroll
        for (int u = 0; u < UN; ++u) {
            const int c = c0 + u * kLdsWaves;  // wave-uniform; chunks past the data load nothing
            raw[u] = buf_ld128<true>(rx, lr.off16(c), 0);
            if constexpr (kBia) rawb[u] = buf_ld128<false>(rb, lr.off16(c), 0);
            else rawb[u] = u32x4{0, 0, 0, 0};
            if constexpr (MASK == Mask::Bytes) mk[u] = buf_ld64(rm, lr.off8(c), 0);
        }
        if constexpr (kRag && MASK == Mask::Bytes) {
            if (lr.head && c0 == 0) {
                const u32x2 hm = ragged_head_mask(rm, lr.first_lane);
                mk[0].x |= hm.x;
                mk[0].y |= hm.y;
            }
        }
#pragma unroll
        for (int u = 0; u < UN; ++u) {
            const int c = c0 + u * kLdsWaves;
            if (c < data_chunks) {
                const int col = lr.pos0(c) - sh;  // first column of the lane, -1 in front of the row
                if constexpr (kRag) {
                    lr.fix16(raw[u], c, rx, tail_x);
                    if constexpr (kBia) lr.fix16(rawb[u], c, rb, tail_b);
                    if constexpr (MASK == Mask::Bytes) {
                        if ((c + 1) * kChunk >= plen) ragged_patch_mask(mk[u], lr.pos0(c), plen, tail_m);
                    }
                }
                // no lane of the wave crosses the row end (or holds the position in front of the row)
                bool plain = (c + 1) * kChunk <= plen && !(lr.head && c == 0);
                if constexpr (MASK == Mask::Bytes) {
                    plain = plain && (__ballot((mk[u].x | mk[u].y) != 0u) == 0ull);
                    if constexpr (kLdsBlankChunks) {
                        // a chunk with no visible key (the hidden tail of a padded row): nothing but -inf to stage
                        if (!plain && __ballot(!all_hidden(mk[u])) == 0ull) {
                            hidden = true;
                            blank |= 1u << (c / kLdsWaves);
                            constexpr uint32_t pair = NegInf16<T>::bits * 0x10001u;
                            *reinterpret_cast<u32x4*>(staged + c * kChunk * 2 + lane * 16) = u32x4{pair, pair, pair, pair};
                            continue;
                        }
                    }
                }
                float xv[8], t[8];
                unpack8<T>(raw[u], xv);
                scores(xv, rawb[u], col, t);
                u32x4 keep_raw = raw[u];
                if (!plain) {
                    hidden = true;
                    uint32_t keep = 0;
#pragma unroll
                    for (int k = 0; k < 8; ++k) {
                        bool kept = (col + k) < len;
                        if constexpr (kRag) kept = kept && (col + k) >= 0;
                        if constexpr (MASK == Mask::Bytes) {
                            const uint32_t w = (k < 4) ? mk[u].x : mk[u].y;
                            kept = kept && (((w >> (8 * (k & 3))) & 0xffu) == 0);
                        }
                        keep |= (kept ? 1u : 0u) << k;
                        t[k] = kept ? t[k] : ninf;
                    }
                    keep_raw = stage_masked<T>(raw[u], keep);
                }
                *reinterpret_cast<u32x4*>(staged + c * kChunk * 2 + lane * 16) = keep_raw;
                float top = mx;
#pragma unroll
                for (int k = 0; k < 8; ++k) top = fmaxf(top, t[k]);
                const float ref = ref_of(top);
                float part = 0.f;
#pragma unroll
                for (int k = 0; k < 8; ++k) part += fast_exp2(t[k] - ref);
                sum = fmaf(sum, fast_exp2(mx - ref), part);
                mx = top;
            }
        }
    }
    {
        // the lanes' sums to the maximum of the wave, the waves' sums to the maximum of the row
        const float lane_mx = mx;
        mx = wave_reduce<OpMax>(mx);
        sum = wave_reduce<OpSum>(sum * fast_exp2(lane_mx - ref_of(mx)));
        if (lane == 0) {
            red_max[wib] = mx;
            red_sum[wib] = sum;
        }
        __syncthreads();
        mx = red_max[0];
#pragma unroll
        for (int w = 1; w < kLdsWaves; ++w) mx = fmaxf(mx, red_max[w]);
        sum = 0.f;
#pragma unroll
        for (int w = 0; w < kLdsWaves; ++w) sum = fmaf(red_sum[w], fast_exp2(red_max[w] - ref_of(mx)), sum);
    }
    // a row whose every key is masked: uniform over the sk columns, as the unfused path gives
    const bool all_masked = (MASK == Mask::Bytes) && (mx == ninf);
    const float inv = all_masked ? 1.0f / (float)len : 1.0f / sum;

    // the bias of the chunks c0, c0 + 16, ... for the second pass (kBias)
    auto load_bias = [&](int c0, u32x4 (&rawb)[UB]) {
#pragma unroll
        for (int u = 0; u < UB; ++u) {
            if constexpr (kBia) rawb[u] = buf_ld128<false>(rb, lr.off16(c0 + u * kLdsWaves), 0);
            else rawb[u] = u32x4{0, 0, 0, 0};
        }
        if constexpr (kBia && kRag) {
#pragma unroll
            for (int u = 0; u < UB; ++u) lr.fix16(rawb[u], c0 + u * kLdsWaves, rb, tail_b);
        }
    };

    // ---- pass 2: normalise and store, from LDS; chunks above the diagonal store zeros.  Only a wave
    // that staged a -inf looks for them.
    const rsrc_t ry = make_rsrc(static_cast<char*>(a.out) + (size_t)pos.row * sk * 2, (uint32_t)sk * 2u);
    rsrc_t ry2 = ry;
    if constexpr (kDrp) ry2 = make_rsrc(static_cast<char*>(a.out2) + (size_t)pos.row * sk * 2, (uint32_t)sk * 2u);
    auto store_chunks = [&](auto with_hidden) {
        for (int c0 = wib; c0 < all_chunks; c0 += kLdsWaves * UB) {
            u32x4 rawb[UB];
            load_bias(c0, rawb);
#pragma unroll
            for (int u = 0; u < UB; ++u) {
                const int c = c0 + u * kLdsWaves;
                if (c >= all_chunks) continue;
                u32x4 o = u32x4{0, 0, 0, 0}, o2 = u32x4{0, 0, 0, 0};
                // (a chunk with no visible key stores zeros, unless the whole row has none)
                if (c < data_chunks && (all_masked || ((blank >> (c / kLdsWaves)) & 1u) == 0u)) {
                    float xv[8], t[8];
                    unpack8<T>(*reinterpret_cast<const u32x4*>(staged + c * kChunk * 2 + lane * 16), xv);
                    const int col = lr.pos0(c) - sh;
                    scores(xv, rawb[u], col, t);
#pragma unroll
                    for (int k = 0; k < 8; ++k) {
                        const float e = fast_exp2(t[k] - mx) * inv;
                        if constexpr (decltype(with_hidden)::value) {
                            t[k] = (xv[k] == ninf) ? 0.f : e;
                            if (all_masked) t[k] = ((col + k) < len && (col + k) >= 0) ? inv : 0.f;
                        } else {
                            t[k] = e;
                        }
                    }
                    o = pack8<T>(t);
                    if constexpr (kDrp) o2 = dropout8<T>(o, keep_bits_row8<kRag>(drop, pos.row, sk, col), drop.scale);
                }
                lr.template store<kRag>(ry, o, c, sk);
                if constexpr (kDrp) lr.template store<kRag>(ry2, o2, c, sk);
            }
        }
    };
    if (hidden) store_chunks(std::true_type{});
    else store_chunks(std::false_type{});
}

// NCH: chunks per wave, kLdsWaves * NCH * 512 >= sk (sk + 1 with kRagged); BYTES: size of the
// staging area, at least twice that many bytes.
template <typename T, Mask MASK, int NCH, int BYTES, int FLAGS = 0>
__global__ __launch_bounds__(kLdsThreads, lds_waves_per_simd(BYTES)) void softmax_bwd_lds_kernel(SoftmaxArgs a) {
    static_assert(NCH * kLdsWaves * kChunk * 2 >= BYTES, "the waves' chunks must cover the staging area");
    static_assert((FLAGS & ~(kRagged | kDropout)) == 0, "features only: the memory hints are fixed here");
    static_assert(FLAGS != (kRagged | kDropout) || BYTES > kLdsHalf, "both features together do not fit 64 registers per lane");
    constexpr bool kRag = (FLAGS & kRagged) != 0, kDrp = (FLAGS & kDropout) != 0;
    // chunks of a wave whose probabilities are in flight together: the keep bits need registers too,
    // of which the kernels that share a CU have 64 per lane
    constexpr int UN = (kDrp && BYTES <= kLdsHalf) ? 2 : kLdsUnroll;
    __shared__ __align__(16) char staged[BYTES];  // the probabilities of the row
    __shared__ float red_sum[kLdsWaves];
    const int sk = a.sk;
    const RowPos pos = locate<MASK>(blockIdx.x, a);
    const LdsRow lr = lds_row<kRag>(a.in0, pos, sk);
    const int lane = lr.lane, wib = lr.wib, sh = lr.sh;
    const int len = pos.len, plen = lr.plen;
    const int data_chunks = (plen + kChunk - 1) / kChunk;
    const uint32_t bytes = (uint32_t)(kRag ? len : (len + kVec - 1) & ~(kVec - 1)) * 2u;
    const rsrc_t bg = make_rsrc(static_cast<const char*>(a.in0) + (size_t)pos.row * sk * 2, bytes);
    const rsrc_t by = make_rsrc(static_cast<const char*>(a.in1) + (size_t)pos.row * sk * 2, bytes);
    uint32_t tail_g = 0, tail_p = 0;  // kRagged: what the range check drops at the row end
    if constexpr (kRag) {
        tail_g = ragged_tail16(bg, len, sh);
        tail_p = ragged_tail16(by, len, sh);
    }
    DropoutArgs drop = a.drop;
    if constexpr (kDrp) drop = resolve(drop);

    // ---- pass 1: the gradient into registers (chunk wib + 16 u; chunks past the data load
    // nothing), the probabilities into LDS, their dot product on the way
    u32x4 rg[NCH];
    uint32_t kb[(NCH + 3) / 4];  // kDropout: keep bits of the lane's 8 columns, a byte per chunk
#pragma unroll
    for (int u = 0; u < (NCH + 3) / 4; ++u) kb[u] = 0u;
#pragma unroll
    for (int u = 0; u < NCH; ++u) rg[u] = buf_ld128<true>(bg, lr.off16(wib + u * kLdsWaves), 0);
    float dot = 0.f;
#pragma unroll
    for (int u0 = 0; u0 < NCH; u0 += UN) {
        u32x4 rp[UN];
#pragma unroll
        for (int u = 0; u < UN; ++u)
            if (u0 + u < NCH) rp[u] = buf_ld128<true>(by, lr.off16(wib + (u0 + u) * kLdsWaves), 0);
#pragma unroll
        for (int u = 0; u < UN; ++u) {
            if (u0 + u >= NCH) continue;
            const int c = wib + (u0 + u) * kLdsWaves;
            if (c < data_chunks) {
                const int col = lr.pos0(c) - sh;
                if constexpr (kRag) {
                    // (the position in front of a row that lies one later stays zero in both tensors)
                    lr.fix16(rg[u0 + u], c, bg, tail_g);
                    lr.fix16(rp[u], c, by, tail_p);
                }
                float gv[8], pv[8];
                unpack8<T>(rg[u0 + u], gv);
                unpack8<T>(rp[u], pv);
                u32x4 keep = rp[u];
                if ((c + 1) * kChunk > plen) {
                    // the lane at the diagonal may have loaded columns past it
#pragma unroll
                    for (int k = 0; k < 8; ++k)
                        if ((col + k) >= len) gv[k] = pv[k] = 0.f;
                    keep = pack8<T>(pv);
                    rg[u0 + u] = pack8<T>(gv);
                }
                if constexpr (kDrp) {
                    const uint32_t bits = keep_bits_row8<kRag>(drop, pos.row, sk, col);
                    kb[(u0 + u) / 4] |= bits << (8 * ((u0 + u) % 4));
#pragma unroll
                    for (int k = 0; k < 8; ++k) gv[k] = ((bits >> k) & 1u) ? gv[k] * drop.scale : 0.f;
                }
#pragma unroll
                for (int k = 0; k < 8; ++k) dot = fmaf(gv[k], pv[k], dot);
                *reinterpret_cast<u32x4*>(staged + c * kChunk * 2 + lane * 16) = keep;
            }
        }
        // the loads of the next group are not to be moved up here: they would not fit the registers
        __builtin_amdgcn_sched_barrier(0);
    }
    dot = wave_reduce<OpSum>(dot);
    if (lane == 0) red_sum[wib] = dot;
    __syncthreads();
    dot = red_sum[0];
#pragma unroll
    for (int w = 1; w < kLdsWaves; ++w) dot += red_sum[w];

    // ---- pass 2: dx.  It may alias dy: a wave has read its chunks of the row before it writes them
#pragma unroll
    for (int u = 0; u < NCH; ++u) forget_origin(rg[u]);  // the gradient stays packed in between
    const rsrc_t rdx = make_rsrc(static_cast<char*>(a.out) + (size_t)pos.row * sk * 2, (uint32_t)sk * 2u);
#pragma unroll
    for (int u = 0; u < NCH; ++u) {
        const int c = wib + u * kLdsWaves;
        u32x4 o = u32x4{0, 0, 0, 0};
        if (c < data_chunks) {
            float gv[8], pv[8];
            unpack8<T>(rg[u], gv);
            unpack8<T>(*reinterpret_cast<const u32x4*>(staged + c * kChunk * 2 + lane * 16), pv);
#pragma unroll
            for (int k = 0; k < 8; ++k) {
                if constexpr (kDrp) gv[k] = ((kb[u / 4] >> (8 * (u % 4) + k)) & 1u) ? gv[k] * drop.scale : 0.f;
                gv[k] = a.scale * (pv[k] * (gv[k] - dot));  // pv = 0 past the row
            }
            o = pack8<T>(gv);
        }
        lr.template store<kRag>(rdx, o, c, sk);  // chunks past the row end store nothing
    }
}

// ---------------------------------------------------------------------------------
// Any-shape kernels: one 256-thread block per row, element-wise accesses, the row
// is re-read for each pass (from L2).  Used for what no other kernel takes: rows shorter
// than 8 columns, rows beyond the LDS-staged limit, ragged rows (sk not a multiple of 8 or
// a pointer not 16-byte aligned) beyond the register-resident limit, and rows beyond the
// register-resident limit with ALiBi, a bias tensor or dropout.
// ---------------------------------------------------------------------------------
constexpr int kGenericThreads = 256;

template <typename Op>
__device__ __forceinline__ float block_reduce(float v, float* red) {
    v = wave_reduce<Op>(v);
    const int lane = threadIdx.x & (kWave - 1);
    const int wib = threadIdx.x >> 6;
    __syncthreads();  // red may still be read from the previous reduction
    if (lane == 0) red[wib] = v;
    __syncthreads();
    typename Op::type r = Op::enc(red[0]);
#pragma unroll
    for (int w = 1; w < kGenericThreads / kWave; ++w) r = Op::f(r, Op::enc(red[w]));
    return Op::dec(r);
}

// keep bit of one element (any alignment): its group's block, its 16-bit field
__device__ __forceinline__ bool keep_element(const DropoutArgs& d, uint32_t row, int sk, int j) {
    const uint64_t e = (uint64_t)row * (uint32_t)sk + (uint32_t)j;
    return (keep_bits8(d, e >> 3) >> (uint32_t)(e & 7u)) & 1u;
}

template <typename T, Mask MASK, int FLAGS = 0>
__global__ __launch_bounds__(kGenericThreads) void softmax_fwd_generic_kernel(SoftmaxArgs a) {
    __shared__ float red[kGenericThreads / kWave];
    const uint32_t row = blockIdx.x;
    const int sk = a.sk;
    const uint32_t i = row % (uint32_t)a.sq;
    DropoutArgs drop = a.drop;
    if constexpr ((FLAGS & kDropout) != 0) drop = resolve(drop);
    const int len = (MASK == Mask::Causal) ? min((int)i + 1, sk) : sk;
    const char* x = static_cast<const char*>(a.in0) + (size_t)row * sk * 2;
    char* y = static_cast<char*>(a.out) + (size_t)row * sk * 2;
    const uint8_t* mrow = nullptr;
    if constexpr (MASK == Mask::Bytes) {
        const uint32_t mb = a.mask_bcast ? 0u : row / a.rows_per_mask_batch;
        mrow = a.mask + ((size_t)mb * a.sq + i) * sk;
    }
    const float ninf = -__builtin_inff();
    // ALiBi: slopes given -> scores get slope * min(j - i', 0) before the scale (decided at run time here)
    const float slope2 = (a.slopes != nullptr) ? a.slopes[(row / (uint32_t)a.sq) % a.np] * a.scale : 0.f;
    const int ipos = alibi_row_position<MASK>(i, a);
    // bias tensor given -> added to the scores before the scale (decided at run time here)
    const char* brow = nullptr;
    if (a.bias != nullptr) brow = static_cast<const char*>(a.bias) + (size_t)bias_row(row, a) * sk * 2;
    auto score = [&](int j) {
        float xj = Elem<T>::load1(x + (size_t)j * 2);
        if (brow != nullptr) xj += Elem<T>::load1(brow + (size_t)j * 2);
        return fmaf(xj, a.scale, slope2 * alibi_distance<MASK>(j, ipos));
    };

    float mx = ninf;
    for (int j = threadIdx.x; j < len; j += kGenericThreads) {
        bool keep = true;
        if constexpr (MASK == Mask::Bytes) keep = (mrow[j] == 0);
        if (keep) mx = fmaxf(mx, score(j));
    }
    mx = block_reduce<OpMax>(mx, red);
    const bool all_masked = (mx == ninf);

    float sum = 0.f;
    for (int j = threadIdx.x; j < len; j += kGenericThreads) {
        bool keep = true;
        if constexpr (MASK == Mask::Bytes) keep = (mrow[j] == 0);
        float e = keep ? fast_exp2(score(j) - mx) : 0.f;
        if (all_masked) e = 1.f;
        sum += e;
    }
    sum = block_reduce<OpSum>(sum, red);
    const float inv = 1.0f / sum;

    // y may alias x: an element is read and written by the same thread only
    for (int j = threadIdx.x; j < sk; j += kGenericThreads) {
        float o = 0.f;
        if (j < len) {
            bool keep = true;
            if constexpr (MASK == Mask::Bytes) keep = (mrow[j] == 0);
            float e = keep ? fast_exp2(score(j) - mx) : 0.f;
            if (all_masked) e = 1.f;
            o = e * inv;
        }
        Elem<T>::store1(y + (size_t)j * 2, o);
        if constexpr ((FLAGS & kDropout) != 0) {
            float rounded, unused;
            Elem<T>::unpack(Elem<T>::pack(o, 0.f), rounded, unused);
            const bool keep = j < len && keep_element(drop, row, sk, j);
            Elem<T>::store1(static_cast<char*>(a.out2) + ((size_t)row * sk + j) * 2, keep ? rounded * drop.scale : 0.f);
        }
    }
}

template <typename T, Mask MASK, int FLAGS = 0>
__global__ __launch_bounds__(kGenericThreads) void softmax_bwd_generic_kernel(SoftmaxArgs a) {
    __shared__ float red[kGenericThreads / kWave];
    const uint32_t row = blockIdx.x;
    const int sk = a.sk;
    const uint32_t i = row % (uint32_t)a.sq;
    DropoutArgs drop = a.drop;
    if constexpr ((FLAGS & kDropout) != 0) drop = resolve(drop);
    const int len = (MASK == Mask::Causal) ? min((int)i + 1, sk) : sk;
    const char* g = static_cast<const char*>(a.in0) + (size_t)row * sk * 2;
    const char* p = static_cast<const char*>(a.in1) + (size_t)row * sk * 2;
    char* dx = static_cast<char*>(a.out) + (size_t)row * sk * 2;

    auto grad = [&](int j) {
        float gj = Elem<T>::load1(g + (size_t)j * 2);
        if constexpr ((FLAGS & kDropout) != 0) gj = keep_element(drop, row, sk, j) ? gj * drop.scale : 0.f;
        return gj;
    };
    float dot = 0.f;
    for (int j = threadIdx.x; j < len; j += kGenericThreads)
        dot = fmaf(grad(j), Elem<T>::load1(p + (size_t)j * 2), dot);
    dot = block_reduce<OpSum>(dot, red);

    for (int j = threadIdx.x; j < sk; j += kGenericThreads) {
        float o = 0.f;
        if (j < len) {
            const float gj = grad(j);
            const float pj = Elem<T>::load1(p + (size_t)j * 2);
            o = a.scale * (pj * (gj - dot));
        }
        Elem<T>::store1(dx + (size_t)j * 2, o);
    }
}

}  // namespace neox
