// Philox4x32-10 (Salmon et al., SC'11) and the element -> random bits assignment of the
// attention-dropout kernels.
//
// Eight consecutive elements of the score tensor (one 128-bit access) share one Philox
// block: counter = (c_lo, c_hi, group_lo, group_hi) with c = offset / 4 and group = element
// index / 8, key = (seed_lo, seed_hi).  This is the counter layout of torch's device generator
// with the group index in the place of the subsequence: a generator offset counts 32-bit
// outputs, four to a block, so a consumer that owns the offsets [o, o + n) draws from the
// counter values [o / 4, (o + n) / 4).  A call that takes the generator's (seed, offset) and
// advances the offset by 4 therefore owns exactly one counter value, disjoint from what every
// earlier and later consumer of that generator draws.  Element e owns the 16-bit field (word[e/2] >> 16*(e%2)) & 0xffff and is kept
// iff field >= threshold, threshold = round(p * 65536): the drop probability is honoured
// to 2^-16.
#pragma once

#include "wave.hpp"

namespace neox {

struct DropoutArgs {
    uint32_t seed_lo, seed_hi;  // Philox key
    uint32_t off_lo, off_hi;    // low half of the counter: generator offset / 4
    uint32_t threshold;         // 0 .. 65536
    float scale;                // 1/(1-p), 0 for p = 1
    // If not null: {seed, offset} in device memory, read when the kernel runs instead of the
    // four words above.  A launch recorded into a HIP graph then draws a fresh pattern on
    // every replay, provided the graph itself advances the offset stored there.
    const uint64_t* state;
};

// The parameters a kernel works with: the by-value ones, or those in device memory.
__device__ __forceinline__ DropoutArgs resolve(DropoutArgs d) {
    if (d.state != nullptr) {
        const uint64_t seed = d.state[0], block = d.state[1] >> 2;  // wave-uniform loads
        d.seed_lo = (uint32_t)seed;
        d.seed_hi = (uint32_t)(seed >> 32);
        d.off_lo = (uint32_t)block;
        d.off_hi = (uint32_t)(block >> 32);
    }
    return d;
}

__device__ __forceinline__ u32x4 philox4x32_10(u32x4 c, uint32_t k0, uint32_t k1) {
#pragma unroll
    for (int r = 0; r < 10; ++r) {
        const uint64_t p0 = (uint64_t)0xD2511F53u * c.x;
        const uint64_t p1 = (uint64_t)0xCD9E8D57u * c.z;
        c = u32x4{(uint32_t)(p1 >> 32) ^ c.y ^ k0, (uint32_t)p1, (uint32_t)(p0 >> 32) ^ c.w ^ k1,
                  (uint32_t)p0};
        k0 += 0x9E3779B9u;
        k1 += 0xBB67AE85u;
    }
    return c;
}

// Bit k of the result is set iff element k of the group is kept.
__device__ __forceinline__ uint32_t keep_bits8(const DropoutArgs& d, uint64_t group) {
    const u32x4 w = philox4x32_10(u32x4{d.off_lo, d.off_hi, (uint32_t)group, (uint32_t)(group >> 32)},
                                  d.seed_lo, d.seed_hi);
    const uint32_t words[4] = {w.x, w.y, w.z, w.w};
    uint32_t bits = 0;
#pragma unroll
    for (int k = 0; k < 8; ++k) {
        const uint32_t field = (k & 1) ? (words[k >> 1] >> 16) : (words[k >> 1] & 0xffffu);
        bits |= (field >= d.threshold ? 1u : 0u) << k;
    }
    return bits;
}

// Dropout of 8 packed probabilities as the unfused path computes it on the already
// rounded values: kept -> round(float(y) * scale), dropped -> 0.
template <typename T>
__device__ __forceinline__ u32x4 dropout8(const u32x4& packed, uint32_t bits, float scale) {
    float f[8];
    unpack8<T>(packed, f);
#pragma unroll
    for (int k = 0; k < 8; ++k) f[k] = ((bits >> k) & 1u) ? f[k] * scale : 0.f;
    return pack8<T>(f);
}

}  // namespace neox
