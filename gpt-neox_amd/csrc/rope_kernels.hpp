// Rotary positional embedding apply for gfx950: q and k in one launch, in place or
// out of place, over the first d_rot dims of [s, b, h, d] tensors with arbitrary
// s/b/h strides (the inputs are usually views into a fused QKV buffer).
//
// One block serves one sequence position: the position's cos/sin values are loaded
// once into registers and reused for every head of q and k.  Two kernels:
//
// * rope_span_kernel -- the rotated span splits into at most 64 slots of W = 8, 4 or 2 dims
//   (the widest the alignment of the layouts and of d_rot/2 allows).  Each lane owns ONE
//   slot and consecutive lanes own consecutive slots, so a wave access covers whole
//   contiguous spans (64 B for d_rot = 32, 256 B for d_rot = 128, 48 B for d_rot = 24).  The
//   partner dims (j +- d_rot/2) live d_rot/(2W) lanes away and are fetched with a wave
//   shuffle.  q and k of one block iteration are loaded together before any arithmetic.
// * rope_kernel -- the rest (odd d_rot/2, 2-byte aligned layouts, spans of more than 64
//   slots).  threadIdx.x selects a slot of W consecutive dims in the first half of the
//   rotated span; the thread also owns the matching W dims of the second half, so no data
//   crosses lanes (W = 8, 4, 2, 1).
//
// In both, a lane reads everything it needs before it writes, and a pair
// (j, j + d_rot/2) is written by the lane(s) that read it, so in-place operation is
// race-free.  q/k accesses carry the non-temporal hint (each byte is touched once).
//
// The rotation is given as cos/sin tables (fp32 or the storage type) or as fp32 angles (CS =
// Angles): then the block evaluates sincosf once per dim of its position into LDS -- d_rot
// evaluations per block, shared by all its heads -- and the lanes take their values from there.
// Out of place, the kernels also copy the pass-through dims [d_rot, d) of every head in the same
// launch (span kernel: further lanes of the head's lane group; rope_kernel: a 16-bit copy loop).
//
// Arithmetic is fp32 with the two products rounded separately (no fused
// multiply-add), which is bit-identical to evaluating q*cos + rotate_half(q)*sin
// in fp32; the result is rounded once to the storage type.
#pragma once

#include <type_traits>

#include "wave.hpp"

namespace neox {

struct RopeTensor {
    const char* in;
    char* out;
    int64_t in_stride[3];   // elements: position, batch, head
    int64_t out_stride[3];
    int32_t n_outer;        // loop extent addressed by stride[1] (1 when b and h are collapsed)
    int32_t n_inner;        // vectors addressed by stride[2]
};

struct RopeArgs {
    RopeTensor t[2];
    const char* cos;
    const char* sin;
    int64_t cs_stride;   // elements between consecutive positions of cos/sin
    int32_t pos_offset;
    int32_t half;        // d_rot / 2
    int32_t lpv;         // slots per vector = half / W
    int32_t nt;          // 1: q only, 2: q and k
    int32_t pad_slots;   // span kernel: slots after the rotated span that are stored as loaded (in place:
                         // the rest of a 64-byte block; out of place: the pass-through dims)
    int32_t copy_dims;   // out of place: pass-through dims [d_rot, d_rot + copy_dims) to copy, else 0
    // span kernel, filled in by its launcher
    int32_t zsplit;      // blocks sharing the vectors of one (position, outer) pair
    int32_t outer_grid;  // extent of the outer loop in the block index
    int32_t share;       // vectors per block: ceil(vectors of a pair / zsplit)
    int32_t lph;         // lanes per head: slots of the rotated span plus pad_slots, <= 64
    int32_t lph_magic;   // ceil(2^16 / lph): lane / lph == (lane * lph_magic) >> 16 for lane < 64
    int32_t spw;         // heads per wave: 64 / lph
    // piece kernel (dense, identically laid out tensors), filled in by its launcher
    int32_t vec_elems;        // elements between consecutive head vectors (= the head size)
    uint32_t vecs_per_pos;    // b * h head vectors per position
    uint32_t n_units;         // work units: runs of spw consecutive head vectors
    uint32_t units_per_piece; // units per 4 KiB piece, 0 = units in order
    uint32_t affine_blocks;   // leading blocks that take part in the XCD-aware order: a multiple of 8
};

template <int W>
struct Pack;  // W 16-bit elements
template <>
struct Pack<8> { typedef u32x4 type; };
template <>
struct Pack<4> { typedef u32x2 type; };
template <>
struct Pack<2> { typedef uint32_t type; };

template <typename T, int W, bool NT = false>
__device__ __forceinline__ void load_elems(const char* p, float (&f)[W]) {
    if constexpr (W == 1) {
        f[0] = Elem<T>::load1(p);
    } else {
        typedef typename Pack<W>::type P;
        const P w = NT ? __builtin_nontemporal_load(reinterpret_cast<const P*>(p))
                       : *reinterpret_cast<const P*>(p);
        const uint32_t* u = reinterpret_cast<const uint32_t*>(&w);
#pragma unroll
        for (int k = 0; k < W / 2; ++k) Elem<T>::unpack(u[k], f[2 * k], f[2 * k + 1]);
    }
}

template <typename T, int W, bool NT = false>
__device__ __forceinline__ void store_elems(char* p, const float (&f)[W]) {
    if constexpr (W == 1) {
        Elem<T>::store1(p, f[0]);
    } else {
        typedef typename Pack<W>::type P;
        P w;
        uint32_t* u = reinterpret_cast<uint32_t*>(&w);
#pragma unroll
        for (int k = 0; k < W / 2; ++k) u[k] = Elem<T>::pack(f[2 * k], f[2 * k + 1]);
        if constexpr (NT) __builtin_nontemporal_store(w, reinterpret_cast<P*>(p));
        else *reinterpret_cast<P*>(p) = w;
    }
}

// CS tag: the rotation is given as fp32 angles; cos and sin are evaluated in the kernel
struct Angles {};

// One position's cos/sin from its fp32 angles: every thread of the block evaluates sincosf for
// the dims tid, tid + nthreads, ... into LDS (cos at [0, d_rot), sin at [d_rot, 2 d_rot)).  All
// threads of the block must call this (it ends with a barrier).
__device__ __forceinline__ void angles_to_lds(const float* angles, int d_rot, float* tab, int tid, int nthreads) {
    for (int j = tid; j < d_rot; j += nthreads) {
        float sv, cv;
        sincosf(angles[j], &sv, &cv);
        tab[j] = cv;
        tab[d_rot + j] = sv;
    }
    __syncthreads();
}

// cos/sin table element access: CS = float reads fp32, otherwise 16-bit type CS
template <typename CS, int W>
__device__ __forceinline__ void load_table(const char* base, int64_t idx, float (&f)[W]) {
    if constexpr (sizeof(CS) == 4) {
        const float* p = reinterpret_cast<const float*>(base) + idx;
        if constexpr (W >= 4) {
#pragma unroll
            for (int k = 0; k < W / 4; ++k) {
                const f32x4 v = *reinterpret_cast<const f32x4*>(p + 4 * k);
                f[4 * k] = v.x;
                f[4 * k + 1] = v.y;
                f[4 * k + 2] = v.z;
                f[4 * k + 3] = v.w;
            }
        } else {
#pragma unroll
            for (int k = 0; k < W; ++k) f[k] = p[k];
        }
    } else {
        load_elems<CS, W>(base + idx * 2, f);
    }
}

template <typename T, int W, bool BWD>
__device__ __forceinline__ void rotate(const float (&xl)[W], const float (&xh)[W],
                                       const float (&cl)[W], const float (&ch)[W],
                                       const float (&sl)[W], const float (&sh)[W], float (&ol)[W],
                                       float (&oh)[W]) {
#pragma clang fp contract(off)
#pragma unroll
    for (int k = 0; k < W; ++k) {
        if constexpr (!BWD) {
            ol[k] = xl[k] * cl[k] - xh[k] * sl[k];
            oh[k] = xh[k] * ch[k] + xl[k] * sh[k];
        } else {
            ol[k] = xl[k] * cl[k] + xh[k] * sh[k];
            oh[k] = xh[k] * ch[k] - xl[k] * sl[k];
        }
    }
}

template <typename T, typename CS, int W, bool BWD>
__global__ __launch_bounds__(256) void rope_kernel(RopeArgs a) {
    const int slot = threadIdx.x;  // < lpv by construction of the block shape
    const int pos = blockIdx.x;
    const int outer = blockIdx.y;
    const int j = slot * W;
    const int half = a.half;

    float cl[W], ch[W], sl[W], sh[W];
    const int64_t crow = (int64_t)(pos + a.pos_offset) * a.cs_stride;
    if constexpr (std::is_same<CS, Angles>::value) {
        extern __shared__ float lds_tab[];
        angles_to_lds(reinterpret_cast<const float*>(a.cos) + crow, 2 * half, lds_tab,
                      threadIdx.y * blockDim.x + threadIdx.x, blockDim.x * blockDim.y);
#pragma unroll
        for (int k = 0; k < W; ++k) {
            cl[k] = lds_tab[j + k];
            ch[k] = lds_tab[j + half + k];
            sl[k] = lds_tab[2 * half + j + k];
            sh[k] = lds_tab[3 * half + j + k];
        }
    } else {
        load_table<CS, W>(a.cos, crow + j, cl);
        load_table<CS, W>(a.cos, crow + j + half, ch);
        load_table<CS, W>(a.sin, crow + j, sl);
        load_table<CS, W>(a.sin, crow + j + half, sh);
    }

    const int v_step = blockDim.y * gridDim.z;
    const int n0 = (outer < a.t[0].n_outer) ? a.t[0].n_inner : 0;
    const int n1 = (a.nt > 1 && outer < a.t[1].n_outer) ? a.t[1].n_inner : 0;
    const int nmax = max(n0, n1);

    const int64_t qi = (int64_t)pos * a.t[0].in_stride[0] + (int64_t)outer * a.t[0].in_stride[1] + j;
    const int64_t qo = (int64_t)pos * a.t[0].out_stride[0] + (int64_t)outer * a.t[0].out_stride[1] + j;
    const int64_t ki = (int64_t)pos * a.t[1].in_stride[0] + (int64_t)outer * a.t[1].in_stride[1] + j;
    const int64_t ko = (int64_t)pos * a.t[1].out_stride[0] + (int64_t)outer * a.t[1].out_stride[1] + j;

    for (int v = threadIdx.y + blockIdx.z * blockDim.y; v < nmax; v += v_step) {
        float ql[W], qh[W], kl[W], kh[W];
        const bool do_q = v < n0;
        const bool do_k = v < n1;
        const char* qp = a.t[0].in + (qi + (int64_t)v * a.t[0].in_stride[2]) * 2;
        const char* kp = a.t[1].in + (ki + (int64_t)v * a.t[1].in_stride[2]) * 2;
        if (do_q) {
            load_elems<T, W, true>(qp, ql);
            load_elems<T, W, true>(qp + (size_t)half * 2, qh);
        }
        if (do_k) {
            load_elems<T, W, true>(kp, kl);
            load_elems<T, W, true>(kp + (size_t)half * 2, kh);
        }
        if (do_q) {
            float ol[W], oh[W];
            rotate<T, W, BWD>(ql, qh, cl, ch, sl, sh, ol, oh);
            char* op = a.t[0].out + (qo + (int64_t)v * a.t[0].out_stride[2]) * 2;
            store_elems<T, W, true>(op, ol);
            store_elems<T, W, true>(op + (size_t)half * 2, oh);
        }
        if (do_k) {
            float ol[W], oh[W];
            rotate<T, W, BWD>(kl, kh, cl, ch, sl, sh, ol, oh);
            char* op = a.t[1].out + (ko + (int64_t)v * a.t[1].out_stride[2]) * 2;
            store_elems<T, W, true>(op, ol);
            store_elems<T, W, true>(op + (size_t)half * 2, oh);
        }
        if (a.copy_dims > 0) {
            // out of place: the pass-through dims of this head, element by element (the shapes
            // that reach this kernel have no common wider alignment)
            const int e0 = 2 * half - j, e1 = e0 + a.copy_dims;  // relative to the lane's first dim
            for (int e = e0 + (int)threadIdx.x; e < e1; e += blockDim.x) {
                if (do_q)
                    *reinterpret_cast<uint16_t*>(a.t[0].out + (qo + (int64_t)v * a.t[0].out_stride[2] + e) * 2) =
                        *reinterpret_cast<const uint16_t*>(qp + (int64_t)e * 2);
                if (do_k)
                    *reinterpret_cast<uint16_t*>(a.t[1].out + (ko + (int64_t)v * a.t[1].out_stride[2] + e) * 2) =
                        *reinterpret_cast<const uint16_t*>(kp + (int64_t)e * 2);
            }
        }
    }
}

// ---- contiguous-span kernel -----------------------------------------------------------
constexpr int kSpanIters = 2;  // head vectors per thread and tensor whose loads are in flight together

template <int W, bool NT>
__device__ __forceinline__ void load_words(const char* p, uint32_t (&w)[W / 2]) {
    typedef typename Pack<W>::type P;
    const P v = NT ? __builtin_nontemporal_load(reinterpret_cast<const P*>(p)) : *reinterpret_cast<const P*>(p);
    const uint32_t* u = reinterpret_cast<const uint32_t*>(&v);
#pragma unroll
    for (int k = 0; k < W / 2; ++k) w[k] = u[k];
}

template <int W, bool NT>
__device__ __forceinline__ void store_words(char* p, const uint32_t (&w)[W / 2]) {
    typedef typename Pack<W>::type P;
    P v;
    uint32_t* u = reinterpret_cast<uint32_t*>(&v);
#pragma unroll
    for (int k = 0; k < W / 2; ++k) u[k] = w[k];
    if constexpr (NT) __builtin_nontemporal_store(v, reinterpret_cast<P*>(p));
    else *reinterpret_cast<P*>(p) = v;
}

// Each lane owns ONE slot of W dims (16, 8 or 4 bytes) of a head's rotated span; the
// d_rot/W lanes of a span are consecutive, a wave holds floor(64 / lanes-per-span) spans and
// leaves its last few lanes idle when that does not divide 64 (d_rot = 24, 48, 80, 96 ...).
template <typename T, typename CS, int W, bool BWD>
__global__ __launch_bounds__(256) void rope_span_kernel(RopeArgs a) {
    const int hl = a.lpv;    // slots per half span = lane distance to the partner slot
    const int lps = hl * 2;  // slots (lanes) per rotated span
    const int lph = a.lph, spw = a.spw;
    const int lane = threadIdx.x & (kWave - 1);
    const int sw = (lane * a.lph_magic) >> 16;  // head of this lane inside its wave
    const int slot = lane - sw * lph;
    const bool active = sw < spw;
    const bool rotated = slot < lps;  // else: a slot that is stored back as loaded
    const int vib = (threadIdx.x >> 6) * spw + sw;  // vector handled in a block iteration
    const int vpb = (256 / kWave) * spw;            // vectors per block iteration
    // blocks are numbered in memory order -- position, outer, piece of the vector loop -- so that
    // the blocks running at any moment stream through neighbouring addresses
    uint32_t po = blockIdx.x;
    int piece = 0, outer = 0;
    if (a.zsplit > 1) {  // block-uniform branches: the common shapes skip the divisions
        piece = po % (uint32_t)a.zsplit;
        po /= (uint32_t)a.zsplit;
    }
    if (a.outer_grid > 1) {
        outer = po % (uint32_t)a.outer_grid;
        po /= (uint32_t)a.outer_grid;
    }
    const int pos = po;
    const bool second = slot >= hl;
    const int partner = (second ? lane - hl : lane + hl) & (kWave - 1);  // idle lanes: any valid lane
    const int j = slot * W;                                                 // first dim this lane owns
    const int jt = rotated ? j : 0;                                         // its table column
    const int jp = rotated ? (second ? slot - hl : slot + hl) * W : 0;      // the partner lane's

    // out = x*cos[own] + sign * partner * sin[.]: the forward pass takes sin at the lane's own
    // dims with sign -,+ for the first/second half; the backward pass takes sin at the
    // partner's dims with sign +,-.  Folding the sign into sin is exact.
    float c[W], sn[W];
    const int64_t crow = (int64_t)(pos + a.pos_offset) * a.cs_stride;
    if constexpr (std::is_same<CS, Angles>::value) {
        extern __shared__ float lds_tab[];
        angles_to_lds(reinterpret_cast<const float*>(a.cos) + crow, 2 * a.half, lds_tab, threadIdx.x, 256);
#pragma unroll
        for (int k = 0; k < W; ++k) {
            c[k] = lds_tab[jt + k];
            sn[k] = lds_tab[2 * a.half + (BWD ? jp : jt) + k];
        }
    } else {
        load_table<CS, W>(a.cos, crow + jt, c);
        load_table<CS, W>(a.sin, crow + (BWD ? jp : jt), sn);
    }
    if (second == BWD) {
#pragma unroll
        for (int k = 0; k < W; ++k) sn[k] = -sn[k];
    }

    // the blocks of one (position, outer) pair share its vectors evenly: equal work per block keeps
    // the XCDs, which receive consecutive blocks in turn, equally loaded
    const int lo = piece * a.share;
    const int hi = lo + a.share;  // block-uniform loop bound; the per-tensor bounds below clip it
    const int nq_hi = active ? min(a.t[0].n_inner, hi) : 0;
    const int nk_hi = (active && a.nt > 1) ? min(a.t[1].n_inner, hi) : 0;
    const int64_t qi = (int64_t)pos * a.t[0].in_stride[0] + (int64_t)outer * a.t[0].in_stride[1] + j;
    const int64_t qo = (int64_t)pos * a.t[0].out_stride[0] + (int64_t)outer * a.t[0].out_stride[1] + j;
    const int64_t ki = (int64_t)pos * a.t[1].in_stride[0] + (int64_t)outer * a.t[1].in_stride[1] + j;
    const int64_t ko = (int64_t)pos * a.t[1].out_stride[0] + (int64_t)outer * a.t[1].out_stride[1] + j;

    const int step = vpb * kSpanIters;
    // every lane of a wave runs the same number of iterations (the shuffles need all lanes)
    for (int v0 = lo; v0 < hi; v0 += step) {
        uint32_t xq[kSpanIters][W / 2], xk[kSpanIters][W / 2];
#pragma unroll
        for (int u = 0; u < kSpanIters; ++u) {
            const int v = v0 + u * vpb + vib;
#pragma unroll
            for (int k = 0; k < W / 2; ++k) xq[u][k] = xk[u][k] = 0u;
            if (v < nq_hi) load_words<W, true>(a.t[0].in + (qi + (int64_t)v * a.t[0].in_stride[2]) * 2, xq[u]);
            if (v < nk_hi) load_words<W, true>(a.t[1].in + (ki + (int64_t)v * a.t[1].in_stride[2]) * 2, xk[u]);
        }
#pragma unroll
        for (int u = 0; u < kSpanIters; ++u) {
            const int v = v0 + u * vpb + vib;
#pragma unroll
            for (int t = 0; t < 2; ++t) {
                const uint32_t(&x)[W / 2] = t ? xk[u] : xq[u];
                float xf[W], pf[W], o[W];
#pragma unroll
                for (int k = 0; k < W / 2; ++k) {
                    const uint32_t p = (uint32_t)__shfl((int)x[k], partner);
                    Elem<T>::unpack(x[k], xf[2 * k], xf[2 * k + 1]);
                    Elem<T>::unpack(p, pf[2 * k], pf[2 * k + 1]);
                }
                {
#pragma clang fp contract(off)
#pragma unroll
                    for (int k = 0; k < W; ++k) o[k] = xf[k] * c[k] + pf[k] * sn[k];
                }
                uint32_t ow[W / 2];
#pragma unroll
                for (int k = 0; k < W / 2; ++k) {
                    const uint32_t packed = Elem<T>::pack(o[2 * k], o[2 * k + 1]);
                    ow[k] = rotated ? packed : x[k];
                }
                if (v < (t ? nk_hi : nq_hi))
                    store_words<W, true>(a.t[t].out + ((t ? ko : qo) + (int64_t)v * a.t[t].out_stride[2]) * 2, ow);
            }
        }
    }
}


// ---- contiguous-span kernel for dense tensors, XCD-aware ---------------------------------
// The same lane layout as rope_span_kernel for tensors that are dense and laid out alike
// ([s, b, h, d] contiguous, in and out, q and k): the head vectors then form one run in memory and
// the work splits into units of spw consecutive vectors (one wave access per tensor), numbered
// in memory order.  A block of 4 waves takes ITERS units per wave.  Workgroups go to the 8 XCDs of
// the chip in turn, and a store stream runs fastest when every XCD keeps to its own 4 KiB
// pieces of the address space (piece index = XCD mod 8): where the units tile 4 KiB pieces, block
// x of a group of 8 takes the pieces x, x + 8, x + 16, ... of the group instead of consecutive
// ones.  Measured against rope_span_kernel in one process: partial rotary in place
// ([2048, 4, 32, 128], first 32 dims) 24.0 -> 22.5 us, full rotary [8192, 1, 32, 128] 44.5 -> 43.8 us.
// A unit lies inside one position (vecs_per_pos % spw == 0); the cos/sin values are loaded per
// unit unless the wave's previous unit had the same position.
// W 16-bit elements through a range-checked buffer access (non-temporal): lanes whose offset lies
// outside the resource load zeros / store nothing
template <int W>
__device__ __forceinline__ void buf_ld_words(rsrc_t r, uint32_t off, uint32_t (&w)[W / 2]) {
    if constexpr (W == 8) {
        const u32x4 v = __builtin_amdgcn_raw_buffer_load_b128(r, (int)off, 0, kAuxNt);
        w[0] = v.x, w[1] = v.y, w[2] = v.z, w[3] = v.w;
    } else if constexpr (W == 4) {
        const u32x2 v = __builtin_amdgcn_raw_buffer_load_b64(r, (int)off, 0, kAuxNt);
        w[0] = v.x, w[1] = v.y;
    } else {
        w[0] = __builtin_amdgcn_raw_buffer_load_b32(r, (int)off, 0, kAuxNt);
    }
}
template <int W>
__device__ __forceinline__ void buf_st_words(rsrc_t r, uint32_t off, const uint32_t (&w)[W / 2]) {
    if constexpr (W == 8) {
        __builtin_amdgcn_raw_buffer_store_b128(u32x4{w[0], w[1], w[2], w[3]}, r, (int)off, 0, kAuxNt);
    } else if constexpr (W == 4) {
        __builtin_amdgcn_raw_buffer_store_b64(u32x2{w[0], w[1]}, r, (int)off, 0, kAuxNt);
    } else {
        __builtin_amdgcn_raw_buffer_store_b32(w[0], r, (int)off, 0, kAuxNt);
    }
}

template <typename T, typename CS, int W, bool BWD, int ITERS>
__global__ __launch_bounds__(256) void rope_piece_kernel(RopeArgs a) {
    static_assert(!std::is_same<CS, Angles>::value, "angles go through rope_span_kernel");
    const int hl = a.lpv, lps = hl * 2, lph = a.lph, spw = a.spw;
    const int lane = threadIdx.x & (kWave - 1);
    const uint32_t wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int sw = (lane * a.lph_magic) >> 16;
    const int slot = lane - sw * lph;
    const bool rotated = slot < lps;
    const bool second = slot >= hl;
    const int partner = (second ? lane - hl : lane + hl) & (kWave - 1);
    const int j = slot * W;
    const int jt = rotated ? j : 0;
    const int jp = rotated ? (second ? slot - hl : slot + hl) * W : 0;
    constexpr uint32_t U = 4 * ITERS;  // units per block
    // A unit is addressed through buffers of exactly its bytes: the lane's offset inside the unit
    // is the same for every unit, the surplus lanes of a wave (sw == spw) lie outside and move
    // nothing, and no branch surrounds a memory access.
    const uint32_t unit_bytes = (uint32_t)spw * (uint32_t)a.vec_elems * 2u;
    const uint32_t lane_off = ((uint32_t)sw * (uint32_t)a.vec_elems + (uint32_t)j) * 2u;

    uint32_t xq[ITERS][W / 2], xk[ITERS][W / 2];
    float c[ITERS][W], sn[ITERS][W];
    size_t base[ITERS];    // byte offset of the unit in every tensor
    uint32_t bytes[ITERS];  // its size, 0 past the last unit
    uint32_t upos[ITERS];
#pragma unroll
    for (int u = 0; u < ITERS; ++u) {
        // unit of this wave in iteration u: the units of a wave are neighbours, so that they mostly
        // share a position and with it the cos/sin values
        const uint32_t l = wave * ITERS + u;
        uint32_t unit;
        const uint32_t b = blockIdx.x, upp = a.units_per_piece;
        if (upp == 0 || b >= a.affine_blocks) {
            unit = b * U + l;
        } else {
            const uint32_t g = b >> 3, x = b & 7u, pj = l / upp, t = l - pj * upp;
            unit = (g * 8u * (U / upp) + pj * 8u + x) * upp + t;
        }
        const bool live = unit < a.n_units;  // wave-uniform
        const uint32_t v0 = live ? unit * (uint32_t)spw : 0u;
        base[u] = (size_t)v0 * (uint32_t)a.vec_elems * 2u;
        bytes[u] = live ? unit_bytes : 0u;
        buf_ld_words<W>(make_rsrc(a.t[0].in + base[u], bytes[u]), lane_off, xq[u]);
        buf_ld_words<W>(make_rsrc(a.t[1].in + base[u], a.nt > 1 ? bytes[u] : 0u), lane_off, xk[u]);
        upos[u] = v0 / a.vecs_per_pos;
        if (u > 0 && upos[u] == upos[u - 1]) {  // wave-uniform
#pragma unroll
            for (int k = 0; k < W; ++k) {
                c[u][k] = c[u - 1][k];
                sn[u][k] = sn[u - 1][k];
            }
        } else {
            const int64_t crow = (int64_t)(upos[u] + a.pos_offset) * a.cs_stride;
            load_table<CS, W>(a.cos, crow + jt, c[u]);
            load_table<CS, W>(a.sin, crow + (BWD ? jp : jt), sn[u]);
            if (second == BWD) {
#pragma unroll
                for (int k = 0; k < W; ++k) sn[u][k] = -sn[u][k];
            }
        }
    }
#pragma unroll
    for (int u = 0; u < ITERS; ++u) {
#pragma unroll
        for (int t = 0; t < 2; ++t) {
            const uint32_t(&x)[W / 2] = t ? xk[u] : xq[u];
            float xf[W], pf[W], o[W];
#pragma unroll
            for (int k = 0; k < W / 2; ++k) {
                const uint32_t p = (uint32_t)__shfl((int)x[k], partner);
                Elem<T>::unpack(x[k], xf[2 * k], xf[2 * k + 1]);
                Elem<T>::unpack(p, pf[2 * k], pf[2 * k + 1]);
            }
            {
#pragma clang fp contract(off)
#pragma unroll
                for (int k = 0; k < W; ++k) o[k] = xf[k] * c[u][k] + pf[k] * sn[u][k];
            }
            uint32_t ow[W / 2];
#pragma unroll
            for (int k = 0; k < W / 2; ++k) {
                const uint32_t packed = Elem<T>::pack(o[2 * k], o[2 * k + 1]);
                ow[k] = rotated ? packed : x[k];
            }
            buf_st_words<W>(make_rsrc(a.t[t].out + base[u], (t == 0 || a.nt > 1) ? bytes[u] : 0u), lane_off, ow);
        }
    }
}

}  // namespace neox
