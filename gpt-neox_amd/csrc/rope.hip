// Rotary embedding kernels and their launcher.
#include "internal.hpp"

namespace neox {

// LDS for the cos/sin values a block evaluates from angles: 2 x d_rot floats (at most 32 KiB)
template <typename CS>
static size_t angle_lds_bytes(const RopeArgs& a) {
    return std::is_same<CS, Angles>::value ? (size_t)a.half * 4 * sizeof(float) : 0;
}

template <typename T, typename CS, int W, bool BWD>
static hipError_t launch_rope_shape(const RopeArgs& a, int s, int n_outer, hipStream_t st) {
    const int lpv = a.lpv;
    const int vpb = (256 / lpv) > 0 ? (256 / lpv) : 1;  // vectors per block iteration
    int nmax = a.t[0].n_inner;
    if (a.nt > 1 && a.t[1].n_inner > nmax) nmax = a.t[1].n_inner;
    const int iters = (nmax + vpb - 1) / vpb;
    // split the vector loop over blockIdx.z until the grid has a few thousand blocks
    long long blocks = (long long)s * n_outer;
    int zsplit = 1;
    if (blocks < 4096) {
        zsplit = (int)((4096 + blocks - 1) / blocks);
        if (zsplit > iters) zsplit = iters;
        if (zsplit > 65535) zsplit = 65535;
        if (zsplit < 1) zsplit = 1;
    }
    const dim3 grid(s, n_outer, zsplit);
    const dim3 block(lpv, vpb);
    hipLaunchKernelGGL((rope_kernel<T, CS, W, BWD>), grid, block, angle_lds_bytes<CS>(a), st, a);
    return hipGetLastError();
}

template <typename T, typename CS, int W, bool BWD>
static bool try_launch_rope_piece(const RopeArgs& a, int s, int n_outer, hipStream_t st, hipError_t* err);

template <typename T, typename CS, int W, bool BWD>
static hipError_t launch_rope_span(const RopeArgs& a, int s, int n_outer, hipStream_t st) {
    RopeArgs b = a;
    b.lph = a.lpv * 2 + a.pad_slots;
    b.lph_magic = (65536 + b.lph - 1) / b.lph;
    b.spw = kWave / b.lph;
    if constexpr (!std::is_same<CS, Angles>::value) {
        hipError_t err = hipSuccess;
        if (try_launch_rope_piece<T, CS, W, BWD>(b, s, n_outer, st, &err)) return err;
    }
    const int vpb = (256 / kWave) * b.spw * kSpanIters;  // vectors per block iteration
    int nmax = a.t[0].n_inner;
    if (a.nt > 1 && a.t[1].n_inner > nmax) nmax = a.t[1].n_inner;
    // one loop iteration per block: many short-lived blocks measured faster than fewer blocks
    // that loop (the cos/sin values a block reloads come from L2)
    long long zsplit = (nmax + vpb - 1) / vpb;
    const long long pairs = (long long)s * n_outer;
    if (pairs * zsplit > 0x7fffffffLL) zsplit = 0x7fffffffLL / pairs;  // grid.x limit: blocks loop instead
    if (zsplit < 1) return hipErrorInvalidValue;
    b.zsplit = (int)zsplit;
    b.outer_grid = n_outer;
    b.share = (int)((nmax + zsplit - 1) / zsplit);
    hipLaunchKernelGGL((rope_span_kernel<T, CS, W, BWD>), dim3((unsigned)(pairs * zsplit)), dim3(256),
                       angle_lds_bytes<CS>(a), st, b);
    return hipGetLastError();
}

// Dense tensors laid out alike: the XCD-aware piece kernel (see rope_piece_kernel).  `a` comes
// from launch_rope_span's preparation (lph, spw set).  Returns false if the shape does not qualify.
template <typename T, typename CS, int W, bool BWD>
static bool try_launch_rope_piece(const RopeArgs& a, int s, int n_outer, hipStream_t st, hipError_t* err) {
    if (std::is_same<CS, Angles>::value) return false;
    const RopeTensor& q = a.t[0];
    // [s, b, h, d] dense: head vectors `vec` elements apart in one run, in and out, q and k
    const int64_t vec = q.in_stride[2];
    const int64_t vecs_per_pos = (int64_t)n_outer * q.n_inner;
    auto dense = [&](const RopeTensor& t) {
        for (int i = 0; i < 3; ++i)
            if (t.in_stride[i] != q.in_stride[i] || t.out_stride[i] != q.in_stride[i]) return false;
        return t.n_inner == q.n_inner && t.n_outer == q.n_outer;
    };
    if (vec < (int64_t)(a.lpv * 2 + a.pad_slots) * W || vec > 0x7fffffff) return false;
    if (q.in_stride[0] != vecs_per_pos * vec) return false;
    if (n_outer > 1 && q.in_stride[1] != (int64_t)q.n_inner * vec) return false;
    if (!dense(q) || (a.nt > 1 && !dense(a.t[1]))) return false;
    if (vecs_per_pos % a.spw != 0 || vecs_per_pos > 0x7fffffff) return false;
    if ((int64_t)a.spw * vec * 2 > 0x7fffffffLL) return false;  // a unit is addressed through one 32-bit buffer
    const int64_t units = (int64_t)s * vecs_per_pos / a.spw;
    if (units > 0x7fffffffLL || (int64_t)s * vecs_per_pos > 0xffffffffLL) return false;
    RopeArgs b = a;
    b.vec_elems = (int32_t)vec;
    b.vecs_per_pos = (uint32_t)vecs_per_pos;
    b.n_units = (uint32_t)units;
    constexpr int ITERS = kSpanIters;
    const uint32_t U = 4 * ITERS;
    const uint32_t blocks = (uint32_t)((units + U - 1) / U);
    // XCD-aware order where the units tile 4 KiB pieces and the tensors start on a piece boundary
    const int64_t unit_bytes = (int64_t)a.spw * vec * 2;
    auto aligned = [](const void* p) { return (reinterpret_cast<uintptr_t>(p) & 4095u) == 0; };
    b.units_per_piece = 0;
    b.affine_blocks = 0;
    bool on_pieces = unit_bytes <= 4096 && 4096 % unit_bytes == 0 && blocks >= 8 && aligned(q.out) &&
                     (a.nt < 2 || aligned(a.t[1].out));
    if (on_pieces) {
        const uint32_t upp = (uint32_t)(4096 / unit_bytes);
        if (U % upp == 0) {
            b.units_per_piece = upp;
            b.affine_blocks = blocks & ~7u;
        }
    }
    // without that order the kernel has nothing over rope_span_kernel, which loads its cos/sin
    // values once per block (20B shape, 192-byte heads: 45.6 against 42.6 us)
    if (b.units_per_piece == 0) return false;
    hipLaunchKernelGGL((rope_piece_kernel<T, CS, W, BWD, ITERS>), dim3(blocks), dim3(256), 0, st, b);
    *err = hipGetLastError();
    return true;
}

// the rotated span, with the slots stored as loaded behind it, is at most 64 slots of w >= 2 dims:
// the contiguous-span kernel applies (a pass-through copy must be covered by those slots)
static bool span_shape(const RopeArgs& a, int w) {
    return w >= 2 && a.lpv * 2 + a.pad_slots <= kWave && (a.copy_dims == 0 || a.pad_slots * w == a.copy_dims);
}

template <typename T, typename CS, bool BWD>
static hipError_t launch_rope_w(const RopeArgs& a, int s, int n_outer, int w, hipStream_t st) {
    if (span_shape(a, w)) {
        switch (w) {
            case 8: return launch_rope_span<T, CS, 8, BWD>(a, s, n_outer, st);
            case 4: return launch_rope_span<T, CS, 4, BWD>(a, s, n_outer, st);
            default: return launch_rope_span<T, CS, 2, BWD>(a, s, n_outer, st);
        }
    }
    switch (w) {
        case 8: return launch_rope_shape<T, CS, 8, BWD>(a, s, n_outer, st);
        case 4: return launch_rope_shape<T, CS, 4, BWD>(a, s, n_outer, st);
        case 2: return launch_rope_shape<T, CS, 2, BWD>(a, s, n_outer, st);
        case 1: return launch_rope_shape<T, CS, 1, BWD>(a, s, n_outer, st);
        default: return hipErrorInvalidValue;
    }
}

template <typename T, typename CS>
static hipError_t launch_rope_dir(const RopeArgs& a, int s, int n_outer, int w, bool backward,
                                  hipStream_t st) {
    return backward ? launch_rope_w<T, CS, true>(a, s, n_outer, w, st)
                    : launch_rope_w<T, CS, false>(a, s, n_outer, w, st);
}

hipError_t launch_rope(const RopeArgs& a, int s, int n_outer, int w, int dtype, int cs_dtype,
                       bool backward, hipStream_t stream) {
    if (cs_dtype == kRopeAngles) {
        return dtype == NEOX_F16 ? launch_rope_dir<F16, Angles>(a, s, n_outer, w, backward, stream)
                                 : launch_rope_dir<BF16, Angles>(a, s, n_outer, w, backward, stream);
    }
    const bool cs32 = (cs_dtype == NEOX_F32);
    if (dtype == NEOX_F16) {
        return cs32 ? launch_rope_dir<F16, float>(a, s, n_outer, w, backward, stream)
                    : launch_rope_dir<F16, F16>(a, s, n_outer, w, backward, stream);
    }
    return cs32 ? launch_rope_dir<BF16, float>(a, s, n_outer, w, backward, stream)
                : launch_rope_dir<BF16, BF16>(a, s, n_outer, w, backward, stream);
}

}  // namespace neox
