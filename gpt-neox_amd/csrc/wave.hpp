// Device-side building blocks shared by the gfx950 kernels: 128-bit packed
// half/bfloat16 access (flat and range-checked buffer forms), fp32 <-> 16-bit
// conversion, and reductions over a wave64 or over lane groups inside it done with
// DPP row operations, one swizzle and four lane reads (no LDS traffic).
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

namespace neox {

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));
typedef float f32x2 __attribute__((ext_vector_type(2)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef _Float16 f16x2 __attribute__((ext_vector_type(2)));
typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));

constexpr int kWave = 64;         // gfx950 wavefront width
constexpr int kVec = 8;           // 16-bit elements per 128-bit access
constexpr int kChunk = kWave * kVec;  // columns one wave covers per 128-bit access (512)

struct F16 {};   // element tags: the kernels see raw 16-bit storage
struct BF16 {};

template <typename T>
struct Elem;

template <>
struct Elem<F16> {
    static __device__ __forceinline__ void unpack(uint32_t w, float& lo, float& hi) {
        f16x2 v = __builtin_bit_cast(f16x2, w);
        lo = (float)v.x;
        hi = (float)v.y;
    }
    // round-to-nearest-even (v_cvt_pk_f16_f32 under the default rounding mode)
    static __device__ __forceinline__ uint32_t pack(float lo, float hi) {
        f32x2 v = {lo, hi};
        return __builtin_bit_cast(uint32_t, __builtin_convertvector(v, f16x2));
    }
    static __device__ __forceinline__ float load1(const void* p) {
        return (float)*reinterpret_cast<const _Float16*>(p);
    }
    static __device__ __forceinline__ void store1(void* p, float v) {
        *reinterpret_cast<_Float16*>(p) = (_Float16)v;
    }
};

template <>
struct Elem<BF16> {
    static __device__ __forceinline__ void unpack(uint32_t w, float& lo, float& hi) {
        lo = __builtin_bit_cast(float, w << 16);
        hi = __builtin_bit_cast(float, w & 0xffff0000u);
    }
    // round-to-nearest-even (v_cvt_pk_bf16_f32)
    static __device__ __forceinline__ uint32_t pack(float lo, float hi) {
        f32x2 v = {lo, hi};
        return __builtin_bit_cast(uint32_t, __builtin_convertvector(v, bf16x2));
    }
    static __device__ __forceinline__ float load1(const void* p) {
        uint32_t w = *reinterpret_cast<const uint16_t*>(p);
        return __builtin_bit_cast(float, w << 16);
    }
    static __device__ __forceinline__ void store1(void* p, float v) {
        *reinterpret_cast<__bf16*>(p) = (__bf16)v;
    }
};

// 8 packed elements -> 8 floats
template <typename T>
__device__ __forceinline__ void unpack8(const u32x4& w, float (&f)[8]) {
    Elem<T>::unpack(w.x, f[0], f[1]);
    Elem<T>::unpack(w.y, f[2], f[3]);
    Elem<T>::unpack(w.z, f[4], f[5]);
    Elem<T>::unpack(w.w, f[6], f[7]);
}

template <typename T>
__device__ __forceinline__ u32x4 pack8(const float (&f)[8]) {
    u32x4 w;
    w.x = Elem<T>::pack(f[0], f[1]);
    w.y = Elem<T>::pack(f[2], f[3]);
    w.z = Elem<T>::pack(f[4], f[5]);
    w.w = Elem<T>::pack(f[6], f[7]);
    return w;
}

// The compiler learns nothing about `w` across this point: values it derived from `w` earlier
// (an unpacked copy, say) are computed again afterwards rather than kept in registers.
__device__ __forceinline__ void forget_origin(u32x4& w) {
    asm volatile("" : "+v"(w.x), "+v"(w.y), "+v"(w.z), "+v"(w.w));
}

// Streaming 128-bit access: every byte of these kernels is touched exactly once,
// so the loads/stores carry the non-temporal hint and do not displace each other in L2.
__device__ __forceinline__ u32x4 ld128(const void* p) {
    return __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(p));
}
__device__ __forceinline__ void st128(void* p, const u32x4& v) {
    __builtin_nontemporal_store(v, reinterpret_cast<u32x4*>(p));
}

// ---- buffer (range-checked) access --------------------------------------------------
// A buffer resource describes one row: base address and its length in bytes.  Lanes whose
// byte offset falls outside [0, bytes) load zeros / store nothing and cause no memory
// traffic, so partially filled rows need no branch around their loads and stores -- and
// with a fixed number of memory instructions per row the compiler can wait on exactly the
// loads it needs while later stores are still in flight.  The range check covers the
// per-lane offset plus the instruction's immediate; a scalar offset operand is NOT
// checked, so callers keep `soffset` at 0.
typedef __amdgpu_buffer_rsrc_t rsrc_t;
constexpr int kRsrcFlags = 0x00020000;  // raw buffer, 32-bit data format (gfx9 family)
constexpr int kAuxNt = 2;               // non-temporal hint

__device__ __forceinline__ rsrc_t make_rsrc(const void* base, uint32_t bytes) {
    return __builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(base), 0, (int)bytes, kRsrcFlags);
}
template <bool NT>
__device__ __forceinline__ u32x4 buf_ld128(rsrc_t r, int voffset, int soffset) {
    return __builtin_amdgcn_raw_buffer_load_b128(r, voffset, soffset, NT ? kAuxNt : 0);
}
template <bool NT>
__device__ __forceinline__ void buf_st128(rsrc_t r, const u32x4& v, int voffset, int soffset) {
    __builtin_amdgcn_raw_buffer_store_b128(v, r, voffset, soffset, NT ? kAuxNt : 0);
}
__device__ __forceinline__ u32x2 buf_ld64(rsrc_t r, int voffset, int soffset) {
    return __builtin_amdgcn_raw_buffer_load_b64(r, voffset, soffset, 0);
}
// Narrow accesses for the ends of rows that are not a whole number of dwords.
__device__ __forceinline__ uint32_t buf_ld32(rsrc_t r, int voffset) {
    return __builtin_amdgcn_raw_buffer_load_b32(r, voffset, 0, 0);
}
__device__ __forceinline__ uint32_t buf_ld16(rsrc_t r, int voffset) {
    return __builtin_amdgcn_raw_buffer_load_b16(r, voffset, 0, 0);
}
typedef uint32_t u32x3 __attribute__((ext_vector_type(3)));
__device__ __forceinline__ u32x3 buf_ld96(rsrc_t r, int voffset) {
    return __builtin_amdgcn_raw_buffer_load_b96(r, voffset, 0, 0);
}
__device__ __forceinline__ void buf_st96(rsrc_t r, const u32x3& v, int voffset) {
    __builtin_amdgcn_raw_buffer_store_b96(v, r, voffset, 0, 0);
}
__device__ __forceinline__ void buf_st16(rsrc_t r, uint32_t v, int voffset) {
    __builtin_amdgcn_raw_buffer_store_b16((unsigned short)v, r, voffset, 0, 0);
}

// ---- wave64 reductions --------------------------------------------------------
// DPP controls (GCN3+/CDNA encoding)
constexpr int kDppQuadSwap1 = 0xB1;    // quad_perm:[1,0,3,2]
constexpr int kDppQuadSwap2 = 0x4E;    // quad_perm:[2,3,0,1]
constexpr int kDppRowHalfMirror = 0x141;
constexpr int kDppRowMirror = 0x140;
constexpr int kSwizzleXor16 = 0x401F;  // ds_swizzle bit mode: and 0x1f, or 0, xor 0x10

struct OpSum {
    typedef float type;
    static __device__ __forceinline__ float f(float a, float b) { return a + b; }
    static __device__ __forceinline__ float enc(float v) { return v; }
    static __device__ __forceinline__ float dec(float v) { return v; }
};
// Maximum of floats taken on order-preserving integer keys (sign-magnitude -> two's
// complement): v_max_i32 needs no NaN canonicalisation of the shuffled operand, so each
// step is a single DPP instruction.  -inf and finite values order as floats do.
struct OpMax {
    typedef int type;
    static __device__ __forceinline__ int f(int a, int b) { return a > b ? a : b; }
    static __device__ __forceinline__ int enc(float v) {
        const int b = __builtin_bit_cast(int, v);
        return b ^ ((b >> 31) & 0x7fffffff);
    }
    static __device__ __forceinline__ float dec(int k) {
        return __builtin_bit_cast(float, k ^ ((k >> 31) & 0x7fffffff));
    }
};

template <int Ctrl, typename V>
__device__ __forceinline__ V dpp(V v) {
    const int r = __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), Ctrl, 0xF, 0xF, false);
    return __builtin_bit_cast(V, r);
}
template <typename V>
__device__ __forceinline__ V lane_read(V v, int lane) {
    return __builtin_bit_cast(V, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), lane));
}

// Reduce across aligned groups of G consecutive lanes (G a power of two); every lane of a
// group gets the group's result.  Steps of 1..8 lanes are DPP operations, 16 is a
// ds_swizzle (no LDS memory is touched), the last step of a full wave reads four lanes.
// Must be called with all 64 lanes active.
template <typename Op, int G>
__device__ __forceinline__ float group_reduce(float x) {
    static_assert(G == 1 || G == 2 || G == 4 || G == 8 || G == 16 || G == 32 || G == 64, "group size");
    typedef typename Op::type V;
    V v = Op::enc(x);
    if constexpr (G >= 2) v = Op::f(v, dpp<kDppQuadSwap1>(v));
    if constexpr (G >= 4) v = Op::f(v, dpp<kDppQuadSwap2>(v));
    if constexpr (G >= 8) v = Op::f(v, dpp<kDppRowHalfMirror>(v));
    if constexpr (G >= 16) v = Op::f(v, dpp<kDppRowMirror>(v));
    if constexpr (G == 32) {
        const int o = __builtin_amdgcn_ds_swizzle(__builtin_bit_cast(int, v), kSwizzleXor16);
        v = Op::f(v, __builtin_bit_cast(V, o));
    }
    if constexpr (G == 64) {
        const V a = Op::f(lane_read(v, 0), lane_read(v, 16));
        const V b = Op::f(lane_read(v, 32), lane_read(v, 48));
        v = Op::f(a, b);
    }
    return Op::dec(v);
}

// Reduce across the whole wave; the result is wave-uniform.
template <typename Op>
__device__ __forceinline__ float wave_reduce(float v) {
    return group_reduce<Op, kWave>(v);
}

constexpr float kLog2e = 1.4426950408889634f;

__device__ __forceinline__ float fast_exp2(float x) { return __builtin_amdgcn_exp2f(x); }

}  // namespace neox
