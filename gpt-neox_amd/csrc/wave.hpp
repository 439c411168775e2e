// Device-side building blocks shared by the gfx950 kernels: 128-bit packed
// half/bfloat16 access, fp32 <-> 16-bit conversion, and wave64 reductions done
// with DPP row operations plus four lane reads (no LDS traffic).
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

// Streaming 128-bit access: every byte of these kernels is touched exactly once,
// so the loads/stores carry the non-temporal hint and do not displace each other in L2.
__device__ __forceinline__ u32x4 ld128(const void* p) {
    return __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(p));
}
__device__ __forceinline__ void st128(void* p, const u32x4& v) {
    __builtin_nontemporal_store(v, reinterpret_cast<u32x4*>(p));
}
__device__ __forceinline__ u32x2 ld64(const void* p) {
    return __builtin_nontemporal_load(reinterpret_cast<const u32x2*>(p));
}
// cached variants (data that several waves re-read: masks, cos/sin tables)
__device__ __forceinline__ u32x4 ld128_cached(const void* p) {
    return *reinterpret_cast<const u32x4*>(p);
}
__device__ __forceinline__ u32x2 ld64_cached(const void* p) {
    return *reinterpret_cast<const u32x2*>(p);
}

// ---- wave64 reductions --------------------------------------------------------
// DPP controls (GCN3+/CDNA encoding)
constexpr int kDppQuadSwap1 = 0xB1;    // quad_perm:[1,0,3,2]
constexpr int kDppQuadSwap2 = 0x4E;    // quad_perm:[2,3,0,1]
constexpr int kDppRowHalfMirror = 0x141;
constexpr int kDppRowMirror = 0x140;

template <int Ctrl>
__device__ __forceinline__ float dpp(float v) {
    int r = __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), Ctrl, 0xF, 0xF, false);
    return __builtin_bit_cast(float, r);
}

__device__ __forceinline__ float lane_read(float v, int lane) {
    return __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), lane));
}

struct OpMax {
    static __device__ __forceinline__ float f(float a, float b) { return fmaxf(a, b); }
};
struct OpSum {
    static __device__ __forceinline__ float f(float a, float b) { return a + b; }
};

// Reduce across each DPP row (16 consecutive lanes); every lane of the row gets the result.
template <typename Op>
__device__ __forceinline__ float row16_reduce(float v) {
    v = Op::f(v, dpp<kDppQuadSwap1>(v));
    v = Op::f(v, dpp<kDppQuadSwap2>(v));
    v = Op::f(v, dpp<kDppRowHalfMirror>(v));
    v = Op::f(v, dpp<kDppRowMirror>(v));
    return v;
}

// Reduce across the whole wave; the result is wave-uniform.
template <typename Op>
__device__ __forceinline__ float wave_reduce(float v) {
    v = row16_reduce<Op>(v);
    float a = Op::f(lane_read(v, 0), lane_read(v, 16));
    float b = Op::f(lane_read(v, 32), lane_read(v, 48));
    return Op::f(a, b);
}

constexpr float kLog2e = 1.4426950408889634f;

__device__ __forceinline__ float fast_exp2(float x) { return __builtin_amdgcn_exp2f(x); }

}  // namespace neox
