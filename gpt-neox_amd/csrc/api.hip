// extern "C" entry points of libneox_fused.so: argument validation, error
// reporting and hand-off to the launchers.  Validation finishes before the
// first HIP call, so it behaves the same on a host without a GPU.
#include <stdarg.h>
#include <stdio.h>

#include <initializer_list>

#include "internal.hpp"

namespace neox {

static thread_local char g_last_error[256] = {0};

int fail(int status, const char* fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_last_error, sizeof(g_last_error), fmt, ap);
    va_end(ap);
    return status;
}

static inline bool aligned(const void* p, uintptr_t n) {
    return (reinterpret_cast<uintptr_t>(p) & (n - 1)) == 0;
}

static int check_launch(hipError_t e, const char* what) {
    if (e == hipSuccess) return NEOX_OK;
    return fail(NEOX_ERR_LAUNCH, "%s: kernel launch failed: %s", what, hipGetErrorString(e));
}

static int check_dtype(int dtype, const char* what) {
    if (dtype == NEOX_F16 || dtype == NEOX_BF16) return NEOX_OK;
    return fail(NEOX_ERR_BAD_DTYPE, "%s: Only fp16 and bf16 are supported (dtype code %d)", what,
                dtype);
}

// rows of a [.., sq, sk] score tensor must be countable in 31 bits
static int check_rows(int64_t rows, int sq, int sk, const char* what) {
    if (sq < 1 || sk < 1) return fail(NEOX_ERR_BAD_SHAPE, "%s: sq=%d sk=%d must be >= 1", what, sq, sk);
    if (rows < 1 || rows > 0x7fffffffLL)
        return fail(NEOX_ERR_BAD_SHAPE, "%s: row count %lld outside [1, 2^31)", what,
                    (long long)rows);
    return NEOX_OK;
}

// Dropout parameters of a call: threshold in 16-bit units and the fp32 factor 1/(1-p)
// formed as torch's dropout kernel forms it (fp32 keep probability, then the quotient).
static int make_dropout(DropoutArgs& d, float p, uint64_t seed, uint64_t offset,
                        const uint64_t* device_state, const char* what) {
    if (!(p >= 0.f && p <= 1.f))
        return fail(NEOX_ERR_BAD_SHAPE, "%s: dropout probability has to be between 0 and 1, but got %g", what, (double)p);
    if (!aligned(device_state, 8))
        return fail(NEOX_ERR_MISALIGNED, "%s: device_state must be 8-byte aligned", what);
    d.state = device_state;
    d.seed_lo = (uint32_t)seed;
    d.seed_hi = (uint32_t)(seed >> 32);
    d.off_lo = (uint32_t)(offset >> 2);  // the Philox block the offset lies in (4 outputs per block)
    d.off_hi = (uint32_t)(offset >> 34);
    d.threshold = (uint32_t)__builtin_rint((double)p * 65536.0);
    const float keep = (float)(1.0 - (double)p);
    d.scale = p >= 1.f ? 0.f : (float)(1.0 / (double)keep);
    return NEOX_OK;
}

// One softmax call under validation.  The checks run in a fixed order -- null pointers,
// dtype, shape, alignment, then the optional parts -- and the first failure sticks in
// `status`; nothing here touches the GPU.  The 16-bit tensors given to the constructor
// also decide whether 128-bit accesses are legal (`vec_ok`).
struct SoftmaxCall {
    const char* what;
    int dtype;
    int status = NEOX_OK;
    bool vec_ok = true;
    int features = 0;  // kAlibi | kBias | kDropout, by what the call brings along
    SoftmaxArgs a{};

    SoftmaxCall(const char* name, int dtype_code, std::initializer_list<const void*> tensors,
                const void* extra = reinterpret_cast<const void*>(1))
        : what(name), dtype(dtype_code) {
        bool null = (extra == nullptr), odd = false;
        for (const void* t : tensors) {
            null = null || t == nullptr;
            odd = odd || !aligned(t, 2);
            vec_ok = vec_ok && aligned(t, 16);
        }
        if (null) {
            status = fail(NEOX_ERR_NULL_POINTER, "%s: null tensor pointer", what);
        } else if ((status = check_dtype(dtype, what)) == NEOX_OK && odd) {
            misaligned_ = true;  // reported after the shape checks
        }
    }

    // [batches, sq, sk]
    void causal_rows(int64_t batches, int sq, int sk) {
        if (status) return;
        if (batches < 1) {
            status = fail(NEOX_ERR_BAD_SHAPE, "%s: batches=%lld must be >= 1", what, (long long)batches);
            return;
        }
        rows(sq < 1 ? 0 : batches * sq, sq, sk);
    }
    // [b, np, sq, sk]
    void head_rows(int b, int np, int sq, int sk) {
        if (status) return;
        if (b < 1 || np < 1) {
            status = fail(NEOX_ERR_BAD_SHAPE, "%s: b=%d np=%d must be >= 1", what, b, np);
            return;
        }
        rows(sq < 1 ? 0 : (int64_t)b * np * sq, sq, sk);
    }
    // [rows, sk]
    void plain_rows(int64_t n, int sk) { if (!status) rows(n, 1, sk); }

    // mask bytes [mask_b, 1, sq, sk]
    void mask(const uint8_t* m, int b, int np, int mask_b) {
        if (status) return;
        if (mask_b != 1 && mask_b != b) {
            status = fail(NEOX_ERR_BAD_SHAPE, "%s: mask batch dim %d must be 1 or b=%d", what, mask_b, b);
            return;
        }
        a.mask = m;
        a.rows_per_mask_batch = (uint32_t)((int64_t)np * a.sq);
        a.mask_bcast = (mask_b == 1 && b != 1) ? 1 : 0;
        a.mask_bytes = fits32((uint64_t)mask_b * (uint64_t)a.sq * (uint64_t)a.sk);
        vec_ok = vec_ok && aligned(m, 8);
    }
    // bias [bias_b, np, sq, sk] in the dtype of the scores
    void bias(const void* t, int b, int np, int bias_b) {
        if (status) return;
        if (bias_b != 1 && bias_b != b) {
            status = fail(NEOX_ERR_BAD_SHAPE, "%s: bias batch dim %d must be 1 or b=%d", what, bias_b, b);
            return;
        }
        if (!aligned(t, 2)) {
            status = fail(NEOX_ERR_MISALIGNED, "%s: misaligned pointer", what);
            return;
        }
        vec_ok = vec_ok && aligned(t, 16);
        a.bias = t;
        a.bias_rows = (bias_b == 1 && b != 1) ? (uint32_t)((int64_t)np * a.sq) : 0u;
        a.bias_bytes = fits32((uint64_t)bias_b * (uint64_t)np * (uint64_t)a.sq * (uint64_t)a.sk * 2u);
        features |= kBias;
    }
    // which mask row [mask_b, 1, sq, .] a score row belongs to, for a call that brings no mask tensor
    void mask_rows(int b, int np, int mask_b) {
        if (status) return;
        if (mask_b != 1 && mask_b != b) {
            status = fail(NEOX_ERR_BAD_SHAPE, "%s: mask batch dim %d must be 1 or b=%d", what, mask_b, b);
            return;
        }
        a.rows_per_mask_batch = (uint32_t)((int64_t)np * a.sq);
        a.mask_bcast = (mask_b == 1 && b != 1) ? 1 : 0;
    }
    // where the visible keys of every mask row end, int32 [mask_b * sq]; null = no hint
    void row_ends(const int32_t* ends) {
        if (status || !ends) return;
        if (!aligned(ends, 4)) {
            status = fail(NEOX_ERR_MISALIGNED, "%s: misaligned pointer", what);
            return;
        }
        a.row_end = ends;
    }
    // ALiBi slopes, fp32 [np]
    void alibi(const float* slopes, int np) {
        if (status) return;
        if (!aligned(slopes, 4)) {
            status = fail(NEOX_ERR_MISALIGNED, "%s: misaligned pointer", what);
            return;
        }
        a.slopes = slopes;
        a.np = (uint32_t)np;
        features |= kAlibi;
    }
    void dropout(float p, uint64_t seed, uint64_t offset, const uint64_t* device_state) {
        if (!status) status = make_dropout(a.drop, p, seed, offset, device_state, what);
        features |= kDropout;
    }
    void second_output(void* y_drop, const void* y) {
        if (status) return;
        if (y_drop == y) status = fail(NEOX_ERR_BAD_STRIDE, "%s: y_drop must not alias y", what);
        a.out2 = y_drop;
    }

    void forward(void* y, const void* x, float scale) {
        a.out = y;
        a.in0 = x;
        a.scale = scale * kLog2e;
    }
    void backward(void* dx, const void* dy, const void* y, float scale) {
        a.out = dx;
        a.in0 = dy;
        a.in1 = y;
        a.scale = scale;
    }
    // The translation unit of the call's feature set; rows that rule out aligned 128-bit accesses
    // go to its kRagged twin, and outside that twin's range of row lengths to the element-wise kernels.
    int launch(bool backward, Mask m, void* stream) const {
        const bool vec = vec_ok && a.sk % kVec == 0;
        int flags = backward ? (features & kDropout) : features;
        if (!vec && a.sk >= kVec && a.sk < kMaxStagedRow) flags |= kRagged;
        const hipError_t e = backward ? launch_softmax_bwd(flags, a, m, dtype, vec, (hipStream_t)stream)
                                      : launch_softmax_fwd(flags, a, m, dtype, vec, (hipStream_t)stream);
        return check_launch(e, what);
    }

  private:
    bool misaligned_ = false;

    void rows(int64_t n, int sq, int sk) {
        if ((status = check_rows(n, sq, sk, what)) != NEOX_OK) return;
        if (misaligned_) {
            status = fail(NEOX_ERR_MISALIGNED, "%s: misaligned pointer", what);
            return;
        }
        a.rows = (uint32_t)n;
        a.sq = sq;
        a.sk = sk;
    }
    // size of a tensor the packed kernels address through one buffer, 0 if it needs more than 32 bits
    static uint32_t fits32(uint64_t bytes) { return bytes < 0xFFFFFFFFull ? (uint32_t)bytes : 0u; }
};

// The keep pattern of the dropout kernels, one byte per element (1 = kept).
__global__ __launch_bounds__(256) void keep_mask_kernel(uint8_t* keep, DropoutArgs d, uint64_t n) {
    const uint64_t group = (uint64_t)blockIdx.x * 256 + threadIdx.x;
    if (group * 8 >= n) return;
    const uint32_t bits = keep_bits8(resolve(d), group);
    for (int k = 0; k < 8; ++k)
        if (group * 8 + k < n) keep[group * 8 + k] = (bits >> k) & 1u;
}

hipError_t launch_softmax_fwd(int flags, const SoftmaxArgs& a, Mask mask, int dtype, bool vec_ok, hipStream_t stream) {
    switch (flags) {
#define NEOX_CASE(F) \
    case F: return launch_softmax_fwd_flags<F>(a, mask, dtype, vec_ok, stream);
        NEOX_FWD_FEATURE_SETS(NEOX_CASE)
#undef NEOX_CASE
    }
    return hipErrorInvalidValue;
}

hipError_t launch_softmax_bwd(int flags, const SoftmaxArgs& a, Mask mask, int dtype, bool vec_ok, hipStream_t stream) {
    switch (flags) {
#define NEOX_CASE(F) \
    case F: return launch_softmax_bwd_flags<F>(a, mask, dtype, vec_ok, stream);
        NEOX_BWD_FEATURE_SETS(NEOX_CASE)
#undef NEOX_CASE
    }
    return hipErrorInvalidValue;
}

}  // namespace neox

using namespace neox;

#pragma GCC visibility push(default)
extern "C" {

int neox_fused_abi_version(void) { return NEOX_FUSED_ABI_VERSION; }

const char* neox_fused_strerror(int status) {
    switch (status) {
        case NEOX_OK: return "success";
        case NEOX_ERR_NULL_POINTER: return "null pointer";
        case NEOX_ERR_BAD_DTYPE: return "Only fp16 and bf16 are supported";
        case NEOX_ERR_BAD_SHAPE: return "unsupported shape";
        case NEOX_ERR_BAD_STRIDE: return "unsupported stride";
        case NEOX_ERR_MISALIGNED: return "pointer not aligned to the element size";
        case NEOX_ERR_LAUNCH: return "kernel launch failed";
        default: return "unknown status";
    }
}

const char* neox_fused_last_error(void) { return g_last_error; }

int neox_causal_softmax_fwd(void* y, const void* x, float scale, int64_t batches, int32_t sq,
                            int32_t sk, int32_t dtype, void* stream) {
    SoftmaxCall c("neox_causal_softmax_fwd", dtype, {y, x});
    c.causal_rows(batches, sq, sk);
    if (c.status) return c.status;
    c.forward(y, x, scale);
    return c.launch(false, Mask::Causal, stream);
}

int neox_causal_softmax_alibi_fwd(void* y, const void* x, const float* slopes, float scale, int32_t b,
                                  int32_t np, int32_t sq, int32_t sk, int32_t dtype, void* stream) {
    SoftmaxCall c("neox_causal_softmax_alibi_fwd", dtype, {y, x}, slopes);
    c.head_rows(b, np, sq, sk);
    c.alibi(slopes, np);
    if (c.status) return c.status;
    c.forward(y, x, scale);
    return c.launch(false, Mask::Causal, stream);
}

int neox_causal_softmax_bwd(void* dx, const void* dy, const void* y, float scale, int64_t batches,
                            int32_t sq, int32_t sk, int32_t dtype, void* stream) {
    SoftmaxCall c("neox_causal_softmax_bwd", dtype, {dx, dy, y});
    c.causal_rows(batches, sq, sk);
    if (c.status) return c.status;
    c.backward(dx, dy, y, scale);
    return c.launch(true, Mask::Causal, stream);
}

int neox_masked_softmax_ends_fwd(void* y_drop, void* y, const void* x, const uint8_t* mask, const int32_t* row_end,
                                 const float* alibi_slopes, const void* bias, int32_t bias_b, float scale, float p,
                                 uint64_t seed, uint64_t offset, const uint64_t* device_state,
                                 int32_t b, int32_t np, int32_t sq, int32_t sk, int32_t mask_b,
                                 int32_t dtype, void* stream) {
    // y_drop: null = no dropout, and p, seed, offset and device_state are not looked at
    SoftmaxCall c("neox_masked_softmax_ends_fwd", dtype, {y, x, y_drop ? y_drop : y}, mask);
    if (y_drop) c.second_output(y_drop, y);
    c.head_rows(b, np, sq, sk);
    c.mask(mask, b, np, mask_b);
    c.row_ends(row_end);
    if (alibi_slopes) c.alibi(alibi_slopes, np);
    if (bias) c.bias(bias, b, np, bias_b);
    if (y_drop) c.dropout(p, seed, offset, device_state);
    if (c.status) return c.status;
    c.forward(y, x, scale);
    return c.launch(false, Mask::Bytes, stream);
}

int neox_masked_softmax_ends_bwd(void* dx, const void* dy, const void* y, const int32_t* row_end, float scale,
                                 int32_t dropout, float p, uint64_t seed, uint64_t offset, const uint64_t* device_state,
                                 int32_t b, int32_t np, int32_t sq, int32_t sk, int32_t mask_b,
                                 int32_t dtype, void* stream) {
    SoftmaxCall c("neox_masked_softmax_ends_bwd", dtype, {dx, dy, y});
    c.head_rows(b, np, sq, sk);
    c.mask_rows(b, np, mask_b);
    c.row_ends(row_end);
    if (dropout) c.dropout(p, seed, offset, device_state);
    if (c.status) return c.status;
    c.backward(dx, dy, y, scale);
    return c.launch(true, Mask::None, stream);
}

int neox_masked_softmax_fwd(void* y, const void* x, const uint8_t* mask, float scale, int32_t b,
                            int32_t np, int32_t sq, int32_t sk, int32_t mask_b, int32_t dtype,
                            void* stream) {
    SoftmaxCall c("neox_masked_softmax_fwd", dtype, {y, x}, mask);
    c.head_rows(b, np, sq, sk);
    c.mask(mask, b, np, mask_b);
    if (c.status) return c.status;
    c.forward(y, x, scale);
    return c.launch(false, Mask::Bytes, stream);
}

int neox_masked_softmax_bwd(void* dx, const void* dy, const void* y, float scale, int64_t rows,
                            int32_t sk, int32_t dtype, void* stream) {
    SoftmaxCall c("neox_masked_softmax_bwd", dtype, {dx, dy, y});
    c.plain_rows(rows, sk);
    if (c.status) return c.status;
    c.backward(dx, dy, y, scale);
    return c.launch(true, Mask::None, stream);
}

int neox_causal_softmax_bias_fwd(void* y, const void* x, const void* bias, const float* alibi_slopes,
                                 float scale, int32_t b, int32_t np, int32_t sq, int32_t sk, int32_t bias_b,
                                 int32_t dtype, void* stream) {
    SoftmaxCall c("neox_causal_softmax_bias_fwd", dtype, {y, x}, bias);
    c.head_rows(b, np, sq, sk);
    c.bias(bias, b, np, bias_b);
    if (alibi_slopes) c.alibi(alibi_slopes, np);
    if (c.status) return c.status;
    c.forward(y, x, scale);
    return c.launch(false, Mask::Causal, stream);
}

int neox_masked_softmax_alibi_fwd(void* y, const void* x, const uint8_t* mask, const float* slopes, float scale,
                                  int32_t b, int32_t np, int32_t sq, int32_t sk, int32_t mask_b, int32_t dtype,
                                  void* stream) {
    if (!slopes) return fail(NEOX_ERR_NULL_POINTER, "neox_masked_softmax_alibi_fwd: null tensor pointer");
    SoftmaxCall c("neox_masked_softmax_alibi_fwd", dtype, {y, x}, mask);
    c.head_rows(b, np, sq, sk);
    c.mask(mask, b, np, mask_b);
    c.alibi(slopes, np);
    if (c.status) return c.status;
    c.forward(y, x, scale);
    return c.launch(false, Mask::Bytes, stream);
}

int neox_masked_softmax_bias_fwd(void* y, const void* x, const uint8_t* mask, const void* bias,
                                 const float* alibi_slopes, float scale, int32_t b, int32_t np, int32_t sq,
                                 int32_t sk, int32_t mask_b, int32_t bias_b, int32_t dtype, void* stream) {
    if (!bias) return fail(NEOX_ERR_NULL_POINTER, "neox_masked_softmax_bias_fwd: null tensor pointer");
    SoftmaxCall c("neox_masked_softmax_bias_fwd", dtype, {y, x}, mask);
    c.head_rows(b, np, sq, sk);
    c.mask(mask, b, np, mask_b);
    c.bias(bias, b, np, bias_b);
    if (alibi_slopes) c.alibi(alibi_slopes, np);
    if (c.status) return c.status;
    c.forward(y, x, scale);
    return c.launch(false, Mask::Bytes, stream);
}

int neox_causal_softmax_dropout_fwd(void* y_drop, void* y, const void* x, const float* alibi_slopes,
                                    const void* bias, int32_t bias_b, float scale, float p,
                                    uint64_t seed, uint64_t offset, const uint64_t* device_state,
                                    int32_t b, int32_t np, int32_t sq, int32_t sk, int32_t dtype,
                                    void* stream) {
    SoftmaxCall c("neox_causal_softmax_dropout_fwd", dtype, {y_drop, y, x});
    c.second_output(y_drop, y);
    c.head_rows(b, np, sq, sk);
    if (alibi_slopes) c.alibi(alibi_slopes, np);
    if (bias) c.bias(bias, b, np, bias_b);
    c.dropout(p, seed, offset, device_state);
    if (c.status) return c.status;
    c.forward(y, x, scale);
    return c.launch(false, Mask::Causal, stream);
}

int neox_causal_softmax_dropout_bwd(void* dx, const void* dy, const void* y, float scale, float p,
                                    uint64_t seed, uint64_t offset, const uint64_t* device_state,
                                    int64_t batches, int32_t sq,
                                    int32_t sk, int32_t dtype, void* stream) {
    SoftmaxCall c("neox_causal_softmax_dropout_bwd", dtype, {dx, dy, y});
    c.causal_rows(batches, sq, sk);
    c.dropout(p, seed, offset, device_state);
    if (c.status) return c.status;
    c.backward(dx, dy, y, scale);
    return c.launch(true, Mask::Causal, stream);
}

int neox_masked_softmax_dropout_fwd(void* y_drop, void* y, const void* x, const uint8_t* mask,
                                    const float* alibi_slopes, const void* bias, int32_t bias_b, float scale, float p,
                                    uint64_t seed, uint64_t offset, const uint64_t* device_state,
                                    int32_t b, int32_t np, int32_t sq, int32_t sk, int32_t mask_b,
                                    int32_t dtype, void* stream) {
    SoftmaxCall c("neox_masked_softmax_dropout_fwd", dtype, {y_drop, y, x}, mask);
    c.second_output(y_drop, y);
    c.head_rows(b, np, sq, sk);
    c.mask(mask, b, np, mask_b);
    if (alibi_slopes) c.alibi(alibi_slopes, np);
    if (bias) c.bias(bias, b, np, bias_b);
    c.dropout(p, seed, offset, device_state);
    if (c.status) return c.status;
    c.forward(y, x, scale);
    return c.launch(false, Mask::Bytes, stream);
}

int neox_masked_softmax_dropout_bwd(void* dx, const void* dy, const void* y, float scale, float p,
                                    uint64_t seed, uint64_t offset, const uint64_t* device_state,
                                    int64_t rows, int32_t sk,
                                    int32_t dtype, void* stream) {
    SoftmaxCall c("neox_masked_softmax_dropout_bwd", dtype, {dx, dy, y});
    c.plain_rows(rows, sk);
    c.dropout(p, seed, offset, device_state);
    if (c.status) return c.status;
    c.backward(dx, dy, y, scale);
    return c.launch(true, Mask::None, stream);
}

int neox_dropout_keep_mask(uint8_t* keep, float p, uint64_t seed, uint64_t offset,
                           const uint64_t* device_state, int64_t n, void* stream) {
    static const char* what = "neox_dropout_keep_mask";
    if (!keep) return fail(NEOX_ERR_NULL_POINTER, "%s: null pointer", what);
    if (n < 1 || n > (int64_t)1 << 40) return fail(NEOX_ERR_BAD_SHAPE, "%s: n=%lld outside [1, 2^40]", what, (long long)n);
    DropoutArgs d{};
    if (int e = make_dropout(d, p, seed, offset, device_state, what)) return e;
    const uint64_t groups = ((uint64_t)n + 7) / 8;
    hipLaunchKernelGGL(keep_mask_kernel, dim3((unsigned)((groups + 255) / 256)), dim3(256), 0,
                       (hipStream_t)stream, keep, d, (uint64_t)n);
    return check_launch(hipGetLastError(), what);
}

// aligned rows of 513 .. kMaxRegisterRow columns: what the sliding-window kernels take
static int check_window_call(const SoftmaxCall& c, int32_t sq, int32_t sk, int32_t window) {
    if (sq != sk) return fail(NEOX_ERR_BAD_SHAPE, "%s: sq=%d and sk=%d must be equal", c.what, sq, sk);
    if (window < 0) return fail(NEOX_ERR_BAD_SHAPE, "%s: window=%d is negative", c.what, window);
    if (sk <= kChunk || sk > kMaxRegisterRow || sk % kVec != 0)
        return fail(NEOX_ERR_BAD_SHAPE, "%s: sk=%d must be a multiple of %d in (%d, %d]", c.what, sk, kVec, kChunk,
                    kMaxRegisterRow);
    if (!c.vec_ok) return fail(NEOX_ERR_MISALIGNED, "%s: the tensors must be 16-byte aligned", c.what);
    return NEOX_OK;
}

int neox_sliding_window_softmax_fwd(void* y, const void* x, float scale, int64_t batches, int32_t sq, int32_t sk,
                                    int32_t window, int32_t dtype, void* stream) {
    SoftmaxCall c("neox_sliding_window_softmax_fwd", dtype, {y, x});
    c.causal_rows(batches, sq, sk);
    if (c.status) return c.status;
    if (int e = check_window_call(c, sq, sk, window)) return e;
    c.forward(y, x, scale);
    c.a.window = window;
    return check_launch(launch_softmax_band_fwd(c.a, dtype, true, (hipStream_t)stream), c.what);
}

int neox_sliding_window_softmax_bwd(void* dx, const void* dy, const void* y, float scale, int64_t batches,
                                    int32_t sq, int32_t sk, int32_t window, int32_t dtype, void* stream) {
    SoftmaxCall c("neox_sliding_window_softmax_bwd", dtype, {dx, dy, y});
    c.causal_rows(batches, sq, sk);
    if (c.status) return c.status;
    if (int e = check_window_call(c, sq, sk, window)) return e;
    c.backward(dx, dy, y, scale);
    c.a.window = window;
    return check_launch(launch_softmax_band_bwd(c.a, dtype, true, (hipStream_t)stream), c.what);
}

int neox_mask_classify(int32_t* record, const uint8_t* mask, int32_t mask_b, int32_t sq, int32_t sk, void* stream) {
    static const char* what = "neox_mask_classify";
    if (!record || !mask) return fail(NEOX_ERR_NULL_POINTER, "%s: null pointer", what);
    if (mask_b < 1) return fail(NEOX_ERR_BAD_SHAPE, "%s: mask_b=%d must be >= 1", what, mask_b);
    if (int e = check_rows((int64_t)mask_b * (sq < 1 ? 0 : sq), sq, sk, what)) return e;
    if (sq != sk) return fail(NEOX_ERR_BAD_SHAPE, "%s: sq=%d and sk=%d must be equal", what, sq, sk);
    if (!aligned(record, 4)) return fail(NEOX_ERR_MISALIGNED, "%s: misaligned pointer", what);
    return check_launch(launch_mask_classify(record, nullptr, mask, (uint32_t)mask_b * (uint32_t)sq, sq, sk, (hipStream_t)stream), what);
}

int neox_mask_scan(int32_t* record, int32_t* row_end, const uint8_t* mask, int32_t mask_b, int32_t sq, int32_t sk,
                   void* stream) {
    static const char* what = "neox_mask_scan";
    if (!record || !row_end || !mask) return fail(NEOX_ERR_NULL_POINTER, "%s: null pointer", what);
    if (mask_b < 1) return fail(NEOX_ERR_BAD_SHAPE, "%s: mask_b=%d must be >= 1", what, mask_b);
    if (int e = check_rows((int64_t)mask_b * (sq < 1 ? 0 : sq), sq, sk, what)) return e;
    if (!aligned(record, 8) || !aligned(row_end, 4)) return fail(NEOX_ERR_MISALIGNED, "%s: misaligned pointer", what);
    return check_launch(launch_mask_classify(record, row_end, mask, (uint32_t)mask_b * (uint32_t)sq, sq, sk, (hipStream_t)stream), what);
}

int neox_get_batch_per_block(int32_t sq, int32_t sk, int32_t b, int32_t np) {
    (void)sq;
    (void)b;
    (void)np;
    if (sk < 1) return fail(NEOX_ERR_BAD_SHAPE, "neox_get_batch_per_block: sk=%d must be >= 1", sk);
    int log2_elements = 0;
    while ((1LL << log2_elements) < sk) ++log2_elements;
    const long long next_pow2 = 1LL << log2_elements;
    const int wave = (next_pow2 < kWave) ? (int)next_pow2 : kWave;
    const int rows_per_wave = (next_pow2 <= 128) ? 2 : 1;
    const int waves_per_block = 128 / wave;
    return waves_per_block * rows_per_wave;
}

static int check_rope_strides(const int64_t* st, const char* what, const char* name) {
    if (!st) return fail(NEOX_ERR_NULL_POINTER, "%s: %s strides are null", what, name);
    for (int i = 0; i < 3; ++i)
        if (st[i] < 0) return fail(NEOX_ERR_BAD_STRIDE, "%s: %s stride[%d]=%lld is negative", what, name, i, (long long)st[i]);
    return NEOX_OK;
}

}  // extern "C"

// Both rotary entry points.  cs_dtype == kRopeAngles: `cos` holds fp32 angles and `sin` is not used.
static int rope_apply(const char* what, void* out_q, void* out_k, const void* q, const void* k,
                      const void* cos, const void* sin, int32_t s, int32_t b, int32_t h_q, int32_t h_k,
                      int32_t d_rot, int32_t d, const int64_t q_strides[3], const int64_t k_strides[3],
                      const int64_t out_q_strides[3], const int64_t out_k_strides[3],
                      int64_t cs_stride, int32_t pos_offset, int32_t dtype, int32_t cs_dtype,
                      int32_t backward, void* stream) {
    const bool angles = (cs_dtype == kRopeAngles);
    if (angles) sin = cos;
    if (!out_q || !q || !cos || !sin) return fail(NEOX_ERR_NULL_POINTER, "%s: null tensor pointer", what);
    if ((k == nullptr) != (out_k == nullptr))
        return fail(NEOX_ERR_NULL_POINTER, "%s: k and out_k must both be given or both be null", what);
    if (int e = check_dtype(dtype, what)) return e;
    if (!angles && cs_dtype != NEOX_F32 && cs_dtype != dtype)
        return fail(NEOX_ERR_BAD_DTYPE, "%s: cos/sin must be fp32 or have the dtype of q (code %d)", what, cs_dtype);
    const bool has_k = (k != nullptr);
    if (s < 1 || b < 1 || h_q < 1 || (has_k && h_k < 1))
        return fail(NEOX_ERR_BAD_SHAPE, "%s: s=%d b=%d h_q=%d h_k=%d must be >= 1", what, s, b, h_q, h_k);
    if (d_rot < 2 || (d_rot & 1))
        return fail(NEOX_ERR_BAD_SHAPE, "%s: d_rot=%d must be even and >= 2", what, d_rot);
    if (d < d_rot) return fail(NEOX_ERR_BAD_SHAPE, "%s: d=%d is smaller than d_rot=%d", what, d, d_rot);
    if (b > 65535) return fail(NEOX_ERR_BAD_SHAPE, "%s: b=%d exceeds 65535", what, b);
    if (pos_offset < 0) return fail(NEOX_ERR_BAD_SHAPE, "%s: pos_offset=%d is negative", what, pos_offset);
    if (cs_stride < d_rot)
        return fail(NEOX_ERR_BAD_STRIDE, "%s: %s row stride %lld < d_rot=%d", what, angles ? "freqs" : "cos/sin", (long long)cs_stride, d_rot);
    if (int e = check_rope_strides(q_strides, what, "q")) return e;
    if (int e = check_rope_strides(out_q_strides, what, "out_q")) return e;
    if (has_k) {
        if (int e = check_rope_strides(k_strides, what, "k")) return e;
        if (int e = check_rope_strides(out_k_strides, what, "out_k")) return e;
    }
    // the d leading dims of a head must not reach into the next head: the pass-through copy and the
    // padded write-back both move whole heads' worth of dims
    auto heads_apart = [&](const int64_t* st, int h, const char* name) {
        if (h > 1 && st[2] < d)
            return fail(NEOX_ERR_BAD_STRIDE, "%s: %s head stride %lld is smaller than d=%d", what, name, (long long)st[2], d);
        return (int)NEOX_OK;
    };
    if (int e = heads_apart(q_strides, h_q, "q")) return e;
    if (int e = heads_apart(out_q_strides, h_q, "out_q")) return e;
    if (has_k) {
        if (int e = heads_apart(k_strides, h_k, "k")) return e;
        if (int e = heads_apart(out_k_strides, h_k, "out_k")) return e;
    }
    const int cs_size = (angles || cs_dtype == NEOX_F32) ? 4 : 2;
    if (!aligned(q, 2) || !aligned(out_q, 2) || (has_k && (!aligned(k, 2) || !aligned(out_k, 2))) ||
        !aligned(cos, cs_size) || !aligned(sin, cs_size))
        return fail(NEOX_ERR_MISALIGNED, "%s: misaligned pointer", what);

    const int half = d_rot / 2;
    // widest slot (elements) every access of the call can use
    auto fits = [&](int w) {
        if (half % w) return false;
        const uintptr_t bytes = (uintptr_t)w * 2;
        auto ok_t = [&](const void* p, const int64_t* st) {
            return aligned(p, bytes) && st[0] % w == 0 && st[1] % w == 0 && st[2] % w == 0;
        };
        if (!ok_t(q, q_strides) || !ok_t(out_q, out_q_strides)) return false;
        if (has_k && (!ok_t(k, k_strides) || !ok_t(out_k, out_k_strides))) return false;
        if (angles) return true;  // the angles are read one by one
        // table accesses are at most 128 bits wide
        const int tw = (cs_size == 4 && w > 4) ? 4 : w;
        const uintptr_t tbytes = (uintptr_t)tw * cs_size;
        return aligned(cos, tbytes) && aligned(sin, tbytes) && cs_stride % tw == 0;
    };
    int w = 1;
    for (int cand : {8, 4, 2})
        if (fits(cand)) {
            w = cand;
            break;
        }
    const int lpv = half / w;
    if (lpv > 256) return fail(NEOX_ERR_BAD_SHAPE, "%s: d_rot=%d too large for slot width %d", what, d_rot, w);

    // collapse (b, h) into one loop when every layout allows it
    auto collapsible = [&](const int64_t* st, int h) { return b == 1 || st[1] == (int64_t)h * st[2]; };
    bool collapse = collapsible(q_strides, h_q) && collapsible(out_q_strides, h_q);
    if (has_k) collapse = collapse && collapsible(k_strides, h_k) && collapsible(out_k_strides, h_k);

    RopeArgs a{};
    auto fill = [&](RopeTensor& t, const void* in, void* out, const int64_t* is, const int64_t* os, int h) {
        t.in = static_cast<const char*>(in);
        t.out = static_cast<char*>(out);
        for (int i = 0; i < 3; ++i) {
            t.in_stride[i] = is[i];
            t.out_stride[i] = os[i];
        }
        t.n_outer = collapse ? 1 : b;
        t.n_inner = collapse ? b * h : h;
    };
    if ((int64_t)b * h_q > 0x7fffffffLL || (has_k && (int64_t)b * h_k > 0x7fffffffLL))
        return fail(NEOX_ERR_BAD_SHAPE, "%s: b*h exceeds 2^31", what);
    fill(a.t[0], q, out_q, q_strides, out_q_strides, h_q);
    if (has_k) fill(a.t[1], k, out_k, k_strides, out_k_strides, h_k);
    a.cos = static_cast<const char*>(cos);
    a.sin = static_cast<const char*>(sin);
    a.cs_stride = cs_stride;
    a.pos_offset = pos_offset;
    a.half = half;
    a.lpv = lpv;
    a.nt = has_k ? 2 : 1;
    // Out of place, the pass-through dims [d_rot, d) are copied by the same launch: by further
    // lanes of the head's lane group when the whole head splits into at most 64 slots, else by
    // the element-wise loop of the other kernel.
    const bool out_of_place = (q != out_q) || (has_k && k != out_k);
    if (out_of_place && d > d_rot) {
        a.copy_dims = d - d_rot;
        if (w >= 2 && a.copy_dims % w == 0 && d / w <= kWave) a.pad_slots = a.copy_dims / w;
    }
    // In place, a rotated span that ends inside a 64-byte block is written back together with the
    // rest of that block (unchanged pass-through dims the loads fetch anyway): the memory system
    // then sees whole 64-byte writes instead of partial ones.  The padded span must stay inside
    // its head cell (the head stride) and must not reach what the other tensor of the call
    // writes: q and k that interleave in one buffer (views into a fused projection) share their
    // head cells, and then each padded span has to end before the other tensor's span begins.
    // Heads whose stride is a multiple of 32 but not of 64 bytes (80- and 112-dim heads) get the same
    // with 32-byte blocks, which still saves 3-11 % against writing the bare spans.
    for (int block : {64, 32}) {
        if (a.copy_dims != 0 || a.pad_slots != 0) break;
        const int slot_bytes = w * 2, span_bytes = d_rot * 2;
        const int pad_bytes = (block - span_bytes % block) % block;
        auto in_place_blocks = [&](const void* in, const void* out, const int64_t* is, const int64_t* os) {
            if (in != out) return false;
            for (int i = 0; i < 3; ++i)
                if (is[i] != os[i] || (is[i] * 2) % block != 0) return false;
            return aligned(in, block) && is[2] * 2 >= span_bytes + pad_bytes;
        };
        bool ok = w >= 2 && pad_bytes > 0 && pad_bytes % slot_bytes == 0 &&
                  lpv * 2 + pad_bytes / slot_bytes <= kWave &&
                  in_place_blocks(q, out_q, q_strides, out_q_strides);
        if (ok && has_k) ok = in_place_blocks(k, out_k, k_strides, out_k_strides);
        if (ok && has_k) {
            // bytes from the first element to one past the last one a tensor's heads can reach
            auto extent = [&](const int64_t* st, int h) {
                return ((int64_t)(s - 1) * st[0] + (int64_t)(b - 1) * st[1] + (int64_t)(h - 1) * st[2]) * 2 +
                       span_bytes + pad_bytes;
            };
            const char* qb = static_cast<const char*>(q);
            const char* kb = static_cast<const char*>(k);
            const bool apart = qb + extent(q_strides, h_q) <= kb || kb + extent(k_strides, h_k) <= qb;
            if (!apart) {
                // interleaved: same cell size needed, and each padded span ends before the other begins
                const int64_t cell = q_strides[2] * 2;
                bool same = true;
                for (int i = 0; i < 3; ++i) same = same && q_strides[i] == k_strides[i];
                const int64_t shift = same ? ((kb - qb) % cell + cell) % cell : 0;
                // (shift 0: the tensors own different cells, e.g. the q heads and then the k heads of one buffer)
                ok = same && (shift == 0 || (span_bytes + pad_bytes <= shift && span_bytes + pad_bytes <= cell - shift));
            }
        }
        if (ok) a.pad_slots = pad_bytes / slot_bytes;
        if (pad_bytes == 0) break;  // the span already ends on a block boundary
    }
    return check_launch(launch_rope(a, s, collapse ? 1 : b, w, dtype, cs_dtype, backward != 0,
                                    (hipStream_t)stream),
                        what);
}

extern "C" {

int neox_rope_apply(void* out_q, void* out_k, const void* q, const void* k, const void* cos,
                    const void* sin, int32_t s, int32_t b, int32_t h_q, int32_t h_k,
                    int32_t d_rot, int32_t d, const int64_t q_strides[3], const int64_t k_strides[3],
                    const int64_t out_q_strides[3], const int64_t out_k_strides[3],
                    int64_t cs_stride, int32_t pos_offset, int32_t dtype, int32_t cs_dtype,
                    int32_t backward, void* stream) {
    static const char* what = "neox_rope_apply";
    if (cs_dtype != NEOX_F16 && cs_dtype != NEOX_BF16 && cs_dtype != NEOX_F32)
        return fail(NEOX_ERR_BAD_DTYPE, "%s: cos/sin must be fp32 or have the dtype of q (code %d)", what, cs_dtype);
    return rope_apply(what, out_q, out_k, q, k, cos, sin, s, b, h_q, h_k, d_rot, d, q_strides, k_strides,
                      out_q_strides, out_k_strides, cs_stride, pos_offset, dtype, cs_dtype, backward, stream);
}

int neox_rope_apply_freqs(void* out_q, void* out_k, const void* q, const void* k, const float* freqs,
                          int32_t s, int32_t b, int32_t h_q, int32_t h_k, int32_t d_rot, int32_t d,
                          const int64_t q_strides[3], const int64_t k_strides[3],
                          const int64_t out_q_strides[3], const int64_t out_k_strides[3],
                          int64_t freqs_stride, int32_t pos_offset, int32_t dtype, int32_t backward,
                          void* stream) {
    return rope_apply("neox_rope_apply_freqs", out_q, out_k, q, k, freqs, nullptr, s, b, h_q, h_k, d_rot, d,
                      q_strides, k_strides, out_q_strides, out_k_strides, freqs_stride, pos_offset, dtype,
                      kRopeAngles, backward, stream);
}

}  // extern "C"
#pragma GCC visibility pop
