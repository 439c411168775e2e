/*
 * neox_fused.h — C-ABI of libneox_fused.so
 *
 * Hand-written gfx950 (MI355X) kernels for GPT-NeoX's fused attention-softmax
 * and rotary-embedding path.  Every entry point
 *   - takes plain device pointers, sizes and a hipStream_t passed as void*;
 *   - is asynchronous with respect to the host (no allocation, no sync);
 *   - returns NEOX_OK (0) or a negative neox_status; it never throws or exits;
 *   - validates its arguments before the first HIP call, so argument errors
 *     are reported on a machine without a GPU too.
 * The caller owns all memory.  Element type codes are neox_dtype.
 * Pointers need the alignment of their element type only (2 bytes for fp16/bf16
 * tensors) and row lengths need not be multiples of anything: tensors that start
 * on a 16-byte boundary with sk % 8 == 0 take the fastest kernels, any other
 * layout runs vectorised kernels built for rows at arbitrary 2-byte alignment.
 *
 * Each declaration cites the reference interface it replaces (paths relative
 * to the GPT-NeoX source tree).
 */
#ifndef NEOX_FUSED_H
#define NEOX_FUSED_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/*
 * ABI versions.  A version is bumped when an entry point is added or its parameter list changes; the
 * Python binding refuses a library of another version.
 *   4  + neox_mask_scan, neox_masked_softmax_ends_fwd, neox_masked_softmax_ends_bwd
 *   3  + neox_masked_softmax_alibi_fwd, neox_sliding_window_softmax_fwd/_bwd, neox_mask_classify;
 *      neox_*_softmax_bias_fwd and neox_masked_softmax_dropout_fwd take ALiBi slopes too
 *   2  + the dropout, bias and ALiBi entry points, neox_rope_apply_freqs
 *   1  the four softmax entry points, neox_rope_apply, neox_get_batch_per_block
 */
#define NEOX_FUSED_ABI_VERSION 4

typedef enum neox_dtype {
    NEOX_F16 = 0,  /* IEEE binary16 */
    NEOX_BF16 = 1, /* bfloat16 */
    NEOX_F32 = 2   /* only valid for the rotary cos/sin tables */
} neox_dtype;

typedef enum neox_status {
    NEOX_OK = 0,
    NEOX_ERR_NULL_POINTER = -1,  /* a required pointer is NULL */
    NEOX_ERR_BAD_DTYPE = -2,     /* "Only fp16 and bf16 are supported" */
    NEOX_ERR_BAD_SHAPE = -3,     /* a size is <= 0 or out of the supported range */
    NEOX_ERR_BAD_STRIDE = -4,    /* negative stride or overlapping layout */
    NEOX_ERR_MISALIGNED = -5,    /* pointer not aligned to the element size */
    NEOX_ERR_LAUNCH = -6         /* hipLaunchKernel reported an error */
} neox_status;

/* ABI version of the loaded library (NEOX_FUSED_ABI_VERSION at build time). */
int neox_fused_abi_version(void);

/* Static description of a status code. Never NULL. */
const char* neox_fused_strerror(int status);

/* Message of the last failing call on the calling thread ("" if none). */
const char* neox_fused_last_error(void);

/*
 * Scaled upper-triangular (causal) masked softmax, forward.
 *   y[m,i,j] = softmax_j(scale * x[m,i,j]) over j <= i ;  y[m,i,j] = 0 for j > i
 * x, y: [batches, sq, sk] contiguous, same dtype (fp16/bf16); y may alias x.
 * fp32 arithmetic, one rounding on store.  Any sq, sk >= 1 (no 2048 cap).
 * Replaces scaled_upper_triang_masked_softmax_cuda.forward
 *   megatron/fused_kernels/scaled_upper_triang_masked_softmax.cpp:31-39
 *   megatron/fused_kernels/scaled_upper_triang_masked_softmax_cuda.cu:33-59
 */
int neox_causal_softmax_fwd(void* y, const void* x, float scale, int64_t batches, int32_t sq,
                            int32_t sk, int32_t dtype, void* stream);

/*
 * Causal softmax with the ALiBi bias folded in (no separate pass over the scores):
 *   y[n,h,i,j] = softmax_j(scale * (x[n,h,i,j] - slopes[h] * (i - j))) over j <= i ; 0 for j > i
 * x, y: [b, np, sq, sk] contiguous; slopes: fp32 [np] in device memory.  The gradient with
 * respect to x is neox_causal_softmax_bwd (the bias is a constant).
 * Replaces AliBi.forward followed by scaled_upper_triang_masked_softmax_cuda.forward
 *   megatron/model/positional_embeddings.py:210-257, megatron/model/transformer.py:529-534
 */
int neox_causal_softmax_alibi_fwd(void* y, const void* x, const float* slopes, float scale, int32_t b,
                                  int32_t np, int32_t sq, int32_t sk, int32_t dtype, void* stream);

/*
 * Mask-tensor softmax with the ALiBi bias folded in:
 *   y[n,h,i,j] = softmax_j(scale * (x[n,h,i,j] + slopes[h] * min(j - i', 0))),  i' = i + sk - sq,
 * masked keys excluded as in neox_masked_softmax_fwd.  The bias is the reference's matrix
 * -slope * tril(i - j) (zero above the diagonal); with sq == 1 the one query row stands at the
 * last key position, the reference's rule for a decode step against a key/value cache.
 * The gradient with respect to x is neox_masked_softmax_bwd.
 * Replaces AliBi.forward followed by scaled_masked_softmax_cuda.forward or the torch branch
 *   megatron/model/positional_embeddings.py:210-257 (the sq == 1 case: 236-250)
 *   megatron/model/transformer.py:529-534
 */
int neox_masked_softmax_alibi_fwd(void* y, const void* x, const uint8_t* mask, const float* slopes, float scale,
                                  int32_t b, int32_t np, int32_t sq, int32_t sk, int32_t mask_b, int32_t dtype,
                                  void* stream);

/*
 * Causal softmax backward:  dx = scale * y * (dy - sum_j(dy*y)) over j <= i,
 * dx = 0 for j > i.  dx may alias dy (the reference overwrites dy in place).
 * Replaces scaled_upper_triang_masked_softmax_cuda.backward
 *   megatron/fused_kernels/scaled_upper_triang_masked_softmax.cpp:41-56
 *   megatron/fused_kernels/scaled_upper_triang_masked_softmax_cuda.cu:61-90
 */
int neox_causal_softmax_bwd(void* dx, const void* dy, const void* y, float scale, int64_t batches,
                            int32_t sq, int32_t sk, int32_t dtype, void* stream);

/*
 * Scaled masked softmax, forward.
 *   y = softmax_j(mask ? excluded : scale * x);  masked positions are exactly 0;
 *   a row with every key masked yields the uniform 1/sk (the unfused path's result).
 * x, y: [b, np, sq, sk] contiguous.  mask: bytes [mask_b, 1, sq, sk] contiguous,
 * non-zero = masked, mask_b in {1, b} (broadcast over heads, and over samples if 1).
 * Replaces scaled_masked_softmax_cuda.forward
 *   megatron/fused_kernels/scaled_masked_softmax.cpp:33-43
 *   megatron/fused_kernels/scaled_masked_softmax_cuda.cu:38-84
 */
int neox_masked_softmax_fwd(void* y, const void* x, const uint8_t* mask, float scale, int32_t b,
                            int32_t np, int32_t sq, int32_t sk, int32_t mask_b, int32_t dtype,
                            void* stream);

/*
 * Masked softmax backward: dx = scale * y * (dy - sum_j(dy*y)) over each full row.
 * rows = b*np*sq.  dx may alias dy.
 * Replaces scaled_masked_softmax_cuda.backward
 *   megatron/fused_kernels/scaled_masked_softmax.cpp:45-62
 *   megatron/fused_kernels/scaled_masked_softmax_cuda.cu:86-108
 */
int neox_masked_softmax_bwd(void* dx, const void* dy, const void* y, float scale, int64_t rows,
                            int32_t sk, int32_t dtype, void* stream);

/*
 * Softmax of scale * (x + bias) with the bias tensor read inside the kernel (no separate
 * "scores += bias" pass); the sum is taken in fp32.  bias: [bias_b, np, sq, sk] contiguous,
 * dtype of x, bias_b in {1, b} (1 = shared by all samples).  Causal / mask-tensor variants as
 * neox_causal_softmax_fwd / neox_masked_softmax_fwd.  The gradient with respect to x is
 * neox_*_softmax_bwd; the gradient with respect to the bias is that same tensor (summed over
 * the samples that share it).  alibi_slopes (fp32 [np], NULL when absent) adds the ALiBi bias of
 * neox_*_softmax_alibi_fwd on top, as a model with both a relative-position bias and ALiBi has it.
 * Replaces "attention_scores += rpe" (and AliBi.forward) followed by the softmax extension call
 *   megatron/model/transformer.py:526-534, megatron/mpu/layers.py:353-380 (the bias)
 */
int neox_causal_softmax_bias_fwd(void* y, const void* x, const void* bias, const float* alibi_slopes,
                                 float scale, int32_t b, int32_t np, int32_t sq, int32_t sk, int32_t bias_b,
                                 int32_t dtype, void* stream);
int neox_masked_softmax_bias_fwd(void* y, const void* x, const uint8_t* mask, const void* bias,
                                 const float* alibi_slopes, float scale, int32_t b, int32_t np, int32_t sq,
                                 int32_t sk, int32_t mask_b, int32_t bias_b, int32_t dtype, void* stream);

/*
 * Softmax with the attention dropout that follows it folded in (training only).
 * Forward stores two tensors: y, the probabilities exactly as neox_*_softmax_fwd gives
 * them (the backward pass needs them), and y_drop = keep ? round(float(y) / (1-p)) : 0,
 * which is what torch.nn.Dropout computes from y; y_drop must not alias y.  Backward
 * takes dy = the gradient of y_drop, regenerates the keep pattern and returns
 *   dx = scale * y * (g - sum_j(g*y)),  g = keep ? dy / (1-p) : 0  (fp32, never stored).
 * Keep pattern: Philox4x32-10 with key = seed and counter = (offset / 4, e / 8), e the
 * row-major element index into the score tensor; element e owns the 16-bit field e % 8 of
 * its block and is kept iff field >= round(p * 65536).  neox_dropout_keep_mask writes that
 * pattern as bytes (1 = kept) for n elements.  (seed, offset) are the device generator's
 * Philox state, whose offset counts 32-bit outputs, four to a counter value; a call draws
 * from the one counter value offset / 4, so the caller advances the generator's offset by 4
 * per call and no other consumer of the generator draws the same blocks.  0 <= p <= 1.
 * The forward entry points take x as [b, np, sq, sk] and two optional additions to the scores,
 * NULL when absent: alibi_slopes (as neox_*_softmax_alibi_fwd) and a bias tensor
 * [bias_b, np, sq, sk] (as neox_*_softmax_bias_fwd).
 * device_state, if not NULL, points to {seed, offset} (two uint64) in device memory that the
 * kernel reads when it runs, instead of the seed and offset arguments: a launch recorded into
 * a HIP graph then follows a state that the graph itself advances between replays.
 * Replaces scaled_*_softmax_cuda.forward/backward followed by the attention dropout
 *   megatron/model/transformer.py:533-539 (softmax, then dropout under the RNG tracker)
 *   megatron/mpu/random.py:20-37 (the tracker that selects the generator state)
 */
int neox_causal_softmax_dropout_fwd(void* y_drop, void* y, const void* x, const float* alibi_slopes,
                                    const void* bias, int32_t bias_b, float scale, float p,
                                    uint64_t seed, uint64_t offset, const uint64_t* device_state,
                                    int32_t b, int32_t np, int32_t sq, int32_t sk, int32_t dtype,
                                    void* stream);
int neox_causal_softmax_dropout_bwd(void* dx, const void* dy, const void* y, float scale, float p,
                                    uint64_t seed, uint64_t offset, const uint64_t* device_state,
                                    int64_t batches, int32_t sq,
                                    int32_t sk, int32_t dtype, void* stream);
int neox_masked_softmax_dropout_fwd(void* y_drop, void* y, const void* x, const uint8_t* mask,
                                    const float* alibi_slopes, const void* bias, int32_t bias_b, float scale, float p,
                                    uint64_t seed, uint64_t offset, const uint64_t* device_state,
                                    int32_t b, int32_t np, int32_t sq, int32_t sk, int32_t mask_b,
                                    int32_t dtype, void* stream);
int neox_masked_softmax_dropout_bwd(void* dx, const void* dy, const void* y, float scale, float p,
                                    uint64_t seed, uint64_t offset, const uint64_t* device_state,
                                    int64_t rows, int32_t sk,
                                    int32_t dtype, void* stream);
int neox_dropout_keep_mask(uint8_t* keep, float p, uint64_t seed, uint64_t offset,
                           const uint64_t* device_state, int64_t n, void* stream);

/*
 * Causal softmax under a sliding window, forward and backward: row i sees the keys
 * max(0, i - window) .. i, every other position is exactly 0 -- the mask that
 * get_attn_mask(seq_length, device, sliding_window_width) builds, without reading a mask tensor
 * and without reading the scores outside the band.  x, y (dy, dx): [batches, sq, sk] contiguous,
 * 16-byte aligned, sq == sk, sk a multiple of 8 in (512, 32768]; other shapes are served by
 * neox_masked_softmax_fwd with the mask tensor (NEOX_ERR_BAD_SHAPE / NEOX_ERR_MISALIGNED here).
 * window >= sk - 1 is the plain causal softmax.  dx may alias dy.
 * Replaces the torch branch with the sliding-window mask (the reference's fused causal kernel
 * ignores the mask's contents and has no such variant)
 *   megatron/utils.py:67-80, megatron/model/fused_softmax.py:173-199
 */
int neox_sliding_window_softmax_fwd(void* y, const void* x, float scale, int64_t batches, int32_t sq, int32_t sk,
                                    int32_t window, int32_t dtype, void* stream);
int neox_sliding_window_softmax_bwd(void* dx, const void* dy, const void* y, float scale, int64_t batches,
                                    int32_t sq, int32_t sk, int32_t window, int32_t dtype, void* stream);

/*
 * Tells whether a mask tensor [mask_b, 1, sq, sk] (bytes, non-zero = masked, sq == sk) is the causal
 * mask, plain or with a sliding window, so that a caller that is handed only the tensor can use the
 * kernels that never read it.  Asynchronous like every entry point: it writes four int32 to
 * `record` (device memory), which the caller reads once the stream has got there:
 *   record[0]  != 0: some row's visible keys are not a contiguous run that ends on the diagonal
 *   record[1], record[2]  smallest and largest i - lo over the rows whose first visible key lo is > 0
 *                         (INT32_MAX and -1 if there is no such row)
 *   record[3]  largest i over the rows with lo == 0 (-1 if none)
 * Plain causal: record[0] == 0 and record[2] == -1.  Sliding window w: record[0] == 0,
 * record[1] == record[2] == w and record[3] <= w.
 * No counterpart in the reference, whose causal branch trusts the caller
 *   megatron/model/fused_softmax.py:173-179, megatron/utils.py:67-80 (the masks it recognises)
 */
int neox_mask_classify(int32_t* record, const uint8_t* mask, int32_t mask_b, int32_t sq, int32_t sk, void* stream);

/*
 * The same pass over a mask tensor [mask_b, 1, sq, sk] of any shape, which also notes where the
 * visible keys of every row end: row_end[r] (int32 [mask_b * sq], device memory) = last visible key
 * + 1, 0 for a row without a visible key.  `record` takes eight int32 (8-byte aligned): [0..3] as
 * neox_mask_classify writes them (record[0] = 1 for a mask that is not square), [4], [5] the low and
 * the high half of the 64-bit sum of sk - row_end[r] over the rows with a visible key -- the keys
 * that neox_masked_softmax_ends_fwd does not fetch --, [6], [7] zero.
 * No counterpart in the reference: its mask-tensor kernel reads every score and mask byte
 *   megatron/fused_kernels/scaled_masked_softmax.h:123-233
 */
int neox_mask_scan(int32_t* record, int32_t* row_end, const uint8_t* mask, int32_t mask_b, int32_t sq, int32_t sk,
                   void* stream);

/*
 * Mask-tensor softmax forward that is told where the visible keys of every mask row end and need
 * fetch neither scores nor mask bytes (nor bias) behind that point: row_end[r], int32 [mask_b * sq] as
 * neox_mask_scan writes it, is the caller's promise that the mask hides every key j >= row_end[r] of
 * mask row r; 0 (or a value >= sk, or row_end == NULL) promises nothing for that row.  A kernel may use
 * the promise or read the mask bytes (rows of up to 512 columns and of 1025 to 2048 skip hidden keys
 * from the bytes themselves), so a false promise gives an unspecified mixture of the two.  The
 * result is that of the plain entry points, bit for bit: y = softmax over the visible keys, exact
 * zeros elsewhere, a fully hidden row uniform 1/sk.  One entry point for every feature set:
 * alibi_slopes and bias (with bias_b) are optional as in neox_masked_softmax_bias_fwd; y_drop == NULL
 * means no dropout (p, seed, offset and device_state are ignored), otherwise the call is
 * neox_masked_softmax_dropout_fwd with the hint.  The backward pass is the plain one, or
 * neox_masked_softmax_ends_bwd.
 * Replaces, for masks whose rows end early (the padding of a batch of sequences of different
 * lengths),
 *   megatron/model/fused_softmax.py:56-83 (ScaledMaskedSoftmax.forward)
 *   megatron/fused_kernels/scaled_masked_softmax.h:123-233
 */
int neox_masked_softmax_ends_fwd(void* y_drop, void* y, const void* x, const uint8_t* mask, const int32_t* row_end,
                                 const float* alibi_slopes, const void* bias, int32_t bias_b, float scale, float p,
                                 uint64_t seed, uint64_t offset, const uint64_t* device_state,
                                 int32_t b, int32_t np, int32_t sq, int32_t sk, int32_t mask_b,
                                 int32_t dtype, void* stream);

/*
 * The backward pass of the mask-tensor softmax with the same hint: behind row_end[r] the probabilities
 * are zero, so neither they nor the incoming gradient are fetched there, and dx is zero.  The result is
 * that of neox_masked_softmax_bwd -- or, with dropout != 0, of neox_masked_softmax_dropout_bwd with
 * (p, seed, offset, device_state) of the forward call -- bit for bit.  [b, np, sq, sk] and mask_b say
 * which entry of row_end belongs to a row; dx may alias dy.
 * Replaces, for masks whose rows end early,
 *   megatron/model/fused_softmax.py:56-83 (ScaledMaskedSoftmax.backward)
 *   megatron/fused_kernels/scaled_masked_softmax.h:240-335
 */
int neox_masked_softmax_ends_bwd(void* dx, const void* dy, const void* y, const int32_t* row_end, float scale,
                                 int32_t dropout, float p, uint64_t seed, uint64_t offset, const uint64_t* device_state,
                                 int32_t b, int32_t np, int32_t sq, int32_t sk, int32_t mask_b,
                                 int32_t dtype, void* stream);

/*
 * Rows-per-block figure the reference's dispatcher predicate consumes; kept for
 * API compatibility (wave64 values).  Pure host arithmetic.
 * Replaces scaled_masked_softmax_cuda.get_batch_per_block
 *   megatron/fused_kernels/scaled_masked_softmax.h:338-352
 */
int neox_get_batch_per_block(int32_t sq, int32_t sk, int32_t b, int32_t np);

/*
 * Rotary positional embedding over the first d_rot dims of q and (optionally) k
 * in ONE launch.  Layout [s, b, h, d] addressed by element strides
 * {stride_s, stride_b, stride_h}; the last dim has stride 1.
 *   forward : out[j]      = x[j]*cos[j]           - x[j+d_rot/2]*sin[j]
 *             out[j+d/2]  = x[j+d/2]*cos[j+d/2]   + x[j]*sin[j+d/2]
 *   backward: out[j]      = g[j]*cos[j]           + g[j+d/2]*sin[j+d/2]
 *             out[j+d/2]  = g[j+d/2]*cos[j+d/2]   - g[j]*sin[j]
 * cos/sin: [>= pos_offset + s, d_rot] rows of stride cs_stride elements, dtype
 * cs_dtype (NEOX_F32 or the same as dtype).  Arithmetic is fp32 with separately
 * rounded products (bit-equal to torch's fp32 q*cos + rotate_half(q)*sin), one
 * rounding to dtype on store.  out_* may alias the inputs (in place).
 * d >= d_rot is the number of leading dims of every head the call delivers in out_*:
 * out of place (out_q != q, or out_k != k) the pass-through dims [d_rot, d) are copied
 * from the inputs by the same launch, as the reference's kernels do; pass d = d_rot to
 * have only the rotated span written.  In place the dims >= d_rot keep their values; those
 * that share a 64-byte block with the end of the rotated span (a 32-byte block when the heads
 * start on 32-byte boundaries only) may be written back unchanged -- whole blocks are much
 * cheaper for the memory system than partial ones; the block never reaches into the other
 * tensor of the same call, so q and k may be views into one buffer.
 * k / out_k may both be NULL.
 * Replaces apply_rotary_pos_emb / apply_rotary_pos_emb_torch
 *   megatron/model/positional_embeddings.py:103-126
 * and fused_rotary_positional_embedding.forward_cached / backward_cached
 *   megatron/fused_kernels/fused_rotary_positional_embedding.cpp:83-127
 *   megatron/fused_kernels/fused_rotary_positional_embedding.h:126-230 (rotation and tail copy)
 */
int neox_rope_apply(void* out_q, void* out_k, const void* q, const void* k, const void* cos,
                    const void* sin, int32_t s, int32_t b, int32_t h_q, int32_t h_k,
                    int32_t d_rot, int32_t d, const int64_t q_strides[3], const int64_t k_strides[3],
                    const int64_t out_q_strides[3], const int64_t out_k_strides[3],
                    int64_t cs_stride, int32_t pos_offset, int32_t dtype, int32_t cs_dtype,
                    int32_t backward, void* stream);

/*
 * The same rotation given as angles: freqs is fp32 [>= pos_offset + s, d_rot] with rows of
 * stride freqs_stride elements, and cos(freqs), sin(freqs) are evaluated inside the kernel in
 * fp32 (sincosf, once per position and dim, shared by all heads).  Everything else as
 * neox_rope_apply.
 * Replaces fused_rotary_positional_embedding.forward / backward
 *   megatron/fused_kernels/fused_rotary_positional_embedding.cpp:38-81
 *   megatron/fused_kernels/fused_rotary_positional_embedding.h:26-124 (sincosf in the kernel)
 */
int neox_rope_apply_freqs(void* out_q, void* out_k, const void* q, const void* k, const float* freqs,
                          int32_t s, int32_t b, int32_t h_q, int32_t h_k, int32_t d_rot, int32_t d,
                          const int64_t q_strides[3], const int64_t k_strides[3],
                          const int64_t out_q_strides[3], const int64_t out_k_strides[3],
                          int64_t freqs_stride, int32_t pos_offset, int32_t dtype, int32_t backward,
                          void* stream);

#ifdef __cplusplus
}
#endif
#endif /* NEOX_FUSED_H */
