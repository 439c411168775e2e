"""Extension-level API of the mask-tensor softmax.

Same functions and checks as the reference's pybind module ``scaled_masked_softmax_cuda``
(megatron/fused_kernels/scaled_masked_softmax.cpp:33-83,
megatron/fused_kernels/scaled_masked_softmax_cuda.cu:38-108), served by the gfx950
kernels behind ``neox_masked_softmax_fwd/_bwd``.
Differences: no ``key_seq_len <= 2048`` / ``query_seq_len > 1`` limits; masked
scores are excluded (probability exactly 0) instead of being set to -10000; any
non-zero mask byte masks; ``scale`` stays fp32.
"""
import torch

from .. import _lib

from .attention_dropout import state_pointer as _state_ptr

_HALF = (torch.float16, torch.bfloat16)


def _check_forward(input, mask):
    if input.dim() != 4:
        raise RuntimeError("expected 4D tensor")
    if input.dtype not in _HALF:
        raise RuntimeError("Only fp16 and bf16 are supported")
    if mask.dim() != 4:
        raise RuntimeError("expected 4D tensor")
    b, np_, sq, sk = input.shape
    pad_batches = mask.size(0)
    if not (pad_batches == 1 or pad_batches == b):
        raise RuntimeError("mask.size(0) must be 1 or the batch size")
    if mask.size(1) != 1 or mask.size(2) != sq or mask.size(3) != sk:
        raise RuntimeError("mask must have shape [1 or b, 1, sq, sk]")
    if mask.dtype not in (torch.bool, torch.uint8):
        raise RuntimeError("mask must be a bool or uint8 tensor")
    _lib.require_gpu(input, mask)
    return input.contiguous(), mask.contiguous()


def forward(input, mask, scale_factor):
    input, mask = _check_forward(input, mask)
    b, np_, sq, sk = input.shape
    pad_batches = mask.size(0)
    softmax_results = torch.empty_like(input, requires_grad=False)
    if input.numel() == 0:
        return softmax_results
    with _lib.device_guard(input):
        _lib.check(
            _lib.lib().neox_masked_softmax_fwd(
                softmax_results.data_ptr(), input.data_ptr(), mask.data_ptr(), float(scale_factor),
                b, np_, sq, sk, pad_batches, _lib.dtype_code(input.dtype),
                _lib.current_stream(input),
            )
        )
    return softmax_results


def forward_bias(input, mask, bias, scale_factor):
    """Mask-tensor softmax of ``scale * (input + bias)`` with the bias read inside the kernel;
    ``bias``: ``[1 or b, np, sq, sk]`` (megatron/model/transformer.py:526-528).  No counterpart
    in the reference's extension: it adds the bias in a separate pass."""
    from .scaled_upper_triang_masked_softmax_cuda import check_bias

    input, mask = _check_forward(input, mask)
    _lib.require_gpu(bias)
    bias = check_bias(input, bias)
    b, np_, sq, sk = input.shape
    softmax_results = torch.empty_like(input, requires_grad=False)
    if input.numel() == 0:
        return softmax_results
    with _lib.device_guard(input):
        _lib.check(
            _lib.lib().neox_masked_softmax_bias_fwd(
                softmax_results.data_ptr(), input.data_ptr(), mask.data_ptr(), bias.data_ptr(),
                float(scale_factor), b, np_, sq, sk, mask.size(0), bias.size(0),
                _lib.dtype_code(input.dtype), _lib.current_stream(input),
            )
        )
    return softmax_results


def _check_backward(output_grads, softmax_results):
    if output_grads.dim() != 4 or softmax_results.dim() != 4:
        raise RuntimeError("expected 4D tensor")
    if output_grads.dtype not in _HALF or softmax_results.dtype not in _HALF:
        raise RuntimeError("Only fp16 and bf16 are supported")
    if output_grads.dtype != softmax_results.dtype or output_grads.shape != softmax_results.shape:
        raise RuntimeError("output_grads and softmax_results must have the same dtype and shape")
    _lib.require_gpu(output_grads, softmax_results)
    return output_grads.contiguous(), softmax_results.contiguous()


def backward(output_grads, softmax_results, scale_factor):
    """Returns d(input), written into ``output_grads`` itself when it is contiguous."""
    output_grads, softmax_results = _check_backward(output_grads, softmax_results)
    b, np_, sq, sk = output_grads.shape
    if output_grads.numel() == 0:
        return output_grads
    with _lib.device_guard(output_grads):
        _lib.check(
            _lib.lib().neox_masked_softmax_bwd(
                output_grads.data_ptr(), output_grads.data_ptr(), softmax_results.data_ptr(),
                float(scale_factor), b * np_ * sq, sk, _lib.dtype_code(output_grads.dtype),
                _lib.current_stream(output_grads),
            )
        )
    return output_grads


def forward_dropout(input, mask, scale_factor, p, seed, offset, state=None, bias=None):
    """Mask-tensor softmax and the attention dropout that follows it, in one kernel.

    Returns ``(softmax_results, dropped)``: the probabilities as :func:`forward` gives them
    and ``dropout(softmax_results, p)`` as ``torch.nn.Dropout`` computes it from them, with
    the keep pattern drawn from Philox state ``(seed, offset)``
    (megatron/model/transformer.py:533-539).  ``state``, if given, is an int64 device tensor
    ``[seed, offset]`` read by the kernel when it runs (for launches recorded into a HIP graph)
    and replaces the two numbers.  ``bias`` (optional) is added to the scores as in
    :func:`forward_bias`.  No counterpart in the reference's extension.
    """
    input, mask = _check_forward(input, mask)
    if bias is not None:
        from .scaled_upper_triang_masked_softmax_cuda import check_bias

        _lib.require_gpu(bias)
        bias = check_bias(input, bias)
    b, np_, sq, sk = input.shape
    softmax_results = torch.empty_like(input, requires_grad=False)
    dropped = torch.empty_like(input, requires_grad=False)
    if input.numel() == 0:
        return softmax_results, dropped
    with _lib.device_guard(input):
        _lib.check(
            _lib.lib().neox_masked_softmax_dropout_fwd(
                dropped.data_ptr(), softmax_results.data_ptr(), input.data_ptr(), mask.data_ptr(),
                bias.data_ptr() if bias is not None else None, bias.size(0) if bias is not None else 0,
                float(scale_factor), float(p), int(seed), int(offset), _state_ptr(state), b, np_, sq, sk,
                mask.size(0),
                _lib.dtype_code(input.dtype), _lib.current_stream(input),
            )
        )
    return softmax_results, dropped


def backward_dropout(output_grads, softmax_results, scale_factor, p, seed, offset, state=None):
    """d(input) from the gradient of ``dropped``; written into ``output_grads`` itself when
    that tensor is contiguous.  ``(p, seed, offset)`` are those of the forward call."""
    output_grads, softmax_results = _check_backward(output_grads, softmax_results)
    b, np_, sq, sk = output_grads.shape
    if output_grads.numel() == 0:
        return output_grads
    with _lib.device_guard(output_grads):
        _lib.check(
            _lib.lib().neox_masked_softmax_dropout_bwd(
                output_grads.data_ptr(), output_grads.data_ptr(), softmax_results.data_ptr(),
                float(scale_factor), float(p), int(seed), int(offset), _state_ptr(state), b * np_ * sq, sk,
                _lib.dtype_code(output_grads.dtype), _lib.current_stream(output_grads),
            )
        )
    return output_grads


def get_batch_per_block(query_seq_len, key_seq_len, batches, attn_heads):
    """Rows per block of the reference's launch shape on a 64-wide wavefront
    (megatron/fused_kernels/scaled_masked_softmax.h:338-352); host arithmetic only."""
    r = _lib.lib().neox_get_batch_per_block(query_seq_len, key_seq_len, batches, attn_heads)
    if r < 0:
        _lib.check(r)
    return r
