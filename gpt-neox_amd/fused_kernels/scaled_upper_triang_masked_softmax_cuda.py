"""Extension-level API of the causal softmax, as the autograd Function calls it.

Same functions and checks as the reference's pybind module
``scaled_upper_triang_masked_softmax_cuda``
(megatron/fused_kernels/scaled_upper_triang_masked_softmax.cpp:31-70,
megatron/fused_kernels/scaled_upper_triang_masked_softmax_cuda.cu:33-90),
served by the gfx950 kernels behind ``neox_causal_softmax_fwd/_bwd``.
Differences: no ``seq_len <= 2048`` limit; ``scale`` stays fp32 in the forward pass.
"""
import torch

from .. import _lib

from .attention_dropout import state_pointer as _state_ptr

_HALF = (torch.float16, torch.bfloat16)


def forward(input, scale_factor):
    if input.dim() != 3:
        raise RuntimeError("expected 3D tensor")
    if input.dtype not in _HALF:
        raise RuntimeError("Only fp16 and bf16 are supported")
    _lib.require_gpu(input)
    input = input.contiguous()
    attn_batches, sq, sk = input.shape
    softmax_results = torch.empty_like(input, requires_grad=False)
    if input.numel() == 0:
        return softmax_results
    with _lib.device_guard(input):
        _lib.check(
            _lib.lib().neox_causal_softmax_fwd(
                softmax_results.data_ptr(), input.data_ptr(), float(scale_factor), attn_batches,
                sq, sk, _lib.dtype_code(input.dtype), _lib.current_stream(input),
            )
        )
    return softmax_results


def forward_alibi(input, slopes, scale_factor):
    """Causal softmax of ``scale * (input + alibi_bias)`` without materialising the bias.

    ``input``: ``[b, np, sq, sk]`` fp16/bf16; ``slopes``: ``[np]`` (any float dtype), the
    per-head ALiBi slopes; the bias of head h is ``-slopes[h] * (i - j)`` for ``j <= i``
    (megatron/model/positional_embeddings.py:161-176).  No counterpart in the reference's
    extension: it adds the bias in a separate pass before calling ``forward``.
    """
    if input.dim() != 4:
        raise RuntimeError("expected 4D tensor")
    if input.dtype not in _HALF:
        raise RuntimeError("Only fp16 and bf16 are supported")
    b, np_, sq, sk = input.shape
    if slopes.numel() != np_:
        raise RuntimeError(f"expected {np_} ALiBi slopes (one per head), got {slopes.numel()}")
    _lib.require_gpu(input, slopes)
    input = input.contiguous()
    slopes = slopes.detach().to(dtype=torch.float32).contiguous()
    softmax_results = torch.empty_like(input, requires_grad=False)
    if input.numel() == 0:
        return softmax_results
    with _lib.device_guard(input):
        _lib.check(
            _lib.lib().neox_causal_softmax_alibi_fwd(
                softmax_results.data_ptr(), input.data_ptr(), slopes.data_ptr(), float(scale_factor),
                b, np_, sq, sk, _lib.dtype_code(input.dtype), _lib.current_stream(input),
            )
        )
    return softmax_results


def check_bias(input, bias):
    """``bias`` broadcastable to ``input`` ``[b, np, sq, sk]`` over the batch dimension only;
    returns it contiguous and in ``input``'s dtype."""
    b, np_, sq, sk = input.shape
    if bias.dim() != 4 or tuple(bias.shape[1:]) != (np_, sq, sk) or bias.size(0) not in (1, b):
        raise RuntimeError(f"bias must have shape [1 or {b}, {np_}, {sq}, {sk}], got {tuple(bias.shape)}")
    return bias.detach().to(dtype=input.dtype).contiguous()


def forward_bias(input, bias, scale_factor):
    """Causal softmax of ``scale * (input + bias)`` with the bias read inside the kernel.

    ``input``: ``[b, np, sq, sk]`` fp16/bf16; ``bias``: ``[1 or b, np, sq, sk]``, e.g. the
    relative-position bias ``[1, np, sq, sk]`` (megatron/model/transformer.py:526-528).  No
    counterpart in the reference's extension: it adds the bias in a separate pass.
    """
    if input.dim() != 4:
        raise RuntimeError("expected 4D tensor")
    if input.dtype not in _HALF:
        raise RuntimeError("Only fp16 and bf16 are supported")
    _lib.require_gpu(input, bias)
    input = input.contiguous()
    bias = check_bias(input, bias)
    b, np_, sq, sk = input.shape
    softmax_results = torch.empty_like(input, requires_grad=False)
    if input.numel() == 0:
        return softmax_results
    with _lib.device_guard(input):
        _lib.check(
            _lib.lib().neox_causal_softmax_bias_fwd(
                softmax_results.data_ptr(), input.data_ptr(), bias.data_ptr(), float(scale_factor),
                b, np_, sq, sk, bias.size(0), _lib.dtype_code(input.dtype), _lib.current_stream(input),
            )
        )
    return softmax_results


def backward(output_grads, softmax_results, scale_factor):
    """Returns d(input); like the reference, the result is written into
    ``output_grads`` itself when that tensor is contiguous."""
    if output_grads.dim() != 3 or softmax_results.dim() != 3:
        raise RuntimeError("expected 3D tensor")
    if output_grads.dtype not in _HALF or softmax_results.dtype not in _HALF:
        raise RuntimeError("Only fp16 and bf16 are supported")
    if output_grads.dtype != softmax_results.dtype or output_grads.shape != softmax_results.shape:
        raise RuntimeError("output_grads and softmax_results must have the same dtype and shape")
    _lib.require_gpu(output_grads, softmax_results)
    output_grads = output_grads.contiguous()
    softmax_results = softmax_results.contiguous()
    attn_batches, sq, sk = output_grads.shape
    if output_grads.numel() == 0:
        return output_grads
    with _lib.device_guard(output_grads):
        _lib.check(
            _lib.lib().neox_causal_softmax_bwd(
                output_grads.data_ptr(), output_grads.data_ptr(), softmax_results.data_ptr(),
                float(scale_factor), attn_batches, sq, sk, _lib.dtype_code(output_grads.dtype),
                _lib.current_stream(output_grads),
            )
        )
    return output_grads


def forward_dropout(input, scale_factor, p, seed, offset, state=None, slopes=None, bias=None):
    """Causal softmax and the attention dropout that follows it, in one kernel.

    Returns ``(softmax_results, dropped)``: the probabilities as :func:`forward` gives them
    and ``dropout(softmax_results, p)`` as ``torch.nn.Dropout`` computes it from them, with
    the keep pattern drawn from Philox state ``(seed, offset)``
    (megatron/model/transformer.py:533-539).  ``state``, if given, is an int64 device tensor
    ``[seed, offset]`` read by the kernel when it runs (for launches recorded into a HIP graph)
    and replaces the two numbers.  ``input`` is ``[attn_batches, sq, sk]``, or ``[b, np, sq, sk]``
    -- required with ``slopes`` (ALiBi, as :func:`forward_alibi`) or ``bias`` (as
    :func:`forward_bias`), of which at most one may be given.  No counterpart in the
    reference's extension.
    """
    if input.dim() not in (3, 4):
        raise RuntimeError("expected 3D or 4D tensor")
    if input.dim() == 3 and (slopes is not None or bias is not None):
        raise RuntimeError("expected 4D tensor")
    if slopes is not None and bias is not None:
        raise RuntimeError("give ALiBi slopes or a bias tensor, not both")
    if input.dtype not in _HALF:
        raise RuntimeError("Only fp16 and bf16 are supported")
    _lib.require_gpu(input, slopes, bias)
    input = input.contiguous()
    b, np_ = (input.shape[0], 1) if input.dim() == 3 else input.shape[:2]
    sq, sk = input.shape[-2:]
    if slopes is not None:
        if slopes.numel() != np_:
            raise RuntimeError(f"expected {np_} ALiBi slopes (one per head), got {slopes.numel()}")
        slopes = slopes.detach().to(dtype=torch.float32).contiguous()
    if bias is not None:
        bias = check_bias(input, bias)
    softmax_results = torch.empty_like(input, requires_grad=False)
    dropped = torch.empty_like(input, requires_grad=False)
    if input.numel() == 0:
        return softmax_results, dropped
    with _lib.device_guard(input):
        _lib.check(
            _lib.lib().neox_causal_softmax_dropout_fwd(
                dropped.data_ptr(), softmax_results.data_ptr(), input.data_ptr(),
                slopes.data_ptr() if slopes is not None else None,
                bias.data_ptr() if bias is not None else None, bias.size(0) if bias is not None else 0,
                float(scale_factor), float(p), int(seed), int(offset), _state_ptr(state), b, np_, sq, sk,
                _lib.dtype_code(input.dtype), _lib.current_stream(input),
            )
        )
    return softmax_results, dropped


def backward_dropout(output_grads, softmax_results, scale_factor, p, seed, offset, state=None):
    """d(input) from the gradient of ``dropped``; written into ``output_grads`` itself when
    that tensor is contiguous.  ``(p, seed, offset, state)`` are those of the forward call."""
    if output_grads.dim() not in (3, 4) or softmax_results.dim() != output_grads.dim():
        raise RuntimeError("expected 3D or 4D tensor")
    if output_grads.dtype not in _HALF or softmax_results.dtype not in _HALF:
        raise RuntimeError("Only fp16 and bf16 are supported")
    if output_grads.dtype != softmax_results.dtype or output_grads.shape != softmax_results.shape:
        raise RuntimeError("output_grads and softmax_results must have the same dtype and shape")
    _lib.require_gpu(output_grads, softmax_results)
    output_grads = output_grads.contiguous()
    softmax_results = softmax_results.contiguous()
    sq, sk = output_grads.shape[-2:]
    attn_batches = output_grads.numel() // max(1, sq * sk)
    if output_grads.numel() == 0:
        return output_grads
    with _lib.device_guard(output_grads):
        _lib.check(
            _lib.lib().neox_causal_softmax_dropout_bwd(
                output_grads.data_ptr(), output_grads.data_ptr(), softmax_results.data_ptr(),
                float(scale_factor), float(p), int(seed), int(offset), _state_ptr(state), attn_batches, sq, sk,
                _lib.dtype_code(output_grads.dtype), _lib.current_stream(output_grads),
            )
        )
    return output_grads
