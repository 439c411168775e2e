"""Extension-level API of the causal softmax, as the autograd Function calls it.

Same functions and checks as the reference's pybind module
``scaled_upper_triang_masked_softmax_cuda``
(megatron/fused_kernels/scaled_upper_triang_masked_softmax.cpp:31-70,
megatron/fused_kernels/scaled_upper_triang_masked_softmax_cuda.cu:33-90),
served by the gfx950 kernels behind ``neox_causal_softmax_fwd/_bwd``.
Differences: no ``seq_len <= 2048`` limit; ``scale`` stays fp32 in the forward pass.
Additions: ``forward_alibi``, ``forward_bias``, ``forward_window`` / ``backward_window`` and
``forward_dropout`` / ``backward_dropout``.
"""
import torch

from .. import _lib

from .attention_dropout import state_pointer as _state_ptr

_HALF = (torch.float16, torch.bfloat16)
_check, _code, _guard, _stream, _lib_handle = _lib.check, _lib.dtype_code, _lib.device_guard, _lib.current_stream, _lib.lib


def _scores(input, dims):
    """The checks of the reference's entry points on a score tensor; returns it contiguous."""
    if input.dim() not in dims:
        raise RuntimeError("expected %s tensor" % " or ".join(f"{d}D" for d in dims))
    if input.dtype not in _HALF:
        raise RuntimeError("Only fp16 and bf16 are supported")
    if not input.is_cuda:
        _lib.require_gpu(input)
    return input if input.is_contiguous() else input.contiguous()


def _grads(output_grads, softmax_results, dims):
    if output_grads.dim() not in dims or softmax_results.dim() != output_grads.dim():
        raise RuntimeError("expected %s tensor" % " or ".join(f"{d}D" for d in dims))
    if output_grads.dtype not in _HALF or softmax_results.dtype not in _HALF:
        raise RuntimeError("Only fp16 and bf16 are supported")
    if output_grads.dtype != softmax_results.dtype or output_grads.shape != softmax_results.shape:
        raise RuntimeError("output_grads and softmax_results must have the same dtype and shape")
    if not (output_grads.is_cuda and softmax_results.is_cuda):
        _lib.require_gpu(output_grads, softmax_results)
    if not output_grads.is_contiguous():
        output_grads = output_grads.contiguous()
    if not softmax_results.is_contiguous():
        softmax_results = softmax_results.contiguous()
    return output_grads, softmax_results


def check_slopes(slopes, np_):
    """ALiBi slopes, one per head; returns them as contiguous fp32 on their device."""
    if slopes.numel() != np_:
        raise RuntimeError(f"expected {np_} ALiBi slopes (one per head), got {slopes.numel()}")
    _lib.require_gpu(slopes)
    if slopes.dtype is torch.float32 and slopes.is_contiguous() and not slopes.requires_grad:
        return slopes
    return slopes.detach().to(dtype=torch.float32).contiguous()


def check_bias(input, bias):
    """``bias`` broadcastable to ``input`` ``[b, np, sq, sk]`` over the batch dimension only;
    returns it contiguous and in ``input``'s dtype."""
    b, np_, sq, sk = input.shape
    if bias.dim() != 4 or tuple(bias.shape[1:]) != (np_, sq, sk) or bias.size(0) not in (1, b):
        raise RuntimeError(f"bias must have shape [1 or {b}, {np_}, {sq}, {sk}], got {tuple(bias.shape)}")
    _lib.require_gpu(bias)
    return bias.detach().to(dtype=input.dtype).contiguous()


def forward(input, scale_factor):
    return forward_nd(_scores(input, (3,)), scale_factor)


def forward_nd(input, scale_factor):
    """:func:`forward` on ``[..., sq, sk]`` (contiguous, checked by the caller): the leading dims
    count as attention batches, so a ``[b, np, sq, sk]`` tensor needs no view of its own."""
    sq, sk = input.shape[-2:]
    attn_batches = input.numel() // max(1, sq * sk)
    softmax_results = torch.empty_like(input)
    if input.numel() == 0:
        return softmax_results
    with _guard(input):
        status = _lib_handle().neox_causal_softmax_fwd(
            softmax_results.data_ptr(), input.data_ptr(), float(scale_factor), attn_batches, sq, sk,
            _code(input.dtype), _stream(input))
    if status:
        _check(status)
    return softmax_results


def forward_alibi(input, slopes, scale_factor):
    """Causal softmax of ``scale * (input + alibi_bias)`` without materialising the bias.

    ``input``: ``[b, np, sq, sk]`` fp16/bf16; ``slopes``: ``[np]`` (any float dtype), the
    per-head ALiBi slopes; the bias of head h is ``-slopes[h] * (i - j)`` for ``j <= i``
    (megatron/model/positional_embeddings.py:161-176).  No counterpart in the reference's
    extension: it adds the bias in a separate pass before calling ``forward``.
    """
    input = _scores(input, (4,))
    b, np_, sq, sk = input.shape
    slopes = check_slopes(slopes, np_)
    softmax_results = torch.empty_like(input)
    if input.numel() == 0:
        return softmax_results
    with _guard(input):
        _check(_lib_handle().neox_causal_softmax_alibi_fwd(
            softmax_results.data_ptr(), input.data_ptr(), slopes.data_ptr(), float(scale_factor),
            b, np_, sq, sk, _code(input.dtype), _stream(input)))
    return softmax_results


def forward_bias(input, bias, scale_factor, slopes=None):
    """Causal softmax of ``scale * (input + bias)`` with the bias read inside the kernel.

    ``input``: ``[b, np, sq, sk]`` fp16/bf16; ``bias``: ``[1 or b, np, sq, sk]``, e.g. the
    relative-position bias ``[1, np, sq, sk]`` (megatron/model/transformer.py:526-528);
    ``slopes`` (optional) adds the ALiBi bias of :func:`forward_alibi` as well.  No
    counterpart in the reference's extension: it adds the bias in a separate pass.
    """
    input = _scores(input, (4,))
    bias = check_bias(input, bias)
    b, np_, sq, sk = input.shape
    if slopes is not None:
        slopes = check_slopes(slopes, np_)
    softmax_results = torch.empty_like(input)
    if input.numel() == 0:
        return softmax_results
    with _guard(input):
        _check(_lib_handle().neox_causal_softmax_bias_fwd(
            softmax_results.data_ptr(), input.data_ptr(), bias.data_ptr(),
            slopes.data_ptr() if slopes is not None else None, float(scale_factor),
            b, np_, sq, sk, bias.size(0), _code(input.dtype), _stream(input)))
    return softmax_results


def backward(output_grads, softmax_results, scale_factor):
    """Returns d(input); like the reference, the result is written into
    ``output_grads`` itself when that tensor is contiguous."""
    return backward_nd(*_grads(output_grads, softmax_results, (3,)), scale_factor)


def backward_nd(output_grads, softmax_results, scale_factor):
    """:func:`backward` on ``[..., sq, sk]`` (contiguous, checked by the caller)."""
    sq, sk = output_grads.shape[-2:]
    attn_batches = output_grads.numel() // max(1, sq * sk)
    if output_grads.numel() == 0:
        return output_grads
    grads = output_grads.data_ptr()
    with _guard(output_grads):
        status = _lib_handle().neox_causal_softmax_bwd(
            grads, grads, softmax_results.data_ptr(), float(scale_factor), attn_batches, sq, sk,
            _code(output_grads.dtype), _stream(output_grads))
    if status:
        _check(status)
    return output_grads


def window_kernel_takes(input, window):
    """Whether the sliding-window kernels serve this score tensor ``[..., sq, sk]``: square, aligned
    rows of 513 to 32768 columns (a multiple of 8)."""
    sq, sk = input.shape[-2:]
    return (sq == sk and window >= 0 and 512 < sk <= 32768 and sk % 8 == 0 and input.data_ptr() % 16 == 0
            and input.is_contiguous())


def forward_window(input, scale_factor, window):
    """Causal softmax under a sliding window: row i sees the keys ``max(0, i - window) .. i``, the
    mask ``get_attn_mask(seq_length, device, sliding_window_width=window)`` builds
    (megatron/utils.py:67-80) -- without reading a mask and without reading the scores outside
    the band.  ``input``: ``[attn_batches, sq, sk]`` or ``[b, np, sq, sk]``; see :func:`window_kernel_takes`.  No
    counterpart in the reference's extension, whose causal kernel ignores the window."""
    input = _scores(input, (3, 4))
    sq, sk = input.shape[-2:]
    attn_batches = input.numel() // max(1, sq * sk)
    softmax_results = torch.empty_like(input)
    if input.numel() == 0:
        return softmax_results
    with _guard(input):
        _check(_lib_handle().neox_sliding_window_softmax_fwd(
            softmax_results.data_ptr(), input.data_ptr(), float(scale_factor), attn_batches, sq, sk, window,
            _code(input.dtype), _stream(input)))
    return softmax_results


def backward_window(output_grads, softmax_results, scale_factor, window):
    """d(input) of :func:`forward_window`, written into ``output_grads`` itself when it is
    contiguous; gradient and probabilities outside the band are not read."""
    output_grads, softmax_results = _grads(output_grads, softmax_results, (3, 4))
    sq, sk = output_grads.shape[-2:]
    attn_batches = output_grads.numel() // max(1, sq * sk)
    if output_grads.numel() == 0:
        return output_grads
    grads = output_grads.data_ptr()
    with _guard(output_grads):
        _check(_lib_handle().neox_sliding_window_softmax_bwd(
            grads, grads, softmax_results.data_ptr(), float(scale_factor), attn_batches, sq, sk, window,
            _code(output_grads.dtype), _stream(output_grads)))
    return output_grads


def forward_dropout(input, scale_factor, p, seed, offset, state=None, slopes=None, bias=None):
    """Causal softmax and the attention dropout that follows it, in one kernel.

    Returns ``(softmax_results, dropped)``: the probabilities as :func:`forward` gives them
    and ``dropout(softmax_results, p)`` as ``torch.nn.Dropout`` computes it from them, with
    the keep pattern drawn from Philox state ``(seed, offset)``
    (megatron/model/transformer.py:533-539).  ``state``, if given, is an int64 device tensor
    ``[seed, offset]`` read by the kernel when it runs (for launches recorded into a HIP graph)
    and replaces the two numbers.  ``input`` is ``[attn_batches, sq, sk]``, or ``[b, np, sq, sk]``
    -- required with ``slopes`` (ALiBi, as :func:`forward_alibi`) and ``bias`` (as
    :func:`forward_bias`).  No counterpart in the reference's extension.
    """
    input = _scores(input, (3, 4))
    if input.dim() == 3 and (slopes is not None or bias is not None):
        raise RuntimeError("expected 4D tensor")
    b, np_ = (input.shape[0], 1) if input.dim() == 3 else input.shape[:2]
    sq, sk = input.shape[-2:]
    if slopes is not None:
        slopes = check_slopes(slopes, np_)
    if bias is not None:
        bias = check_bias(input, bias)
    softmax_results = torch.empty_like(input)
    dropped = torch.empty_like(input)
    if input.numel() == 0:
        return softmax_results, dropped
    with _guard(input):
        _check(_lib_handle().neox_causal_softmax_dropout_fwd(
            dropped.data_ptr(), softmax_results.data_ptr(), input.data_ptr(),
            slopes.data_ptr() if slopes is not None else None,
            bias.data_ptr() if bias is not None else None, bias.size(0) if bias is not None else 0,
            float(scale_factor), float(p), int(seed), int(offset), _state_ptr(state), b, np_, sq, sk,
            _code(input.dtype), _stream(input)))
    return softmax_results, dropped


def backward_dropout(output_grads, softmax_results, scale_factor, p, seed, offset, state=None):
    """d(input) from the gradient of ``dropped``; written into ``output_grads`` itself when
    that tensor is contiguous.  ``(p, seed, offset, state)`` are those of the forward call."""
    output_grads, softmax_results = _grads(output_grads, softmax_results, (3, 4))
    sq, sk = output_grads.shape[-2:]
    attn_batches = output_grads.numel() // max(1, sq * sk)
    if output_grads.numel() == 0:
        return output_grads
    grads = output_grads.data_ptr()
    with _guard(output_grads):
        _check(_lib_handle().neox_causal_softmax_dropout_bwd(
            grads, grads, softmax_results.data_ptr(), float(scale_factor), float(p), int(seed), int(offset),
            _state_ptr(state), attn_batches, sq, sk, _code(output_grads.dtype), _stream(output_grads)))
    return output_grads
