"""Extension-level API of the mask-tensor softmax.

Same functions and checks as the reference's pybind module ``scaled_masked_softmax_cuda``
(megatron/fused_kernels/scaled_masked_softmax.cpp:33-83,
megatron/fused_kernels/scaled_masked_softmax_cuda.cu:38-108), served by the gfx950
kernels behind ``neox_masked_softmax_fwd/_bwd``.
Differences: no ``key_seq_len <= 2048`` / ``query_seq_len > 1`` limits; masked
scores are excluded (probability exactly 0) instead of being set to -10000; any
non-zero mask byte masks; ``scale`` stays fp32.
Additions: ``forward_alibi``, ``forward_bias``, ``forward_dropout`` / ``backward_dropout``,
``classify_mask``, and ``scan_mask`` with the ``row_end=`` hint of the forward functions: rows whose
visible keys end early (padding) are not fetched behind that point.
"""
import torch

from .. import _lib

from .attention_dropout import state_pointer as _state_ptr
from .scaled_upper_triang_masked_softmax_cuda import _grads, check_bias, check_slopes

_HALF = (torch.float16, torch.bfloat16)
_MASK_TYPES = (torch.bool, torch.uint8)
_check, _code, _guard, _stream, _lib_handle = _lib.check, _lib.dtype_code, _lib.device_guard, _lib.current_stream, _lib.lib


def _check_forward(input, mask):
    if input.dim() != 4:
        raise RuntimeError("expected 4D tensor")
    if input.dtype not in _HALF:
        raise RuntimeError("Only fp16 and bf16 are supported")
    if mask.dim() != 4:
        raise RuntimeError("expected 4D tensor")
    b, np_, sq, sk = input.shape
    mb, m1, msq, msk = mask.shape
    if not (mb == 1 or mb == b):
        raise RuntimeError("mask.size(0) must be 1 or the batch size")
    if m1 != 1 or msq != sq or msk != sk:
        raise RuntimeError("mask must have shape [1 or b, 1, sq, sk]")
    if mask.dtype not in _MASK_TYPES:
        raise RuntimeError("mask must be a bool or uint8 tensor")
    if not (input.is_cuda and mask.is_cuda):
        _lib.require_gpu(input, mask)
    return (input if input.is_contiguous() else input.contiguous(),
            mask if mask.is_contiguous() else mask.contiguous())


def _check_row_end(row_end, mask):
    """``row_end`` as :func:`scan_mask` returns it for ``mask``: int32 ``[mask_b * sq]`` on its device."""
    if (row_end.dtype != torch.int32 or row_end.dim() != 1 or row_end.numel() != mask.size(0) * mask.size(2)
            or row_end.device != mask.device):
        raise RuntimeError("row_end must be an int32 tensor [mask_b * sq] on the mask's device")
    return row_end if row_end.is_contiguous() else row_end.contiguous()


def _forward_ends(input, mask, row_end, scale_factor, slopes=None, bias=None, dropout=None):
    """The forward pass of any feature set with the hint ``row_end`` (see :func:`scan_mask`);
    ``dropout``: ``(p, seed, offset, state)`` or None.  Arguments already checked."""
    b, np_, sq, sk = input.shape
    row_end = _check_row_end(row_end, mask)
    softmax_results = torch.empty_like(input)
    dropped = torch.empty_like(input) if dropout is not None else None
    if input.numel() != 0:
        p, seed, offset, state = dropout if dropout is not None else (0.0, 0, 0, None)
        with _guard(input):
            _check(_lib_handle().neox_masked_softmax_ends_fwd(
                dropped.data_ptr() if dropped is not None else None, softmax_results.data_ptr(), input.data_ptr(),
                mask.data_ptr(), row_end.data_ptr(), slopes.data_ptr() if slopes is not None else None,
                bias.data_ptr() if bias is not None else None, bias.size(0) if bias is not None else 0,
                float(scale_factor), float(p), int(seed), int(offset), _state_ptr(state), b, np_, sq, sk,
                mask.size(0), _code(input.dtype), _stream(input)))
    return softmax_results if dropout is None else (softmax_results, dropped)


def forward(input, mask, scale_factor, row_end=None):
    """``row_end`` (optional, an addition): the hint of :func:`scan_mask` for this mask."""
    input, mask = _check_forward(input, mask)
    if row_end is not None:
        return _forward_ends(input, mask, row_end, scale_factor)
    b, np_, sq, sk = input.shape
    softmax_results = torch.empty_like(input)
    if input.numel() == 0:
        return softmax_results
    with _guard(input):
        status = _lib_handle().neox_masked_softmax_fwd(
            softmax_results.data_ptr(), input.data_ptr(), mask.data_ptr(), float(scale_factor),
            b, np_, sq, sk, mask.size(0), _code(input.dtype), _stream(input))
    if status:
        _check(status)
    return softmax_results


def forward_alibi(input, mask, slopes, scale_factor, row_end=None):
    """Mask-tensor softmax of ``scale * (input + alibi_bias)`` without materialising the bias:
    head h adds ``slopes[h] * min(j - i', 0)`` with ``i' = i + sk - sq``, the matrix the
    reference's ``AliBi`` module adds -- ``-slope * tril(i - j)``, and for a one-query decode step
    its last row (megatron/model/positional_embeddings.py:210-257).  No counterpart in the
    reference's extension: it adds the bias in a separate pass."""
    input, mask = _check_forward(input, mask)
    b, np_, sq, sk = input.shape
    slopes = check_slopes(slopes, np_)
    if row_end is not None:
        return _forward_ends(input, mask, row_end, scale_factor, slopes=slopes)
    softmax_results = torch.empty_like(input)
    if input.numel() == 0:
        return softmax_results
    with _guard(input):
        _check(_lib_handle().neox_masked_softmax_alibi_fwd(
            softmax_results.data_ptr(), input.data_ptr(), mask.data_ptr(), slopes.data_ptr(),
            float(scale_factor), b, np_, sq, sk, mask.size(0), _code(input.dtype), _stream(input)))
    return softmax_results


def forward_bias(input, mask, bias, scale_factor, slopes=None, row_end=None):
    """Mask-tensor softmax of ``scale * (input + bias)`` with the bias read inside the kernel;
    ``bias``: ``[1 or b, np, sq, sk]`` (megatron/model/transformer.py:526-528); ``slopes``
    (optional) adds the ALiBi bias of :func:`forward_alibi` as well.  No counterpart
    in the reference's extension: it adds the bias in a separate pass."""
    input, mask = _check_forward(input, mask)
    bias = check_bias(input, bias)
    b, np_, sq, sk = input.shape
    if slopes is not None:
        slopes = check_slopes(slopes, np_)
    if row_end is not None:
        return _forward_ends(input, mask, row_end, scale_factor, slopes=slopes, bias=bias)
    softmax_results = torch.empty_like(input)
    if input.numel() == 0:
        return softmax_results
    with _guard(input):
        _check(_lib_handle().neox_masked_softmax_bias_fwd(
            softmax_results.data_ptr(), input.data_ptr(), mask.data_ptr(), bias.data_ptr(),
            slopes.data_ptr() if slopes is not None else None, float(scale_factor),
            b, np_, sq, sk, mask.size(0), bias.size(0), _code(input.dtype), _stream(input)))
    return softmax_results


def _backward_ends(output_grads, softmax_results, row_end, scale_factor, dropout=None):
    """The backward pass with the hint ``row_end`` ``[mask_b * sq]`` (see :func:`scan_mask`): nothing is
    fetched behind a row's end, where the probabilities are zero.  ``dropout``: ``(p, seed, offset,
    state)`` of the forward call or None.  Arguments already checked."""
    b, np_, sq, sk = output_grads.shape
    if row_end.dtype != torch.int32 or row_end.dim() != 1 or row_end.numel() not in (sq, b * sq) \
            or row_end.device != output_grads.device:
        raise RuntimeError("row_end must be an int32 tensor [mask_b * sq] on the gradient's device")
    if not row_end.is_contiguous():
        row_end = row_end.contiguous()
    if output_grads.numel() == 0:
        return output_grads
    p, seed, offset, state = dropout if dropout is not None else (0.0, 0, 0, None)
    grads = output_grads.data_ptr()
    with _guard(output_grads):
        _check(_lib_handle().neox_masked_softmax_ends_bwd(
            grads, grads, softmax_results.data_ptr(), row_end.data_ptr(), float(scale_factor),
            0 if dropout is None else 1, float(p), int(seed), int(offset), _state_ptr(state),
            b, np_, sq, sk, row_end.numel() // sq, _code(output_grads.dtype), _stream(output_grads)))
    return output_grads


def backward(output_grads, softmax_results, scale_factor, row_end=None):
    """Returns d(input), written into ``output_grads`` itself when it is contiguous.  ``row_end``
    (optional, an addition): the hint of :func:`scan_mask` for the mask of the forward call."""
    output_grads, softmax_results = _grads(output_grads, softmax_results, (4,))
    if row_end is not None:
        return _backward_ends(output_grads, softmax_results, row_end, scale_factor)
    b, np_, sq, sk = output_grads.shape
    if output_grads.numel() == 0:
        return output_grads
    grads = output_grads.data_ptr()
    with _guard(output_grads):
        status = _lib_handle().neox_masked_softmax_bwd(
            grads, grads, softmax_results.data_ptr(), float(scale_factor), b * np_ * sq, sk,
            _code(output_grads.dtype), _stream(output_grads))
    if status:
        _check(status)
    return output_grads


def forward_dropout(input, mask, scale_factor, p, seed, offset, state=None, bias=None, slopes=None, row_end=None):
    """Mask-tensor softmax and the attention dropout that follows it, in one kernel.

    Returns ``(softmax_results, dropped)``: the probabilities as :func:`forward` gives them
    and ``dropout(softmax_results, p)`` as ``torch.nn.Dropout`` computes it from them, with
    the keep pattern drawn from Philox state ``(seed, offset)``
    (megatron/model/transformer.py:533-539).  ``state``, if given, is an int64 device tensor
    ``[seed, offset]`` read by the kernel when it runs (for launches recorded into a HIP graph)
    and replaces the two numbers.  ``bias`` and ``slopes`` (optional) add to the scores as in
    :func:`forward_bias` and :func:`forward_alibi`.  No counterpart in the reference's extension.
    """
    input, mask = _check_forward(input, mask)
    if bias is not None:
        bias = check_bias(input, bias)
    b, np_, sq, sk = input.shape
    if slopes is not None:
        slopes = check_slopes(slopes, np_)
    if row_end is not None:
        return _forward_ends(input, mask, row_end, scale_factor, slopes=slopes, bias=bias,
                             dropout=(p, seed, offset, state))
    softmax_results = torch.empty_like(input)
    dropped = torch.empty_like(input)
    if input.numel() == 0:
        return softmax_results, dropped
    with _guard(input):
        _check(_lib_handle().neox_masked_softmax_dropout_fwd(
            dropped.data_ptr(), softmax_results.data_ptr(), input.data_ptr(), mask.data_ptr(),
            slopes.data_ptr() if slopes is not None else None,
            bias.data_ptr() if bias is not None else None, bias.size(0) if bias is not None else 0,
            float(scale_factor), float(p), int(seed), int(offset), _state_ptr(state), b, np_, sq, sk,
            mask.size(0), _code(input.dtype), _stream(input)))
    return softmax_results, dropped


def backward_dropout(output_grads, softmax_results, scale_factor, p, seed, offset, state=None, row_end=None):
    """d(input) from the gradient of ``dropped``; written into ``output_grads`` itself when
    that tensor is contiguous.  ``(p, seed, offset)`` are those of the forward call; ``row_end``
    (optional) as in :func:`backward`."""
    output_grads, softmax_results = _grads(output_grads, softmax_results, (4,))
    if row_end is not None:
        return _backward_ends(output_grads, softmax_results, row_end, scale_factor, (p, seed, offset, state))
    b, np_, sq, sk = output_grads.shape
    if output_grads.numel() == 0:
        return output_grads
    grads = output_grads.data_ptr()
    with _guard(output_grads):
        _check(_lib_handle().neox_masked_softmax_dropout_bwd(
            grads, grads, softmax_results.data_ptr(), float(scale_factor), float(p), int(seed), int(offset),
            _state_ptr(state), b * np_ * sq, sk, _code(output_grads.dtype), _stream(output_grads)))
    return output_grads


def classify_mask(mask):
    """Folds a mask ``[mask_b, 1, s, s]`` (bool/uint8 on the GPU) into four int32 on its device, from
    which :func:`decode_mask_record` tells a causal mask -- plain or with a sliding window
    (megatron/utils.py:67-80) -- from any other.  Asynchronous: the record is valid once the
    current stream has got there.  No counterpart in the reference, whose causal branch never
    looks at the mask (megatron/model/fused_softmax.py:173-179)."""
    if mask.dim() != 4 or mask.size(1) != 1 or mask.size(2) != mask.size(3):
        raise RuntimeError("mask must have shape [mask_b, 1, s, s]")
    if mask.dtype not in _MASK_TYPES:
        raise RuntimeError("mask must be a bool or uint8 tensor")
    _lib.require_gpu(mask)
    if not mask.is_contiguous():
        mask = mask.contiguous()
    record = torch.empty(4, dtype=torch.int32, device=mask.device)
    with _guard(mask):
        _check(_lib_handle().neox_mask_classify(record.data_ptr(), mask.data_ptr(), mask.size(0), mask.size(2),
                                                mask.size(3), _stream(mask)))
    return record


def scan_mask(mask):
    """:func:`classify_mask` for a mask ``[mask_b, 1, sq, sk]`` of any shape, which also notes where
    every row's visible keys end.  Returns ``(record, row_end)`` on the mask's device: eight int32 --
    the first four as :func:`classify_mask` gives them, then the 64-bit number of hidden keys behind
    the rows' last visible ones (see :func:`hidden_tail_keys`) -- and int32 ``[mask_b * sq]``, the
    ``row_end=`` hint of the forward functions (last visible key + 1; 0 for a row with none).
    Asynchronous like every call.  No counterpart in the reference."""
    if mask.dim() != 4 or mask.size(1) != 1:
        raise RuntimeError("mask must have shape [mask_b, 1, sq, sk]")
    if mask.dtype not in _MASK_TYPES:
        raise RuntimeError("mask must be a bool or uint8 tensor")
    _lib.require_gpu(mask)
    if not mask.is_contiguous():
        mask = mask.contiguous()
    record = torch.empty(8, dtype=torch.int32, device=mask.device)
    row_end = torch.empty(mask.size(0) * mask.size(2), dtype=torch.int32, device=mask.device)
    if row_end.numel() == 0 or mask.size(3) == 0:
        record.copy_(torch.tensor([1, 2**31 - 1, -1, -1, 0, 0, 0, 0], dtype=torch.int32))
        return record, row_end.zero_()
    with _guard(mask):
        _check(_lib_handle().neox_mask_scan(record.data_ptr(), row_end.data_ptr(), mask.data_ptr(), mask.size(0),
                                            mask.size(2), mask.size(3), _stream(mask)))
    return record, row_end


def launch_stream(tensor):
    """The raw handle of the stream a call on ``tensor`` is launched on now."""
    return _stream(tensor)


def hidden_tail_keys(record):
    """The number of keys that the ``row_end`` hint of :func:`scan_mask` saves: the sum over the
    mask rows of ``sk - row_end`` (rows without a visible key not counted), from the eight numbers
    of the record."""
    return (int(record[4]) & 0xFFFFFFFF) | ((int(record[5]) & 0xFFFFFFFF) << 32)


def decode_mask_record(record):
    """What the (first) four numbers of :func:`classify_mask` / :func:`scan_mask` say: ``"causal"``, a
    sliding-window width (int), or False for any other mask."""
    bad, wmin, wmax, top = (int(v) for v in record[:4])
    if bad:
        return False
    if wmax < 0:
        return "causal"
    if wmin == wmax and top <= wmin:
        return wmin
    return False


def get_batch_per_block(query_seq_len, key_seq_len, batches, attn_heads):
    """Rows per block of the reference's launch shape on a 64-wide wavefront
    (megatron/fused_kernels/scaled_masked_softmax.h:338-352); host arithmetic only."""
    r = _lib_handle().neox_get_batch_per_block(query_seq_len, key_seq_len, batches, attn_heads)
    if r < 0:
        _check(r)
    return r
