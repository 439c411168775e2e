"""Extension-level API of the rotary embedding kernels.

Same functions and checks as the reference's pybind module
``fused_rotary_positional_embedding``
(megatron/fused_kernels/fused_rotary_positional_embedding.cpp:38-139,
megatron/fused_kernels/fused_rotary_positional_embedding_cuda.cu:24-216):
``t`` is ``[s, b, h, d]`` with any s/b/h strides, the table is ``[s, 1, 1, d2]``
with ``d2 <= d``; dims ``>= d2`` are copied through by the same launch;
``transpose_output`` makes the result's memory ``[b, s, h, d]``.  The cached variants are
served by ``neox_rope_apply``, the ``freqs`` variants by ``neox_rope_apply_freqs``, which
evaluates cos and sin of the angles inside the kernel as the reference's does.
Differences: arithmetic is fp32 with one rounding (the reference rounds cos/sin to
the dtype of ``t`` first); ``t`` must be fp16 or bf16.
"""
import torch

from .. import _lib

_HALF = (torch.float16, torch.bfloat16)


def rope_launch(out_q, out_k, q, k, cos, sin, d_rot, pos_offset, backward, d=None):
    """One launch over q (and k, unless None).  Tensors are 4-D ``[s, b, h, >=d_rot]``
    with last-dim stride 1; cos/sin are ``[>= pos_offset + s, .., d_rot]`` contiguous
    in their last dim, fp32 or of q's dtype; ``sin is None`` means that ``cos`` holds fp32
    angles whose cos and sin the kernel evaluates.  ``d`` (default ``d_rot``): leading dims
    of every head delivered in the outputs -- out of place the dims ``[d_rot, d)`` are copied
    from the inputs."""
    s, b, h_q = q.shape[0], q.shape[1], q.shape[2]
    h_k = k.shape[2] if k is not None else 0
    lib = _lib.lib()
    head = (
        out_q.data_ptr(), out_k.data_ptr() if k is not None else None,
        q.data_ptr(), k.data_ptr() if k is not None else None,
    )
    shape = (
        s, b, h_q, h_k, d_rot, d_rot if d is None else d,
        _lib.strides3(q), _lib.strides3(k) if k is not None else None,
        _lib.strides3(out_q), _lib.strides3(out_k) if k is not None else None,
        cos.stride(0) if cos.shape[0] > 1 else d_rot, pos_offset, _lib.dtype_code(q.dtype),
    )
    tail = (1 if backward else 0, _lib.current_stream(q))
    with _lib.device_guard(q):
        if sin is None:
            _lib.check(lib.neox_rope_apply_freqs(*head, cos.data_ptr(), *shape, *tail))
        else:
            _lib.check(lib.neox_rope_apply(*head, cos.data_ptr(), sin.data_ptr(), *shape,
                                           _lib.dtype_code(cos.dtype), *tail))


def _check_table(t, table, name):
    if t.dim() != 4 or table.dim() != 4:
        raise RuntimeError("expected 4D tensor")
    if t.size(0) != table.size(0):
        raise RuntimeError(f"expected input and {name} tensor have the same sequence length")
    if table.size(1) != 1 or table.size(2) != 1:
        raise RuntimeError(f"expected the second and third dims of the {name} tensor equal 1")
    if t.size(3) < table.size(3):
        raise RuntimeError(
            f"expected the last dim of the input tensor equals or is greater than the {name} tensor"
        )


def _apply(t, cos, sin, transpose_output, backward):
    """Out-of-place rotation of ``t`` by tables (``cos``, ``sin``) or by angles (``cos`` = freqs,
    ``sin`` None); one launch, which also copies the dims ``>= d2``."""
    if t.dtype not in _HALF:
        raise RuntimeError("Only fp16 and bf16 are supported")
    _lib.require_gpu(t, cos, sin)
    s, b, h, d = t.shape
    d2 = cos.size(3)
    if t.stride(3) != 1:
        t = t.contiguous()
    cos = cos.contiguous()
    if sin is not None:
        sin = sin.contiguous()
    if transpose_output:
        out = torch.empty((b, s, h, d), dtype=t.dtype, device=t.device).transpose(0, 1)
    else:
        out = torch.empty((s, b, h, d), dtype=t.dtype, device=t.device)
    if t.numel() == 0:
        return out
    rope_launch(out, None, t, None, cos, sin, d2, 0, backward, d=d)
    return out


def forward_cached(input, cos, sin, transpose_output=False):
    _check_table(input, cos, "cos")
    _check_table(input, sin, "sin")
    if cos.size(3) != sin.size(3):
        raise RuntimeError("expected cos and sin tensor have the same last dim")
    if cos.dtype != sin.dtype:
        raise RuntimeError("expected cos and sin tensor have the same dtype")
    if cos.dtype != torch.float32 and cos.dtype != input.dtype:
        raise RuntimeError("cos/sin must be float32 or have the dtype of the input")
    return _apply(input, cos, sin, transpose_output, backward=False)


def backward_cached(output_grads, cos, sin, transpose_output=False):
    _check_table(output_grads, cos, "cos")
    _check_table(output_grads, sin, "sin")
    if cos.size(3) != sin.size(3):
        raise RuntimeError("expected cos and sin tensor have the same last dim")
    if cos.dtype != sin.dtype:
        raise RuntimeError("expected cos and sin tensor have the same dtype")
    if cos.dtype != torch.float32 and cos.dtype != output_grads.dtype:
        raise RuntimeError("cos/sin must be float32 or have the dtype of the input")
    return _apply(output_grads, cos, sin, transpose_output, backward=True)


def forward(input, freqs, transpose_output=False):
    """Rotation angles given as ``freqs`` (fp32); cos/sin are evaluated in fp32 inside the kernel."""
    _check_table(input, freqs, "freqs")
    if freqs.dtype != torch.float32:
        raise RuntimeError("Dtype of the freqs tensor must be float")
    return _apply(input, freqs, None, transpose_output, backward=False)


def backward(output_grads, freqs, transpose_output=False):
    _check_table(output_grads, freqs, "freqs")
    if freqs.dtype != torch.float32:
        raise RuntimeError("Dtype of the freqs tensor must be float")
    return _apply(output_grads, freqs, None, transpose_output, backward=True)
