"""Drop-in for ``megatron/model/fused_rope.py`` (the ``rope_fusion`` path,
megatron/model/transformer.py:844-848).

``fused_apply_rotary_pos_emb`` / ``fused_apply_rotary_pos_emb_cached`` and the two
autograd Functions keep the reference's names, arguments and return values
(megatron/model/fused_rope.py:18-141); the work is done by the gfx950 rotary kernel
through ``fused_kernels.fused_rotary_positional_embedding``.

Both variants rotate ``t`` ``[s, b, h, d]`` (any s/b/h strides) over its first ``d2`` dims
and pass the others through; they differ only in how the rotation is given: as angles
``freqs`` ``[s, 1, 1, d2]`` (fp32), or as ready ``cos`` / ``sin`` tables of that shape (fp32
or the dtype of ``t``).  With ``transpose_output_memory`` the result's memory is
``[b, s, h, d]``, so that ``output.transpose(0, 1)`` is contiguous.  Gradients flow to ``t``
only.
"""
from typing import Tuple, Union

import torch

from .fused_kernels import fused_rotary_positional_embedding as _ext


def _make_rope_function(name, n_tables, fwd, bwd, doc):
    """One autograd Function per way of giving the rotation: ``apply(t, *tables, transpose)``
    saves the ``n_tables`` table tensors and runs the extension's ``fwd``; the backward pass
    runs ``bwd`` on the incoming gradient with the same tables."""

    def forward(ctx, t: torch.Tensor, *rest) -> torch.Tensor:
        tables, flags = rest[:n_tables], rest[n_tables:]
        transpose_output_memory = bool(flags[0]) if flags else False
        ctx.save_for_backward(*tables)
        ctx.transpose_output_memory = transpose_output_memory
        ctx.n_inputs = 1 + len(rest)
        return fwd(t, *tables, transpose_output_memory)

    def backward(ctx, grad_output: torch.Tensor) -> Tuple[Union[torch.Tensor, None], ...]:
        grad_input = bwd(grad_output, *ctx.saved_tensors, ctx.transpose_output_memory)
        return (grad_input,) + (None,) * (ctx.n_inputs - 1)

    return type(name, (torch.autograd.Function,),
                {"forward": staticmethod(forward), "backward": staticmethod(backward), "__doc__": doc})


FusedRoPEFunc = _make_rope_function(
    "FusedRoPEFunc", 1, _ext.forward, _ext.backward,
    "``apply(t, freqs, transpose_output_memory=False)``: rotation by the angles ``freqs``, whose "
    "cos/sin are evaluated in fp32 (megatron/model/fused_rope.py:18-54).")

FusedRoPECachedFunc = _make_rope_function(
    "FusedRoPECachedFunc", 2, _ext.forward_cached, _ext.backward_cached,
    "``apply(t, cos_, sin_, transpose_output_memory=False)``: rotation by cached tables "
    "(megatron/model/fused_rope.py:83-120).")


def fused_apply_rotary_pos_emb(
    t: torch.Tensor, freqs: torch.Tensor, transpose_output_memory: bool = False
) -> torch.Tensor:
    """``t``: ``[s, b, h, d]``; ``freqs``: ``[s, 1, 1, d2]`` float
    (megatron/model/fused_rope.py:57-80)."""
    return FusedRoPEFunc.apply(t, freqs, transpose_output_memory)


def fused_apply_rotary_pos_emb_cached(
    t: torch.Tensor, cos_: torch.Tensor, sin_: torch.Tensor, transpose_output_memory: bool = False
) -> torch.Tensor:
    """``t``: ``[s, b, h, d]``; ``cos_``, ``sin_``: ``[s, 1, 1, d2]``
    (megatron/model/fused_rope.py:123-141)."""
    return FusedRoPECachedFunc.apply(t, cos_, sin_, transpose_output_memory)
