"""Drop-in for ``megatron/model/fused_rope.py`` (the ``rope_fusion`` path,
megatron/model/transformer.py:844-848).

``fused_apply_rotary_pos_emb`` / ``fused_apply_rotary_pos_emb_cached`` and the two
autograd Functions keep the reference's names, arguments and return values
(megatron/model/fused_rope.py:18-141); the work is done by the gfx950 rotary kernel
through ``fused_kernels.fused_rotary_positional_embedding``.
"""
from typing import Tuple, Union

import torch

from .fused_kernels import fused_rotary_positional_embedding as _ext


class FusedRoPEFunc(torch.autograd.Function):
    """Rotary embedding from rotation angles ``freqs`` ``[s, 1, 1, d2]`` (fp32) on an
    ``[s, b, h, d]`` tensor of any s/b/h strides; dims ``>= d2`` pass through."""

    @staticmethod
    def forward(ctx, t: torch.Tensor, freqs: torch.Tensor, transpose_output_memory: bool = False):
        output = _ext.forward(t, freqs, transpose_output_memory)
        ctx.save_for_backward(freqs)
        ctx.transpose_output_memory = transpose_output_memory
        return output

    @staticmethod
    def backward(ctx, grad_output: torch.Tensor) -> Tuple[Union[torch.Tensor, None], ...]:
        (freqs,) = ctx.saved_tensors
        grad_input = _ext.backward(grad_output, freqs, ctx.transpose_output_memory)
        return grad_input, None, None


def fused_apply_rotary_pos_emb(
    t: torch.Tensor, freqs: torch.Tensor, transpose_output_memory: bool = False
) -> torch.Tensor:
    """``t``: ``[s, b, h, d]``; ``freqs``: ``[s, 1, 1, d2]`` float.  With
    ``transpose_output_memory`` the result's memory is ``[b, s, h, d]`` (so that
    ``output.transpose(0, 1)`` is contiguous)."""
    return FusedRoPEFunc.apply(t, freqs, transpose_output_memory)


class FusedRoPECachedFunc(torch.autograd.Function):
    """Rotary embedding from cached ``cos`` / ``sin`` tables ``[s, 1, 1, d2]`` that are
    fp32 or of ``t``'s dtype."""

    @staticmethod
    def forward(ctx, t: torch.Tensor, cos_: torch.Tensor, sin_: torch.Tensor,
                transpose_output_memory: bool = False):
        output = _ext.forward_cached(t, cos_, sin_, transpose_output_memory)
        ctx.save_for_backward(cos_, sin_)
        ctx.transpose_output_memory = transpose_output_memory
        return output

    @staticmethod
    def backward(ctx, grad_output: torch.Tensor) -> Tuple[Union[torch.Tensor, None], ...]:
        cos_, sin_ = ctx.saved_tensors
        grad_input = _ext.backward_cached(grad_output, cos_, sin_, ctx.transpose_output_memory)
        return grad_input, None, None, None


def fused_apply_rotary_pos_emb_cached(
    t: torch.Tensor, cos_: torch.Tensor, sin_: torch.Tensor, transpose_output_memory: bool = False
) -> torch.Tensor:
    """``t``: ``[s, b, h, d]``; ``cos_``, ``sin_``: ``[s, 1, 1, d2]``."""
    return FusedRoPECachedFunc.apply(t, cos_, sin_, transpose_output_memory)
