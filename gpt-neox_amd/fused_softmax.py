"""Drop-in for ``megatron/model/fused_softmax.py`` on MI355X.

Same public names, constructor arguments, call signatures and tensor layouts as
the reference module (megatron/model/fused_softmax.py:24-205):
``ScaledUpperTriangMaskedSoftmax``, ``ScaledMaskedSoftmax``, ``SoftmaxFusionTypes``,
``FusedScaleMaskSoftmax``.  The fused branches run hand-written gfx950 kernels
through the C-ABI library; the unfused branch is the same sequence of torch ops
as the reference's ``forward_torch_softmax``.

What differs from the reference, on purpose:

* the fused kernels take any ``sk`` (the reference stops at 2048 and silently
  runs the torch path beyond it) and need none of the ``sq % 4``,
  ``attn_batches % 4`` or ``% batch_per_block`` divisibility rules, which were
  artefacts of the CUDA launch shape -- see :meth:`is_kernel_available`;
* masked scores are excluded, so their probability is exactly 0 as in the torch
  path (the reference's padded kernel fills -10000), and a fully masked row is
  uniform ``1/sk`` as in the torch path;
* ``scale`` is applied in fp32 (the reference's forward narrows it to fp16/bf16);
* a missing kernel library raises ``ImportError`` instead of calling ``exit()``.
"""
import enum

import torch
import torch.nn as nn

from .fused_kernels import load_fused_kernels
from .fused_kernels import scaled_masked_softmax_cuda
from .fused_kernels import scaled_upper_triang_masked_softmax_cuda


class ScaledUpperTriangMaskedSoftmax(torch.autograd.Function):
    """
    Fused operation which performs following three operations in sequence
    1. Scale the tensor.
    2. Apply upper triangular mask (typically used in gpt models).
    3. Perform softmax.

    ``inputs`` is ``[attn_batches, sq, sk]`` fp16/bf16; reference:
    megatron/model/fused_softmax.py:24-53.
    """

    @staticmethod
    def forward(ctx, inputs, scale):
        scale_t = torch.tensor([scale])  # 1-element fp32 CPU tensor, as in the reference
        softmax_results = scaled_upper_triang_masked_softmax_cuda.forward(inputs, scale_t[0].item())
        ctx.save_for_backward(softmax_results, scale_t)
        return softmax_results

    @staticmethod
    def backward(ctx, output_grads):
        softmax_results, scale_t = ctx.saved_tensors
        input_grads = scaled_upper_triang_masked_softmax_cuda.backward(
            output_grads, softmax_results, scale_t[0].item()
        )
        return input_grads, None


class ScaledMaskedSoftmax(torch.autograd.Function):
    """
    Fused operation which performs following three operations in sequence
    1. Scale the tensor.
    2. Apply the mask.
    3. Perform softmax.

    ``inputs`` is ``[b, np, sq, sk]`` fp16/bf16, ``mask`` is ``[1 or b, 1, sq, sk]``
    bool/uint8 with True = masked; reference: megatron/model/fused_softmax.py:56-83.
    """

    @staticmethod
    def forward(ctx, inputs, mask, scale):
        scale_t = torch.tensor([scale])
        softmax_results = scaled_masked_softmax_cuda.forward(inputs, mask, scale_t[0].item())
        ctx.save_for_backward(softmax_results, scale_t)
        return softmax_results

    @staticmethod
    def backward(ctx, output_grads):
        softmax_results, scale_t = ctx.saved_tensors
        input_grads = scaled_masked_softmax_cuda.backward(
            output_grads, softmax_results, scale_t[0].item()
        )
        return input_grads, None, None


class SoftmaxFusionTypes(enum.Enum):
    upper_triang = 1  # causal mask
    general = 2  # general mask
    none = 3  # no fusion


class FusedScaleMaskSoftmax(nn.Module):
    """
    fused operation: scaling + mask + softmax
    Arguments:
        input_in_fp16: flag to indicate if input in fp16 data format.
        input_in_bf16: flag to indicate if input in bf16 data format.
        fusion_type: type of fusion to perform, should be either upper_triang, general or none. None will perform a regular torch softmax.
        mask_func: mask function to be applied.
        softmax_in_fp32: if true, softmax in performed at fp32 precision.
        scale: scaling factor used in input tensor scaling.

    Reference: megatron/model/fused_softmax.py:92-205.
    """

    def __init__(
        self,
        input_in_fp16,
        input_in_bf16,
        fusion_type,
        mask_func,
        softmax_in_fp32,
        scale,
    ):
        super().__init__()
        self.input_in_fp16 = input_in_fp16
        self.input_in_bf16 = input_in_bf16
        self.input_in_float16 = self.input_in_fp16 or self.input_in_bf16

        assert fusion_type in [
            SoftmaxFusionTypes.upper_triang,
            SoftmaxFusionTypes.general,
            SoftmaxFusionTypes.none,
        ], f"Invalid fusion type {fusion_type}"

        if fusion_type != SoftmaxFusionTypes.none:
            load_fused_kernels()  # check fused kernels are installed

        self.upper_triang_mask_fusion = fusion_type == SoftmaxFusionTypes.upper_triang
        self.general_mask_fusion = fusion_type == SoftmaxFusionTypes.general
        self.fusion = fusion_type != SoftmaxFusionTypes.none

        self.mask_func = mask_func
        self.softmax_in_fp32 = softmax_in_fp32
        self.scale = scale

        assert (
            self.scale is None or softmax_in_fp32
        ), "softmax should be in fp32 when scaled"

    def forward(self, input, mask):
        # [b, np, sq, sk]
        assert input.dim() == 4
        if self.is_kernel_available(mask, *input.size()):
            return self.forward_fused_softmax(input, mask)
        else:
            return self.forward_torch_softmax(input, mask)

    def is_kernel_available(self, mask, b, np, sq, sk):
        """Whether the fused branch serves this call.

        Kept from the reference predicate (megatron/model/fused_softmax.py:148-168):
        the user asked for fusion, the input is fp16/bf16, a mask tensor is given.
        Dropped: ``16 < sk <= 2048``, ``sq % 4``, ``(b*np) % 4`` and the
        ``batch_per_block`` rules.  Added: the causal branch needs ``sq == sk`` (the
        reference asserts it later; a decode step with ``sq == 1`` goes to the torch path
        with the mask it was given), and the tensor must not be empty.
        """
        if not (self.fusion and self.input_in_float16 and mask is not None):
            return False
        if b * np * sq * sk == 0:
            return False
        if self.upper_triang_mask_fusion:
            return sq == sk
        return True

    @staticmethod
    def reference_is_kernel_available(fusion, upper_triang, input_in_float16, mask, b, np, sq, sk):
        """The reference's own predicate (megatron/model/fused_softmax.py:148-168),
        evaluated with wave64 ``get_batch_per_block`` values; for comparison only."""
        attn_batches = b * np
        if (
            fusion
            and input_in_float16
            and mask is not None
            and 16 < sk <= 2048
            and sq % 4 == 0
            and attn_batches % 4 == 0
        ):
            batch_per_block = FusedScaleMaskSoftmax.get_batch_per_block(sq, sk, b, np)
            if upper_triang:
                return attn_batches % batch_per_block == 0
            return sq % batch_per_block == 0
        return False

    def forward_fused_softmax(self, input, mask):
        b, np, sq, sk = input.size()
        scale = self.scale if self.scale is not None else 1.0
        if self.upper_triang_mask_fusion:
            assert sq == sk, "causal mask is only for self attention"

            # input is 3D tensor (attn_batches, sq, sk)
            input = input.view(-1, sq, sk)
            probs = ScaledUpperTriangMaskedSoftmax.apply(input, scale)
            return probs.view(b, np, sq, sk)
        else:
            # input is 4D tensor (b, np, sq, sk)
            return ScaledMaskedSoftmax.apply(input, mask, scale)

    def forward_torch_softmax(self, input, mask):
        if self.input_in_float16 and self.softmax_in_fp32:
            input = input.float()

        if self.scale is not None:
            input = input * self.scale
        mask_output = self.mask_func(input, mask) if mask is not None else input
        probs = torch.nn.Softmax(dim=-1)(mask_output)

        if self.input_in_float16 and self.softmax_in_fp32:
            if self.input_in_fp16:
                probs = probs.half()
            else:
                probs = probs.bfloat16()

        return probs

    @staticmethod
    def get_batch_per_block(sq, sk, b, np):
        return scaled_masked_softmax_cuda.get_batch_per_block(sq, sk, b, np)
