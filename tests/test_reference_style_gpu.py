"""The reference's own two fused-kernel tests, on synthetic attention scores.

tests/model/test_fused_kernels.py:48-253 of the reference builds layer-0 attention scores
of a downloaded BERT / GPT-2, runs ``FusedScaleMaskSoftmax`` once with a fused fusion
type and once with ``SoftmaxFusionTypes.none`` (fp16, ``scale=None``,
``softmax_in_fp32=False``) and prints whether the mean absolute difference is <= 1e-3.
The checkpoints cannot be fetched here, so the scores come from a random embedding and
random query/key projections of the same sizes (12 heads of 64 dims); the modules, their
arguments and the bar are the reference's, and the bar is asserted instead of printed.
"""
import math

import pytest
import torch

from gpt_neox_amd.fused_kernels import load
from gpt_neox_amd.fused_softmax import FusedScaleMaskSoftmax, SoftmaxFusionTypes
from oracle.torch_ref import gpt2_attention_mask_func as attention_mask_func

pytestmark = pytest.mark.gpu


def layer0_scores(device, batch, seq, heads=12, head_dim=64, seed=0):
    g = torch.Generator(device=device).manual_seed(seed)
    hidden = heads * head_dim
    embedding_output = torch.randn(batch, seq, hidden, device=device, generator=g).half()
    wq = (torch.randn(hidden, hidden, device=device, generator=g) * 0.05).half()
    wk = (torch.randn(hidden, hidden, device=device, generator=g) * 0.05).half()

    def transpose_for_scores(x):
        return x.view(batch, seq, heads, head_dim).permute(0, 2, 1, 3)

    query_layer = transpose_for_scores(embedding_output @ wq)
    key_layer = transpose_for_scores(embedding_output @ wk)
    attention_scores = torch.matmul(query_layer, key_layer.transpose(-1, -2))
    attention_scores /= math.sqrt(key_layer.size()[-1])
    return attention_scores


def softmax_pair(fusion_type):
    def make(ft):
        return FusedScaleMaskSoftmax(
            input_in_fp16=True, input_in_bf16=False, fusion_type=ft, mask_func=attention_mask_func,
            scale=None, softmax_in_fp32=False).cuda().half()

    return make(fusion_type), make(SoftmaxFusionTypes.none)


def mean_difference(a, b):
    test_result = (a - b).abs()
    while test_result.dim() != 1:
        test_result = test_result.mean(dim=-1)
    return test_result.mean(dim=-1).item()


def test_load_fused_kernels():
    load()
    import scaled_masked_softmax_cuda  # noqa: F401  (registered by load_fused_kernels)
    import scaled_upper_triang_masked_softmax_cuda  # noqa: F401
    import fused_rotary_positional_embedding  # noqa: F401


def test_fused_softmax(device):
    batch, seq = 4, 36  # four copies of one tokenised sentence; the last 4 positions are padding
    attention_scores = layer0_scores(device, batch, seq)
    attention_mask = torch.ones(batch, seq, device=device)
    attention_mask[:, -4:] = 0
    extended = (1.0 - attention_mask[:, None, None, :]) * torch.finfo(torch.float16).min  # (bsz, 1, 1, seq)
    mask = extended.repeat(1, 1, seq, 1)  # (bsz, 1, seq, seq)
    fused_softmax, torch_softmax = softmax_pair(SoftmaxFusionTypes.general)
    assert fused_softmax.is_kernel_available(mask != 0, *attention_scores.shape)
    fused_softmax_output = fused_softmax(attention_scores, (mask != 0))
    torch_softmax_output = torch_softmax(attention_scores.clone(), (mask != 0))
    assert mean_difference(fused_softmax_output, torch_softmax_output) <= 1e-3
    assert (fused_softmax_output - torch_softmax_output).abs().max().item() <= 2e-3
    assert (fused_softmax_output[..., -4:] == 0).all()


def test_fused_upper_triangle_mask_softmax(device):
    batch, seq = 4, 24
    attention_scores = layer0_scores(device, batch, seq, seed=1)
    attn_mask = torch.tril(torch.ones(seq, seq, device=device)).view(1, 1, seq, seq) < 0.5
    total_mask = attn_mask.repeat(batch, 1, 1, 1)
    fused_softmax, torch_softmax = softmax_pair(SoftmaxFusionTypes.upper_triang)
    assert fused_softmax.is_kernel_available(total_mask, *attention_scores.shape)
    fused_softmax_output = fused_softmax(attention_scores, total_mask)
    torch_softmax_output = torch_softmax(attention_scores.clone(), total_mask)
    assert mean_difference(fused_softmax_output, torch_softmax_output) <= 1e-3
    assert (fused_softmax_output - torch_softmax_output).abs().max().item() <= 2e-3
    assert (fused_softmax_output[total_mask.expand_as(fused_softmax_output)] == 0).all()
