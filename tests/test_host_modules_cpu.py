"""Host-side logic of the drop-in modules that runs without a GPU: the unfused
branch of FusedScaleMaskSoftmax, the rotary tables, the torch branch of the rotary
apply for non-GPU tensors, and the plain-torch Sinusoidal / AliBi modules."""
import math

import pytest
import torch

from gpt_neox_amd.fused_softmax import FusedScaleMaskSoftmax, SoftmaxFusionTypes
from gpt_neox_amd.positional_embeddings import (
    AliBi,
    RotaryEmbedding,
    SinusoidalPositionalEmbedding,
    apply_rotary_pos_emb,
    apply_rotary_pos_emb_,
    apply_rotary_pos_emb_torch,
    rotate_half,
)
from oracle import torch_ref as R


@pytest.mark.parametrize("dtype,fp16,bf16", [(torch.float16, True, False), (torch.bfloat16, False, True)])
def test_unfused_branch_equals_the_oracle(dtype, fp16, bf16):
    x = (torch.randn(2, 3, 8, 8) * 8).to(dtype)
    mask = R.get_attn_mask(8)
    mod = FusedScaleMaskSoftmax(fp16, bf16, SoftmaxFusionTypes.none, R.gpt2_attention_mask_func, True, 0.125)
    y = mod(x, mask)
    want = R.forward_torch_softmax(x, mask, 0.125, fp16, bf16, True)
    assert y.dtype == dtype and torch.equal(y, want)
    # mask None -> plain scaled softmax
    assert torch.equal(mod(x, None), R.forward_torch_softmax(x, None, 0.125, fp16, bf16, True))


def test_unfused_branch_taken_when_predicate_fails_even_with_fusion_requested():
    mod = FusedScaleMaskSoftmax(False, False, SoftmaxFusionTypes.general, R.gpt2_attention_mask_func, True, None)
    x = torch.randn(1, 2, 4, 4)  # fp32 input: not a fused case
    y = mod(x, R.get_attn_mask(4))
    assert torch.allclose(y.sum(-1), torch.ones(1, 2, 4))


def test_rotary_embedding_tables_equal_the_oracle():
    for prec in (torch.float, torch.half, torch.bfloat16):
        emb = RotaryEmbedding(32, 64, base=10000, precision=prec)
        cos, sin = R.rotary_tables(32, 64, 10000, prec)
        assert torch.equal(emb.cos_cached, cos) and torch.equal(emb.sin_cached, sin)
        c, s = emb(torch.zeros(10, 1, 1, 32))
        assert c.shape == (10, 1, 1, 32) and torch.equal(c, cos[:10]) and torch.equal(s, sin[:10])
        c, s = emb(torch.zeros(3, 1), seq_len=64)
        assert c.shape[0] == 64
        assert emb.inv_freq.dtype == prec and emb.inv_freq.shape == (16,)
    with pytest.raises(AssertionError):
        emb(torch.zeros(65, 1, 1, 32))


def test_rotary_embedding_state_dict_and_attributes():
    assert "inv_freq" not in RotaryEmbedding(8, 16).state_dict()
    assert "inv_freq" in RotaryEmbedding(8, 16, save_inv_freqs=True).state_dict()
    emb = RotaryEmbedding(8, 16, base=500, precision=torch.float)
    assert (emb.dim, emb.max_seq_len, emb.base, emb.precision) == (8, 16, 500, torch.float)
    assert emb.emb.shape == (16, 1, 1, 8) and emb.emb.dtype == torch.float32
    assert emb.inv_freq[1].item() == pytest.approx(500 ** (-2 / 8), rel=1e-6)


def test_rotary_apply_on_cpu_or_fp32_is_the_torch_expression():
    cos, sin = R.rotary_tables(8, 12)
    q, k = torch.randn(5, 2, 3, 8), torch.randn(5, 2, 3, 8)
    for fn in (apply_rotary_pos_emb, apply_rotary_pos_emb_torch):
        oq, ok = fn(q, k, cos, sin, offset=4)
        rq, rk = R.apply_rotary_pos_emb(q, k, cos, sin, 4)
        assert torch.equal(oq, rq) and torch.equal(ok, rk)
    assert torch.equal(rotate_half(q), R.rotate_half(q))
    with pytest.raises(RuntimeError, match="GPU tensors"):
        apply_rotary_pos_emb_(q.half(), k.half(), cos, sin)


def test_sinusoidal_embedding():
    mod = SinusoidalPositionalEmbedding(8, base=10000, precision=torch.float)
    out = mod(torch.zeros(2, 5, 8))
    assert out.shape == (1, 5, 8)
    for t in range(5):
        for i in range(4):
            ang = t * 10000.0 ** (-2.0 * i / 8)
            assert out[0, t, i].item() == pytest.approx(math.sin(ang), abs=1e-6)
            assert out[0, t, 4 + i].item() == pytest.approx(math.cos(ang), abs=1e-6)
    assert SinusoidalPositionalEmbedding(8, precision=torch.bfloat16)(torch.zeros(1, 3, 8)).dtype == torch.bfloat16


def test_alibi_slopes_and_bias():
    assert AliBi(8)._get_slopes(8) == pytest.approx([2.0 ** -(i + 1) for i in range(8)])
    s6 = AliBi(6, mp_size=1, mp_rank=0)._get_slopes(6)
    assert s6[:4] == pytest.approx([2.0 ** -(2 * (i + 1)) for i in range(4)])
    assert s6[4:] == pytest.approx([2.0 ** -1, 2.0 ** -3])
    a = AliBi(4, mp_size=2, mp_rank=1)  # second half of the heads
    assert torch.allclose(a.slopes, torch.tensor([2.0 ** -6, 2.0 ** -8]))
    x = torch.zeros(1, 2, 5, 5)
    y = a(x)
    for h in range(2):
        for i in range(5):
            for j in range(5):
                want = -a.slopes[h].item() * (i - j) if j <= i else 0.0
                assert y[0, h, i, j].item() == pytest.approx(want, abs=1e-7)
    # decode step: one query against 5 keys uses the last row of the bias
    y1 = a(torch.zeros(1, 2, 1, 5))
    assert torch.allclose(y1[0, :, 0, :], y[0, :, 4, :])
    assert a.cached_seq_len == 5
    a(torch.zeros(1, 2, 7, 7))
    assert a.cached_seq_len == 20  # grown 4x
    assert torch.equal(a.bias(7, 7, "cpu", torch.float32), a(torch.zeros(1, 2, 7, 7))[0])


def test_alibi_bias_helper_equals_the_alibi_module_and_the_oracle():
    from gpt_neox_amd.fused_softmax import alibi_bias

    mod = AliBi(6, mp_size=1, mp_rank=0)
    assert mod.slopes.tolist() == pytest.approx(R.alibi_slopes(6))
    for dtype in (torch.float32, torch.bfloat16):
        x = torch.zeros(2, 6, 9, 9, dtype=dtype)
        assert torch.equal(mod(x)[0], alibi_bias(mod.slopes, 9, 9, "cpu", dtype))
    assert torch.equal(alibi_bias(mod.slopes, 9, 9, "cpu", torch.float32), R.alibi_bias_fp32(mod.slopes, 9, 9))
    one = AliBi(6, mp_size=1, mp_rank=0)
    assert torch.equal(one(torch.zeros(2, 6, 1, 9))[0], alibi_bias(mod.slopes, 1, 9, "cpu", torch.float32))


def test_alibi_slopes_argument_on_the_unfused_branch():
    mod = AliBi(4, mp_size=1, mp_rank=0)
    x = torch.randn(2, 4, 8, 8)
    mask = R.get_attn_mask(8)
    sm = FusedScaleMaskSoftmax(False, False, SoftmaxFusionTypes.none, R.gpt2_attention_mask_func, True, 0.5)
    assert torch.equal(sm(x.clone(), mask, alibi_slopes=mod.slopes), sm(mod(x.clone()), mask))


def test_get_fusion_type_prefers_the_causal_kernel():
    from types import SimpleNamespace

    from gpt_neox_amd.utils import get_fusion_type

    def args(causal, general):
        return SimpleNamespace(scaled_upper_triang_masked_softmax_fusion=causal,
                               scaled_masked_softmax_fusion=general)

    assert get_fusion_type(args(False, False)) is SoftmaxFusionTypes.none
    assert get_fusion_type(args(False, True)) is SoftmaxFusionTypes.general
    assert get_fusion_type(args(True, False)) is SoftmaxFusionTypes.upper_triang
    assert get_fusion_type(args(True, True)) is SoftmaxFusionTypes.upper_triang


def test_dropout_and_bias_arguments_on_the_unfused_branch():
    # fusion off: softmax of (scores + bias) by the torch expression, then torch's dropout
    m = FusedScaleMaskSoftmax(False, True, SoftmaxFusionTypes.none, R.gpt2_attention_mask_func, True, 0.5)
    g = torch.Generator().manual_seed(3)
    x = (torch.randn(2, 2, 16, 16, generator=g) * 4).bfloat16()
    bias = torch.randn(1, 2, 16, 16, generator=g).bfloat16()
    mask = R.get_attn_mask(16)
    assert torch.equal(m(x, mask, bias=bias), m(x + bias, mask))
    torch.manual_seed(5)
    out = m(x, mask, dropout_p=0.5)
    base = m(x, mask)
    kept = out != 0
    assert 0.2 < kept[..., ~mask[0, 0]].float().mean() < 0.8
    assert torch.allclose(out[kept].float(), 2 * base[kept].float(), rtol=1e-2)
    assert torch.equal(m(x, mask, dropout_p=0.0), base)
