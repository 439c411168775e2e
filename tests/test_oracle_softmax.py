"""Pins of the softmax oracle (oracle/torch_ref.py, oracle/brute.py) -- CPU only.

The reference has no golden vectors or asserting tests for this path
(tests/model/test_fused_kernels.py only prints a mean difference on model
activations it downloads), so the restated torch path is pinned by closed forms,
invariants, an independent float64 loop evaluation, finite differences and the
committed fixtures.  Each check is chosen so that a plausible slip (scale applied
after the mask, mask polarity flipped, softmax over the wrong dim, dropped
``- y*sum`` term, missing scale in the backward) fails it.
"""
import math

import numpy as np
import pytest
import torch

from oracle import brute
from oracle import torch_ref as R


def test_attn_mask_is_strict_upper_triangle():
    m = R.get_attn_mask(5)
    assert m.shape == (1, 1, 5, 5) and m.dtype == torch.bool
    expect = torch.tensor([[c > r for c in range(5)] for r in range(5)])
    assert torch.equal(m[0, 0], expect)


def test_attn_mask_sliding_window():
    m = R.get_attn_mask(6, sliding_window_width=2)[0, 0]
    for r in range(6):
        for c in range(6):
            assert bool(m[r, c]) == (c > r or c < r - 2)


def test_mask_func_fills_lowest_finite_value_in_place():
    for dt in (torch.float32, torch.float16, torch.bfloat16):
        s = torch.zeros(1, 1, 2, 2, dtype=dt)
        out = R.gpt2_attention_mask_func(s, torch.tensor([[[[False, True], [False, False]]]]))
        assert out is s
        assert s[0, 0, 0, 1].item() == torch.finfo(dt).min and s[0, 0, 0, 0].item() == 0


def test_causal_constant_input_closed_form():
    # equal scores: row i is 1/(i+1) on j <= i, exactly 0 elsewhere
    s = 7
    x = torch.full((1, 1, s, s), 3.0)
    y = R.forward_torch_softmax(x, R.get_attn_mask(s), scale=0.37)
    for i in range(s):
        assert torch.allclose(y[0, 0, i, : i + 1], torch.full((i + 1,), 1.0 / (i + 1)), atol=1e-7)
        assert (y[0, 0, i, i + 1 :] == 0).all()


def test_causal_row0_is_one_hot():
    x = torch.randn(2, 3, 6, 6) * 8
    y = R.forward_torch_softmax(x, R.get_attn_mask(6), 0.125)
    assert torch.equal(y[..., 0, 0], torch.ones(2, 3)) and (y[..., 0, 1:] == 0).all()


def test_two_element_row_is_logistic_of_scaled_difference():
    # softmax([a, b] * s) = [sigmoid(s(a-b)), sigmoid(s(b-a))]: pins where the scale enters
    a, b, s = 1.25, -0.5, 0.3
    y = R.forward_torch_softmax(torch.tensor([[[[a, b]]]]), None, s)
    assert y[0, 0, 0, 0].item() == pytest.approx(1 / (1 + math.exp(-s * (a - b))), abs=1e-7)


def test_padding_constant_input_is_one_over_len():
    lens = [3, 8, 1]
    mask = R.padding_mask(lens, sq=4, sk=8)
    y = R.forward_torch_softmax(torch.zeros(3, 2, 4, 8), mask, 0.125)
    for b, n in enumerate(lens):
        assert torch.allclose(y[b, :, :, :n], torch.full((2, 4, n), 1.0 / n), atol=1e-7)
        assert (y[b, :, :, n:] == 0).all()


def test_fully_masked_row_is_uniform():
    mask = torch.ones(1, 1, 2, 8, dtype=torch.bool)
    y = R.forward_torch_softmax(torch.randn(1, 3, 2, 8), mask, 0.5)
    assert torch.allclose(y, torch.full_like(y, 1 / 8))


def test_rows_sum_to_one_and_shift_invariance():
    x = torch.randn(2, 2, 9, 9, dtype=torch.float64) * 4
    m = R.get_attn_mask(9)
    y = R.forward_torch_softmax(x, m, 0.2)
    assert torch.allclose(y.sum(-1), torch.ones(2, 2, 9, dtype=torch.float64), atol=1e-12)
    y2 = R.forward_torch_softmax(x + 11.0, m, 0.2)
    assert torch.allclose(y, y2, atol=1e-12)


def test_half_input_goes_through_fp32_and_is_cast_back():
    x = (torch.randn(1, 2, 8, 8) * 8).to(torch.bfloat16)
    m = R.get_attn_mask(8)
    y = R.forward_torch_softmax(x, m, 0.125, input_in_bf16=True, softmax_in_fp32=True)
    assert y.dtype == torch.bfloat16
    assert torch.equal(y, R.softmax_fp32(x, m, 0.125).bfloat16())
    assert torch.equal(x, x.clone())  # the half input itself is not modified


@pytest.mark.parametrize("seed", [0, 1, 2])
def test_torch_ref_matches_float64_loops(seed):
    rng = np.random.default_rng(seed)
    x = rng.normal(size=(6, 6)) * 8
    y_loop = brute.softmax_rows(x, 0.3, brute.causal_hidden(6, 6))
    y_t = R.forward_torch_softmax(torch.tensor(x)[None, None], R.get_attn_mask(6), 0.3)[0, 0]
    assert np.allclose(y_t.numpy(), y_loop, atol=1e-12)
    hidden = rng.random((6, 6)) < 0.4
    hidden[2, :] = True
    y_loop = brute.softmax_rows(x, 0.3, hidden)
    y_t = R.forward_torch_softmax(torch.tensor(x)[None, None], torch.tensor(hidden)[None, None], 0.3)
    assert np.allclose(y_t[0, 0].numpy(), y_loop, atol=1e-12)


def test_fixtures_forward(golden):
    for name in ("causal_8", "causal_40"):
        f = golden[name]
        s = f["x"].shape[-1]
        y = R.softmax_fp32(torch.tensor(f["x"])[None], R.get_attn_mask(s), float(f["scale"]))[0]
        assert np.allclose(y.numpy(), f["y"], atol=2e-7), name
        assert (y.numpy()[f["y"] == 0] == 0).all()
    for name in ("masked_4x16", "masked_3x37"):
        f = golden[name]
        y = R.softmax_fp32(torch.tensor(f["x"]), torch.tensor(f["mask"]).bool(), float(f["scale"]))
        assert np.allclose(y.numpy(), f["y"], atol=2e-7), name
        assert (y.numpy()[f["y"] == 0] == 0).all()


# ---- backward -----------------------------------------------------------------------


def test_backward_closed_form_matches_autograd_fp64():
    x = torch.randn(1, 2, 5, 5, dtype=torch.float64)
    g = torch.randn(1, 2, 5, 5, dtype=torch.float64)
    m = R.get_attn_mask(5)
    xr = x.clone().requires_grad_(True)
    y = torch.softmax(R.gpt2_attention_mask_func(xr * 0.7, m), -1)
    y.backward(g)
    dx = R.softmax_backward_fp32(g, y.detach(), 0.7)  # float() of float64 loses bits: compare at 1e-6
    assert torch.allclose(dx.double(), xr.grad, atol=1e-6)
    assert (xr.grad.masked_select(m.expand_as(xr.grad)) == 0).all()


def test_backward_finite_differences():
    # d/dx of L = sum(g * softmax(s x)) by central differences, float64 loops only
    rng = np.random.default_rng(5)
    x = rng.normal(size=(1, 6))
    g = rng.normal(size=(1, 6))
    s = 0.45
    y = brute.softmax_rows(x, s)
    dx = brute.softmax_rows_backward(g, y, s)
    for j in range(6):
        xp, xm = x.copy(), x.copy()
        xp[0, j] += 1e-6
        xm[0, j] -= 1e-6
        num = ((g * brute.softmax_rows(xp, s)).sum() - (g * brute.softmax_rows(xm, s)).sum()) / 2e-6
        assert dx[0, j] == pytest.approx(num, abs=1e-8)
    dxt = R.softmax_backward_fp32(torch.tensor(g), torch.tensor(y), s)
    assert np.allclose(dxt.numpy(), dx, atol=1e-6)


def test_backward_invariants():
    y = torch.softmax(torch.randn(4, 9, dtype=torch.float64), -1)
    g = torch.randn(4, 9, dtype=torch.float64)
    dx = R.softmax_backward_fp32(g, y, 1.0)
    assert torch.allclose(dx.sum(-1), torch.zeros(4), atol=1e-6)  # rows of dx sum to 0
    const = R.softmax_backward_fp32(torch.full((4, 9), 2.5), y, 1.0)
    assert torch.allclose(const, torch.zeros(4, 9), atol=1e-6)  # constant g -> zero gradient
    assert torch.allclose(R.softmax_backward_fp32(g, y, 3.0), 3.0 * dx)  # linear in scale


def test_autograd_helper_matches_closed_form():
    x = (torch.randn(2, 2, 6, 6) * 8).half()
    g = torch.randn(2, 2, 6, 6).half()
    m = R.get_attn_mask(6)
    y, dx = R.softmax_autograd_fp32(x, m, 0.125, g)
    assert torch.allclose(dx, R.softmax_backward_fp32(g, y, 0.125), atol=1e-6)


def test_fixtures_backward(golden):
    for name in ("causal_8", "causal_40", "masked_4x16", "masked_3x37"):
        f = golden[name]
        dx = R.softmax_backward_fp32(torch.tensor(f["g"]), torch.tensor(f["y"]), float(f["scale"]))
        assert np.allclose(dx.numpy(), f["dx"], atol=1e-5), name


# ---- ALiBi bias -----------------------------------------------------------------------


def test_alibi_slopes_and_bias_closed_forms():
    assert R.alibi_slopes(8) == pytest.approx([2.0 ** -(k + 1) for k in range(8)])
    assert R.alibi_slopes(4) == pytest.approx([2.0 ** -2, 2.0 ** -4, 2.0 ** -6, 2.0 ** -8])
    s6 = R.alibi_slopes(6)  # 4 slopes of n=4, then slopes 0 and 2 of n=8
    assert s6 == pytest.approx([2.0 ** -2, 2.0 ** -4, 2.0 ** -6, 2.0 ** -8, 2.0 ** -1, 2.0 ** -3])
    bias = R.alibi_bias_fp32([0.5, 0.25], 4, 4)
    assert bias.shape == (2, 4, 4)
    for h, m in enumerate((0.5, 0.25)):
        for i in range(4):
            for j in range(4):
                assert bias[h, i, j].item() == (-m * (i - j) if j <= i else 0.0)
    # one query against a key/value cache: the query stands at the last key position
    last = R.alibi_bias_fp32([0.5, 0.25], 1, 5)
    assert last.shape == (2, 1, 5)
    assert last[0, 0].tolist() == [-2.0, -1.5, -1.0, -0.5, 0.0] and last[1, 0].tolist() == [-1.0, -0.75, -0.5, -0.25, 0.0]
    with pytest.raises(AssertionError):
        R.alibi_bias_fp32([0.5], 2, 5)


def test_alibi_softmax_row_closed_form():
    # zero scores: row i of head h is softmax_j(-m (i - j)) = a geometric distribution
    m, s = 0.5, 6
    y = R.softmax_fp32(torch.zeros(1, 1, s, s) + R.alibi_bias_fp32([m], s, s), R.get_attn_mask(s), 1.0)
    for i in range(s):
        w = [math.exp(-m * (i - j)) for j in range(i + 1)]
        for j in range(i + 1):
            assert y[0, 0, i, j].item() == pytest.approx(w[j] / sum(w), abs=1e-6)
