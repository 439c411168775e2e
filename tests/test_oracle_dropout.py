"""Pins of the attention-dropout oracle (oracle/philox.py, oracle/torch_ref.py) on the CPU.

The reference draws its mask with torch.nn.Dropout under the RNG tracker
(megatron/model/transformer.py:536-539) and ships no vectors for it.  What can be pinned
without a GPU: the Philox block function against the known-answer vectors published with
Random123, the element -> field assignment against a per-element restatement written with
Python integers only, the statistics of the keep pattern, and the dropout arithmetic
against autograd of the same expression.
"""
import ctypes

import numpy as np
import pytest
import torch

from oracle import brute, philox, torch_ref

gpt_neox_amd = pytest.importorskip("gpt_neox_amd")
from gpt_neox_amd import _lib  # noqa: E402


# Random123 kat_vectors, the three "philox4x32 10" lines: counter[4], key[2] -> output[4]
KAT = [
    ((0, 0, 0, 0), (0, 0), (0x6627E8D5, 0xE169C58D, 0xBC57AC4C, 0x9B00DBD8)),
    ((0xFFFFFFFF,) * 4, (0xFFFFFFFF,) * 2, (0x408F276D, 0x41C83B0E, 0xA20BC7C6, 0x6D5451FD)),
    ((0x243F6A88, 0x85A308D3, 0x13198A2E, 0x03707344), (0xA4093822, 0x299F31D0),
     (0xD16CFE09, 0x94FDCCEB, 0x5001E420, 0x24126EA1)),
]


@pytest.mark.parametrize("counter,key,expected", KAT)
def test_philox_known_answers(counter, key, expected):
    out = philox.philox4x32_10(np.array(counter, dtype=np.uint64), key)
    assert tuple(int(v) for v in out) == expected


@pytest.mark.parametrize("counter,key,expected", KAT)
def test_integer_philox_known_answers(counter, key, expected):
    assert tuple(brute.philox4x32_10(counter, key)) == expected


@pytest.mark.parametrize("seed,offset", [(0, 0), (1234, 8), (2**63 + 12345, 2**40 + 4)])
def test_keep_mask_matches_the_per_element_restatement(seed, offset):
    n = 203
    mask = philox.keep_mask(n, 0.3, seed, offset)
    assert mask.dtype == np.bool_ and mask.shape == (n,)
    assert [bool(v) for v in mask] == [brute.keep_element(e, 0.3, seed, offset) for e in range(n)]


def test_keep_mask_statistics_and_structure():
    n = 1 << 20
    for p in (0.05, 0.1, 0.5, 0.9):
        kept = philox.keep_mask(n, p, 42, 0).mean()
        sigma = (p * (1 - p) / n) ** 0.5
        assert abs(kept - (1 - p)) < 5 * sigma + 2.0**-16, (p, kept)
    assert philox.keep_mask(4096, 0.0, 7, 0).all()
    assert not philox.keep_mask(4096, 1.0, 7, 0).any()
    a = philox.keep_mask(4096, 0.5, 7, 0)
    assert (a == philox.keep_mask(4096, 0.5, 7, 0)).all()  # a function of (seed, offset)
    assert (a[:1000] == philox.keep_mask(1000, 0.5, 7, 0)).all()  # and of the element index only
    for other in (philox.keep_mask(4096, 0.5, 8, 0), philox.keep_mask(4096, 0.5, 7, 4)):
        assert 0.4 < (a != other).mean() < 0.6  # another seed / offset: an unrelated pattern
    # a lower p keeps a superset (same bits, lower threshold)
    assert (philox.keep_mask(4096, 0.2, 7, 0) | ~a).all()
    # neighbouring elements are uncorrelated
    x = philox.keep_mask(n, 0.5, 3, 0).astype(np.float64) - 0.5
    for lag in (1, 2, 7, 8, 512):
        assert abs((x[:-lag] * x[lag:]).mean()) < 5 * 0.25 / n**0.5
    with pytest.raises(ValueError):
        philox.threshold(1.5)


def test_dropout_scale_and_expression():
    assert torch_ref.dropout_scale(0.0) == 1.0
    assert torch_ref.dropout_scale(1.0) == 0.0
    assert torch_ref.dropout_scale(0.5) == 2.0
    assert torch_ref.dropout_scale(0.1) == float(np.float32(1.0 / np.float64(np.float32(0.9))))
    assert float(philox.dropout_scale(0.1)) == torch_ref.dropout_scale(0.1)
    g = torch.Generator().manual_seed(5)
    probs = torch.softmax(torch.randn(4, 16, generator=g), -1).to(torch.bfloat16)
    keep = torch.from_numpy(philox.keep_mask(64, 0.25, 9, 0)).view(4, 16)
    out = torch_ref.dropout_with_mask(probs, keep, 0.25)
    assert out.dtype == torch.bfloat16
    assert (out[~keep] == 0).all()
    expect = (probs.float() * torch.tensor(4.0 / 3.0, dtype=torch.float32)).to(torch.bfloat16)
    assert torch.equal(out[keep], expect[keep])


def test_softmax_dropout_backward_matches_autograd_of_the_unfused_expression():
    g = torch.Generator().manual_seed(11)
    x = torch.randn(3, 5, 24, generator=g, dtype=torch.float64, requires_grad=True)
    grad_out = torch.randn(3, 5, 24, generator=g, dtype=torch.float64)
    keep = torch.from_numpy(philox.keep_mask(x.numel(), 0.3, 77, 4)).view(x.shape)
    scale, p = 0.7, 0.3
    probs = torch.softmax(scale * x, -1)
    dropped = probs * keep / (1 - p)
    (dx,) = torch.autograd.grad(dropped, x, grad_out)
    got = torch_ref.softmax_dropout_backward_fp32(grad_out.float(), probs.detach().float(), keep, p, scale)
    assert torch.allclose(got.double(), dx, atol=2e-6, rtol=1e-5)


@pytest.mark.parametrize("name", ["dropout_causal_16", "dropout_causal_37"])
def test_golden_dropout_vectors(golden, name):
    f = golden[name]
    p, seed, offset, scale = float(f["p"]), int(f["seed"]), int(f["offset"]), float(f["scale"])
    keep = philox.keep_mask(f["x"].size, p, seed, offset).reshape(f["x"].shape)
    assert np.array_equal(keep, f["keep"].astype(bool))
    x = torch.tensor(f["x"])
    s = x.shape[-1]
    probs = torch_ref.softmax_fp32(x.unsqueeze(1), torch_ref.get_attn_mask(s), scale).squeeze(1)
    assert np.abs(probs.numpy() - f["y"]).max() < 1e-6
    dropped = torch_ref.dropout_with_mask(probs, torch.from_numpy(keep), p)
    assert np.abs(dropped.numpy() - f["y_drop"]).max() < 1e-6
    dx = torch_ref.softmax_dropout_backward_fp32(torch.tensor(f["g"]), probs, torch.from_numpy(keep), p, scale)
    assert np.abs(dx.numpy() - f["dx"]).max() < 1e-5 * max(1.0, np.abs(f["dx"]).max())


def _call(name, *args):
    handle = _lib.lib()
    status = getattr(handle, name)(*args)
    return status, handle.neox_fused_last_error().decode()


def test_dropout_and_bias_entry_points_validate_before_touching_the_gpu():
    buf = (ctypes.c_uint16 * 64)()
    other = (ctypes.c_uint16 * 64)()
    third = (ctypes.c_uint16 * 64)()
    a, b, c = (ctypes.addressof(v) for v in (buf, other, third))
    status, msg = _call("neox_causal_softmax_dropout_fwd", a, b, c, None, None, 0, 1.0, 1.5, 0, 0, None, 1, 1, 8, 8, 0, None)
    assert status == -3 and "between 0 and 1" in msg
    status, msg = _call("neox_causal_softmax_dropout_fwd", a, a, c, None, None, 0, 1.0, 0.1, 0, 0, None, 1, 1, 8, 8, 0, None)
    assert status == -4 and "alias" in msg
    status, msg = _call("neox_causal_softmax_dropout_fwd", None, b, c, None, None, 0, 1.0, 0.1, 0, 0, None, 1, 1, 8, 8, 0, None)
    assert status == -1
    status, msg = _call("neox_causal_softmax_dropout_bwd", a, b, c, 1.0, -0.1, 0, 0, None, 1, 8, 8, 0, None)
    assert status == -3
    status, msg = _call("neox_masked_softmax_dropout_fwd", a, b, c, None, None, None, 0, 1.0, 0.1, 0, 0, None, 1, 1, 8, 8, 1, 0, None)
    assert status == -1
    status, msg = _call("neox_masked_softmax_dropout_fwd", a, b, c, a, None, None, 0, 1.0, 0.1, 0, 0, None, 2, 1, 8, 8, 3, 0, None)
    assert status == -3 and "mask batch" in msg
    status, msg = _call("neox_masked_softmax_dropout_bwd", a, b, c, 1.0, 0.1, 0, 0, None, 0, 8, 0, None)
    assert status == -3
    status, msg = _call("neox_masked_softmax_dropout_bwd", a, b, c, 1.0, 0.1, 0, 0, None, 4, 8, 2, None)
    assert status == -2
    # ALiBi slopes that are not aligned to their element size, with and without a bias tensor
    status, msg = _call("neox_causal_softmax_dropout_fwd", a, b, c, a + 2, b, 1, 1.0, 0.1, 0, 0, None, 1, 1, 8, 8, 0, None)
    assert status == -5
    status, msg = _call("neox_masked_softmax_dropout_fwd", a, b, c, a, a + 2, None, 0, 1.0, 0.1, 0, 0, None, 1, 1, 8, 8, 1, 0, None)
    assert status == -5
    status, msg = _call("neox_causal_softmax_dropout_fwd", a, b, c, None, a, 3, 1.0, 0.1, 0, 0, None, 2, 1, 8, 8, 0, None)
    assert status == -3 and "bias batch" in msg
    status, msg = _call("neox_masked_softmax_dropout_fwd", a, b, c, a, None, a + 1, 1, 1.0, 0.1, 0, 0, None, 1, 1, 8, 8, 1, 0, None)
    assert status == -5
    status, msg = _call("neox_causal_softmax_bias_fwd", a, b, c, None, 1.0, 2, 1, 8, 8, 3, 0, None)
    assert status == -3 and "bias batch" in msg
    status, msg = _call("neox_causal_softmax_bias_fwd", a, b, None, None, 1.0, 2, 1, 8, 8, 1, 0, None)
    assert status == -1
    status, msg = _call("neox_masked_softmax_bias_fwd", a, b, c, a, None, 1.0, 2, 1, 8, 8, 1, 4, 0, None)
    assert status == -3 and "bias batch" in msg
    status, msg = _call("neox_masked_softmax_bias_fwd", a, b, c, a, None, 1.0, 2, 1, 8, 8, 1, 1, 7, None)
    assert status == -2
    status, msg = _call("neox_masked_softmax_alibi_fwd", a, b, c, None, 1.0, 2, 1, 8, 8, 1, 0, None)
    assert status == -1
    status, msg = _call("neox_masked_softmax_alibi_fwd", a, b, c, a, 1.0, 2, 1, 8, 8, 3, 0, None)
    assert status == -3 and "mask batch" in msg
    # the sliding-window entry points take aligned square rows of 513 to 32768 columns only
    status, msg = _call("neox_sliding_window_softmax_fwd", a, b, 1.0, 1, 512, 512, 4, 0, None)
    assert status == -3 and "sk=512" in msg
    status, msg = _call("neox_sliding_window_softmax_fwd", a, b, 1.0, 1, 1024, 2048, 4, 0, None)
    assert status == -3 and "equal" in msg
    status, msg = _call("neox_sliding_window_softmax_fwd", a, b, 1.0, 1, 1024, 1024, -1, 0, None)
    assert status == -3 and "window" in msg
    status, msg = _call("neox_sliding_window_softmax_bwd", a, b, c + 2, 1.0, 1, 1024, 1024, 4, 1, None)
    assert status == -5
    status, msg = _call("neox_sliding_window_softmax_bwd", a, None, c, 1.0, 1, 1024, 1024, 4, 1, None)
    assert status == -1
    status, msg = _call("neox_mask_classify", None, a, 1, 8, 8, None)
    assert status == -1
    status, msg = _call("neox_mask_classify", a, b, 1, 8, 9, None)
    assert status == -3 and "equal" in msg
    status, msg = _call("neox_mask_classify", a, b, 0, 8, 8, None)
    assert status == -3
    status, msg = _call("neox_dropout_keep_mask", None, 0.1, 0, 0, None, 8, None)
    assert status == -1
    status, msg = _call("neox_dropout_keep_mask", a, float("nan"), 0, 0, None, 8, None)
    assert status == -3
    status, msg = _call("neox_dropout_keep_mask", a, 0.1, 0, 0, None, 0, None)
    assert status == -3
    status, msg = _call("neox_dropout_keep_mask", a, 0.1, 0, 0, a + 4, 8, None)  # state not 8-byte aligned
    assert status == -5 and "device_state" in msg
