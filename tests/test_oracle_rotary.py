"""Pins of the rotary oracle (oracle/torch_ref.py, oracle/brute.py) -- CPU only.

No rotary test exists in the reference.  Pins: closed forms (position 0 is the
identity, a 2-dim head is the 2x2 rotation matrix, the frequency formula), the
invariants of a rotation (pair norms, inverse = transpose, relative-position
property), an independent float64 loop evaluation, the committed fixtures, and
the GPT-NeoX rotary of the installed ``transformers`` library (same half-split
pairing, different tensor layout).  A swapped sign, an interleaved (2j, 2j+1)
pairing or a wrong exponent fails at least one of them.
"""
import math

import numpy as np
import pytest
import torch

from oracle import brute
from oracle import torch_ref as R


def test_table_shapes_dtype_and_frequency_formula():
    cos, sin = R.rotary_tables(8, 16, base=10000, precision=torch.float)
    assert cos.shape == sin.shape == (16, 1, 1, 8) and cos.dtype == torch.float32
    for t in (0, 1, 7, 15):
        for j in range(8):
            ang = t * 10000.0 ** (-2.0 * (j % 4) / 8)
            assert cos[t, 0, 0, j].item() == pytest.approx(math.cos(ang), abs=2e-6)
            assert sin[t, 0, 0, j].item() == pytest.approx(math.sin(ang), abs=2e-6)
    assert torch.equal(cos[..., :4], cos[..., 4:])  # both halves carry the same angles
    ch, _ = R.rotary_tables(8, 16, precision=torch.bfloat16)
    assert ch.dtype == torch.bfloat16 and torch.equal(ch, cos.bfloat16())


def test_position_zero_is_identity():
    cos, sin = R.rotary_tables(16, 4)
    q, k = torch.randn(4, 2, 3, 16), torch.randn(4, 2, 3, 16)
    oq, ok = R.apply_rotary_pos_emb(q, k, cos, sin)
    assert torch.equal(oq[0], q[0]) and torch.equal(ok[0], k[0])


def test_two_dim_head_is_plane_rotation():
    cos, sin = R.rotary_tables(2, 6)  # single frequency base^0 = 1: angle = position
    q = torch.tensor([1.0, 0.0]).expand(6, 1, 1, 2).contiguous()
    oq, _ = R.apply_rotary_pos_emb(q, q, cos, sin)
    for t in range(6):
        assert oq[t, 0, 0, 0].item() == pytest.approx(math.cos(t), abs=1e-6)
        assert oq[t, 0, 0, 1].item() == pytest.approx(math.sin(t), abs=1e-6)


def test_rotate_half_is_not_interleaved():
    x = torch.arange(6.0)
    assert torch.equal(R.rotate_half(x), torch.tensor([-3.0, -4.0, -5.0, 0.0, 1.0, 2.0]))


def test_pair_norms_and_relative_position_property():
    d = 8
    cos, sin = (t.double() for t in R.rotary_tables(d, 32))
    q = torch.randn(1, 1, 1, d, dtype=torch.float64).expand(32, 1, 1, d)
    k = torch.randn(1, 1, 1, d, dtype=torch.float64).expand(32, 1, 1, d)
    oq, ok = R.apply_rotary_pos_emb(q, k, cos, sin)
    n_in = q[..., : d // 2] ** 2 + q[..., d // 2 :] ** 2
    n_out = oq[..., : d // 2] ** 2 + oq[..., d // 2 :] ** 2
    assert torch.allclose(n_in, n_out, atol=1e-6)
    # <R_m q, R_n k> depends on m - n only
    dots = {(m, n): float((oq[m, 0, 0] * ok[n, 0, 0]).sum()) for m in range(32) for n in range(32)}
    for (m, n), v in dots.items():
        if m + 3 < 32 and n + 3 < 32:
            assert v == pytest.approx(dots[(m + 3, n + 3)], abs=1e-4)


def test_offset_slices_the_tables():
    cos, sin = R.rotary_tables(8, 20)
    q, k = torch.randn(5, 1, 2, 8), torch.randn(5, 1, 2, 8)
    a = R.apply_rotary_pos_emb(q, k, cos, sin, offset=7)
    b = R.apply_rotary_pos_emb(q, k, cos[7:12], sin[7:12], offset=0)
    assert torch.equal(a[0], b[0]) and torch.equal(a[1], b[1])


def test_matches_float64_loops_and_fixtures(golden):
    for name in ("rotary_d8", "rotary_d32", "rotary_d24"):
        f = golden[name]
        s, _, _, d = f["q"].shape
        off = int(f["offset"])
        cos, sin = R.rotary_tables(d, s + off, float(f["base"]))
        oq, ok = R.apply_rotary_pos_emb(torch.tensor(f["q"]), torch.tensor(f["k"]), cos, sin, off)
        assert np.allclose(oq.numpy(), f["oq"], atol=2e-5), name
        assert np.allclose(ok.numpy(), f["ok"], atol=2e-5), name
        dq, dk = R.rotary_autograd_fp32(
            torch.tensor(f["q"]), torch.tensor(f["k"]), cos, sin, torch.tensor(f["gq"]),
            torch.tensor(f["gk"]), off,
        )
        assert np.allclose(dq.numpy(), f["dq"], atol=2e-5), name
        assert np.allclose(dk.numpy(), f["dk"], atol=2e-5), name


def test_backward_is_inverse_rotation():
    x = np.random.default_rng(3).normal(size=12)
    assert np.allclose(brute.rotary_vec_backward(brute.rotary_vec(x, 9), 9), x, atol=1e-12)
    d = 12
    cos, sin = R.rotary_tables(d, 10)
    q, k = torch.randn(10, 2, 2, d), torch.randn(10, 2, 2, d)
    oq, ok = R.apply_rotary_pos_emb(q, k, cos, sin)
    bq, bk = R.rotary_autograd_fp32(q, k, cos, sin, oq, ok)  # grad = transpose applied to oq
    assert torch.allclose(bq, q, atol=1e-5) and torch.allclose(bk, k, atol=1e-5)


def test_against_transformers_gpt_neox_rotary():
    hf = pytest.importorskip("transformers.models.gpt_neox.modeling_gpt_neox")
    s, b, h, hn, rot = 9, 2, 3, 16, 8
    q, k = torch.randn(s, b, h, hn), torch.randn(s, b, h, hn)
    cos, sin = R.rotary_tables(rot, s)
    oq, ok = R.partial_rotary(q, k, cos, sin, rot)
    # transformers layout: q [b, h, s, hn]; cos/sin [b, s, rot]
    cq = cos[:, 0, 0, :].unsqueeze(0).expand(b, s, rot)
    sq_ = sin[:, 0, 0, :].unsqueeze(0).expand(b, s, rot)
    hq, hk = hf.apply_rotary_pos_emb(q.permute(1, 2, 0, 3), k.permute(1, 2, 0, 3), cq, sq_)
    assert torch.allclose(hq.permute(2, 0, 1, 3), oq, atol=1e-6)
    assert torch.allclose(hk.permute(2, 0, 1, 3), ok, atol=1e-6)


def test_partial_rotary_passes_remaining_dims_through():
    q, k = torch.randn(4, 1, 2, 16), torch.randn(4, 1, 2, 16)
    cos, sin = R.rotary_tables(4, 4)
    oq, ok = R.partial_rotary(q, k, cos, sin, 4)
    assert torch.equal(oq[..., 4:], q[..., 4:]) and torch.equal(ok[..., 4:], k[..., 4:])
    assert not torch.equal(oq[1:, ..., :4], q[1:, ..., :4])


def test_tables_from_freqs_are_fp32_cos_and_sin_of_the_angles():
    # pins rotary_tables_from_freqs: against float64 cos/sin of the same fp32 angles (1 ulp of
    # fp32 at magnitude 1, angles up to thousands of radians), and against rotary_tables, which
    # forms the same angles itself
    freqs = torch.outer(torch.arange(4096).float(), 1.0 / (10000 ** (torch.arange(0, 32, 2).float() / 32)))
    freqs = torch.cat((freqs, freqs), -1)[:, None, None, :]
    cos, sin = R.rotary_tables_from_freqs(freqs)
    assert cos.dtype == torch.float32 and cos.shape == freqs.shape
    assert (cos.double() - freqs.double().cos()).abs().max().item() <= 1.2e-7
    assert (sin.double() - freqs.double().sin()).abs().max().item() <= 1.2e-7
    c2, s2 = R.rotary_tables(32, 4096)
    assert torch.equal(cos, c2) and torch.equal(sin, s2)
