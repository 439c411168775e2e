"""Kernel instantiations that only unusual calls reach, each against the oracle (through the C-ABI).

* rows that the packed kernels take (at most 512 columns; 513-2048 with a mask tensor)
  whose mask or bias tensor is larger than a 32-bit buffer range (4 GiB): the row kernels with a
  64-bit address per row instead;
* packed kernels on tensors beyond 4 GiB;
* the XCD-aware rotary kernel with 2-, 4- and 8-element slots, fp32 and 16-bit tables, forward and
  backward (it takes dense tensors that start on a 4 KiB boundary);
* the element-wise rotary kernel with kernel-evaluated angles and 4-element slots, and with
  1-element slots, 16-bit tables, backward.

Bars as in the other parity tests: softmax within 2e-3 (bf16) / 1e-3 (fp16) of the fp32 expression
with hidden positions exactly 0, dropout output bit-equal to torch's expression on the kernel's own
probabilities and the oracle's keep pattern, rotary bit-equal to the fp32 expression rounded once
(kernel-evaluated angles: within one unit in the last place).
"""
import pytest
import torch

from gpt_neox_amd.fused_kernels import attention_dropout as rng
from gpt_neox_amd.fused_kernels import fused_rotary_positional_embedding as rope_ext
from gpt_neox_amd.fused_kernels import scaled_masked_softmax_cuda as masked_ext
from gpt_neox_amd.fused_kernels import scaled_upper_triang_masked_softmax_cuda as causal_ext
from gpt_neox_amd.positional_embeddings import apply_rotary_pos_emb, apply_rotary_pos_emb_
from oracle import torch_ref as R

pytestmark = pytest.mark.gpu

TOL = {torch.bfloat16: 2e-3, torch.float16: 1e-3}
DTYPES = [torch.float16, torch.bfloat16]
FOUR_GIB = 1 << 32


def gen(device, seed):
    return torch.Generator(device=device).manual_seed(seed)


def big_normal(shape, dtype, device, seed, times=1.0):
    """Normal values in `dtype`, drawn directly in that type (no fp32 copy of a multi-GiB tensor)."""
    t = torch.empty(shape, dtype=dtype, device=device)
    t.normal_(0.0, times, generator=gen(device, seed))
    return t


def max_err(a, b):
    return (a.float() - b.float()).abs().max().item()


def sample_rows(n, device, seed):
    """Row numbers at both ends of [0, n), around the middle and at random."""
    fixed = torch.tensor([0, 1, 2, 3, n // 2 - 1, n // 2, n - 4, n - 3, n - 2, n - 1], device=device)
    rand = torch.randint(0, n, (54,), device=device, generator=gen(device, seed))
    return torch.cat((fixed, rand)).unique()


# ---------------------------------------------------------------------------------
# softmax: short rows with tensors beyond 4 GiB
# ---------------------------------------------------------------------------------
@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("sk", [512, 511, 640, 1536, 2048])  # aligned / ragged short rows; the packed kernels' longer rows
def test_rows_with_a_mask_tensor_beyond_4_gib(device, sk, dtype):
    sq = FOUR_GIB // sk + 16
    assert sq * sk > FOUR_GIB
    scale, p, seed, offset = 0.5, 0.25, 99, 8
    x = big_normal((1, 1, sq, sk), dtype, device, 1, times=8.0)
    mask = torch.empty((1, 1, sq, sk), dtype=torch.uint8, device=device)
    mask.random_(0, 10, generator=gen(device, 2))
    mask = mask < 3
    bias = big_normal((1, 1, sq, sk), dtype, device, 3)
    rows = sample_rows(sq, device, 4)
    xs, ms, bs = x[0, 0][rows].float(), mask[0, 0][rows], bias[0, 0][rows].float()
    # ALiBi for sq != sk as the C-ABI defines it: slope * min(j - i', 0), i' = i + sk - sq (only the last sk rows get any)
    slopes = torch.tensor([0.37], device=device)
    ab = (torch.arange(sk, device=device).view(1, sk) - (rows.view(-1, 1) + sk - sq)).clamp(max=0).float() * slopes[0]
    want = {False: R.softmax_fp32(xs, ms, scale), True: R.softmax_fp32(xs + bs, ms, scale),
            "alibi": R.softmax_fp32(xs + ab, ms, scale), "alibi+bias": R.softmax_fp32(xs + ab + bs, ms, scale)}
    keep = rng.keep_mask(x.numel(), p, seed, offset, device).view(x.shape)[0, 0][rows]

    def check(y, with_bias, dropped=None):
        got = y[0, 0][rows]
        assert max_err(got, want[with_bias]) <= TOL[dtype]
        assert (got[ms & ~ms.all(-1, keepdim=True)] == 0).all()
        if dropped is not None:
            assert torch.equal(dropped[0, 0][rows], R.dropout_with_mask(got, keep, p))

    check(masked_ext.forward(x, mask, scale), False)
    check(masked_ext.forward_bias(x, mask, bias, scale), True)
    y, dropped = masked_ext.forward_dropout(x, mask, scale, p, seed, offset)
    check(y, False, dropped)
    check(masked_ext.forward_alibi(x, mask, slopes, scale), "alibi")
    check(masked_ext.forward_bias(x, mask, bias, scale, slopes), "alibi+bias")
    y, dropped = masked_ext.forward_dropout(x, mask, scale, p, seed, offset, slopes=slopes)
    check(y, "alibi", dropped)
    y, dropped = masked_ext.forward_dropout(x, mask, scale, p, seed, offset, bias=bias, slopes=slopes)
    check(y, "alibi+bias", dropped)
    y, dropped = masked_ext.forward_dropout(x, mask, scale, p, seed, offset, bias=bias)
    check(y, True, dropped)
    # the backward pass reads neither mask nor bias: packed kernels on tensors beyond 4 GiB
    g = bias
    dx = masked_ext.backward(g.clone(), y, scale)
    assert max_err(dx[0, 0][rows], R.softmax_backward_fp32(g[0, 0][rows], y[0, 0][rows], scale)) <= TOL[dtype] * 4
    dx = masked_ext.backward_dropout(g.clone(), y, scale, p, seed, offset)
    ref = R.softmax_dropout_backward_fp32(g[0, 0][rows], y[0, 0][rows], keep, p, scale)
    assert max_err(dx[0, 0][rows], ref) <= TOL[dtype] * 4


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("s", [512, 511])
def test_short_causal_rows_with_a_bias_tensor_beyond_4_gib(device, s, dtype):
    heads = FOUR_GIB // (2 * s * s) + 8
    assert heads * s * s * 2 > FOUR_GIB
    scale, p, seed, offset = 0.25, 0.5, 5, 12
    x = big_normal((1, heads, s, s), dtype, device, 11, times=8.0)
    bias = big_normal((1, heads, s, s), dtype, device, 12)
    pick = sample_rows(heads, device, 13)[::4]  # whole heads
    mask = R.get_attn_mask(s, device)[0]  # [1, s, s]
    want_plain = R.softmax_fp32(x[0, pick].float(), mask, scale)
    want_bias = R.softmax_fp32(x[0, pick].float() + bias[0, pick].float(), mask, scale)
    hidden = mask.expand(pick.numel(), s, s)
    keep = rng.keep_mask(x.numel(), p, seed, offset, device).view(x.shape)[0, pick]

    def check(y, want, dropped=None):
        got = y.view(x.shape)[0, pick]
        assert max_err(got, want) <= TOL[dtype]
        assert (got[hidden] == 0).all()
        if dropped is not None:
            assert torch.equal(dropped.view(x.shape)[0, pick], R.dropout_with_mask(got, keep, p))

    check(causal_ext.forward(x.view(-1, s, s), scale), want_plain)  # packed kernel beyond 4 GiB
    check(causal_ext.forward_bias(x, bias, scale), want_bias)
    slopes = torch.rand(heads, device=device, generator=gen(device, 14)) * 0.5
    ab = R.alibi_bias_fp32(slopes[pick], s, s, device)
    want_both = R.softmax_fp32(x[0, pick].float() + bias[0, pick].float() + ab, mask, scale)
    check(causal_ext.forward_bias(x, bias, scale, slopes), want_both)
    y, dropped = causal_ext.forward_dropout(x, scale, p, seed, offset, bias=bias, slopes=slopes)
    check(y, want_both, dropped)
    y, dropped = causal_ext.forward_dropout(x, scale, p, seed, offset, bias=bias)
    check(y, want_bias, dropped)
    g = bias
    dx = causal_ext.backward(g.clone().view(-1, s, s), y.view(-1, s, s), scale).view(x.shape)
    assert max_err(dx[0, pick], R.softmax_backward_fp32(g[0, pick], y[0, pick], scale)) <= TOL[dtype] * 4
    assert (dx[0, pick][hidden] == 0).all()


# ---------------------------------------------------------------------------------
# rotary
# ---------------------------------------------------------------------------------
def on_a_4k_boundary(t):
    """A copy of `t` whose storage starts on a 4 KiB boundary."""
    flat = torch.empty(t.numel() + 2048, dtype=t.dtype, device=t.device)
    skip = (-flat.data_ptr() % 4096) // t.element_size()
    out = flat[skip : skip + t.numel()].view(t.shape)
    out.copy_(t)
    assert out.data_ptr() % 4096 == 0
    return out


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("half_tables", [False, True])
@pytest.mark.parametrize("shape,d_rot", [
    ((64, 2, 16, 128), 32),  # 8-element slots
    ((64, 2, 16, 64), 8),    # 4-element slots
    ((96, 1, 32, 64), 4),    # 2-element slots
    ((40, 2, 32, 16), 8),    # 4-element slots, pass-through dims copied by the same lanes
])
def test_xcd_aware_rotary_kernel_slot_widths_and_table_types(device, shape, d_rot, half_tables, dtype):
    s, b, h, hn = shape
    q = on_a_4k_boundary(big_normal(shape, dtype, device, 21))
    k = on_a_4k_boundary(big_normal(shape, dtype, device, 22))
    cos, sin = (t.to(device) for t in R.rotary_tables(d_rot, s + 2, 10000, dtype if half_tables else torch.float))
    want_q, want_k = R.partial_rotary(q.float(), k.float(), cos.float(), sin.float(), d_rot, offset=2)
    cosf, sinf = cos.float(), sin.float()
    gq, gk = R.rotary_autograd_fp32(q[..., :d_rot], k[..., :d_rot], cosf, sinf, q[..., :d_rot], k[..., :d_rot], offset=2)

    def rotated(got, want, untouched):
        return torch.equal(got[..., :d_rot], want.to(dtype)) and torch.equal(got[..., d_rot:], untouched[..., d_rot:])

    # in place on q and k (one launch), forward and backward
    q1, k1 = on_a_4k_boundary(q), on_a_4k_boundary(k)
    apply_rotary_pos_emb_(q1, k1, cos, sin, 2, d_rot)
    assert torch.equal(q1, want_q.to(dtype)) and torch.equal(k1, want_k.to(dtype))
    q1, k1 = on_a_4k_boundary(q), on_a_4k_boundary(k)
    rope_ext.rope_launch(q1, k1, q1, k1, cos, sin, d_rot, 2, True)
    assert rotated(q1, gq, q) and rotated(k1, gk, k)
    # out of place into outputs on a 4 KiB boundary, the other dims copied by the same launch
    for backward, wq, wk in ((False, want_q[..., :d_rot], want_k[..., :d_rot]), (True, gq, gk)):
        oq, ok = on_a_4k_boundary(torch.zeros_like(q)), on_a_4k_boundary(torch.zeros_like(k))
        rope_ext.rope_launch(oq, ok, q, k, cos, sin, d_rot, 2, backward, d=hn)
        assert rotated(oq, wq, q) and rotated(ok, wk, k)
    # and through the extension's functions, wherever their output lands
    c, sn = cos[2 : 2 + s].contiguous(), sin[2 : 2 + s].contiguous()
    assert torch.equal(rope_ext.forward_cached(q, c, sn, False), want_q.to(dtype))
    assert rotated(rope_ext.backward_cached(k, c, sn, False), gk, k)


ULP = {torch.bfloat16: 2.0**-7, torch.float16: 2.0**-10}


def assert_within_one_ulp(got, want, dtype):
    diff = (got.float() - want.float()).abs()
    assert (diff <= ULP[dtype] * want.float().abs() + 1e-6).all(), diff.max().item()
    assert (got != want).float().mean().item() <= 1e-3


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("transpose", [False, True])
def test_element_wise_rotary_kernel_with_angles_and_4_element_slots(device, dtype, transpose):
    # 24 rotated dims (12 per half: 4-element slots) of 512: too many pass-through slots for the
    # span kernel, so the element-wise kernel evaluates the angles and copies the other dims
    s, b, h, d, d2 = 9, 2, 3, 512, 24
    t = big_normal((s, b, h, d), dtype, device, 31)
    rates = torch.rand(d2, device=device, generator=gen(device, 32))
    freqs = (torch.arange(s, device=device).float()[:, None] * rates).view(s, 1, 1, d2)
    cos, sin = R.rotary_tables_from_freqs(freqs)
    rot, _ = R.rotary_fp32(t[..., :d2], t[..., :d2], cos, sin)
    got = rope_ext.forward(t, freqs, transpose)
    assert got.shape == t.shape
    assert got.transpose(0, 1).is_contiguous() == transpose
    assert_within_one_ulp(got[..., :d2], rot.to(dtype), dtype)
    assert torch.equal(got[..., d2:], t[..., d2:])
    gq, _ = R.rotary_autograd_fp32(t[..., :d2], t[..., :d2], cos, sin, t[..., :d2], t[..., :d2])
    back = rope_ext.backward(t, freqs, transpose)
    assert_within_one_ulp(back[..., :d2], gq.to(dtype), dtype)
    assert torch.equal(back[..., d2:], t[..., d2:])


@pytest.mark.parametrize("dtype", DTYPES)
def test_element_wise_rotary_kernel_with_1_element_slots_and_16_bit_tables(device, dtype):
    s, b, h, hn, d_rot = 7, 2, 3, 16, 6  # 3 dims per half
    q, k = big_normal((s, b, h, hn), dtype, device, 41), big_normal((s, b, h, hn), dtype, device, 42)
    cos, sin = (t.to(device) for t in R.rotary_tables(d_rot, s, 10000, dtype))
    qr = q[..., :d_rot].detach().requires_grad_(True)
    kr = k[..., :d_rot].detach().requires_grad_(True)
    oq, ok = apply_rotary_pos_emb(qr, kr, cos, sin, 0)
    rq, rk = R.rotary_fp32(q[..., :d_rot], k[..., :d_rot], cos, sin)
    assert torch.equal(oq, rq.to(dtype)) and torch.equal(ok, rk.to(dtype))
    torch.autograd.backward([oq, ok], [k[..., :d_rot], q[..., :d_rot]])
    dq, dk = R.rotary_autograd_fp32(q[..., :d_rot], k[..., :d_rot], cos.float(), sin.float(), k[..., :d_rot], q[..., :d_rot])
    assert torch.equal(qr.grad, dq.to(dtype)) and torch.equal(kr.grad, dk.to(dtype))
