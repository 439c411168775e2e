"""Rows beyond the register budget (more than 32768 columns, staged in a CU's LDS) with everything a
call can bring along: ALiBi slopes, a bias tensor, dropout, rows at any alignment (sk % 8 != 0 or
tensors that start off a 16-byte boundary), under a mask tensor and under the causal mask, forward
and backward, through the C-ABI.  Two staging sizes exist (half of a CU's LDS up to 40448 positions,
all of it up to 81408) and both are taken here, at and next to their limits.

Bars as in the other parity tests: within 2e-3 (bf16) / 1e-3 (fp16) of the fp32 expression of the
oracle on the same inputs, hidden positions exactly 0, the dropout output bit-equal to torch's
expression on the kernel's own probabilities and the oracle's keep pattern, the backward pass within
the same bars of the fp32 closed form on the kernel's probabilities (gradients of unit variance).
"""
import pytest
import torch

from gpt_neox_amd.fused_kernels import attention_dropout as rng
from gpt_neox_amd.fused_kernels import scaled_masked_softmax_cuda as masked_ext
from gpt_neox_amd.fused_kernels import scaled_upper_triang_masked_softmax_cuda as causal_ext
from oracle import torch_ref as R

from bars import assert_grad

pytestmark = pytest.mark.gpu

TOL = {torch.bfloat16: 2e-3, torch.float16: 1e-3}
DTYPES = [torch.float16, torch.bfloat16]


def gen(device, seed):
    return torch.Generator(device=device).manual_seed(seed)


def max_err(a, b):
    return (a.float() - b.float()).abs().max().item()


def normal_at(shape, dtype, device, seed, skip, times=1.0):
    """Normal values in a tensor that starts `skip` elements behind a 16-byte boundary."""
    n = 1
    for d in shape:
        n *= d
    flat = torch.empty(n + 8, dtype=dtype, device=device)
    first = (-flat.data_ptr() % 16) // 2 + skip
    out = flat[first : first + n].view(shape)
    out.normal_(0.0, times, generator=gen(device, seed))
    assert out.data_ptr() % 16 == 2 * skip
    return out


def copy_at(t, skip):
    """A copy of `t` that starts `skip` elements behind a 16-byte boundary."""
    out = normal_at(t.shape, t.dtype, t.device, 0, skip)
    out.copy_(t)
    return out


def alibi_any_shape(slopes, sq, sk, device):
    """slope * min(j - i', 0), i' = i + sk - sq: fp32 [np, sq, sk]"""
    i = torch.arange(sq, device=device).view(sq, 1) + (sk - sq)
    j = torch.arange(sk, device=device).view(1, sk)
    return (j - i).clamp(max=0).float() * slopes.float().view(-1, 1, 1)


# (sk, elements behind a 16-byte boundary).  Positions = sk, plus one for rows that lie one later.
STAGED = [
    (33280, 0),   # aligned, half of the LDS
    (50008, 0),   # aligned, all of it
    (40448, 0),   # the longest row of the half
    (40456, 0),   # the shortest row that needs all
    (33001, 0),   # odd length: rows alternate between the two alignments
    (40447, 1),   # odd length from an odd element on; 40448 positions
    (40448, 3),   # aligned length off the boundary: the ragged kernels, 40449 positions
    (65537, 2),
    (81407, 1),   # the longest ragged row
    (81408, 0),   # the longest row
]


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("sk,skip", STAGED)
def test_staged_rows_under_a_mask_tensor_with_every_feature(device, sk, skip, dtype):
    b, heads, sq = 2, 2, 3
    scale, p, seed, offset = 0.25, 0.25, 1234, 16
    shape = (b, heads, sq, sk)
    x = normal_at(shape, dtype, device, sk, skip, times=4.0)
    g = normal_at(shape, dtype, device, sk + 1, skip)
    bias = normal_at(shape, dtype, device, sk + 2, skip)
    shared = normal_at((1, heads, sq, sk), dtype, device, sk + 3, skip)
    mask = torch.rand(b, 1, sq, sk, device=device, generator=gen(device, sk + 4)) < 0.3
    mask[0, 0, 1, :] = True            # every key hidden: uniform over the row
    mask[1, 0, 2, 100:] = True         # a row that ends early
    mask[1, 0, 0, :] = False           # nothing hidden
    mask[1, 0, 1, : sk - 3] = True     # only the last three keys visible
    mask[1, 0, 1, sk - 3 :] = False
    slopes = torch.tensor([0.5, 0.03125], device=device)
    ab = alibi_any_shape(slopes, sq, sk, device)
    keep = rng.keep_mask(x.numel(), p, seed, offset, device).view(shape)
    hidden = mask.expand(shape).clone()
    hidden[0, :, 1, :] = False
    xf = x.float()

    def check(y, want, dropped=None):
        assert max_err(y, want) <= TOL[dtype]
        assert (y[hidden] == 0).all()
        if dropped is not None:
            assert torch.equal(dropped, R.dropout_with_mask(y, keep, p))

    plain = masked_ext.forward(x, mask, scale)
    check(plain, R.softmax_fp32(xf, mask, scale))
    assert torch.allclose(plain[0, :, 1, :].float(), torch.full((heads, sk), 1.0 / sk, device=device), rtol=1e-2)
    check(masked_ext.forward_alibi(x, mask, slopes, scale), R.softmax_fp32(xf + ab, mask, scale))
    check(masked_ext.forward_bias(x, mask, bias, scale), R.softmax_fp32(xf + bias.float(), mask, scale))
    check(masked_ext.forward_bias(x, mask, shared, scale, slopes), R.softmax_fp32(xf + shared.float() + ab, mask, scale))
    y, dropped = masked_ext.forward_dropout(x, mask, scale, p, seed, offset)
    check(y, R.softmax_fp32(xf, mask, scale), dropped)
    assert torch.equal(y, plain)
    y, dropped = masked_ext.forward_dropout(x, mask, scale, p, seed, offset, bias=bias, slopes=slopes)
    check(y, R.softmax_fp32(xf + bias.float() + ab, mask, scale), dropped)
    y, dropped = masked_ext.forward_dropout(x, mask, scale, p, seed, offset, slopes=slopes)
    check(y, R.softmax_fp32(xf + ab, mask, scale), dropped)
    y, dropped = masked_ext.forward_dropout(x, mask, scale, p, seed, offset, bias=shared)
    check(y, R.softmax_fp32(xf + shared.float(), mask, scale), dropped)

    # in place on copies of the gradient that start where it starts
    dx = masked_ext.backward(copy_at(g, skip), y, scale)
    assert_grad(dx, R.softmax_backward_fp32(g, y, scale), dtype, "plain")
    assert (dx[hidden] == 0).all()
    buf = copy_at(g, skip)
    dxd = masked_ext.backward_dropout(buf, y, scale, p, seed, offset)
    assert dxd.data_ptr() == buf.data_ptr()
    assert_grad(dxd, R.softmax_dropout_backward_fp32(g, y, keep, p, scale), dtype, "dropout")
    assert (dxd[hidden] == 0).all()


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("s,skip", [(33000, 0), (40968, 0), (33001, 0), (40449, 1)])
def test_staged_causal_rows_with_every_feature(device, s, skip, dtype):
    heads = 2
    scale, p, seed, offset = 0.05, 0.5, 77, 24
    shape = (1, heads, s, s)
    x = normal_at(shape, dtype, device, s, skip, times=4.0)
    bias = normal_at((1, heads, s, s), dtype, device, s + 1, skip)
    g = bias  # any values do
    slopes = torch.tensor([0.25, 0.0078125], device=device)
    # rows at both ends, at the chunk and staging limits, around the middle and at random
    rows = torch.tensor([0, 1, 2, 7, 8, 511, 512, 513, 32767, 32768, 32769, s // 2, s - 2, s - 1], device=device)
    rows = torch.cat((rows, torch.randint(0, s, (18,), device=device, generator=gen(device, s + 2)))).unique()
    mask = (torch.arange(s, device=device).view(1, s) > rows.view(-1, 1))  # [rows, s]
    ab = (torch.arange(s, device=device).view(1, 1, s) - rows.view(1, -1, 1)).clamp(max=0).float() * slopes.view(-1, 1, 1)
    xs, bs = x[0][:, rows].float(), bias[0][:, rows].float()  # [heads, rows, s]
    keep = rng.keep_mask(x.numel(), p, seed, offset, device).view(shape)[0][:, rows]
    hidden = mask.expand(heads, -1, -1)

    def check(y, want, dropped=None):
        got = y.view(shape)[0][:, rows]
        assert max_err(got, want) <= TOL[dtype]
        assert (got[hidden] == 0).all()
        if dropped is not None:
            assert torch.equal(dropped.view(shape)[0][:, rows], R.dropout_with_mask(got, keep, p))

    plain = causal_ext.forward(x.view(-1, s, s), scale)
    check(plain, R.softmax_fp32(xs, mask, scale))
    check(causal_ext.forward_alibi(x, slopes, scale), R.softmax_fp32(xs + ab, mask, scale))
    check(causal_ext.forward_bias(x, bias, scale), R.softmax_fp32(xs + bs, mask, scale))
    check(causal_ext.forward_bias(x, bias, scale, slopes), R.softmax_fp32(xs + bs + ab, mask, scale))
    y, dropped = causal_ext.forward_dropout(x, scale, p, seed, offset)
    check(y, R.softmax_fp32(xs, mask, scale), dropped)
    assert torch.equal(y.view(-1, s, s), plain)
    y, dropped = causal_ext.forward_dropout(x, scale, p, seed, offset, slopes=slopes)
    check(y, R.softmax_fp32(xs + ab, mask, scale), dropped)
    y, dropped = causal_ext.forward_dropout(x, scale, p, seed, offset, bias=bias)
    check(y, R.softmax_fp32(xs + bs, mask, scale), dropped)
    y, dropped = causal_ext.forward_dropout(x, scale, p, seed, offset, slopes=slopes, bias=bias)
    check(y, R.softmax_fp32(xs + bs + ab, mask, scale), dropped)

    y3, g3 = y.view(-1, s, s), g.view(-1, s, s)
    dx = causal_ext.backward(copy_at(g3, skip), y3, scale).view(shape)[0][:, rows]
    gs, ys = g[0][:, rows], y.view(shape)[0][:, rows]
    assert_grad(dx, R.softmax_backward_fp32(gs, ys, scale), dtype, "plain")
    assert (dx[hidden] == 0).all()
    dxd = causal_ext.backward_dropout(copy_at(g3, skip), y3, scale, p, seed, offset).view(shape)[0][:, rows]
    assert_grad(dxd, R.softmax_dropout_backward_fp32(gs, ys, keep, p, scale), dtype, "dropout")
    assert (dxd[hidden] == 0).all()
