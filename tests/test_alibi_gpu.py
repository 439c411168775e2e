"""ALiBi folded into every softmax kernel family: with a mask tensor, together with a bias tensor,
with dropout, for a one-query decode step (through the C-ABI).

Oracle: the reference's sequence -- AliBi.forward adds -slope * tril(i - j) (its last row for
sq == 1), megatron/model/positional_embeddings.py:210-257; then the bias tensor, the mask and the
softmax, megatron/model/transformer.py:526-534 -- evaluated in fp32.  Bars: 2e-3 (bf16) / 1e-3
(fp16) on the probabilities and, against fp32 autograd from x, on the gradient; hidden positions
exactly 0; dropped outputs bit-equal to torch's dropout expression on the kernel's own probabilities.
"""
import pytest
import torch

from gpt_neox_amd.fused_kernels import attention_dropout as rng
from gpt_neox_amd.fused_kernels import scaled_masked_softmax_cuda as masked_ext
from gpt_neox_amd.fused_kernels import scaled_upper_triang_masked_softmax_cuda as causal_ext
from gpt_neox_amd.fused_softmax import (FusedScaleMaskSoftmax, ScaledMaskedSoftmaxAlibi, ScaledMaskedSoftmaxBias,
                                       ScaledUpperTriangMaskedSoftmaxBias, SoftmaxFusionTypes)
from gpt_neox_amd.positional_embeddings import AliBi
from bars import assert_grad
from oracle import torch_ref as R

pytestmark = pytest.mark.gpu

TOL = {torch.bfloat16: 2e-3, torch.float16: 1e-3}
DTYPES = [torch.float16, torch.bfloat16]


def gen(device, seed):
    return torch.Generator(device=device).manual_seed(seed)


def scores(shape, dtype, device, seed):
    return (torch.randn(shape, device=device, generator=gen(device, seed)) * 8).to(dtype)


def normal(shape, dtype, device, seed):
    return torch.randn(shape, device=device, generator=gen(device, seed)).to(dtype)


def max_err(a, b):
    return (a.float() - b.float()).abs().max().item()


def slopes_for(heads, device):
    return torch.tensor(R.alibi_slopes(heads), device=device)


def random_mask(b, sq, sk, device, seed, density=0.3):
    m = torch.rand(b, 1, sq, sk, device=device, generator=gen(device, seed)) < density
    m[..., -1] = False  # every row keeps a key: fully hidden rows have their own test
    return m


def oracle(x, mask, slopes, scale, bias=None):
    b, heads, sq, sk = x.shape
    t = x.float() + R.alibi_bias_fp32(slopes, sq, sk, x.device)
    if bias is not None:
        t = t + bias.float()
    return R.softmax_fp32(t, mask, scale)


# [b, np, sq, sk]: packed kernels (<= 512 columns; 513-2048 with a mask tensor), one to
# sixteen waves per row, ragged rows (sk % 8 != 0), the element-wise kernels (sk < 8), rows staged in LDS (sk > 32768),
# and one-query decode steps
MASKED_ALIBI_SHAPES = [(2, 3, 8, 8), (1, 4, 40, 40), (2, 2, 136, 136), (1, 6, 512, 512), (1, 2, 640, 640), (2, 2, 1000, 1000),
                       (1, 2, 1280, 1280), (1, 3, 2048, 2048), (1, 2, 2568, 2568), (1, 2, 4104, 4104), (1, 1, 9000, 9000),
                       (2, 3, 37, 37), (1, 2, 1001, 1001), (1, 2, 2047, 2047), (2, 2, 5, 5),
                       (2, 4, 1, 33), (1, 8, 1, 512), (3, 2, 1, 2049), (1, 2, 1, 8192), (1, 2, 1, 33000)]


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("shape", MASKED_ALIBI_SHAPES)
def test_alibi_with_a_mask_tensor(device, shape, dtype):
    b, heads, sq, sk = shape
    x = scores(shape, dtype, device, sk)
    slopes = slopes_for(heads, device)
    for mask in (random_mask(b, sq, sk, device, sk + 1), random_mask(1, sq, sk, device, sk + 2, 0.05)):
        got = masked_ext.forward_alibi(x, mask, slopes, 0.25)
        assert max_err(got, oracle(x, mask, slopes, 0.25)) <= TOL[dtype], shape
        assert (got[mask.expand_as(got)] == 0).all()
    if sq == sk:
        # under the causal mask: the causal kernel's function (bits may differ: other chunks summed)
        causal = R.get_attn_mask(sk, device)
        assert max_err(masked_ext.forward_alibi(x, causal, slopes, 0.25), causal_ext.forward_alibi(x, slopes, 0.25)) <= 2.0 ** -8
        # nothing hidden (bidirectional attention): keys after the query get no bias
        nothing = torch.zeros(1, 1, sq, sk, dtype=torch.bool, device=device)
        assert max_err(masked_ext.forward_alibi(x, nothing, slopes, 0.25), oracle(x, nothing, slopes, 0.25)) <= TOL[dtype]
    # zero slopes: the plain kernel's result
    zero = masked_ext.forward_alibi(x, mask, torch.zeros_like(slopes), 0.25)
    assert max_err(zero, masked_ext.forward(x, mask, 0.25)) <= 2.0 ** -8


BOTH_SHAPES = [(2, 3, 8, 8), (2, 2, 136, 136), (1, 4, 512, 512), (1, 2, 640, 640), (2, 2, 1024, 1024), (1, 2, 1280, 1280),
               (1, 2, 2048, 2048), (1, 2, 4096, 4096), (2, 2, 37, 37), (1, 2, 1001, 1001), (1, 1, 5, 5), (1, 1, 33000, 33000)]


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("shared", [True, False])
@pytest.mark.parametrize("shape", BOTH_SHAPES)
def test_alibi_and_a_bias_tensor_together(device, shape, shared, dtype):
    b, heads, s, _ = shape
    if s > 30000:
        if not shared or dtype is torch.float16:
            pytest.skip("one case of the very long row is enough")
        rows = torch.tensor([0, 1, 511, 512, s // 2, s - 1], device=device)
    x = scores(shape, dtype, device, 70)
    bias = scores((1 if shared else b, heads, s, s), dtype, device, 71) * 0.25
    slopes = slopes_for(heads, device)
    causal = R.get_attn_mask(s, device)
    mask = random_mask(b, s, s, device, 72)
    got_c = causal_ext.forward_bias(x, bias, 0.125, slopes)
    got_m = masked_ext.forward_bias(x, mask, bias, 0.125, slopes)
    if s > 30000:
        dist = (torch.arange(s, device=device).view(1, s) - rows.view(-1, 1)).clamp(max=0).float()  # -tril(i - j), these rows
        t = x[0, 0][rows].float() + slopes[0] * dist + bias[0, 0][rows].float()
        assert max_err(got_c[0, 0][rows], R.softmax_fp32(t, causal[0, 0][rows], 0.125)) <= TOL[dtype]
        assert max_err(got_m[0, 0][rows], R.softmax_fp32(t, mask[0, 0][rows], 0.125)) <= TOL[dtype]
        return
    assert max_err(got_c, oracle(x, causal, slopes, 0.125, bias)) <= TOL[dtype]
    assert (got_c[causal.expand_as(got_c)] == 0).all()
    assert max_err(got_m, oracle(x, mask, slopes, 0.125, bias)) <= TOL[dtype]
    assert (got_m[mask.expand_as(got_m)] == 0).all()
    # a zero bias tensor is the ALiBi kernel, a zero slope the bias kernel: bit for bit
    assert torch.equal(causal_ext.forward_bias(x, torch.zeros_like(bias), 0.125, slopes), causal_ext.forward_alibi(x, slopes, 0.125))
    assert torch.equal(masked_ext.forward_bias(x, mask, bias, 0.125, torch.zeros_like(slopes)), masked_ext.forward_bias(x, mask, bias, 0.125))


DROP_SHAPES = [(2, 3, 8, 8), (2, 2, 5, 5), (2, 2, 136, 136), (1, 4, 512, 512), (1, 2, 640, 640), (2, 2, 1024, 1024), (1, 2, 2048, 2048),
               (1, 2, 4096, 4096), (2, 2, 37, 37), (1, 2, 1001, 1001), (2, 3, 1, 520)]


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("shape", DROP_SHAPES)
def test_dropout_with_alibi_on_every_kernel_family(device, shape, dtype):
    b, heads, sq, sk = shape
    x = scores(shape, dtype, device, 40)
    g = normal(shape, dtype, device, 41)
    slopes = slopes_for(heads, device)
    bias = scores((1, heads, sq, sk), dtype, device, 42) * 0.25
    mask = random_mask(b, sq, sk, device, 43)
    p, seed, offset, scale = 0.2, 77, 16, 0.125
    keep = rng.keep_mask(x.numel(), p, seed, offset, device).view(shape)
    cases = [(dict(slopes=slopes), masked_ext.forward_alibi(x, mask, slopes, scale)),
             (dict(slopes=slopes, bias=bias), masked_ext.forward_bias(x, mask, bias, scale, slopes))]
    for kwargs, plain in cases:
        y, dropped = masked_ext.forward_dropout(x, mask, scale, p, seed, offset, **kwargs)
        assert torch.equal(y, plain)  # the probabilities kept for the backward pass: the undropped kernel's bits
        assert torch.equal(dropped, R.dropout_with_mask(y, keep, p))
        dx = masked_ext.backward_dropout(g.clone(), y, scale, p, seed, offset)
        ref = R.softmax_dropout_backward_fp32(g, y, keep, p, scale)
        assert max_err(dx, ref) <= TOL[dtype] * max(1.0, ref.abs().max().item())
    y, dropped = masked_ext.forward_dropout(x, mask, scale, p, seed, offset, bias=bias)
    assert torch.equal(y, masked_ext.forward_bias(x, mask, bias, scale))
    assert torch.equal(dropped, R.dropout_with_mask(y, keep, p))
    if sq == sk:
        for kwargs, plain in ((dict(slopes=slopes, bias=bias), causal_ext.forward_bias(x, bias, scale, slopes)),
                              (dict(slopes=slopes), causal_ext.forward_alibi(x, slopes, scale)),
                              (dict(bias=bias), causal_ext.forward_bias(x, bias, scale))):
            y, dropped = causal_ext.forward_dropout(x, scale, p, seed, offset, **kwargs)
            assert torch.equal(y, plain)
            assert torch.equal(dropped, R.dropout_with_mask(y, keep, p))


def test_autograd_functions_with_slopes(device):
    b, heads, s, dtype = 2, 4, 200, torch.bfloat16
    x = scores((b, heads, s, s), dtype, device, 3)
    g = normal((b, heads, s, s), dtype, device, 4)
    slopes = slopes_for(heads, device)
    mask = random_mask(b, s, s, device, 5)
    rpe = (scores((1, heads, s, s), dtype, device, 6) * 0.25).requires_grad_(True)
    abias = R.alibi_bias_fp32(slopes, s, s, device)

    def reference(with_bias, m):
        xr = x.float().requires_grad_(True)
        br = rpe.detach().float().requires_grad_(True)
        t = xr + abias + (br if with_bias else 0.0)
        yr = torch.softmax(R.gpt2_attention_mask_func(t * 0.5, m), -1)
        yr.backward(g.float())
        return yr.detach(), xr.grad, br.grad

    # mask tensor + slopes
    xin = x.clone().requires_grad_(True)
    y = ScaledMaskedSoftmaxAlibi.apply(xin, mask, slopes, 0.5)
    y.backward(g.clone())
    yr, dxr, _ = reference(False, mask)
    assert max_err(y, yr) <= TOL[dtype]
    assert_grad(xin.grad, dxr, dtype, y=y.detach(), g=g, scale=0.5)
    # mask tensor + bias + slopes, causal + bias + slopes: gradients for the scores and the bias
    for fn, m in ((lambda t: ScaledMaskedSoftmaxBias.apply(t, mask, rpe, 0.5, slopes), mask),
                  (lambda t: ScaledUpperTriangMaskedSoftmaxBias.apply(t, rpe, 0.5, slopes), R.get_attn_mask(s, device))):
        xin = x.clone().requires_grad_(True)
        rpe.grad = None
        y = fn(xin)
        y.backward(g.clone())
        yr, dxr, dbr = reference(True, m)
        assert max_err(y, yr) <= TOL[dtype]
        assert_grad(xin.grad, dxr, dtype, y=y.detach(), g=g, scale=0.5)
        # the bias gradient sums the two samples in the storage type: two roundings
        assert max_err(rpe.grad, dbr) <= 2 * TOL[dtype] + 2.0 ** -8 * dbr.abs().max().item()


def test_module_folds_alibi_whatever_the_mask(device):
    heads, s, dtype = 4, 256, torch.bfloat16
    alibi = AliBi(heads, mp_size=1, mp_rank=0).to(device)
    x = scores((2, heads, s, s), dtype, device, 11)
    rpe = scores((1, heads, s, s), dtype, device, 12) * 0.25
    pad = R.padding_mask(torch.tensor([100, 256]), s, s, device)
    window = R.get_attn_mask(s, device, sliding_window_width=31)
    causal = R.get_attn_mask(s, device)
    general = FusedScaleMaskSoftmax(False, True, SoftmaxFusionTypes.general, R.gpt2_attention_mask_func, True, 0.5)
    upper = FusedScaleMaskSoftmax(False, True, SoftmaxFusionTypes.upper_triang, R.gpt2_attention_mask_func, True, 0.5,
                                  causal_mask_check="verify")
    unfused = FusedScaleMaskSoftmax(False, True, SoftmaxFusionTypes.none, R.gpt2_attention_mask_func, True, 0.5)
    for mod, mask in ((general, pad), (general, causal), (upper, window), (upper, causal)):
        for bias in (None, rpe):
            got = mod(x, mask, alibi_slopes=alibi.slopes, bias=bias)
            assert max_err(got, oracle(x, mask, alibi.slopes, 0.5, bias)) <= TOL[dtype]
            assert (got[mask.expand_as(got) & ~mask.expand_as(got).all(-1, keepdim=True)] == 0).all()
            # the reference's sequence of passes (sums rounded to bf16 on the way) stays within bf16 noise of it
            two_pass = unfused(alibi(x if bias is None else x + bias), mask)
            assert max_err(got, two_pass) <= 0.08
    # dropout on top: one kernel, the same probabilities dropped as torch drops them
    torch.manual_seed(5)
    off = torch.cuda.default_generators[device.index].get_offset()
    out = general(x, pad, alibi_slopes=alibi.slopes, bias=rpe, dropout_p=0.1)
    keep = rng.keep_mask(x.numel(), 0.1, 5, off, device).view(x.shape)
    assert torch.equal(out, R.dropout_with_mask(general(x, pad, alibi_slopes=alibi.slopes, bias=rpe), keep, 0.1))
    # one new token against 300 cached keys: the query stands at the last key position
    xd = scores((2, heads, 1, 300), dtype, device, 13)
    seen = torch.zeros(2, 1, 1, 300, dtype=torch.bool, device=device)
    seen[1, ..., :40] = True  # left padding of the second sample
    for mod in (general, upper):
        got = mod(xd, seen, alibi_slopes=alibi.slopes)
        assert max_err(got, oracle(xd, seen, alibi.slopes, 0.5)) <= TOL[dtype]
        assert max_err(got, unfused(alibi(xd), seen)) <= 0.08
    with pytest.raises(AssertionError, match="sq == 1"):
        general(scores((1, heads, 5, 300), dtype, device, 14), torch.zeros(1, 1, 5, 300, dtype=torch.bool, device=device),
                alibi_slopes=alibi.slopes)
