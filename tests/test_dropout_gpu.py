"""Parity of the fused softmax + attention-dropout kernels (through the C-ABI) with the oracle.

Bars: the keep pattern is bit-equal to oracle/philox.py; the undropped probabilities are
bit-equal to the plain softmax kernels'; the dropped output is bit-equal to torch's
dropout expression evaluated on those probabilities with that pattern; the backward pass
meets the softmax bars (2e-3 bf16 / 1e-3 fp16, masked positions exactly 0) against the
fp32 closed form.
"""
import numpy as np
import pytest
import torch

from gpt_neox_amd.fused_kernels import attention_dropout as rng
from gpt_neox_amd.fused_kernels import scaled_masked_softmax_cuda as masked_ext
from gpt_neox_amd.fused_kernels import scaled_upper_triang_masked_softmax_cuda as causal_ext
from gpt_neox_amd.fused_softmax import (
    FusedScaleMaskSoftmax,
    ScaledMaskedSoftmaxDropout,
    ScaledUpperTriangMaskedSoftmaxDropout,
    SoftmaxFusionTypes,
)
from oracle import philox
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


# ---------------------------------------------------------------------------------
# the generator
# ---------------------------------------------------------------------------------
@pytest.mark.parametrize("n", [1, 7, 8, 9, 4099, 1 << 20])
@pytest.mark.parametrize("p,seed,offset", [(0.1, 1234, 0), (0.5, 2**63 + 5, 2**40 + 8), (0.9, 0, 4)])
def test_keep_mask_kernel_is_bit_equal_to_the_oracle(device, n, p, seed, offset):
    got = rng.keep_mask(n, p, seed, offset, device).cpu().numpy()
    assert np.array_equal(got, philox.keep_mask(n, p, seed, offset))


def test_keep_mask_edge_probabilities(device):
    assert rng.keep_mask(5000, 0.0, 3, 0, device).all()
    assert not rng.keep_mask(5000, 1.0, 3, 0, device).any()
    with pytest.raises(RuntimeError, match="between 0 and 1"):
        rng.keep_mask(8, 1.25, 3, 0, device)


def test_oracle_philox_agrees_with_the_device_library_generator(device):
    # torch.rand on the device draws Philox4x32-10 blocks with key = seed and
    # counter = (offset, thread index); in a launch with one element per thread, thread t
    # converts the first word of its block to a float in (0, 1].
    torch.manual_seed(987654321)
    u = torch.rand(256, device=device, dtype=torch.float32).cpu().numpy().astype(np.float64)
    ctr = np.zeros((256, 4), dtype=np.uint64)
    ctr[:, 2] = np.arange(256, dtype=np.uint64)
    words = philox.philox4x32_10(ctr, (987654321, 0)).astype(np.float64)  # [256, 4]
    want = words[:, 0] / 2.0**32  # element t <- first word of thread t's first block
    assert np.abs(u - want).max() < 2.0**-23
    # a generator offset counts 32-bit outputs, four to a counter value: at offset 400 the same
    # launch draws at counter 100 -- the kernels' keep pattern uses offset / 4 likewise, so a call
    # that owns the offsets [o, o + 4) shares no block with any other consumer
    torch.cuda.default_generators[device.index].set_offset(400)
    u = torch.rand(256, device=device, dtype=torch.float32).cpu().numpy().astype(np.float64)
    ctr[:, 0] = 100
    words = philox.philox4x32_10(ctr, (987654321, 0)).astype(np.float64)
    assert np.abs(u - words[:, 0] / 2.0**32).max() < 2.0**-23
    got = rng.keep_mask(2048, 0.5, 987654321, 400, device).cpu().numpy()
    fields = philox.philox4x32_10(ctr, (987654321, 0))[:, 0] & 0xFFFF  # element 8 t <- low half of word 0
    assert np.array_equal(got[0::8], fields >= 32768)


def test_dropout_scale_is_the_device_library_s(device):
    # kept entries of torch's own dropout equal round(float(y) * scale) for the oracle's scale
    y = torch.rand(1 << 16, device=device).to(torch.bfloat16)
    for p in (0.1, 0.25, 0.3):
        out = torch.nn.functional.dropout(y, p, True)
        kept = out != 0
        want = R.dropout_with_mask(y, kept, p)
        assert torch.equal(out, want)


# ---------------------------------------------------------------------------------
# golden vectors
# ---------------------------------------------------------------------------------
@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", ["dropout_causal_16", "dropout_causal_37"])
def test_golden_dropout(device, golden, name, dtype):
    f = golden[name]
    p, seed, offset, scale = float(f["p"]), int(f["seed"]), int(f["offset"]), float(f["scale"])
    x = torch.tensor(f["x"], device=device).to(dtype)
    assert torch.equal(x.float().cpu(), torch.tensor(f["x"]))  # inputs are exact in both types
    y, dropped = causal_ext.forward_dropout(x, scale, p, seed, offset)
    keep = torch.tensor(f["keep"], device=device).bool()
    assert torch.equal(rng.keep_mask(x.numel(), p, seed, offset, device).view(x.shape), keep)
    assert torch.equal(dropped != 0, keep & (y != 0))
    assert max_err(y, torch.tensor(f["y"], device=device)) <= TOL[dtype]
    # values up to 1/(1-p) > 1: the error of y scaled up, plus half an ulp of the second rounding
    half_ulp = 2.0**-8 if dtype == torch.bfloat16 else 2.0**-11
    assert max_err(dropped, torch.tensor(f["y_drop"], device=device)) <= (TOL[dtype] + half_ulp) / (1 - p)
    g = torch.tensor(f["g"], device=device).to(dtype)
    dx = causal_ext.backward_dropout(g.clone(), y, scale, p, seed, offset)
    assert max_err(dx, torch.tensor(f["dx"], device=device)) <= 4 * TOL[dtype] * max(1.0, np.abs(f["dx"]).max())


# ---------------------------------------------------------------------------------
# forward
# ---------------------------------------------------------------------------------
def check_forward(y, dropped, y_plain, p, seed, offset, device):
    assert torch.equal(y, y_plain)  # the saved probabilities are the plain kernels'
    keep = rng.keep_mask(y.numel(), p, seed, offset, device).view(y.shape)
    assert torch.equal(dropped, R.dropout_with_mask(y, keep, p))
    return keep


CAUSAL_SHAPES = [(3, 8, 8), (5, 24, 24), (2, 72, 72), (3, 128, 128), (2, 264, 264), (2, 512, 512),
                 (2, 1024, 1024), (1, 1032, 1032), (2, 2048, 2048), (1, 4096, 4096), (1, 8192, 8192),
                 (3, 7, 7), (2, 100, 100), (1, 1001, 1001),
                 # ragged rows: a lane's 8 columns straddle two Philox groups
                 (3, 9, 9), (3, 33, 33), (2, 129, 129), (2, 515, 515), (2, 2047, 2047), (1, 4099, 4099)]


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("shape", CAUSAL_SHAPES)
def test_causal_forward(device, shape, dtype):
    x = scores(shape, dtype, device, 3)
    p, seed, offset = 0.1, 1234 + shape[1], 4 * shape[0]
    y, dropped = causal_ext.forward_dropout(x, 0.125, p, seed, offset)
    keep = check_forward(y, dropped, causal_ext.forward(x, 0.125), p, seed, offset, device)
    if shape[1] <= 1024:
        # the device-side pattern is the oracle's (row-major element index of the [B, sq, sk] tensor)
        want = philox.keep_mask(x.numel(), p, seed, offset).reshape(shape)
        assert np.array_equal(keep.cpu().numpy(), want)
    upper = torch.triu(torch.ones(shape[1:], dtype=torch.bool, device=device), 1).expand(shape)
    assert (dropped[upper] == 0).all()


MASKED_SHAPES = [(2, 3, 5, 8), (2, 2, 9, 40), (1, 3, 16, 136), (2, 2, 8, 512), (2, 2, 16, 1024),
                 (1, 2, 8, 1536), (1, 2, 8, 2048), (1, 1, 4, 4096), (1, 1, 2, 16384), (1, 1, 2, 32768),
                 (2, 2, 5, 37), (1, 2, 3, 1001), (1, 1, 2, 40000), (1, 1, 2, 81416),  # ... staged in LDS, beyond it
                 (2, 2, 5, 9), (2, 3, 7, 129), (2, 2, 3, 515), (1, 2, 3, 2050), (1, 1, 3, 4099), (1, 1, 2, 9001)]


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("shape", MASKED_SHAPES)
def test_masked_forward(device, shape, dtype):
    b, np_, sq, sk = shape
    x = scores(shape, dtype, device, 4)
    lengths = torch.randint(1, sk + 1, (b,), generator=gen(device, 5), device=device)
    mask = R.padding_mask(lengths, sq, sk, device)
    mask[0, 0, 0, :] = True  # one fully hidden row: uniform 1/sk, then dropout
    p, seed, offset = 0.25, 99, 8
    y, dropped = masked_ext.forward_dropout(x, mask, 0.5, p, seed, offset)
    check_forward(y, dropped, masked_ext.forward(x, mask, 0.5), p, seed, offset, device)
    hidden = mask.expand(shape).clone()
    hidden[0, :, 0, :] = False
    assert (dropped[hidden] == 0).all()


@pytest.mark.parametrize("p", [0.0, 1.0])
def test_forward_edge_probabilities(device, p):
    x = scores((2, 64, 64), torch.bfloat16, device, 6)
    y, dropped = causal_ext.forward_dropout(x, 1.0, p, 1, 0)
    assert torch.equal(dropped, y if p == 0.0 else torch.zeros_like(y))


# ---------------------------------------------------------------------------------
# backward
# ---------------------------------------------------------------------------------
@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("shape", CAUSAL_SHAPES)
def test_causal_backward(device, shape, dtype):
    x = scores(shape, dtype, device, 7)
    g = normal(shape, dtype, device, 8)
    p, seed, offset, scale = 0.2, 4321, 12, 0.125
    y, _ = causal_ext.forward_dropout(x, scale, p, seed, offset)
    keep = rng.keep_mask(y.numel(), p, seed, offset, device).view(shape)
    ref = R.softmax_dropout_backward_fp32(g, y, keep, p, scale)
    dx = causal_ext.backward_dropout(g.clone(), y, scale, p, seed, offset)
    assert max_err(dx, ref) <= TOL[dtype] * max(1.0, ref.abs().max().item())
    assert (dx[y == 0] == 0).all()
    # in place on the gradient buffer, as the plain backward
    buf = g.clone()
    out = causal_ext.backward_dropout(buf, y, scale, p, seed, offset)
    assert out.data_ptr() == buf.data_ptr() and torch.equal(out, dx)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("shape", MASKED_SHAPES)
def test_masked_backward(device, shape, dtype):
    b, np_, sq, sk = shape
    x = scores(shape, dtype, device, 9)
    g = normal(shape, dtype, device, 10)
    mask = R.padding_mask(torch.randint(1, sk + 1, (b,), generator=gen(device, 11), device=device), sq, sk, device)
    p, seed, offset, scale = 0.1, 2**50 + 3, 2**33, 1.0
    y, _ = masked_ext.forward_dropout(x, mask, scale, p, seed, offset)
    keep = rng.keep_mask(y.numel(), p, seed, offset, device).view(shape)
    ref = R.softmax_dropout_backward_fp32(g, y, keep, p, scale)
    dx = masked_ext.backward_dropout(g.clone(), y, scale, p, seed, offset)
    assert max_err(dx, ref) <= TOL[dtype] * max(1.0, ref.abs().max().item())
    assert (dx[mask.expand(shape)] == 0).all()


def test_backward_against_fp64_autograd_of_the_unfused_expression(device):
    shape = (2, 3, 48, 48)
    x = scores(shape, torch.float16, device, 12)
    g = normal(shape, torch.float16, device, 13)
    mask = R.get_attn_mask(48, device)
    p, seed, offset, scale = 0.3, 5, 0, 0.25
    y, dropped = masked_ext.forward_dropout(x, mask, scale, p, seed, offset)
    keep = rng.keep_mask(y.numel(), p, seed, offset, device).view(shape)
    xd = x.double().requires_grad_(True)
    probs = torch.softmax((scale * xd).masked_fill(mask, float("-inf")), -1)
    out = probs * keep / (1 - p)
    (want,) = torch.autograd.grad(out, xd, g.double())
    assert max_err(dropped, out) <= 2 * TOL[torch.float16] / (1 - p)
    dx = masked_ext.backward_dropout(g.clone(), y, scale, p, seed, offset)
    assert max_err(dx, want) <= 4 * TOL[torch.float16] * max(1.0, want.abs().max().item())


# ---------------------------------------------------------------------------------
# the benchmark shapes at full size
# ---------------------------------------------------------------------------------
def test_full_size_padded_config(device):
    shape = (8, 16, 1024, 1024)
    x = scores(shape, torch.float16, device, 1235)
    g = normal(shape, torch.float16, device, 1236)
    lengths = torch.randint(256, 1025, (8,), generator=gen(device, 1237), device=device)
    mask = R.padding_mask(lengths, 1024, 1024, device)
    p, seed, offset = 0.1, 17, 400
    y, dropped = masked_ext.forward_dropout(x, mask, 0.125, p, seed, offset)
    keep = check_forward(y, dropped, masked_ext.forward(x, mask, 0.125), p, seed, offset, device)
    frac = keep.float().mean().item()
    assert abs(frac - 0.9) < 5 * (0.09 / keep.numel()) ** 0.5 + 2.0**-16
    dx = masked_ext.backward_dropout(g.clone(), y, 0.125, p, seed, offset)
    for s in range(0, 8, 4):  # fp32 reference in slices
        ref = R.softmax_dropout_backward_fp32(g[s:s + 4], y[s:s + 4], keep[s:s + 4], p, 0.125)
        assert max_err(dx[s:s + 4], ref) <= TOL[torch.float16] * max(1.0, ref.abs().max().item())


def test_full_size_long_causal_config(device):
    shape = (32, 8192, 8192)
    x = scores((4, 8192, 8192), torch.bfloat16, device, 1238).repeat(8, 1, 1)
    p, seed, offset = 0.1, 23, 2**35
    y, dropped = causal_ext.forward_dropout(x, 0.0884, p, seed, offset)
    assert y.shape == shape
    y_plain = causal_ext.forward(x, 0.0884)
    assert torch.equal(y, y_plain)
    del y_plain
    for s in range(0, 32, 8):  # element indices beyond 2^31: groups are 64-bit
        n0 = s * 8192 * 8192
        keep = rng.keep_mask(n0 + 8 * 8192 * 8192, p, seed, offset, device)[n0:].view(8, 8192, 8192)
        assert torch.equal(dropped[s:s + 8], R.dropout_with_mask(y[s:s + 8], keep, p))
        del keep
    g = normal((4, 8192, 8192), torch.bfloat16, device, 1239).repeat(8, 1, 1)
    dx = causal_ext.backward_dropout(g.clone(), y, 0.0884, p, seed, offset)
    s = 24
    n0 = s * 8192 * 8192
    keep = rng.keep_mask(n0 + 2 * 8192 * 8192, p, seed, offset, device)[n0:].view(2, 8192, 8192)
    ref = R.softmax_dropout_backward_fp32(g[s:s + 2], y[s:s + 2], keep, p, 0.0884)
    assert max_err(dx[s:s + 2], ref) <= TOL[torch.bfloat16] * max(1.0, ref.abs().max().item())
    assert (dx[s:s + 2][y[s:s + 2] == 0] == 0).all()


# ---------------------------------------------------------------------------------
# autograd Functions, module, generator plumbing
# ---------------------------------------------------------------------------------
def test_functions_follow_the_default_generator(device):
    x = scores((4, 256, 256), torch.bfloat16, device, 20).requires_grad_(True)
    gen0 = torch.cuda.default_generators[device.index]
    torch.manual_seed(555)
    off0 = gen0.get_offset()
    a = ScaledUpperTriangMaskedSoftmaxDropout.apply(x, 0.5, 0.1)
    assert gen0.get_offset() == off0 + rng.OFFSET_STEP
    b = ScaledUpperTriangMaskedSoftmaxDropout.apply(x, 0.5, 0.1)
    assert not torch.equal(a, b)  # the generator moved on
    torch.manual_seed(555)
    c = ScaledUpperTriangMaskedSoftmaxDropout.apply(x, 0.5, 0.1)
    assert torch.equal(a, c)  # same generator state, same pattern
    # the call with the state spelled out
    _, want = causal_ext.forward_dropout(x.detach(), 0.5, 0.1, 555, off0)
    assert torch.equal(a, want)
    # a torch random call in between shifts the pattern: the state is shared, not private
    torch.manual_seed(555)
    torch.rand(4, device=device)
    d = ScaledUpperTriangMaskedSoftmaxDropout.apply(x, 0.5, 0.1)
    assert not torch.equal(a, d)
    # saved and restored generator state (what the RNG tracker's fork() does)
    torch.manual_seed(777)
    state = torch.cuda.get_rng_state(device)
    e = ScaledUpperTriangMaskedSoftmaxDropout.apply(x, 0.5, 0.1)
    torch.cuda.set_rng_state(state, device)
    f = ScaledUpperTriangMaskedSoftmaxDropout.apply(x, 0.5, 0.1)
    assert torch.equal(e, f)


@pytest.mark.parametrize("dtype", DTYPES)
def test_function_gradients(device, dtype):
    shape = (2, 4, 128, 128)
    x = scores(shape, dtype, device, 21).requires_grad_(True)
    g = normal(shape, dtype, device, 22)
    mask = R.padding_mask(torch.tensor([100, 128]), 128, 128, device)
    torch.manual_seed(31)
    off = torch.cuda.default_generators[device.index].get_offset()
    out = ScaledMaskedSoftmaxDropout.apply(x, mask, 0.5, 0.15)
    out.backward(g.clone())
    y = masked_ext.forward(x.detach(), mask, 0.5)
    keep = rng.keep_mask(y.numel(), 0.15, 31, off, device).view(shape)
    assert torch.equal(out, R.dropout_with_mask(y, keep, 0.15))
    ref = R.softmax_dropout_backward_fp32(g, y, keep, 0.15, 0.5)
    assert max_err(x.grad, ref) <= TOL[dtype] * max(1.0, ref.abs().max().item())

    x3 = scores((6, 128, 128), dtype, device, 23).requires_grad_(True)
    torch.manual_seed(32)
    off = torch.cuda.default_generators[device.index].get_offset()
    out = ScaledUpperTriangMaskedSoftmaxDropout.apply(x3, 0.5, 0.15)
    out.backward(g.view(8, 128, 128)[:6].clone())
    y = causal_ext.forward(x3.detach(), 0.5)
    keep = rng.keep_mask(y.numel(), 0.15, 32, off, device).view(y.shape)
    ref = R.softmax_dropout_backward_fp32(g.view(8, 128, 128)[:6], y, keep, 0.15, 0.5)
    assert max_err(x3.grad, ref) <= TOL[dtype] * max(1.0, ref.abs().max().item())


def test_module_dropout_argument(device):
    b, np_, s = 2, 4, 256
    x = scores((b, np_, s, s), torch.bfloat16, device, 24)
    causal = R.get_attn_mask(s, device)
    m = FusedScaleMaskSoftmax(False, True, SoftmaxFusionTypes.upper_triang, R.gpt2_attention_mask_func, True, 0.5)
    plain = m(x, causal)
    assert torch.equal(m(x, causal, dropout_p=0.0), plain)
    torch.manual_seed(41)
    off = torch.cuda.default_generators[device.index].get_offset()
    out = m(x, causal, dropout_p=0.1)
    keep = rng.keep_mask(x.numel(), 0.1, 41, off, device).view(x.shape)
    assert torch.equal(out, R.dropout_with_mask(plain, keep, 0.1))
    # a sliding-window mask goes to the mask-tensor kernel, same pattern assignment
    window = R.get_attn_mask(s, device, sliding_window_width=32)
    torch.manual_seed(41)
    out = m(x, window, dropout_p=0.1)
    assert torch.equal(out, R.dropout_with_mask(m(x, window), keep, 0.1))
    # general fusion with a padding mask
    mg = FusedScaleMaskSoftmax(False, True, SoftmaxFusionTypes.general, R.gpt2_attention_mask_func, True, None)
    pad = R.padding_mask(torch.tensor([200, 256]), s, s, device)
    torch.manual_seed(41)
    out = mg(x, pad, dropout_p=0.1)
    assert torch.equal(out, R.dropout_with_mask(mg(x, pad), keep, 0.1))
    # ALiBi slopes or a bias tensor are folded into the same kernel: the pattern is still ours
    slopes = torch.tensor(R.alibi_slopes(np_), device=device)
    torch.manual_seed(41)
    out = m(x, causal, alibi_slopes=slopes, dropout_p=0.1)
    assert torch.equal(out, R.dropout_with_mask(m(x, causal, alibi_slopes=slopes), keep, 0.1))
    rpe = scores((1, np_, s, s), torch.bfloat16, device, 26) * 0.25
    torch.manual_seed(41)
    out = m(x, causal, bias=rpe, dropout_p=0.1)
    assert torch.equal(out, R.dropout_with_mask(m(x, causal, bias=rpe), keep, 0.1))
    torch.manual_seed(41)
    out = mg(x, pad, bias=rpe, dropout_p=0.1)
    assert torch.equal(out, R.dropout_with_mask(mg(x, pad, bias=rpe), keep, 0.1))
    # both at once, or ALiBi with a mask that is not the plain triangle: the softmax kernel
    # followed by torch's dropout -- same law, torch's pattern
    for kwargs, mask in ((dict(alibi_slopes=slopes, bias=rpe), causal), (dict(alibi_slopes=slopes), window)):
        out = m(x, mask, dropout_p=0.5, **kwargs)
        base = m(x, mask, **kwargs)
        kept = out != 0
        assert torch.equal(out, R.dropout_with_mask(base, kept, 0.5))
        frac = (kept & (base != 0)).float().sum().item() / (base != 0).float().sum().item()
        assert 0.45 < frac < 0.55
    # the unfused module (fusion off) takes torch's dropout as well
    mt = FusedScaleMaskSoftmax(False, True, SoftmaxFusionTypes.none, R.gpt2_attention_mask_func, True, 0.5)
    out = mt(x, causal, dropout_p=0.5)
    assert torch.equal(out, R.dropout_with_mask(mt(x, causal), out != 0, 0.5))


def test_statistics_of_the_fused_output(device):
    # E[dropout(y)] = y: averaged over many patterns the dropped output returns the probabilities
    x = scores((1, 64, 64), torch.float16, device, 25)
    y = causal_ext.forward(x, 0.25).float()
    acc = torch.zeros_like(y)
    n = 400
    for i in range(n):
        _, d = causal_ext.forward_dropout(x, 0.25, 0.3, 1000, 4 * i)
        acc += d.float()
    err = (acc / n - y).abs()
    bound = 5 * y * (0.3 / 0.7 / n) ** 0.5 + 1e-3
    assert (err <= bound).all()


# ---------------------------------------------------------------------------------
# HIP graphs: the pattern follows a device-resident state that the graph advances
# ---------------------------------------------------------------------------------
def test_device_state_argument_equals_the_numbers_it_holds(device):
    x = scores((3, 264, 264), torch.bfloat16, device, 30)
    g = normal((3, 264, 264), torch.bfloat16, device, 31)
    seed, offset = 2**45 + 17, rng.GRAPH_OFFSET_BASE + 40
    state = torch.tensor([seed, offset], dtype=torch.int64, device=device)
    y0, d0 = causal_ext.forward_dropout(x, 0.25, 0.2, seed, offset)
    y1, d1 = causal_ext.forward_dropout(x, 0.25, 0.2, 0, 0, state)
    assert torch.equal(y0, y1) and torch.equal(d0, d1)
    assert torch.equal(causal_ext.backward_dropout(g.clone(), y0, 0.25, 0.2, seed, offset),
                       causal_ext.backward_dropout(g.clone(), y0, 0.25, 0.2, 0, 0, state))
    assert torch.equal(rng.keep_mask(1000, 0.2, seed, offset, device), rng.keep_mask(1000, 0.2, 0, 0, device, state))
    with pytest.raises(RuntimeError, match="int64 device tensor"):
        causal_ext.forward_dropout(x, 0.25, 0.2, 0, 0, state.int())


def test_fused_dropout_in_a_hip_graph_draws_a_fresh_pattern_per_replay(device):
    shape = (2, 4, 256, 256)
    x = scores(shape, torch.float16, device, 32).requires_grad_(True)
    g = normal(shape, torch.float16, device, 33)
    pad = R.padding_mask(torch.tensor([256, 100]), 256, 256, device)
    causal = R.get_attn_mask(256, device)
    mc = FusedScaleMaskSoftmax(True, False, SoftmaxFusionTypes.upper_triang, R.gpt2_attention_mask_func, True, 0.5,
                               causal_mask_check="verify")
    mg = FusedScaleMaskSoftmax(True, False, SoftmaxFusionTypes.general, R.gpt2_attention_mask_func, True, 0.5)
    assert mc.mask_is_plain_causal(causal)  # decided (with a host sync) before the capture
    torch.manual_seed(99)
    live = rng.graph_state(device, reseed=True)
    first = live.tolist()
    assert first == [99, rng.GRAPH_OFFSET_BASE + torch.cuda.default_generators[device.index].get_offset()]

    out = {}

    def step():
        a = ScaledUpperTriangMaskedSoftmaxDropout.apply(x.view(-1, 256, 256), 0.5, 0.1)
        b = mg(x, pad, dropout_p=0.1)
        # the backward kernels write into the gradient they are given: hand them copies
        (ga,) = torch.autograd.grad(a, x, g.view(-1, 256, 256).clone(), retain_graph=False)
        (gb,) = torch.autograd.grad(b, x, g.clone(), retain_graph=False)
        out.update(a=a, b=b, ga=ga, gb=gb)

    graph = torch.cuda.CUDAGraph()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        step()  # eager warm-up on the capture stream: takes the host generator, not the device state
        side.synchronize()
        assert live.tolist() == first
        fresh_mask = causal.clone()
        with torch.cuda.graph(graph, stream=side):
            step()
            # a mask decided before the capture keeps its verdict; one first seen inside it cannot
            # be examined (that would synchronise) and goes to the mask-tensor kernel
            verdicts = (mc.mask_is_plain_causal(causal), mc.mask_is_plain_causal(fresh_mask))
    assert verdicts == (True, False)
    assert live.tolist() == first  # capturing executes nothing

    seen = []
    for rep in range(3):
        for t in out.values():
            t.fill_(float("nan"))  # eager work between the replays
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        seed, off_a = first[0], first[1] + 2 * rep * rng.OFFSET_STEP
        off_b = off_a + rng.OFFSET_STEP
        assert live.tolist() == [seed, first[1] + 2 * (rep + 1) * rng.OFFSET_STEP]
        xd = x.detach()
        ya, want_a = causal_ext.forward_dropout(xd.view(-1, 256, 256), 0.5, 0.1, seed, off_a)
        yb, want_b = masked_ext.forward_dropout(xd, pad, 0.5, 0.1, seed, off_b)
        assert torch.equal(out["a"], want_a) and torch.equal(out["b"], want_b)
        assert torch.equal(out["ga"].view(-1, 256, 256),
                           causal_ext.backward_dropout(g.view(-1, 256, 256).clone(), ya, 0.5, 0.1, seed, off_a))
        assert torch.equal(out["gb"], masked_ext.backward_dropout(g.clone(), yb, 0.5, 0.1, seed, off_b))
        seen.append(out["a"].clone())
    assert not torch.equal(seen[0], seen[1]) and not torch.equal(seen[1], seen[2])
    # capture without the state prepared is refused with a clear message
    rng._graph_states.pop(device.index)
    with pytest.raises(RuntimeError, match="graph_state"):
        with torch.cuda.stream(side):
            with torch.cuda.graph(torch.cuda.CUDAGraph(), stream=side):
                mg(x.detach(), pad, dropout_p=0.1)


# ---------------------------------------------------------------------------------
# ALiBi slopes / bias tensor together with dropout
# ---------------------------------------------------------------------------------
COMBO_SHAPES = [(2, 3, 8, 8), (2, 2, 136, 136), (1, 4, 512, 512), (2, 2, 1024, 1024), (1, 2, 2048, 2048),
                (1, 2, 4096, 4096), (2, 2, 37, 37)]


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("shape", COMBO_SHAPES)
def test_causal_dropout_with_alibi_or_bias(device, shape, dtype):
    b, np_, s, _ = shape
    x = scores(shape, dtype, device, 40)
    g = normal(shape, dtype, device, 41)
    slopes = torch.tensor(R.alibi_slopes(np_), device=device)
    bias = scores((1, np_, s, s), dtype, device, 42) * 0.25
    p, seed, offset, scale = 0.2, 77, 16, 0.125
    keep = rng.keep_mask(x.numel(), p, seed, offset, device).view(shape)
    for kwargs, plain in ((dict(slopes=slopes), causal_ext.forward_alibi(x, slopes, scale)),
                          (dict(bias=bias), causal_ext.forward_bias(x, bias, scale))):
        y, dropped = causal_ext.forward_dropout(x, scale, p, seed, offset, **kwargs)
        assert torch.equal(y, plain)
        assert torch.equal(dropped, R.dropout_with_mask(y, keep, p))
        dx = causal_ext.backward_dropout(g.clone(), y, scale, p, seed, offset)
        ref = R.softmax_dropout_backward_fp32(g, y, keep, p, scale)
        assert max_err(dx, ref) <= TOL[dtype] * max(1.0, ref.abs().max().item())
    # both at once: the probabilities of the bias kernel with the slopes on top, dropped alike
    y, dropped = causal_ext.forward_dropout(x, scale, p, seed, offset, slopes=slopes, bias=bias)
    assert torch.equal(y, causal_ext.forward_bias(x, bias, scale, slopes))
    assert torch.equal(dropped, R.dropout_with_mask(y, keep, p))
    with pytest.raises(RuntimeError, match="4D"):
        causal_ext.forward_dropout(x.view(-1, s, s), scale, p, seed, offset, slopes=slopes)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("shape", [(2, 3, 5, 8), (1, 3, 16, 136), (2, 2, 8, 512), (2, 2, 16, 1024), (1, 2, 8, 2048),
                                   (2, 2, 5, 37)])
def test_masked_dropout_with_bias(device, shape, dtype):
    b, np_, sq, sk = shape
    x = scores(shape, dtype, device, 43)
    bias = scores((b, np_, sq, sk), dtype, device, 44) * 0.25
    mask = R.padding_mask(torch.randint(1, sk + 1, (b,), generator=gen(device, 45), device=device), sq, sk, device)
    p, seed, offset = 0.3, 5, 2**34
    y, dropped = masked_ext.forward_dropout(x, mask, 0.5, p, seed, offset, bias=bias)
    assert torch.equal(y, masked_ext.forward_bias(x, mask, bias, 0.5))
    keep = rng.keep_mask(x.numel(), p, seed, offset, device).view(shape)
    assert torch.equal(dropped, R.dropout_with_mask(y, keep, p))


@pytest.mark.parametrize("shared", [True, False])
def test_dropout_function_gradient_reaches_the_bias(device, shared):
    b, np_, s = 3, 2, 64
    shape = (b, np_, s, s)
    x = scores(shape, torch.bfloat16, device, 46).requires_grad_(True)
    bias = (scores((1 if shared else b, np_, s, s), torch.bfloat16, device, 47) * 0.25).requires_grad_(True)
    g = normal(shape, torch.bfloat16, device, 48)
    causal = R.get_attn_mask(s, device)
    pad = R.padding_mask(torch.tensor([40, 64, 9]), s, s, device)
    for fn, mask in ((lambda: ScaledUpperTriangMaskedSoftmaxDropout.apply(x, 0.5, 0.2, None, bias), causal),
                     (lambda: ScaledMaskedSoftmaxDropout.apply(x, pad, 0.5, 0.2, bias), pad)):
        x.grad = bias.grad = None
        torch.manual_seed(61)
        off = torch.cuda.default_generators[device.index].get_offset()
        fn().backward(g.clone())
        keep = rng.keep_mask(x.numel(), 0.2, 61, off, device).view(shape)
        xr = x.detach().float().requires_grad_(True)
        br = bias.detach().float().requires_grad_(True)
        probs = R.softmax_fp32(xr + br, mask, 0.5)
        (probs * keep * R.dropout_scale(0.2)).backward(g.float())
        tol = 4 * TOL[torch.bfloat16]
        assert max_err(x.grad, xr.grad) <= tol * max(1.0, xr.grad.abs().max().item())
        assert bias.grad.shape == bias.shape
        assert max_err(bias.grad, br.grad) <= tol * max(1.0, br.grad.abs().max().item()) * (b if shared else 1)


def alibi_bias_any_shape(slopes, sq, sk, device):
    """The ALiBi bias as the C-ABI defines it for any sq: slope * min(j - i', 0) with i' = i + sk - sq,
    fp32 [np, sq, sk].  For sq == sk and sq == 1 -- all the reference's module produces -- it is the
    oracle's matrix (asserted in test_alibi_definition_for_any_query_count)."""
    i = torch.arange(sq, device=device).view(sq, 1) + (sk - sq)
    j = torch.arange(sk, device=device).view(1, sk)
    return (j - i).clamp(max=0).float() * slopes.float().view(-1, 1, 1)


def test_alibi_definition_for_any_query_count(device):
    slopes = torch.tensor(R.alibi_slopes(6), device=device)
    for sq, sk in ((9, 9), (1, 9), (1, 1), (520, 520), (1, 777)):
        assert torch.equal(alibi_bias_any_shape(slopes, sq, sk, device), R.alibi_bias_fp32(slopes, sq, sk, device))


def check_combination(device, dtype, causal, b, heads, sq, sk, scale, p, extra, shift, case):
    """One call of the kernels with the given mask kind (causal / random mask bytes), optional bias
    tensor ("bias", "shared bias") and / or ALiBi slopes ("alibi", "alibi+bias", "alibi+shared bias"),
    dropout probability p and every tensor (those of the backward pass too) starting `shift` elements
    into its allocation: forward and backward against the oracle's fp32 expressions, with the
    kernels' own keep pattern."""

    def shifted(t, by):
        flat = torch.empty(t.numel() + by, dtype=t.dtype, device=device)
        flat[by:] = t.reshape(-1)
        return flat[by:].view(t.shape)

    tag = (case, str(dtype), causal, b, heads, sq, sk, scale, p, extra, shift)
    x = shifted(scores((b, heads, sq, sk), dtype, device, case), shift)
    g = shifted(normal((b, heads, sq, sk), dtype, device, 1000 + case), shift)
    bias = slopes = None
    logits = x.float()
    if "bias" in extra:
        bias = shifted(normal((1 if "shared bias" in extra else b, heads, sq, sk), dtype, device, 2000 + case), shift)
        logits = logits + bias.float()
    if "alibi" in extra:
        slopes = torch.rand(heads, device=device, generator=gen(device, case)) * 0.5
        logits = logits + alibi_bias_any_shape(slopes, sq, sk, device)
    if causal:
        mask = R.get_attn_mask(sk, device)
    else:
        mask = torch.rand(1 if case % 2 else b, 1, sq, sk, device=device, generator=gen(device, 3000 + case)) < 0.3
        mask = shifted(mask, shift)
    want = R.softmax_fp32(logits, mask, scale)
    del logits
    seed, offset = 77 + case, 4 * case
    if p == 0.0:
        if causal:
            if bias is not None:
                y = causal_ext.forward_bias(x, bias, scale, slopes)
            elif slopes is not None:
                y = causal_ext.forward_alibi(x, slopes, scale)
            else:
                y = causal_ext.forward(x.view(-1, sq, sk), scale).view(x.shape)
            dx = causal_ext.backward(shifted(g, shift).view(-1, sq, sk), shifted(y, shift).view(-1, sq, sk), scale).view(x.shape)
        else:
            if bias is not None:
                y = masked_ext.forward_bias(x, mask, bias, scale, slopes)
            elif slopes is not None:
                y = masked_ext.forward_alibi(x, mask, slopes, scale)
            else:
                y = masked_ext.forward(x, mask, scale)
            dx = masked_ext.backward(shifted(g, shift), shifted(y, shift), scale)
        want_dx = R.softmax_backward_fp32(g, y, scale)
    else:
        if causal:
            y, dropped = causal_ext.forward_dropout(x, scale, p, seed, offset, slopes=slopes, bias=bias)
            dx = causal_ext.backward_dropout(shifted(g, shift), shifted(y, shift), scale, p, seed, offset)
        else:
            y, dropped = masked_ext.forward_dropout(x, mask, scale, p, seed, offset, bias=bias, slopes=slopes)
            dx = masked_ext.backward_dropout(shifted(g, shift), shifted(y, shift), scale, p, seed, offset)
        keep = rng.keep_mask(y.numel(), p, seed, offset, device).view(y.shape)
        if y.numel() <= 1 << 20:
            assert np.array_equal(keep.cpu().numpy().reshape(-1), philox.keep_mask(y.numel(), p, seed, offset)), tag
        assert torch.equal(dropped, R.dropout_with_mask(y, keep, p)), tag
        want_dx = R.softmax_dropout_backward_fp32(g, y, keep, p, scale)
    assert max_err(y, want) <= TOL[dtype], tag
    hidden = mask.expand_as(y)
    full_rows = hidden.all(-1, keepdim=True).expand_as(y)
    assert (y[hidden & ~full_rows] == 0).all(), tag
    # the bound scales with the largest gradient and allows for the rounding of values above 1
    top = want_dx.abs().max().item()
    half_ulp = top * (2.0**-8 if dtype == torch.bfloat16 else 2.0**-11)
    assert max_err(dx, want_dx) <= TOL[dtype] * max(1.0, top) + half_ulp, tag
    assert (dx[hidden & ~full_rows] == 0).all(), tag


def test_seeded_random_row_lengths_alignments_and_feature_combinations(device):
    # any row length (mostly not a multiple of 8), tensors starting at a random element of their
    # allocation, and a random choice of mask kind, bias / ALiBi and dropout
    import random

    rnd = random.Random(20250101)
    for case in range(90):
        dtype = rnd.choice(DTYPES)
        sk = rnd.choice([rnd.randint(8, 70), rnd.randint(71, 520), rnd.randint(521, 2100), rnd.randint(2101, 9000)])
        causal = rnd.random() < 0.5
        b, heads = rnd.randint(1, 2), rnd.randint(1, 3)
        sq = sk if causal else rnd.randint(1, 6)
        if causal and sk > 2100:
            b, heads = 1, 1
        scale = rnd.choice([0.125, 0.5, 1.0])
        p = rnd.choice([0.0, 0.0, 0.1, 0.5])
        extra = rnd.choice(["none", "none", "bias", "shared bias", "alibi", "alibi+bias", "alibi+shared bias"])
        check_combination(device, dtype, causal, b, heads, sq, sk, scale, p, extra, rnd.randint(0, 9), case)


# one row length per kernel shape of the dispatcher: lane groups of 1 .. 64 lanes (those of 32 and 64
# lanes also three quarters full or less: 160 and 320 columns; 640 and 1280: the forward passes'
# two- and three-chunk packed kernels), then 1, 2, 4, 8 and 16 waves per row
# with 2, 3 or 4 chunks per wave
SHAPE_LENGTHS = [8, 16, 32, 64, 128, 160, 256, 320, 512, 640, 1024, 1280, 1536, 2048, 2560, 4096, 5120, 8192, 10240, 13312, 16384,
                 20480, 28672]


@pytest.mark.parametrize("extra", ["none", "bias", "shared bias", "alibi", "alibi+bias", "alibi+shared bias"])
@pytest.mark.parametrize("p", [0.0, 0.25])
def test_every_kernel_shape_with_every_feature_combination(device, extra, p):
    # each length as it is (aligned rows) and one column shorter (ragged rows of odd length), in
    # both storage types, through the mask-tensor kernels (three rows) and through the causal
    # kernels (two heads up to 4096 columns, one beyond); 8 columns also as ragged rows, which
    # only a tensor that starts off a 16-byte boundary makes of them
    case = 0
    for n in SHAPE_LENGTHS:
        for sk, shift in ((n, 0), (n - 1, 0) if n > 8 else (9, 0)) + (((8, 3),) if n == 8 else ()):
            for dtype in DTYPES:
                case += 1
                check_combination(device, dtype, False, 2, 2, 3, sk, 0.25, p, extra, shift, case)
                check_combination(device, dtype, True, 1, 2 if sk <= 4096 else 1, sk, sk, 0.25, p, extra, shift, 500 + case)
        if n > 4096:
            torch.cuda.empty_cache()
