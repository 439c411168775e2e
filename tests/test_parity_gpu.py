"""Parity of the gfx950 kernels (called through the C-ABI) with the oracle.

Bars: softmax |err| <= 2e-3 (bf16) / 1e-3 (fp16)
against the fp32 computation of the reference's unfused path, masked positions
exactly 0; rotary is bit-equal to the fp32 expression rounded once to the storage
type.  The backward pass is compared with the fp32 closed form evaluated on the
same saved (rounded) probabilities, which is what the reference's fused backward
consumes, at the same bars.
"""
import numpy as np
import pytest
import torch

from gpt_neox_amd import _lib
from gpt_neox_amd.fused_kernels import (
    fused_rotary_positional_embedding as rope_ext,
    scaled_masked_softmax_cuda as masked_ext,
    scaled_upper_triang_masked_softmax_cuda as causal_ext,
)
from gpt_neox_amd.fused_softmax import (
    FusedScaleMaskSoftmax,
    ScaledMaskedSoftmax,
    ScaledUpperTriangMaskedSoftmax,
    SoftmaxFusionTypes,
)
from gpt_neox_amd.positional_embeddings import (
    RotaryEmbedding,
    apply_rotary_pos_emb,
    apply_rotary_pos_emb_,
    apply_rotary_pos_emb_qkv_,
    apply_rotary_pos_emb_torch,
)
from gpt_neox_amd.fused_kernels.attention_dropout import keep_mask as rng_keep
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


# ---------------------------------------------------------------------------------
# 16-bit conversions used by every kernel
# ---------------------------------------------------------------------------------
@pytest.mark.parametrize("dtype", DTYPES)
def test_rounding_is_nearest_even(device, dtype):
    # q = 1, sin = 0: the kernel stores round(cos).  cos walks through quarter-ulp steps of
    # the storage type, so every fourth value is an exact tie (must go to the even neighbour).
    p = 7 if dtype == torch.bfloat16 else 10  # explicit mantissa bits
    steps = torch.arange(64, device=device, dtype=torch.float32)
    cos = (1.0 + steps * 2.0 ** -(p + 2)).view(1, 1, 1, 64).expand(4, 1, 1, 64).contiguous()
    sin = torch.zeros_like(cos)
    q = torch.ones(4, 2, 3, 64, dtype=dtype, device=device)
    oq, ok = apply_rotary_pos_emb(q, q, cos, sin)
    want = cos.to(dtype).expand_as(q)
    assert torch.equal(oq, want) and torch.equal(ok, want)
    # identity table: every stored value survives unchanged
    x = normal((8, 2, 4, 64), dtype, device, 1)
    oq, _ = apply_rotary_pos_emb(x, x, torch.ones(8, 1, 1, 64, device=device), torch.zeros(8, 1, 1, 64, device=device))
    assert torch.equal(oq, x)


def grad_bar(ref, dtype):
    """north_star's absolute bar for a gradient compared with one that torch's autograd has itself
    rounded to the storage type: the bar plus half an ulp of the largest comparator value."""
    ulp = 2.0 ** -8 if dtype == torch.bfloat16 else 2.0 ** -11
    return TOL[dtype] + ulp * ref.float().abs().max().item()


# ---------------------------------------------------------------------------------
# golden vectors
# ---------------------------------------------------------------------------------
@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", ["causal_8", "causal_40"])
def test_golden_causal(device, golden, name, dtype):
    f = golden[name]
    x = torch.tensor(f["x"], device=device).to(dtype)
    assert torch.equal(x.float().cpu(), torch.tensor(f["x"]))  # inputs are exact in both types
    y = causal_ext.forward(x, float(f["scale"]))
    want = torch.tensor(f["y"], device=device)
    assert max_err(y, want) <= TOL[dtype]
    assert (y[want == 0] == 0).all()
    g = torch.tensor(f["g"], device=device).to(dtype)
    dx = causal_ext.backward(g.clone(), y, float(f["scale"]))
    ref = R.softmax_backward_fp32(g, y, float(f["scale"]))
    assert max_err(dx, ref) <= TOL[dtype] * max(1.0, ref.abs().max().item())
    # against the float64 fixture: adds the effect of the rounded probabilities
    assert max_err(dx, torch.tensor(f["dx"], device=device)) <= 4 * TOL[dtype] * max(1.0, np.abs(f["dx"]).max())
    assert (dx[want == 0] == 0).all()


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", ["masked_4x16", "masked_3x37"])
def test_golden_masked(device, golden, name, dtype):
    f = golden[name]
    x = torch.tensor(f["x"], device=device).to(dtype)
    mask_u8 = torch.tensor(f["mask"], device=device)
    want = torch.tensor(f["y"], device=device)
    for mask in (mask_u8, mask_u8.bool(), mask_u8 * 7):  # any non-zero byte masks
        y = masked_ext.forward(x, mask, float(f["scale"]))
        assert max_err(y, want) <= TOL[dtype]
        assert (y[want == 0] == 0).all()
    g = torch.tensor(f["g"], device=device).to(dtype)
    dx = masked_ext.backward(g.clone(), y, float(f["scale"]))
    ref = R.softmax_backward_fp32(g, y, float(f["scale"]))
    assert max_err(dx, ref) <= TOL[dtype] * max(1.0, ref.abs().max().item())
    assert (dx[want == 0] == 0).all()


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", ["rotary_d8", "rotary_d32", "rotary_d24"])
def test_golden_rotary(device, golden, name, dtype):
    f = golden[name]
    s, _, _, d = f["q"].shape
    off = int(f["offset"])
    cos, sin = (t.to(device) for t in R.rotary_tables(d, s + off, float(f["base"])))
    q = torch.tensor(f["q"], device=device).to(dtype).requires_grad_(True)
    k = torch.tensor(f["k"], device=device).to(dtype).requires_grad_(True)
    oq, ok = apply_rotary_pos_emb(q, k, cos, sin, off)
    ulp = 2.0**-8 if dtype == torch.bfloat16 else 2.0**-11
    for got, key in ((oq, "oq"), (ok, "ok")):
        want = torch.tensor(f[key], device=device)
        assert ((got.double() - want).abs() <= ulp * want.abs().clamp(min=1.0) + 1e-4).all(), key
    torch.autograd.backward([oq, ok], [torch.tensor(f["gq"], device=device).to(dtype),
                                       torch.tensor(f["gk"], device=device).to(dtype)])
    for got, key in ((q.grad, "dq"), (k.grad, "dk")):
        want = torch.tensor(f[key], device=device)
        assert ((got.double() - want).abs() <= ulp * want.abs().clamp(min=1.0) + 1e-4).all(), key


# ---------------------------------------------------------------------------------
# causal softmax
# ---------------------------------------------------------------------------------
def check_causal(device, batches, s, dtype, scale, seed, chunk=4, absolute=False):
    x = scores((batches, s, s), dtype, device, seed)
    g = normal((batches, s, s), dtype, device, seed + 1000)
    x_copy = x.clone()
    y = causal_ext.forward(x, scale)
    assert torch.equal(x, x_copy)  # the input is not modified
    assert y.dtype == dtype and y.shape == x.shape and y.is_contiguous()
    dx = causal_ext.backward(g.clone(), y, scale)
    mask = R.get_attn_mask(s, device)
    for i in range(0, batches, chunk):
        ref = R.softmax_fp32(x[i : i + chunk].unsqueeze(0), mask, scale)[0]
        assert max_err(y[i : i + chunk], ref) <= TOL[dtype], (batches, s, dtype)
        hidden = mask[0].expand_as(y[i : i + chunk])
        assert (y[i : i + chunk][hidden] == 0).all()
        refb = R.softmax_backward_fp32(g[i : i + chunk], y[i : i + chunk], scale)
        assert max_err(dx[i : i + chunk], refb) <= TOL[dtype] * max(1.0, refb.abs().max().item())
        assert (dx[i : i + chunk][hidden] == 0).all()
        # the bar itself: autograd of the unfused fp32 path from x (not from the kernel's rounded
        # probabilities)
        _, auto = R.softmax_autograd_fp32(x[i : i + chunk].unsqueeze(0), mask, scale, g[i : i + chunk].unsqueeze(0))
        assert_grad(dx[i : i + chunk], auto[0], dtype, (batches, s, dtype), absolute,
                    y=y[i : i + chunk], g=g[i : i + chunk], scale=scale)
    return x, y, g, dx


# row lengths chosen to hit: 1 column; lanes partly filled; not a multiple of 8 (element-wise
# kernels); 1 and 2 chunks of 512 columns on one wave; the 2-, 4- and 8-wave kernels with rows
# that fill their last chunk exactly, partly, or leave whole chunks of a wave empty.
CAUSAL_SIZES = [1, 2, 7, 8, 16, 24, 37, 40, 64, 72, 120, 128, 200, 256, 264, 384, 504, 512, 520, 1000, 1024, 1536, 2048, 2056, 2560, 3072,
                4096, 4104, 5000, 6144, 8192]


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("s", CAUSAL_SIZES)
def test_causal_sizes(device, s, dtype):
    batches = 3 if s <= 2056 else 1
    check_causal(device, batches, s, dtype, 0.125, seed=s)


@pytest.mark.parametrize("s", [8200, 10240, 12288, 13312, 14336, 16384, 20000, 28672, 33000, 40448, 40456, 40968])
def test_causal_very_long_rows(device, s):
    # 16 waves per row with 2, 3 and 4 chunks per wave; from 33000 on the row exceeds the register
    # budget and is staged in LDS: in half of a CU's LDS up to 40448 columns, in all of it beyond
    x = scores((1, s, s), torch.bfloat16, device, s)
    y = causal_ext.forward(x, 0.05)
    rows = torch.tensor([0, 1, 511, 512, 513, s // 2, s - 2, s - 1], device=device)
    mask = R.get_attn_mask(s, device)[0, 0][rows]
    ref = R.softmax_fp32(x[0][rows], mask, 0.05)
    assert max_err(y[0][rows], ref) <= TOL[torch.bfloat16]
    assert (y[0][rows][mask] == 0).all()
    assert torch.allclose(y.float().sum(-1), torch.ones(1, s, device=device), atol=3e-2)
    g = normal((1, s, s), torch.bfloat16, device, 5)
    dx = causal_ext.backward(g.clone(), y, 0.05)
    refb = R.softmax_backward_fp32(g[0][rows], y[0][rows], 0.05)
    assert max_err(dx[0][rows], refb) <= TOL[torch.bfloat16]
    assert (dx[0][rows][mask] == 0).all()


@pytest.mark.parametrize("s", [8, 24, 200, 512, 1000, 1536, 2048, 3000, 4104, 9000, 20000, 33000, 41000])
def test_causal_kernels_ignore_what_lies_past_the_diagonal(device, s):
    # The reference reads scores, gradient and probabilities up to the diagonal only
    # (scaled_upper_triang_masked_softmax.h:180-196 and 304-325): NaN and Inf above it, also in
    # the columns that share a 128-bit access with the diagonal, change nothing.
    batches = 2 if s <= 4104 else 1
    upper = torch.ones(s, s, dtype=torch.bool, device=device).triu_(1)
    for dtype in (DTYPES if s <= 4104 else [torch.bfloat16]):
        x = scores((batches, s, s), dtype, device, s)
        g = normal((batches, s, s), dtype, device, s + 1)
        y = causal_ext.forward(x, 0.125)
        dx = causal_ext.backward(g.clone(), y, 0.125)
        y_poisoned = causal_ext.forward(x.masked_fill(upper, float("nan")), 0.125)
        assert torch.equal(y_poisoned, y)
        y_poisoned = causal_ext.forward(x.masked_fill(upper, float("inf")), 0.125)
        assert torch.equal(y_poisoned, y)
        for poison_g, poison_y in ((float("nan"), float("nan")), (float("inf"), 0.0), (1.0, float("-inf"))):
            got = causal_ext.backward(g.masked_fill(upper, poison_g), y.masked_fill(upper, poison_y), 0.125)
            assert torch.equal(got, dx), (s, dtype, poison_g, poison_y)


@pytest.mark.parametrize("s", [520, 1032, 2056, 4104, 8200])
def test_nothing_is_written_past_the_end_of_the_output(device, s):
    # rows that do not fill the last chunk of their waves: lanes past the row end must
    # store nothing, neither into the next row nor behind the tensor
    lib = _lib.lib()
    stream = torch.cuda.current_stream().cuda_stream
    n = 2 * s * s
    x = scores((2, s, s), torch.float16, device, s)
    g = normal((2, s, s), torch.float16, device, s + 1)
    guard = 4096
    for kind in ("causal", "masked"):
        out = torch.full((n + guard,), 7.0, dtype=torch.float16, device=device)
        dxo = torch.full((n + guard,), 7.0, dtype=torch.float16, device=device)
        if kind == "causal":
            _lib.check(lib.neox_causal_softmax_fwd(out.data_ptr(), x.data_ptr(), 0.125, 2, s, s, _lib.NEOX_F16, stream))
            _lib.check(lib.neox_causal_softmax_bwd(dxo.data_ptr(), g.data_ptr(), out.data_ptr(), 0.125, 2, s, s,
                                                   _lib.NEOX_F16, stream))
            want = causal_ext.forward(x, 0.125)
        else:
            mask = torch.zeros(1, 1, s, s, dtype=torch.bool, device=device)
            _lib.check(lib.neox_masked_softmax_fwd(out.data_ptr(), x.data_ptr(), mask.data_ptr(), 0.125, 1, 2, s, s,
                                                   1, _lib.NEOX_F16, stream))
            _lib.check(lib.neox_masked_softmax_bwd(dxo.data_ptr(), g.data_ptr(), out.data_ptr(), 0.125, 2 * s, s,
                                                   _lib.NEOX_F16, stream))
            want = masked_ext.forward(x.view(1, 2, s, s), mask, 0.125)
        assert torch.equal(out[:n].view(2, s, s), want.view(2, s, s))
        assert (out[n:] == 7.0).all() and (dxo[n:] == 7.0).all(), kind


@pytest.mark.parametrize("dtype", DTYPES)
def test_short_rows_packed_several_per_wave(device, dtype):
    # sk <= 512 packs 64/G rows into a wave (G lanes per row): row counts that do not fill the
    # last wave / block, fully masked rows inside a packed wave, per-sample masks, in-place
    for batches, s in ((1, 8), (5, 8), (7, 16), (3, 24), (9, 40), (2, 136), (3, 264), (1, 512)):
        check_causal(device, batches, s, dtype, 0.3, seed=batches * 1000 + s)
    b, heads, sq, sk = 3, 2, 21, 48
    pattern = torch.rand(b, 1, sq, sk, device=device, generator=gen(device, 3)) < 0.4
    pattern[1, 0, 5, :] = True
    pattern[2, 0, 20, :] = True
    x, mask, y, g, dx = check_masked(device, b, heads, sq, sk, dtype, 0.2, 9, mask=pattern)
    assert torch.allclose(y[1, :, 5, :].float(), torch.full((heads, sk), 1.0 / sk, device=device), atol=2e-4)
    check_masked(device, b, heads, sq, sk, dtype, 0.2, 10, mask=pattern[:1].contiguous())
    x2 = x.clone()
    _lib.check(_lib.lib().neox_masked_softmax_fwd(x2.data_ptr(), x2.data_ptr(), mask.data_ptr(), 0.2, b, heads,
                                                  sq, sk, b, _lib.dtype_code(dtype),
                                                  torch.cuda.current_stream().cuda_stream))
    assert torch.equal(x2, y)


def test_seeded_random_shapes_around_every_dispatch_boundary(device):
    # row lengths next to each kernel-shape boundary (8 lanes-per-row steps, 512, 1024, 2048,
    # 4096, 8192) and odd row counts, both storage types, both mask kinds, forward + backward
    import random

    rnd = random.Random(20240611)
    edges = [8, 16, 32, 64, 128, 256, 512, 1024, 2048, 4096, 8192]
    for case in range(40):
        edge = rnd.choice(edges)
        sk = max(8, edge + 8 * rnd.choice([-2, -1, 0, 0, 1, 2]))
        dtype = rnd.choice(DTYPES)
        scale = rnd.choice([0.125, 0.5, 1.0, 2.0])
        if rnd.random() < 0.5:
            batches = rnd.randint(1, 3) if sk <= 2064 else 1
            check_causal(device, batches, sk, dtype, scale, seed=case, chunk=1)
        else:
            b, heads = rnd.randint(1, 3), rnd.randint(1, 3)
            sq = rnd.randint(1, 70) if sk <= 1040 else rnd.randint(1, 9)
            mask = None
            if rnd.random() < 0.5:
                mb = rnd.choice([1, b])
                mask = torch.rand(mb, 1, sq, sk, device=device, generator=gen(device, case)) < rnd.random()
            check_masked(device, b, heads, sq, sk, dtype, scale, seed=case, mask=mask)


def test_causal_negative_and_large_scale(device):
    for scale in (-0.25, 4.0, 1.0):
        check_causal(device, 2, 96, torch.float16, scale, seed=3)


def test_causal_forward_in_place_alias(device):
    x = scores((2, 520, 520), torch.bfloat16, device, 9)
    want = causal_ext.forward(x, 0.125)
    ptr = x.data_ptr()
    lib = _lib.lib()
    _lib.check(lib.neox_causal_softmax_fwd(ptr, ptr, 0.125, 2, 520, 520, _lib.NEOX_BF16,
                                           torch.cuda.current_stream().cuda_stream))
    assert torch.equal(x, want)


def test_causal_backward_overwrites_contiguous_grad_like_the_reference(device):
    y = causal_ext.forward(scores((2, 64, 64), torch.float16, device, 1), 0.125)
    g = normal((2, 64, 64), torch.float16, device, 2)
    keep = g.clone()
    dx = causal_ext.backward(g, y, 0.125)
    assert dx.data_ptr() == g.data_ptr()
    g_t = keep.transpose(1, 2)  # non-contiguous: a copy is made, the argument survives
    dx2 = causal_ext.backward(g_t, y, 0.125)
    assert dx2.data_ptr() != g_t.data_ptr() and torch.equal(g_t, keep.transpose(1, 2))
    assert torch.equal(dx2, causal_ext.backward(g_t.contiguous(), y, 0.125))


def test_causal_other_stream(device):
    x = scores((4, 256, 256), torch.float16, device, 11)
    want = causal_ext.forward(x, 0.5)
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        got = causal_ext.forward(x, 0.5)
    side.synchronize()
    assert torch.equal(got, want)


def test_causal_autograd_function_and_module(device):
    for dtype, fp16, bf16 in ((torch.float16, True, False), (torch.bfloat16, False, True)):
        b, heads, s = 2, 3, 72
        x = scores((b, heads, s, s), dtype, device, 21)
        mask = R.get_attn_mask(s, device)
        fused = FusedScaleMaskSoftmax(fp16, bf16, SoftmaxFusionTypes.upper_triang,
                                      R.gpt2_attention_mask_func, True, 0.3)
        plain = FusedScaleMaskSoftmax(fp16, bf16, SoftmaxFusionTypes.none,
                                      R.gpt2_attention_mask_func, True, 0.3)
        xf = x.clone().requires_grad_(True)
        xp = x.clone().requires_grad_(True)
        yf, yp = fused(xf, mask), plain(xp, mask)
        assert yf.shape == (b, heads, s, s) and yf.dtype == dtype
        assert max_err(yf, yp) <= 2 * TOL[dtype]  # two roundings apart at most
        g = normal(yf.shape, dtype, device, 22)
        yf.backward(g.clone())
        yp.backward(g.clone())
        # the fused backward consumes the rounded probabilities, autograd the fp32 ones
        assert max_err(xf.grad, xp.grad) <= grad_bar(xp.grad, dtype)
        # scale None means 1.0
        f1 = FusedScaleMaskSoftmax(fp16, bf16, SoftmaxFusionTypes.upper_triang, None, True, None)
        assert torch.equal(f1(x, mask), ScaledUpperTriangMaskedSoftmax.apply(x.view(-1, s, s), 1.0).view_as(x))


def test_causal_module_honours_masks_that_are_not_plain_causal(device):
    # a sliding-window mask (megatron/utils.py:75-77) given to the causal-fusion module: the
    # result is what the torch path computes from that mask, at any length -- the reference's
    # causal kernel would ignore the window below 2048 and apply it (torch path) above
    for s, dtype, fp16, bf16 in ((40, torch.float16, True, False), (2560, torch.bfloat16, False, True)):
        x = scores((1, 2, s, s), dtype, device, 4)
        fused = FusedScaleMaskSoftmax(fp16, bf16, SoftmaxFusionTypes.upper_triang,
                                      R.gpt2_attention_mask_func, True, 0.25, causal_mask_check="verify")
        plain = R.get_attn_mask(s, device)
        window = R.get_attn_mask(s, device, sliding_window_width=3)
        assert fused.mask_is_plain_causal(plain) and not fused.mask_is_plain_causal(window)
        assert fused.mask_is_plain_causal(plain)  # remembered verdict
        assert fused.classify_mask(window) == 3  # (at 2560 columns the sliding-window kernel serves it)
        a, b = fused(x, plain), fused(x, window)
        assert max_err(a, R.softmax_fp32(x, plain, 0.25)) <= TOL[dtype]
        assert max_err(b, R.softmax_fp32(x, window, 0.25)) <= TOL[dtype]
        assert (b[window.expand_as(b)] == 0).all() and not torch.equal(a, b)
        # an in-place edit of a remembered mask is noticed
        plain[0, 0, s - 1, 0] = True
        assert not fused.mask_is_plain_causal(plain)
        assert max_err(fused(x, plain), R.softmax_fp32(x, plain, 0.25)) <= TOL[dtype]


@pytest.mark.parametrize("sk", [64, 128, 256, 512, 1024, 2048])
def test_xcd_aware_block_order_covers_every_row_once(device, sk):
    # Rows of 4096 / 2^k bytes: the kernels hand the 4 KiB pieces of the tensors to their blocks so
    # that block x of every group of 8 keeps to the pieces x, x + 8, ... (one XCD, one piece
    # residue).  Whatever the order, every row must be computed exactly once -- with a grid that
    # is not a multiple of 8 blocks, a last block that is only partly filled, and several matrices.
    dtype = torch.float16
    for batches, sq in ((3, 1000), (5, 333), (1, 77)):
        x = scores((batches, sq, sk), dtype, device, 7 + sk)
        g = normal((batches, sq, sk), dtype, device, 8 + sk)
        causal = torch.ones(sq, sk, dtype=torch.bool, device=device).triu_(1)
        y = causal_ext.forward(x, 0.25)
        assert max_err(y, R.softmax_fp32(x, causal, 0.25)) <= TOL[dtype]
        assert (y[:, causal] == 0).all()
        dx = causal_ext.backward(g.clone(), y, 0.25)
        assert max_err(dx, R.softmax_backward_fp32(g, y, 0.25)) <= TOL[dtype]
        lens = torch.randint(1, sk + 1, (batches,), device=device, generator=gen(device, sk))
        mask = R.padding_mask(lens, sq, sk, device)
        x4 = x.view(batches, 1, sq, sk).expand(batches, 2, sq, sk).contiguous()
        y4 = masked_ext.forward(x4, mask, 0.25)
        assert max_err(y4, R.softmax_fp32(x4, mask, 0.25)) <= TOL[dtype]
        assert (y4[mask.expand_as(y4)] == 0).all()
        g4 = g.view(batches, 1, sq, sk).expand(batches, 2, sq, sk).contiguous()
        dx4 = masked_ext.backward(g4.clone(), y4, 0.25)
        assert max_err(dx4, R.softmax_backward_fp32(g4, y4, 0.25)) <= TOL[dtype]


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("batches,sq,sk", [(3, 4096, 4096), (2, 8192, 8192), (5, 100, 4096), (2, 5000, 6144),
                                           (1, 9000, 8192), (3, 2052, 16384), (7, 8, 8192)])
def test_long_causal_rows_store_every_piece_exactly_once(device, dtype, batches, sq, sk):
    # rows of several KiB, most of them zeros above the diagonal, in matrices that are square, wide
    # and tall.  Outputs pre-filled with NaN: every element must have been written, the zeros
    # included; forward, backward and the two outputs of the dropout forward.
    lib = _lib.lib()
    stream = torch.cuda.current_stream().cuda_stream
    code = _lib.dtype_code(dtype)
    x = scores((batches, sq, sk), dtype, device, 13)
    g = normal((batches, sq, sk), dtype, device, 14)
    hidden = torch.ones(sq, sk, dtype=torch.bool, device=device).triu_(1)
    y = torch.full_like(x, float("nan"))
    _lib.check(lib.neox_causal_softmax_fwd(y.data_ptr(), x.data_ptr(), 0.125, batches, sq, sk, code, stream))
    assert not torch.isnan(y).any() and (y[:, hidden] == 0).all()
    for m in range(batches):
        assert max_err(y[m], R.softmax_fp32(x[m], hidden, 0.125)) <= TOL[dtype]
    dx = torch.full_like(x, float("nan"))
    _lib.check(lib.neox_causal_softmax_bwd(dx.data_ptr(), g.data_ptr(), y.data_ptr(), 0.125, batches, sq, sk, code, stream))
    assert not torch.isnan(dx).any() and (dx[:, hidden] == 0).all()
    for m in range(batches):
        assert max_err(dx[m], R.softmax_backward_fp32(g[m], y[m], 0.125)) <= TOL[dtype]
    y1, y2 = torch.full_like(x, float("nan")), torch.full_like(x, float("nan"))
    _lib.check(lib.neox_causal_softmax_dropout_fwd(y2.data_ptr(), y1.data_ptr(), x.data_ptr(), None, None, 0, 0.125, 0.25,
                                                   77, 8, None, batches, 1, sq, sk, code, stream))
    assert torch.equal(y1, y) and not torch.isnan(y2).any() and (y2[:, hidden] == 0).all()
    keep = rng_keep(y.numel(), 0.25, 77, 8, device).view(y.shape)
    assert torch.equal(y2, R.dropout_with_mask(y, keep, 0.25))
    # in place (the reference overwrites the gradient): the zero pieces are written, not left
    buf = g.clone()
    _lib.check(lib.neox_causal_softmax_bwd(buf.data_ptr(), buf.data_ptr(), y.data_ptr(), 0.125, batches, sq, sk, code, stream))
    assert torch.equal(buf, dx)


@pytest.mark.parametrize("shape,d_rot", [((37, 3, 16, 128), 32), ((37, 3, 16, 128), 128), ((129, 1, 24, 64), 64),
                                         ((50, 2, 8, 256), 64), ((9, 5, 32, 128), 32)])
def test_rotary_piece_order_covers_every_head_once(device, shape, d_rot):
    # dense q and k whose heads tile 4 KiB pieces take the XCD-aware kernel: unit counts that are
    # not a multiple of a block's 8 units or of a group of 8 blocks, in place and out of place
    s, b, h, hn = shape
    dtype = torch.bfloat16
    q, k = normal(shape, dtype, device, 3), normal(shape, dtype, device, 4)
    cos, sin = (t.to(device) for t in R.rotary_tables(d_rot, s + 5))
    want_q, want_k = R.partial_rotary(q.float(), k.float(), cos, sin, d_rot, offset=5)
    q1, k1 = q.clone(), k.clone()
    apply_rotary_pos_emb_(q1, k1, cos, sin, 5, d_rot)
    assert torch.equal(q1, want_q.to(dtype)) and torch.equal(k1, want_k.to(dtype))
    out = rope_ext.forward_cached(q, cos[5 : 5 + s], sin[5 : 5 + s], False)
    assert torch.equal(out, want_q.to(dtype))
    gq, gk = R.rotary_autograd_fp32(q[..., :d_rot], k[..., :d_rot], cos, sin, q[..., :d_rot], k[..., :d_rot], offset=5)
    back = rope_ext.backward_cached(q, cos[5 : 5 + s], sin[5 : 5 + s], False)
    assert torch.equal(back[..., :d_rot], gq.to(dtype)) and torch.equal(back[..., d_rot:], q[..., d_rot:])


def test_causal_mask_check_lazy_and_trust(device):
    # "lazy": no host synchronisation -- while the device-side comparison of a new mask is in
    # flight the mask-tensor kernel serves the call (right for any mask), afterwards the causal
    # kernel; "trust": the mask is never read, as in megatron/model/fused_softmax.py:173-179
    from gpt_neox_amd import fused_softmax as fs

    s, dtype = 520, torch.bfloat16
    x = scores((2, 3, s, s), dtype, device, 91)
    g = normal((2, 3, s, s), dtype, device, 92)
    mods = {m: FusedScaleMaskSoftmax(False, True, SoftmaxFusionTypes.upper_triang, R.gpt2_attention_mask_func,
                                     True, 0.25, causal_mask_check=m) for m in ("verify", "lazy", "trust")}
    plain = R.get_attn_mask(s, device)
    want = R.softmax_fp32(x, plain, 0.25)
    ref = mods["verify"](x, plain)
    assert max_err(ref, want) <= TOL[dtype]
    for fresh in (plain.clone(), plain.clone()):
        assert fs._causal_memo.lookup(fresh) is None
        first = mods["lazy"](x, fresh)  # verdict possibly still in flight
        torch.cuda.synchronize()
        assert fs._causal_memo.lookup(fresh) == "causal"  # arrived: read without a synchronisation
        assert fs._causal_memo.lookup(fresh.detach()) == "causal"
        second = mods["lazy"](x, fresh)
        assert torch.equal(first, ref) and torch.equal(second, ref)  # both kernels give the same bits
    window = R.get_attn_mask(s, device, sliding_window_width=5)
    for _ in range(2):
        out = mods["lazy"](x, window)
        assert max_err(out, R.softmax_fp32(x, window, 0.25)) <= TOL[dtype]
        torch.cuda.synchronize()
    assert fs._causal_memo.lookup(window) == 5
    # more new masks than the memo has result slots: an entry that never looked at its verdict
    # keeps the right one when its slot is handed on
    old = R.get_attn_mask(16, device, sliding_window_width=2)
    assert fs._causal_memo.is_plain_causal(old, wait=False) in (None, False)
    for n in range(300):
        fs._causal_memo.is_plain_causal(torch.zeros(1, 1, 4, 4, dtype=torch.bool, device=device).triu_(1) if n % 2
                                        else R.get_attn_mask(4, device), wait=False)
    assert fs._causal_memo.is_plain_causal(old, wait=True) is False
    # trust: the window mask is ignored, the plain triangle applied
    assert torch.equal(mods["trust"](x, window), ref)
    # gradients through the lazy module, first call (mask-tensor kernels) and later (causal kernels)
    dx_want = R.softmax_backward_fp32(g, ref, 0.25)
    for fresh in (plain.clone(), plain):
        xin = x.clone().requires_grad_(True)
        mods["lazy"](xin, fresh).backward(g.clone())
        assert max_err(xin.grad, dx_want) <= TOL[dtype]


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("shape", [(2, 4, 8), (1, 6, 40), (2, 3, 136), (1, 8, 520), (2, 2, 1000), (1, 4, 2048),
                                   (1, 2, 2568), (1, 2, 4104), (1, 3, 37)])
def test_alibi_folded_into_the_causal_kernel(device, shape, dtype):
    # scale * (x + alibi) evaluated in fp32, against the fp32 oracle; every kernel family
    # (packed, one/several waves per row, element-wise)
    b, heads, s = shape
    x = scores((b, heads, s, s), dtype, device, s)
    slopes = torch.tensor(R.alibi_slopes(heads), device=device)
    mask = R.get_attn_mask(s, device)
    want = R.softmax_fp32(x.float() + R.alibi_bias_fp32(slopes.cpu(), s, s).to(device), mask, 0.25)
    got = causal_ext.forward_alibi(x, slopes, 0.25)
    assert max_err(got, want) <= TOL[dtype]
    assert (got[mask.expand_as(got)] == 0).all()
    zero = causal_ext.forward_alibi(x, torch.zeros_like(slopes), 0.25)  # zero slopes: the plain kernel's result
    assert max_err(zero, causal_ext.forward(x.view(-1, s, s), 0.25).view_as(x)) <= 2.0 ** -8


def test_alibi_module_argument_and_gradient(device):
    from gpt_neox_amd.positional_embeddings import AliBi

    b, heads, s, dtype = 2, 4, 72, torch.bfloat16
    alibi = AliBi(heads, mp_size=1, mp_rank=0).to(device)
    mask = R.get_attn_mask(s, device)
    fused = FusedScaleMaskSoftmax(False, True, SoftmaxFusionTypes.upper_triang,
                                  R.gpt2_attention_mask_func, True, 0.5)
    x = scores((b, heads, s, s), dtype, device, 3)
    xf = x.clone().requires_grad_(True)
    y = fused(xf, mask, alibi_slopes=alibi.slopes)
    # fp32 oracle, forward and autograd backward
    xr = x.float().requires_grad_(True)
    bias = R.alibi_bias_fp32(alibi.slopes.cpu(), s, s).to(device)
    yr = torch.softmax(R.gpt2_attention_mask_func((xr + bias) * 0.5, mask), -1)
    assert max_err(y, yr) <= TOL[dtype]
    g = normal(y.shape, dtype, device, 4)
    y.backward(g.clone())
    yr.backward(g.float())
    assert max_err(xf.grad, xr.grad) <= grad_bar(xr.grad, dtype)
    # the reference's two-pass sequence (bias added in bf16) stays within bf16 noise of it
    two_pass = fused(alibi(x), mask)
    assert max_err(y, two_pass) <= 0.06
    # a sliding-window mask: the mask-tensor kernel with the slopes, the mask honoured
    window = R.get_attn_mask(s, device, sliding_window_width=5)
    yw = fused(x, window, alibi_slopes=alibi.slopes)
    assert max_err(yw, R.softmax_fp32(x.float() + bias, window, 0.5)) <= TOL[dtype]
    assert (yw[window.expand_as(yw)] == 0).all()


def test_causal_fusion_against_a_key_value_cache(device):
    # sq != sk: the reference's causal branch asserts; here the mask-tensor kernel serves the call
    # with the mask it is given, and a mask of another layout still goes to the torch branch
    fused = FusedScaleMaskSoftmax(True, False, SoftmaxFusionTypes.upper_triang,
                                  R.gpt2_attention_mask_func, True, None)
    x = scores((1, 2, 1, 33), torch.float16, device, 4)  # one new token, 33 keys
    mask = torch.zeros(1, 1, 1, 33, dtype=torch.bool, device=device)
    assert fused.is_kernel_available(mask, *x.shape)
    assert max_err(fused(x, mask), R.softmax_fp32(x, mask, None)) <= TOL[torch.float16]
    # prefill of 5 tokens after 28 cached ones: query i sees keys j <= 28 + i
    x = scores((2, 3, 5, 33), torch.float16, device, 5).requires_grad_(True)
    mask = (torch.arange(33, device=device)[None, :] > (28 + torch.arange(5, device=device))[:, None]).view(1, 1, 5, 33)
    y = fused(x, mask)
    ref = R.softmax_fp32(x.detach(), mask, None)
    assert max_err(y, ref) <= TOL[torch.float16] and (y[mask.expand_as(y)] == 0).all()
    g = normal(x.shape, torch.float16, device, 6)
    y.backward(g.clone())
    want = R.softmax_backward_fp32(g, y.detach(), None)
    assert max_err(x.grad, want) <= TOL[torch.float16] * max(1.0, want.abs().max().item())
    broadcast = torch.zeros(1, 1, 1, 1, dtype=torch.bool, device=device)  # not the kernel's layout
    assert not fused.is_kernel_available(broadcast, 2, 3, 5, 33)
    xd = x.detach()
    assert torch.equal(fused(xd, broadcast), R.forward_torch_softmax(xd, broadcast, None, True, False, True))


# ---------------------------------------------------------------------------------
# mask-tensor softmax
# ---------------------------------------------------------------------------------
def check_masked(device, b, heads, sq, sk, dtype, scale, seed, mask=None, lo=1, absolute=False):
    x = scores((b, heads, sq, sk), dtype, device, seed)
    g = normal((b, heads, sq, sk), dtype, device, seed + 1)
    if mask is None:
        lens = torch.randint(lo, sk + 1, (b,), device=device, generator=gen(device, seed + 2))
        mask = R.padding_mask(lens, sq, sk, device)
    y = masked_ext.forward(x, mask, scale)
    ref = R.softmax_fp32(x, mask.bool(), scale)
    assert max_err(y, ref) <= TOL[dtype], (b, heads, sq, sk, dtype)
    hidden = mask.bool().expand_as(y)
    full_rows = hidden.all(-1, keepdim=True).expand_as(y)
    assert (y[hidden & ~full_rows] == 0).all()
    dx = masked_ext.backward(g.clone(), y, scale)
    refb = R.softmax_backward_fp32(g, y, scale)
    assert max_err(dx, refb) <= TOL[dtype] * max(1.0, refb.abs().max().item())
    assert (dx[hidden & ~full_rows] == 0).all()
    # the bar itself: autograd of the unfused fp32 path from x.  Rows whose every key is
    # hidden are the one place where the two differ by design: autograd returns 0 there (every
    # score went through masked_fill_), the kernels -- like the reference's -- apply the softmax
    # gradient to the uniform row they emitted: dx = scale * (g - mean(g)) / sk.
    _, auto = R.softmax_autograd_fp32(x, mask.bool(), scale, g)
    assert_grad(dx.float().masked_fill(full_rows, 0.0), auto, dtype, (b, heads, sq, sk, dtype), absolute,
                y=y.float().masked_fill(full_rows, 0.0), g=g, scale=scale)
    if full_rows.any():
        assert (auto[full_rows] == 0).all()
        gf = g.float()
        uniform = scale * (gf - gf.mean(-1, keepdim=True)) / sk
        ulp = 2.0 ** -8 if dtype == torch.bfloat16 else 2.0 ** -11  # 1/sk is rounded to the storage type in y
        assert ((dx.float() - uniform).abs()[full_rows] <= TOL[dtype] + 2 * ulp * uniform.abs()[full_rows]).all()
    return x, mask, y, g, dx


MASKED_SHAPES = [(2, 3, 4, 1), (2, 2, 5, 37), (1, 2, 8, 8), (3, 5, 7, 8), (2, 3, 5, 16), (2, 2, 33, 24), (2, 2, 16, 64),
                 (3, 3, 50, 72), (2, 2, 31, 128), (2, 3, 17, 200), (2, 2, 65, 256), (1, 3, 129, 384), (2, 2, 9, 512), (3, 2, 9, 520),
                 (2, 2, 33, 1000), (2, 2, 8, 1024), (1, 2, 6, 2048), (1, 1, 4, 3072), (1, 2, 3, 4096),
                 (1, 1, 3, 8192), (1, 1, 2, 12000), (1, 1, 2, 20000), (1, 1, 2, 30000), (1, 1, 2, 40000), (1, 3, 1, 77),
                 (2, 2, 3, 32776), (1, 2, 2, 65536), (1, 1, 3, 81408), (1, 1, 2, 81416),
                 (1, 2, 3, 2560), (1, 2, 3, 4104), (1, 1, 3, 10240), (1, 1, 2, 13312), (1, 1, 2, 14344)]


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("shape", MASKED_SHAPES)
def test_masked_shapes(device, shape, dtype):
    check_masked(device, *shape, dtype, 0.125, seed=sum(shape))


def test_masked_broadcast_over_batch_and_arbitrary_pattern(device):
    b, heads, sq, sk = 3, 2, 24, 136
    pattern = torch.rand(1, 1, sq, sk, device=device, generator=gen(device, 5)) < 0.5
    pattern[0, 0, 3, :] = True  # fully masked row -> uniform 1/sk
    pattern[0, 0, 4, :] = False
    x, mask, y, g, dx = check_masked(device, b, heads, sq, sk, torch.float16, 0.2, 6, mask=pattern)
    assert torch.allclose(y[:, :, 3, :].float(), torch.full((b, heads, sk), 1.0 / sk, device=device), atol=1e-5)
    per_sample = torch.rand(b, 1, sq, sk, device=device, generator=gen(device, 7)) < 0.3
    check_masked(device, b, heads, sq, sk, torch.bfloat16, 0.2, 8, mask=per_sample)
    check_masked(device, b, heads, sq, sk, torch.bfloat16, 0.2, 8, mask=per_sample.to(torch.uint8) * 255)


def test_masked_autograd_function_and_module(device):
    b, heads, sq, sk = 2, 4, 48, 200
    dtype = torch.bfloat16
    x = scores((b, heads, sq, sk), dtype, device, 31)
    lens = torch.tensor([200, 77], device=device)
    mask = R.padding_mask(lens, sq, sk, device)
    fused = FusedScaleMaskSoftmax(False, True, SoftmaxFusionTypes.general, R.gpt2_attention_mask_func, True, 0.125)
    plain = FusedScaleMaskSoftmax(False, True, SoftmaxFusionTypes.none, R.gpt2_attention_mask_func, True, 0.125)
    xf, xp = x.clone().requires_grad_(True), x.clone().requires_grad_(True)
    yf, yp = fused(xf, mask), plain(xp, mask)
    assert max_err(yf, yp) <= 2 * TOL[dtype]
    g = normal(yf.shape, dtype, device, 32)
    yf.backward(g.clone())
    yp.backward(g.clone())
    assert max_err(xf.grad, xp.grad) <= grad_bar(xp.grad, dtype)
    assert torch.equal(ScaledMaskedSoftmax.apply(x, mask, 0.125), yf.detach())


def test_masked_non_contiguous_input_is_accepted(device):
    x = scores((2, 2, 64, 32), torch.float16, device, 1).transpose(2, 3)  # [2,2,32,64] strided
    mask = torch.zeros(2, 1, 32, 64, dtype=torch.bool, device=device)
    y = masked_ext.forward(x, mask, 1.0)
    assert max_err(y, R.softmax_fp32(x, mask, 1.0)) <= TOL[torch.float16]


def test_empty_tensors(device):
    assert causal_ext.forward(torch.empty(0, 8, 8, dtype=torch.float16, device=device), 1.0).shape == (0, 8, 8)
    m = torch.zeros(1, 1, 4, 8, dtype=torch.bool, device=device)
    assert masked_ext.forward(torch.empty(0, 2, 4, 8, dtype=torch.float16, device=device), m[:0], 1.0).numel() == 0


# ---------------------------------------------------------------------------------
# rotary
# ---------------------------------------------------------------------------------
def check_rotary(device, s, b, hq, hk, hn, d_rot, dtype, seed, offset=0, table_dtype=torch.float,
                 qkv_view=False):
    if qkv_view:  # q, k as slices of a fused [s, b, h, 3*hn] projection (hq == hk)
        qkv = normal((s, b, hq, 3 * hn), dtype, device, seed)
        q_full, k_full = qkv[..., :hn], qkv[..., hn : 2 * hn]
    else:
        q_full = normal((s, b, hq, hn), dtype, device, seed)
        k_full = normal((s, b, hk, hn), dtype, device, seed + 1)
    cos, sin = (t.to(device) for t in R.rotary_tables(d_rot, s + offset + 3, 10000, table_dtype))
    q, k = q_full[..., :d_rot], k_full[..., :d_rot]
    # leaves that keep the strides of the slices: the kernels see the strided views
    qr, kr = q.detach().requires_grad_(True), k.detach().requires_grad_(True)
    oq, ok = apply_rotary_pos_emb(qr, kr, cos, sin, offset)
    assert oq.dtype == dtype and oq.shape == q.shape and ok.shape == k.shape
    rq, rk = R.rotary_fp32(q, k, cos, sin, offset)
    assert torch.equal(oq, rq.to(dtype)) and torch.equal(ok, rk.to(dtype)), "forward not bit-equal"
    gq = normal(oq.shape, dtype, device, seed + 2)
    gk = normal(ok.shape, dtype, device, seed + 3)
    torch.autograd.backward([oq, ok], [gq, gk])
    dq, dk = R.rotary_autograd_fp32(q, k, cos, sin, gq, gk, offset)
    assert torch.equal(qr.grad, dq.to(dtype)) and torch.equal(kr.grad, dk.to(dtype)), "backward not bit-equal"
    # in place over whole heads: rotated span as above, remaining dims untouched
    q2, k2 = q_full.clone(), k_full.clone()
    r1, r2 = apply_rotary_pos_emb_(q2, k2, cos, sin, offset, d_rot)
    assert r1.data_ptr() == q2.data_ptr() and r2.data_ptr() == k2.data_ptr()
    assert torch.equal(q2[..., :d_rot], oq) and torch.equal(k2[..., :d_rot], ok)
    assert torch.equal(q2[..., d_rot:], q_full[..., d_rot:]) and torch.equal(k2[..., d_rot:], k_full[..., d_rot:])


ROTARY_CASES = [
    # s, b, hq, hk, hn, d_rot
    (16, 2, 4, 4, 64, 64), (16, 2, 4, 4, 128, 32), (9, 3, 5, 5, 96, 24), (7, 2, 3, 3, 80, 80),
    (5, 1, 2, 2, 16, 6), (33, 2, 8, 2, 128, 128), (12, 2, 6, 6, 96, 96), (4, 5, 3, 3, 256, 256),
    (1, 7, 9, 9, 64, 16), (300, 1, 1, 1, 8, 2), (64, 4, 32, 32, 128, 32), (6, 2, 4, 4, 64, 48),
]


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("case", ROTARY_CASES)
def test_rotary_cases(device, case, dtype):
    check_rotary(device, *case, dtype, seed=sum(case))


@pytest.mark.parametrize("dtype", DTYPES)
def test_rotary_offset_and_qkv_views(device, dtype):
    check_rotary(device, 20, 2, 4, 4, 64, 16, dtype, seed=1, offset=5)
    check_rotary(device, 20, 2, 4, 4, 64, 64, dtype, seed=2, offset=0, qkv_view=True)
    check_rotary(device, 11, 3, 4, 4, 128, 32, dtype, seed=3, offset=2, qkv_view=True)


@pytest.mark.parametrize("hn,d_rot,parts", [(48, 40, 2), (48, 24, 2), (48, 40, 3), (80, 20, 3), (80, 40, 2), (112, 28, 3),
                                            (96, 24, 3), (64, 40, 2)])
def test_rotary_in_place_on_q_and_k_interleaved_in_one_buffer(device, hn, d_rot, parts):
    # q and k as views into one [s, b, h, parts * hn] buffer: the kernels write a rotated span back
    # together with the rest of its 64- or 32-byte block, and that block must never reach into the
    # other tensor's span, which the same launch rewrites (48-dim heads with 40 rotated dims: the
    # 64-byte block of q's span end would cover the first 32 bytes of k)
    s, b, h, dtype = 33, 2, 8, torch.bfloat16
    for seed in range(3):
        buf = normal((s, b, h, parts * hn), dtype, device, 70 + seed)
        before = buf.clone()
        q, k = buf[..., :hn], buf[..., hn : 2 * hn]
        cos, sin = (t.to(device) for t in R.rotary_tables(d_rot, s + 1))
        want_q, want_k = R.partial_rotary(before[..., :hn].float(), before[..., hn : 2 * hn].float(), cos, sin, d_rot, offset=1)
        apply_rotary_pos_emb_(q, k, cos, sin, 1, d_rot)
        assert torch.equal(buf[..., :hn], want_q.to(dtype)) and torch.equal(buf[..., hn : 2 * hn], want_k.to(dtype))
        assert torch.equal(buf[..., 2 * hn :], before[..., 2 * hn :])


@pytest.mark.parametrize("dtype", DTYPES)
def test_rotary_half_precision_tables(device, dtype):
    # tables in the dtype of q (the model's usual setting): fp32 arithmetic on the table
    # values as stored, one rounding
    s, b, h, d = 24, 2, 4, 32
    q, k = normal((s, b, h, d), dtype, device, 1), normal((s, b, h, d), dtype, device, 2)
    emb = RotaryEmbedding(d, 64, precision=dtype)
    cos, sin = emb(q, seq_len=s)
    assert cos.device == q.device and cos.dtype == dtype
    oq, ok = apply_rotary_pos_emb_torch(q, k, cos, sin)
    rq, rk = R.rotary_fp32(q, k, cos, sin)
    assert torch.equal(oq, rq.to(dtype)) and torch.equal(ok, rk.to(dtype))
    # and within the bf16/fp16 noise of the all-half-precision torch expression
    tq, _ = R.apply_rotary_pos_emb(q, k, cos, sin)
    assert max_err(oq, tq) <= (0.05 if dtype == torch.bfloat16 else 0.01)
    assert emb(q, seq_len=s)[0].data_ptr() == cos.data_ptr()  # device copy is kept, not re-made


@pytest.mark.parametrize("d_rot", [64, 48, 24, 6])
def test_rotary_head_loop_split_over_blocks(device, d_rot):
    # few positions, many heads: the head loop of a position is split over blockIdx.z
    # (contiguous-span kernel for d_rot = 64, the per-pair kernel with 8/4/1-element slots otherwise)
    s, b, h, hn = 2, 1, 600, 64
    q, k = normal((s, b, h, hn), torch.float16, device, 1), normal((s, b, 77, hn), torch.float16, device, 2)
    cos, sin = (t.to(device) for t in R.rotary_tables(d_rot, s))
    oq, ok = apply_rotary_pos_emb(q[..., :d_rot], k[..., :d_rot], cos, sin)
    rq, rk = R.rotary_fp32(q[..., :d_rot], k[..., :d_rot], cos, sin)
    assert torch.equal(oq, rq.half()) and torch.equal(ok, rk.half())


@pytest.mark.parametrize("d_rot", [32, 24, 48])
def test_rotary_strided_batch_and_half_tables_on_every_kernel(device, d_rot):
    # [s, b, h, d] view of a [b, s, h, d] buffer (batch stride cannot be folded into the head
    # stride) with tables stored in the dtype of q
    s, b, h, hn = 10, 3, 4, 64
    for dtype in DTYPES:
        q = normal((b, s, h, hn), dtype, device, 1).transpose(0, 1)
        k = normal((b, s, h, hn), dtype, device, 2).transpose(0, 1)
        cos, sin = (t.to(device) for t in R.rotary_tables(d_rot, s + 2, 10000, dtype))
        oq, ok = apply_rotary_pos_emb(q[..., :d_rot], k[..., :d_rot], cos, sin, offset=2)
        rq, rk = R.rotary_fp32(q[..., :d_rot], k[..., :d_rot], cos, sin, offset=2)
        assert torch.equal(oq, rq.to(dtype)) and torch.equal(ok, rk.to(dtype))
        q2, k2 = q.clone(memory_format=torch.preserve_format), k.clone(memory_format=torch.preserve_format)
        apply_rotary_pos_emb_(q2, k2, cos, sin, 2, d_rot)
        assert torch.equal(q2[..., :d_rot], oq) and torch.equal(q2[..., d_rot:], q[..., d_rot:])


def test_rotary_non_collapsible_layout(device):
    # [s, b, h, d] view of a [b, s, h, d] buffer: stride_b != h * stride_h
    s, b, h, d = 10, 3, 4, 32
    base_q = normal((b, s, h, d), torch.bfloat16, device, 1)
    base_k = normal((b, s, h, d), torch.bfloat16, device, 2)
    q, k = base_q.transpose(0, 1), base_k.transpose(0, 1)
    cos, sin = (t.to(device) for t in R.rotary_tables(d, s))
    oq, ok = apply_rotary_pos_emb(q, k, cos, sin)
    rq, rk = R.rotary_fp32(q, k, cos, sin)
    assert torch.equal(oq, rq.bfloat16()) and torch.equal(ok, rk.bfloat16())


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("transpose", [False, True])
def test_fused_rope_extension_api(device, dtype, transpose):
    s, b, h, d, d2 = 12, 2, 3, 64, 16
    t = normal((s, b, h, d), dtype, device, 5)
    cos, sin = (x.to(device) for x in R.rotary_tables(d2, s))
    out = rope_ext.forward_cached(t, cos, sin, transpose)
    want, _ = R.partial_rotary(t.float(), t.float(), cos, sin, d2)
    assert out.shape == (s, b, h, d) and torch.equal(out, want.to(dtype))
    assert out.transpose(0, 1).is_contiguous() == transpose
    g = normal((s, b, h, d), dtype, device, 6)
    gin = rope_ext.backward_cached(g, cos, sin, transpose)
    dq, _ = R.rotary_autograd_fp32(t[..., :d2], t[..., :d2], cos, sin, g[..., :d2], g[..., :d2])
    assert torch.equal(gin[..., :d2], dq.to(dtype)) and torch.equal(gin[..., d2:], g[..., d2:])
    # angles given instead of tables
    freqs = torch.outer(torch.arange(s, device=device).float(),
                        1.0 / (10000 ** (torch.arange(0, d2, 2, device=device).float() / d2)))
    freqs = torch.cat((freqs, freqs), -1)[:, None, None, :]
    # (the kernel evaluates sincosf itself: two fp32 evaluations of cos/sin may differ in the last
    # bit, so the bar is 1 ulp of the storage type; tests/test_fused_rope_gpu.py covers this path)
    out2 = rope_ext.forward(t, freqs, transpose)
    w2, _ = R.partial_rotary(t.float(), t.float(), freqs.cos(), freqs.sin(), d2)
    ulp = 2.0 ** -10 if dtype == torch.float16 else 2.0 ** -7
    assert ((out2.float() - w2).abs() <= ulp * w2.abs() + 1e-6).all()
    assert torch.equal(out2[..., d2:], t[..., d2:])


def test_rotary_in_place_on_views_of_a_fused_qkv_buffer(device):
    # megatron/model/transformer.py:798-809 produces [sq, b, np, 3*hn] and splits it into q, k, v
    # views; rotating q and k in place must leave v and the pass-through dims untouched
    s, b, h, hn, d_rot = 48, 2, 6, 64, 16
    qkv = normal((s, b, h, 3 * hn), torch.float16, device, 77)
    before = qkv.clone()
    q, k, v = qkv[..., :hn], qkv[..., hn : 2 * hn], qkv[..., 2 * hn :]
    cos, sin = (t.to(device) for t in R.rotary_tables(d_rot, s))
    apply_rotary_pos_emb_(q, k, cos, sin, 0, d_rot)
    rq, rk = R.rotary_fp32(before[..., :d_rot], before[..., hn : hn + d_rot], cos, sin)
    assert torch.equal(qkv[..., :d_rot], rq.half()) and torch.equal(qkv[..., hn : hn + d_rot], rk.half())
    assert torch.equal(qkv[..., d_rot:hn], before[..., d_rot:hn])
    assert torch.equal(qkv[..., hn + d_rot : 2 * hn], before[..., hn + d_rot : 2 * hn])
    assert torch.equal(v, before[..., 2 * hn :])


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("rotary_ndims,offset", [(None, 0), (16, 0), (32, 3)])
def test_rotary_call_site_fusion_matches_slice_rotate_concatenate(device, dtype, rotary_ndims, offset):
    # the sequence of megatron/model/transformer.py:807-860 on a fused projection, against
    # one in-place launch; forward values and the gradient of the projection output
    s, b, h, hn = 24, 2, 4, 64
    d_rot = hn if rotary_ndims is None else rotary_ndims
    w = normal((s, b, h, 3 * hn), dtype, device, 11)
    cos, sin = (t.to(device) for t in R.rotary_tables(d_rot, s + offset))

    def reference(mixed):  # fp32 arithmetic, rounded once where the kernels round
        q, k, v = mixed[..., :hn], mixed[..., hn : 2 * hn], mixed[..., 2 * hn :]
        oq, ok = R.partial_rotary(q, k, cos, sin, d_rot, offset)
        return oq, ok, v

    wr = w.detach().float().requires_grad_(True)
    rq, rk, rv = reference(wr * 1.0)
    wf = w.detach().clone().requires_grad_(True)
    fq, fk, fv = apply_rotary_pos_emb_qkv_(wf * 1, cos, sin, offset, rotary_ndims)
    assert fq.shape == (s, b, h, hn) and fq.data_ptr() + 2 * hn == fk.data_ptr()  # views of one buffer
    assert torch.equal(fq, rq.to(dtype)) and torch.equal(fk, rk.to(dtype)) and torch.equal(fv, rv.to(dtype))
    gq, gk, gv = (normal((s, b, h, hn), dtype, device, 20 + i) for i in range(3))
    torch.autograd.backward([rq, rk, rv], [gq.float(), gk.float(), gv.float()])
    torch.autograd.backward([fq, fk, fv], [gq, gk, gv])
    assert torch.equal(wf.grad, wr.grad.to(dtype))
    with torch.no_grad():  # inference: same values, really in place
        buf = w.clone()
        q2, k2, v2 = apply_rotary_pos_emb_qkv_(buf, cos, sin, offset, rotary_ndims)
        assert q2.data_ptr() == buf.data_ptr() and torch.equal(q2, fq) and torch.equal(k2, fk)


def test_rotary_in_place_autograd(device):
    s, b, h, hn, d_rot = 16, 2, 3, 32, 16
    q0 = normal((s, b, h, hn), torch.bfloat16, device, 1)
    k0 = normal((s, b, h, hn), torch.bfloat16, device, 2)
    cos, sin = (t.to(device) for t in R.rotary_tables(d_rot, s))
    qa, ka = q0.clone().requires_grad_(True), k0.clone().requires_grad_(True)
    oq, ok = apply_rotary_pos_emb_(qa * 1, ka * 1, cos, sin, 0, d_rot)  # in place on non-leaf copies
    gq, gk = normal(oq.shape, torch.bfloat16, device, 3), normal(ok.shape, torch.bfloat16, device, 4)
    torch.autograd.backward([oq, ok], [gq, gk])
    dq, dk = R.rotary_autograd_fp32(q0[..., :d_rot], k0[..., :d_rot], cos, sin, gq[..., :d_rot], gk[..., :d_rot])
    assert torch.equal(qa.grad[..., :d_rot], dq.bfloat16()) and torch.equal(ka.grad[..., :d_rot], dk.bfloat16())
    assert torch.equal(qa.grad[..., d_rot:], gq[..., d_rot:]) and torch.equal(ka.grad[..., d_rot:], gk[..., d_rot:])


def test_entry_points_can_be_captured_in_a_hip_graph(device):
    # no allocation, no synchronisation inside the library: a captured sequence replays to the
    # same result as the eager one, also with other work between the replays
    lib = _lib.lib()
    B, n = 4, 520
    x = scores((B, n, n), torch.float16, device, 5)
    g = normal((B, n, n), torch.float16, device, 6)
    y, dx = torch.empty_like(x), torch.empty_like(x)
    q = normal((64, 2, 4, 64), torch.float16, device, 7)
    k = normal((64, 2, 4, 64), torch.float16, device, 8)
    oq, ok = torch.empty_like(q), torch.empty_like(k)
    cos, sin = (t.to(device).reshape(64, 64).contiguous() for t in R.rotary_tables(64, 64))

    def run():
        st = torch.cuda.current_stream().cuda_stream
        _lib.check(lib.neox_causal_softmax_fwd(y.data_ptr(), x.data_ptr(), 0.125, B, n, n, _lib.NEOX_F16, st))
        _lib.check(lib.neox_causal_softmax_bwd(dx.data_ptr(), g.data_ptr(), y.data_ptr(), 0.125, B, n, n,
                                               _lib.NEOX_F16, st))
        rope_ext.rope_launch(oq, ok, q, k, cos, sin, 64, 0, backward=False)

    run()
    torch.cuda.synchronize()
    want = [t.clone() for t in (y, dx, oq, ok)]
    graph = torch.cuda.CUDAGraph()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        run()  # warm-up on the capture stream
        side.synchronize()
        with torch.cuda.graph(graph, stream=side):
            run()
    for rep in range(3):
        for t in (y, dx, oq, ok):
            t.fill_(float(rep))  # eager work between the replays
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        for got, ref in zip((y, dx, oq, ok), want):
            assert torch.equal(got, ref), rep


def test_rotary_round_trip_property(device):
    # backward is the inverse rotation: bwd(fwd(x)) == x up to two roundings
    s, b, h, d = 128, 2, 8, 64
    q, k = normal((s, b, h, d), torch.float16, device, 1), normal((s, b, h, d), torch.float16, device, 2)
    cos, sin = (t.to(device).reshape(s, d) for t in R.rotary_tables(d, s))
    oq, ok = torch.empty_like(q), torch.empty_like(k)
    rope_ext.rope_launch(oq, ok, q, k, cos, sin, d, 0, backward=False)
    bq, bk = torch.empty_like(q), torch.empty_like(k)
    rope_ext.rope_launch(bq, bk, oq, ok, cos, sin, d, 0, backward=True)
    assert max_err(bq, q) <= 8e-3 and max_err(bk, k) <= 8e-3


# ---------------------------------------------------------------------------------
# the benchmark shapes at full size
# ---------------------------------------------------------------------------------
def test_config1_causal_fwd_125m(device):
    x, y, g, dx = check_causal(device, 48, 2048, torch.bfloat16, 0.125, seed=1234, absolute=True)
    sums = y.float().sum(-1)
    assert (sums - 1).abs().max().item() < 2e-2  # bf16-rounded rows still sum to ~1


def test_config2_padding_fwd_bwd(device):
    # backward: |dx - autograd of the fp32 torch path from x| <= 1e-3, absolute
    x, mask, y, g, dx = check_masked(device, 8, 16, 1024, 1024, torch.float16, 0.125, seed=1235, lo=256, absolute=True)
    assert (y.float().sum(-1) - 1).abs().max().item() < 5e-3
    assert dx.float().sum(-1).abs().max().item() < 5e-2  # rows of dx sum to 0


def test_config3_partial_rotary(device):
    check_rotary(device, 2048, 4, 32, 32, 128, 32, torch.bfloat16, seed=1236)


def test_config4_causal_20b(device):
    # backward: |dx - autograd of the fp32 torch path from x| <= 1e-3, absolute
    x, y, g, dx = check_causal(device, 64, 2048, torch.float16, 96**-0.5, seed=1237, absolute=True)
    assert dx.float().sum(-1).abs().max().item() < 5e-2


def test_config5_long_context(device):
    # backward: |dx - autograd of the fp32 torch path from x| <= 2e-3, absolute
    x, y, g, dx = check_causal(device, 32, 8192, torch.bfloat16, 128**-0.5, seed=1238, chunk=2, absolute=True)
    del x, g, dx
    assert (y.float().sum(-1) - 1).abs().max().item() < 3e-2
    del y
    torch.cuda.empty_cache()
    check_rotary(device, 8192, 1, 32, 32, 128, 128, torch.bfloat16, seed=1239)


def test_in_place_rotary_without_grad_is_still_seen_by_autograd(device):
    # q and k need no gradient, so the in-place rotation skips the autograd Function -- but another
    # op has saved q for its own backward pass: the write must bump q's version counter, so that
    # autograd refuses the stale tensor instead of computing a wrong gradient silently
    s, d = 16, 64
    q = normal((s, 1, 2, d), torch.float16, device, 1)
    k = normal((s, 1, 2, d), torch.float16, device, 2)
    cos, sin = (t.to(device) for t in R.rotary_tables(d, s))
    w = torch.ones(d, dtype=torch.float16, device=device, requires_grad=True)
    out = q * w  # saves q for dw
    before = q._version
    apply_rotary_pos_emb_(q, k, cos, sin)
    assert q._version > before and k._version > 0
    with pytest.raises(RuntimeError, match="modified by an inplace operation"):
        out.sum().backward()
    mixed = normal((s, 1, 2, 3 * d), torch.float16, device, 3)
    out = mixed * 2.0 * w.repeat(3)
    before = mixed._version
    apply_rotary_pos_emb_qkv_(mixed, cos, sin)
    assert mixed._version > before


# ---------------------------------------------------------------------------------
# additive bias tensor (relative-position bias) read inside the softmax kernels
# ---------------------------------------------------------------------------------
from gpt_neox_amd.fused_softmax import ScaledMaskedSoftmaxBias, ScaledUpperTriangMaskedSoftmaxBias  # noqa: E402

BIAS_SHAPES = [(2, 3, 8, 8), (3, 2, 40, 40), (2, 2, 136, 136), (2, 3, 512, 512), (2, 2, 1024, 1024),
               (2, 1, 2048, 2048), (1, 2, 4096, 4096), (2, 2, 37, 37), (1, 2, 1001, 1001)]


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("shared", [True, False])
@pytest.mark.parametrize("shape", BIAS_SHAPES)
def test_causal_softmax_with_bias_tensor(device, shape, shared, dtype):
    b, np_, s, _ = shape
    x = scores(shape, dtype, device, 70)
    bias = scores((1 if shared else b, np_, s, s), dtype, device, 71) * 0.25
    y = causal_ext.forward_bias(x, bias, 0.125)
    mask = R.get_attn_mask(s, device)
    ref = R.softmax_fp32(x.float() + bias.float(), mask, 0.125)
    assert max_err(y, ref) <= TOL[dtype]
    assert (y[mask.expand(shape)] == 0).all()
    # a zero bias is the plain kernel, bit for bit
    assert torch.equal(causal_ext.forward_bias(x, torch.zeros_like(bias), 0.125),
                       causal_ext.forward(x.view(-1, s, s), 0.125).view(shape))


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("shared", [True, False])
@pytest.mark.parametrize("shape", [(2, 3, 5, 8), (2, 2, 9, 40), (1, 3, 16, 136), (2, 2, 8, 512), (2, 2, 16, 1024),
                                   (1, 2, 8, 2048), (2, 1, 4, 4096), (2, 2, 5, 37), (1, 2, 3, 1001)])
def test_masked_softmax_with_bias_tensor(device, shape, shared, dtype):
    b, np_, sq, sk = shape
    x = scores(shape, dtype, device, 72)
    bias = scores((1 if shared else b, np_, sq, sk), dtype, device, 73) * 0.25
    lengths = torch.randint(1, sk + 1, (b,), generator=gen(device, 74), device=device)
    mask = R.padding_mask(lengths, sq, sk, device)
    y = masked_ext.forward_bias(x, mask, bias, 0.5)
    ref = R.softmax_fp32(x.float() + bias.float(), mask, 0.5)
    assert max_err(y, ref) <= TOL[dtype]
    assert (y[mask.expand(shape)] == 0).all()
    assert torch.equal(masked_ext.forward_bias(x, mask, torch.zeros_like(bias), 0.5),
                       masked_ext.forward(x, mask, 0.5))


def test_bias_argument_checks(device):
    x = scores((2, 3, 16, 16), torch.float16, device, 75)
    with pytest.raises(RuntimeError, match="bias must have shape"):
        causal_ext.forward_bias(x, x[:, :2], 1.0)
    with pytest.raises(RuntimeError, match="bias must have shape"):
        causal_ext.forward_bias(x, x[0], 1.0)
    # other dtypes and layouts are converted: the result is that of the converted bias
    bias = scores((1, 3, 16, 16), torch.float32, device, 76)
    permuted = bias.permute(0, 2, 3, 1).contiguous().permute(0, 3, 1, 2)  # the layout movedim(2, 0) leaves
    assert not permuted.is_contiguous()
    assert torch.equal(causal_ext.forward_bias(x, permuted, 1.0), causal_ext.forward_bias(x, bias.half(), 1.0))


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("shared", [True, False])
def test_bias_functions_gradients(device, shared, dtype):
    b, np_, s = 3, 2, 64
    shape = (b, np_, s, s)
    x = scores(shape, dtype, device, 77).requires_grad_(True)
    bias = (scores((1 if shared else b, np_, s, s), dtype, device, 78) * 0.25).requires_grad_(True)
    g = normal(shape, dtype, device, 79)
    causal = R.get_attn_mask(s, device)
    pad = R.padding_mask(torch.tensor([40, 64, 9]), s, s, device)
    for fn, mask in ((lambda: ScaledUpperTriangMaskedSoftmaxBias.apply(x, bias, 0.5), causal),
                     (lambda: ScaledMaskedSoftmaxBias.apply(x, pad, bias, 0.5), pad)):
        x.grad = bias.grad = None
        y = fn()
        y.backward(g.clone())
        xr = x.detach().float().requires_grad_(True)
        br = bias.detach().float().requires_grad_(True)
        R.softmax_fp32(xr + br, mask, 0.5).backward(g.float())
        scale = max(1.0, xr.grad.abs().max().item())
        assert max_err(x.grad, xr.grad) <= 4 * TOL[dtype] * scale
        assert bias.grad.shape == bias.shape
        assert max_err(bias.grad, br.grad) <= 4 * TOL[dtype] * max(1.0, br.grad.abs().max().item()) * (b if shared else 1)
    # no bias gradient is formed when the bias does not ask for one
    x.grad = None
    fixed = bias.detach()
    ScaledUpperTriangMaskedSoftmaxBias.apply(x, fixed, 0.5).backward(g.clone())
    assert fixed.grad is None and x.grad is not None


def test_module_bias_argument(device):
    b, np_, s = 2, 4, 128
    x = scores((b, np_, s, s), torch.bfloat16, device, 80)
    rpe = (scores((s, s, np_), torch.bfloat16, device, 81) * 0.25).movedim(2, 0).unsqueeze(0)  # [1, np, s, s] view
    causal = R.get_attn_mask(s, device)
    m = FusedScaleMaskSoftmax(False, True, SoftmaxFusionTypes.upper_triang, R.gpt2_attention_mask_func, True, 0.5)
    y = m(x, causal, bias=rpe)
    ref = R.softmax_fp32(x.float() + rpe.float(), causal, 0.5)
    assert max_err(y, ref) <= TOL[torch.bfloat16]
    # the reference's two passes round x + rpe to bf16 first: close, not identical
    two_pass = m(x + rpe, causal)
    assert max_err(y, two_pass) <= 0.1
    assert max_err(two_pass, ref) >= max_err(y, ref)
    # sliding-window mask, general fusion and the unfused module give the same function
    window = R.get_attn_mask(s, device, sliding_window_width=16)
    assert max_err(m(x, window, bias=rpe), R.softmax_fp32(x.float() + rpe.float(), window, 0.5)) <= TOL[torch.bfloat16]
    mg = FusedScaleMaskSoftmax(False, True, SoftmaxFusionTypes.general, R.gpt2_attention_mask_func, True, 0.5)
    pad = R.padding_mask(torch.tensor([100, 128]), s, s, device)
    assert max_err(mg(x, pad, bias=rpe), R.softmax_fp32(x.float() + rpe.float(), pad, 0.5)) <= TOL[torch.bfloat16]
    mt = FusedScaleMaskSoftmax(False, True, SoftmaxFusionTypes.none, R.gpt2_attention_mask_func, True, 0.5)
    assert torch.equal(mt(x, causal, bias=rpe), mt(x + rpe, causal))
    # bias and dropout together, in one kernel: the same probabilities, dropped as torch drops them
    out = m(x, causal, bias=rpe, dropout_p=0.5)
    assert torch.equal(out, R.dropout_with_mask(y, out != 0, 0.5))


# ---------------------------------------------------------------------------------
# in-place partial rotary whose span ends inside a 64-byte block (head sizes of real models)
# ---------------------------------------------------------------------------------
@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("hn,d_rot,qkv", [(96, 24, False), (96, 24, True), (64, 16, False), (64, 16, True),
                                          (80, 20, False), (256, 64, False), (48, 24, False), (24, 24, False),
                                          (96, 48, True), (160, 40, False)])
def test_in_place_partial_rotary_keeps_pass_through_bits(device, hn, d_rot, qkv, dtype):
    s, b, h = 33, 2, 5
    width = 3 * hn if qkv else hn
    base = normal((s, b, h, width), dtype, device, 90)
    # pass-through dims hold every kind of bit pattern: they must come back bit for bit
    special = torch.tensor([float("nan"), float("inf"), -float("inf"), -0.0, 65504.0, 6e-8], device=device).to(dtype)
    bits = base.view(torch.int16).clone()
    fill = special.view(torch.int16).repeat((width + 5) // 6)[:width]
    passthrough = torch.ones(width, dtype=torch.bool, device=device)
    for start in ((0, hn) if qkv else (0,)):
        passthrough[start:start + d_rot] = False
    bits[..., passthrough] = fill[passthrough]
    x = bits.view(dtype)
    cos, sin = (t.to(device) for t in R.rotary_tables(d_rot, s + 3))
    q_ref, k_ref = x[..., :d_rot].float(), (x[..., hn:hn + d_rot] if qkv else x[..., :d_rot]).float()
    want_q, want_k = R.rotary_fp32(q_ref, k_ref, cos, sin, offset=3)
    work = x.clone()
    if qkv:
        q, k, v = apply_rotary_pos_emb_qkv_(work, cos, sin, offset=3, rotary_ndims=d_rot)
    else:
        other = x.clone()
        q, k = apply_rotary_pos_emb_(work, other, cos, sin, offset=3, rotary_ndims=d_rot)
        assert torch.equal(other.view(torch.int16)[..., d_rot:], bits[..., d_rot:])
    assert torch.equal(q[..., :d_rot], want_q.to(dtype)) and torch.equal(k[..., :d_rot], want_k.to(dtype))
    assert torch.equal(work.view(torch.int16)[..., passthrough], bits[..., passthrough])


def test_seeded_random_rotary_layouts(device):
    """Random head sizes, rotary widths, head counts (q and k differ), batch layouts that can and
    cannot be collapsed, table dtypes, offsets, in place and out of place: every kernel shape the
    launcher can pick, each bit-equal to the fp32 expression rounded once."""
    rs = np.random.RandomState(2024)
    for case in range(80):
        dtype = DTYPES[case % 2]
        d_rot = int(rs.choice([2, 4, 6, 8, 12, 16, 20, 24, 32, 40, 48, 64, 72, 80, 96, 128, 160, 256, 512]))
        extra = int(rs.choice([0, 0, 8, 16, 24, 2, 96]))
        hn = d_rot + extra
        s, b = int(rs.randint(1, 9)), int(rs.randint(1, 4))
        h_q, h_k = int(rs.randint(1, 9)), int(rs.randint(1, 9))
        offset = int(rs.randint(0, 5))
        pad_b = int(rs.choice([0, 0, 8, 3]))  # extra elements between batch entries: (b, h) no longer collapse
        in_place = bool(rs.randint(0, 2))
        half_tables = bool(rs.randint(0, 2))

        def make(h, seed):
            buf = normal((s, b, h * hn + pad_b), dtype, device, seed)
            return buf[..., : h * hn].view(s, b, h, hn)

        q, k = make(h_q, 1000 + case), make(h_k, 2000 + case)
        cos, sin = (t.to(device) for t in R.rotary_tables(d_rot, s + offset))
        if half_tables:
            cos, sin = cos.to(dtype), sin.to(dtype)
        want_q, want_k = R.rotary_fp32(q[..., :d_rot], k[..., :d_rot], cos, sin, offset=offset)
        tag = (case, dtype, d_rot, hn, s, b, h_q, h_k, offset, pad_b, in_place, half_tables)
        if in_place:
            q0, k0 = q.clone(), k.clone()  # clones are dense: a second layout for the same data
            for qq, kk in ((q, k), (q0, k0)):
                keep_q, keep_k = qq[..., d_rot:].clone(), kk[..., d_rot:].clone()
                oq, ok = apply_rotary_pos_emb_(qq, kk, cos, sin, offset=offset, rotary_ndims=d_rot)
                assert torch.equal(oq[..., :d_rot], want_q.to(dtype)) and torch.equal(ok[..., :d_rot], want_k.to(dtype)), tag
                assert torch.equal(oq[..., d_rot:], keep_q) and torch.equal(ok[..., d_rot:], keep_k), tag
                if h_q != h_k:
                    break  # one layout is enough for the rarer case
        else:
            oq, ok = apply_rotary_pos_emb(q[..., :d_rot], k[..., :d_rot], cos, sin, offset=offset)
            assert torch.equal(oq, want_q.to(dtype)) and torch.equal(ok, want_k.to(dtype)), tag


# ---------------------------------------------------------------------------------
# rows beyond the register budget: staged in LDS
# ---------------------------------------------------------------------------------
@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("scale", [0.5, -0.25])
@pytest.mark.parametrize("sk", [33280, 50008])  # staged in half of a CU's LDS / in all of it
def test_lds_staged_rows_masks_scales_and_aliasing(device, dtype, scale, sk):
    b, heads, sq = 2, 2, 3
    x = scores((b, heads, sq, sk), dtype, device, 91)
    g = normal((b, heads, sq, sk), dtype, device, 92)
    mask = torch.rand(b, 1, sq, sk, device=device, generator=gen(device, 93)) < 0.3  # arbitrary pattern
    mask[0, 0, 1, :] = True        # a row with every key hidden: uniform 1/sk
    mask[1, 0, 2, 100:] = True     # a row that ends early
    y = masked_ext.forward(x, mask, scale)
    ref = R.softmax_fp32(x, mask, scale)
    assert max_err(y, ref) <= TOL[dtype]
    hidden = mask.expand_as(y).clone()
    hidden[0, :, 1, :] = False
    assert (y[hidden] == 0).all()
    assert torch.allclose(y[0, :, 1, :].float(), torch.full((heads, sk), 1.0 / sk, device=device), rtol=1e-2)
    dx = masked_ext.backward(g.clone(), y, scale)
    refb = R.softmax_backward_fp32(g, y, scale)
    assert max_err(dx, refb) <= TOL[dtype] * max(1.0, refb.abs().max().item())
    buf = g.clone()  # in place on the gradient buffer
    assert masked_ext.backward(buf, y, scale).data_ptr() == buf.data_ptr() and torch.equal(buf, dx)
    # the mask shared by all samples
    y1 = masked_ext.forward(x, mask[:1], scale)
    assert max_err(y1, R.softmax_fp32(x, mask[:1], scale)) <= TOL[dtype]


# ---------------------------------------------------------------------------------
# ragged rows: sk not a multiple of 8, tensors at any 2-byte alignment
# ---------------------------------------------------------------------------------
RAGGED_CAUSAL = [9, 15, 17, 33, 63, 65, 127, 129, 255, 511, 513, 1001, 1023, 1025, 1537, 2047, 2049, 3001, 4095, 4097,
                 5003, 8191, 10001, 20003, 32767]


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("s", RAGGED_CAUSAL)
def test_ragged_causal_sizes(device, s, dtype):
    # three matrices: rows start at every 2-byte alignment, row lengths of both parities
    check_causal(device, 3 if s <= 2049 else 1, s, dtype, 0.125, seed=s, chunk=1)


RAGGED_MASKED = [(2, 3, 5, 9), (2, 2, 7, 33), (3, 2, 9, 129), (2, 2, 6, 250), (2, 3, 5, 515), (2, 2, 5, 1001), (1, 2, 3, 2047),
                 (2, 2, 3, 2050), (1, 2, 3, 4099), (1, 1, 3, 9001), (1, 1, 3, 16388), (1, 1, 2, 32767)]


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("shape", RAGGED_MASKED)
def test_ragged_masked_shapes(device, shape, dtype):
    b, heads, sq, sk = shape
    check_masked(device, b, heads, sq, sk, dtype, 0.125, seed=sum(shape))
    # an arbitrary pattern, and the last one to three keys of a row hidden or alone visible: the
    # mask bytes next to the row end travel by an access of their own
    pattern = torch.rand(b, 1, sq, sk, device=device, generator=gen(device, sk)) < 0.4
    for i in range(sq):
        tail = 1 + i % 3
        pattern[0, 0, i, :] = False
        pattern[0, 0, i, sk - tail:] = True
        if b > 1:
            pattern[1, 0, i, :] = True
            pattern[1, 0, i, sk - tail:] = False
    check_masked(device, b, heads, sq, sk, dtype, 0.5, seed=sk, mask=pattern)
    check_masked(device, b, heads, sq, sk, dtype, 0.5, seed=sk, mask=pattern[:1])


@pytest.mark.parametrize("offset", [1, 2, 3, 4, 7])
@pytest.mark.parametrize("sk", [16, 512, 1000, 1001, 2048, 4099])
def test_tensors_at_any_two_byte_alignment(device, sk, offset):
    # every tensor of the call starts `offset` elements into its allocation (the mask `offset` bytes)
    dtype, b, heads, sq, scale = torch.float16, 2, 2, 5, 0.25

    def shifted(t):
        flat = torch.empty(t.numel() + offset, dtype=t.dtype, device=device)
        flat[offset:] = t.reshape(-1)
        return flat[offset:].view(t.shape)

    x = scores((b, heads, sq, sk), dtype, device, sk)
    g = normal((b, heads, sq, sk), dtype, device, sk + 1)
    mask = torch.rand(b, 1, sq, sk, device=device, generator=gen(device, sk + 2)) < 0.3
    xs, gs, ms = shifted(x), shifted(g), shifted(mask)
    assert xs.data_ptr() % 16 == (2 * offset) % 16 and xs.is_contiguous()
    y = masked_ext.forward(xs, ms, scale)
    assert max_err(y, R.softmax_fp32(x, mask, scale)) <= TOL[dtype]
    assert (y[mask.expand_as(y)] == 0).all()
    ys = shifted(y)
    dx = masked_ext.backward(gs, ys, scale)
    assert dx.data_ptr() == gs.data_ptr()
    assert max_err(dx, R.softmax_backward_fp32(g, y, scale)) <= TOL[dtype]
    # causal, square
    n = min(sk, 1001)
    xc = scores((3, n, n), dtype, device, sk + 3)
    yc = causal_ext.forward(shifted(xc), scale)
    assert max_err(yc.unsqueeze(0), R.softmax_fp32(xc.unsqueeze(0), R.get_attn_mask(n, device), scale)) <= TOL[dtype]
    gc = normal((3, n, n), dtype, device, sk + 4)
    dxc = causal_ext.backward(shifted(gc), shifted(yc), scale)
    assert max_err(dxc, R.softmax_backward_fp32(gc, yc, scale)) <= TOL[dtype]


@pytest.mark.parametrize("sk", [9, 515, 1001, 2047, 4099, 9001])
def test_ragged_rows_write_exactly_their_output(device, sk):
    # outputs surrounded by guard elements, every element of the output pre-set: the kernels
    # write each element of the rows (zeros above the diagonal included) and nothing else
    lib = _lib.lib()
    stream = torch.cuda.current_stream().cuda_stream
    guard = 64
    for dtype in DTYPES:
        code = _lib.dtype_code(dtype)
        for kind in ("causal", "masked"):
            rows_shape = (2, sk, sk) if kind == "causal" and sk <= 2047 else (2, 1, 5, sk)
            causal = len(rows_shape) == 3
            x = scores(rows_shape, dtype, device, sk)
            g = normal(rows_shape, dtype, device, sk + 1)
            n = x.numel()
            for pad in (guard, guard + 1, guard + 3):  # output base at different alignments
                out = torch.full((n + 2 * guard + 8,), 7.0, dtype=dtype, device=device)
                dxo = torch.full((n + 2 * guard + 8,), 7.0, dtype=dtype, device=device)
                y, dx = out[pad : pad + n], dxo[pad : pad + n]
                if causal:
                    _lib.check(lib.neox_causal_softmax_fwd(y.data_ptr(), x.data_ptr(), 0.125, 2, sk, sk, code, stream))
                    want = R.softmax_fp32(x.unsqueeze(0), R.get_attn_mask(sk, device), 0.125)[0]
                    _lib.check(lib.neox_causal_softmax_bwd(dx.data_ptr(), g.data_ptr(), y.data_ptr(), 0.125, 2, sk, sk, code, stream))
                else:
                    mask = torch.rand(2, 1, 5, sk, device=device, generator=gen(device, sk)) < 0.3
                    _lib.check(lib.neox_masked_softmax_fwd(y.data_ptr(), x.data_ptr(), mask.data_ptr(), 0.125, 2, 1, 5, sk, 2, code, stream))
                    want = R.softmax_fp32(x, mask, 0.125)
                    _lib.check(lib.neox_masked_softmax_bwd(dx.data_ptr(), g.data_ptr(), y.data_ptr(), 0.125, 10, sk, code, stream))
                assert max_err(y.view(rows_shape), want) <= TOL[dtype], (sk, kind, pad)
                wantb = R.softmax_backward_fp32(g, y.view(rows_shape), 0.125)
                assert max_err(dx.view(rows_shape), wantb) <= TOL[dtype], (sk, kind, pad)
                for buf in (out, dxo):
                    assert (buf[:pad] == 7.0).all() and (buf[pad + n:] == 7.0).all(), (sk, kind, pad)


@pytest.mark.parametrize("s", [9, 513, 1001, 2047, 4099])
def test_ragged_causal_kernels_ignore_what_lies_past_the_diagonal(device, s):
    upper = torch.ones(s, s, dtype=torch.bool, device=device).triu_(1)
    for dtype in DTYPES:
        x = scores((2, s, s), dtype, device, s)
        g = normal((2, s, s), dtype, device, s + 1)
        y = causal_ext.forward(x, 0.125)
        dx = causal_ext.backward(g.clone(), y, 0.125)
        assert torch.equal(causal_ext.forward(x.masked_fill(upper, float("nan")), 0.125), y)
        for poison_g, poison_y in ((float("nan"), float("nan")), (float("inf"), 0.0), (1.0, float("-inf"))):
            got = causal_ext.backward(g.masked_fill(upper, poison_g), y.masked_fill(upper, poison_y), 0.125)
            assert torch.equal(got, dx), (s, dtype, poison_g, poison_y)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("shape", [(2, 3, 9, 9), (2, 2, 65, 65), (1, 3, 513, 513), (2, 2, 1001, 1001), (1, 2, 2047, 2047)])
def test_ragged_rows_with_alibi_and_bias(device, shape, dtype):
    b, heads, sq, sk = shape
    x = scores(shape, dtype, device, sk)
    slopes = torch.rand(heads, device=device, generator=gen(device, 3)) * 0.5
    causal = R.get_attn_mask(sk, device)
    y = causal_ext.forward_alibi(x, slopes, 0.25)
    bias = R.alibi_bias_fp32(slopes.cpu(), sq, sk).to(device)
    assert max_err(y, R.softmax_fp32(x.float() + bias, causal, 0.25)) <= TOL[dtype]
    for shared in (True, False):
        rpe = normal((1 if shared else b, heads, sq, sk), dtype, device, sk + 5)
        yb = causal_ext.forward_bias(x, rpe, 0.25)
        assert max_err(yb, R.softmax_fp32(x.float() + rpe.float(), causal, 0.25)) <= TOL[dtype]
        assert (yb[causal.expand_as(yb)] == 0).all()
        pad = torch.rand(b, 1, sq, sk, device=device, generator=gen(device, sk + 6)) < 0.3
        ym = masked_ext.forward_bias(x, pad, rpe, 0.25)
        assert max_err(ym, R.softmax_fp32(x.float() + rpe.float(), pad, 0.25)) <= TOL[dtype]


def test_ragged_short_rows_every_row_end_and_group_size(device):
    # rows of 8m + r columns, r = 1..7, for every lane-group size of the several-rows-per-wave
    # kernels: the lane at a row end moves its r columns in pieces of 4, 2 and 1
    for m in (1, 2, 3, 4, 8, 16, 32, 63):
        for r in range(1, 8):
            sk = 8 * m + r
            dtype = DTYPES[(m + r) % 2]
            check_causal(device, 3, sk, dtype, 0.25, seed=sk, chunk=3)
            mask = torch.rand(2, 1, 5, sk, device=device, generator=gen(device, sk)) < 0.3
            mask[0, 0, 1, :] = True                      # a row with every key hidden
            mask[1, 0, 2, :] = False
            mask[1, 0, 2, sk - r:] = True                # exactly the columns of the row-end lane hidden
            mask[1, 0, 3, :] = True
            mask[1, 0, 3, sk - r:] = False               # ... and those alone visible
            check_masked(device, 2, 3, 5, sk, dtype, 0.25, seed=sk, mask=mask)
            check_masked(device, 2, 3, 5, sk, dtype, 0.25, seed=sk, mask=mask[:1])


def test_module_through_a_generation_loop_at_arbitrary_lengths(device):
    # a prefill at an odd prompt length (causal kernel), then single-token steps against a growing
    # key/value cache (mask-tensor kernel): the fused module against its own unfused branch
    b, heads = 2, 4
    for dtype in DTYPES:
        fused = FusedScaleMaskSoftmax(dtype == torch.float16, dtype == torch.bfloat16, SoftmaxFusionTypes.upper_triang,
                                      R.gpt2_attention_mask_func, True, 0.125)
        plain = FusedScaleMaskSoftmax(dtype == torch.float16, dtype == torch.bfloat16, SoftmaxFusionTypes.none,
                                      R.gpt2_attention_mask_func, True, 0.125)
        for prompt in (37, 1001, 1537):
            full_mask = R.get_attn_mask(prompt + 6, device)
            x = scores((b, heads, prompt, prompt), dtype, device, prompt)
            mask = full_mask[..., :prompt, :prompt].contiguous()
            with torch.no_grad():
                assert max_err(fused(x, mask), plain(x.clone(), mask)) <= 2 * TOL[dtype]
                for t in range(prompt + 1, prompt + 6):
                    x = scores((b, heads, 1, t), dtype, device, t)
                    # the mask row of the one query, at position t - 1, against the t cached keys
                    step_mask = full_mask[..., t - 1, :t].unsqueeze(2).contiguous()
                    assert fused.is_kernel_available(step_mask, b, heads, 1, t)
                    y = fused(x, step_mask)
                    assert max_err(y, plain(x.clone(), step_mask)) <= 2 * TOL[dtype]
                    assert torch.allclose(y.float().sum(-1), torch.ones(b, heads, 1, device=device), atol=2e-2)


# ---------------------------------------------------------------------------------
# kernel variants the cases above do not reach
# ---------------------------------------------------------------------------------
@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("half_tables", [False, True])
@pytest.mark.parametrize("case", [
    # rotated spans of more than 64 slots of 8, 4 and 2 dims (the pair-in-lane kernel)
    (5, 2, 3, 3, 1024, 1024), (4, 2, 2, 2, 1028, 520), (4, 2, 2, 2, 134, 132),
    # spans of 8-, 4- and 2-dim slots (the span kernel), also backward with half-precision tables
    (16, 2, 4, 4, 64, 64), (9, 3, 5, 5, 96, 24), (4, 2, 3, 3, 20, 20),
])
def test_rotary_slot_widths_table_types_and_directions(device, case, half_tables, dtype):
    check_rotary(device, *case, dtype, seed=sum(case), table_dtype=dtype if half_tables else torch.float)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("s", [33000, 40968])  # staged in half of a CU's LDS / in all of it
def test_lds_staged_causal_rows_in_both_storage_types(device, dtype, s):
    x = scores((1, s, s), dtype, device, 7)
    y = causal_ext.forward(x, 0.05)
    rows = torch.tensor([0, 1, 700, s // 2, s - 1], device=device)
    mask = R.get_attn_mask(s, device)[0, 0][rows]
    assert max_err(y[0][rows], R.softmax_fp32(x[0][rows], mask, 0.05)) <= TOL[dtype]
    assert (y[0][rows][mask] == 0).all()
    g = normal((1, s, s), dtype, device, 8)
    dx = causal_ext.backward(g.clone(), y, 0.05)
    assert max_err(dx[0][rows], R.softmax_backward_fp32(g[0][rows], y[0][rows], 0.05)) <= TOL[dtype]


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("sk", [5, 33000])
def test_bias_tensor_on_very_short_and_very_long_rows(device, sk, dtype):
    # rows shorter than 8 columns (element-wise kernels), and rows beyond the register budget (staged in LDS)
    b, heads, sq = 2, 2, (sk if sk < 8 else 3)
    x = scores((b, heads, sq, sk), dtype, device, sk)
    rpe = normal((1, heads, sq, sk), dtype, device, sk + 1)
    pad = torch.rand(b, 1, sq, sk, device=device, generator=gen(device, sk + 2)) < 0.3
    pad[..., 0] = False
    y = masked_ext.forward_bias(x, pad, rpe, 0.25)
    assert max_err(y, R.softmax_fp32(x.float() + rpe.float(), pad, 0.25)) <= TOL[dtype]
    assert (y[pad.expand_as(y)] == 0).all()
    if sk < 8:
        causal = R.get_attn_mask(sk, device)
        yc = causal_ext.forward_bias(x, rpe, 0.25)
        assert max_err(yc, R.softmax_fp32(x.float() + rpe.float(), causal, 0.25)) <= TOL[dtype]


@pytest.mark.parametrize("offset", [1, 2, 4])
def test_one_lane_rows_at_any_alignment(device, offset):
    # sk = 8: one lane per row; the tensors start `offset` elements into their allocations
    dtype, b, heads, sq, sk = torch.bfloat16, 2, 3, 8, 8
    flat = torch.empty(b * heads * sq * sk + offset, dtype=dtype, device=device)
    flat[offset:] = scores((b, heads, sq, sk), dtype, device, offset).reshape(-1)
    x = flat[offset:].view(b, heads, sq, sk)
    mask = torch.rand(b, 1, sq, sk, device=device, generator=gen(device, offset)) < 0.3
    mask[..., 0] = False
    y = masked_ext.forward(x, mask, 0.5)
    assert max_err(y, R.softmax_fp32(x, mask, 0.5)) <= TOL[dtype]
    yc = causal_ext.forward(x.view(-1, sq, sk), 0.5)
    assert max_err(yc.view(x.shape), R.softmax_fp32(x, R.get_attn_mask(sk, device), 0.5)) <= TOL[dtype]
    gflat = torch.empty_like(flat)
    gflat[offset:] = normal((b, heads, sq, sk), dtype, device, offset + 1).reshape(-1)
    g = gflat[offset:].view(b, heads, sq, sk)
    want = R.softmax_backward_fp32(g, y, 0.5)
    assert max_err(masked_ext.backward(g, y, 0.5), want) <= TOL[dtype]
    # the same rows with a bias tensor, ALiBi slopes and dropout
    rpe = normal((1, heads, sq, sk), dtype, device, offset + 2)
    want_b = R.softmax_fp32(x.float() + rpe.float(), mask, 0.5)
    assert max_err(masked_ext.forward_bias(x, mask, rpe, 0.5), want_b) <= TOL[dtype]
    causal = R.get_attn_mask(sk, device)
    assert max_err(causal_ext.forward_bias(x, rpe, 0.5), R.softmax_fp32(x.float() + rpe.float(), causal, 0.5)) <= TOL[dtype]
    slopes = torch.tensor([0.5, 0.25, 0.125], device=device)
    want_a = R.softmax_fp32(x.float() + R.alibi_bias_fp32(slopes.cpu(), sq, sk).to(device), causal, 0.5)
    assert max_err(causal_ext.forward_alibi(x, slopes, 0.5), want_a) <= TOL[dtype]
    from gpt_neox_amd.fused_kernels import attention_dropout as rng
    for fwd, kw in ((lambda **k: masked_ext.forward_dropout(x, mask, 0.5, 0.25, 5, 8, **k), [{}, {"bias": rpe}]),
                    (lambda **k: causal_ext.forward_dropout(x, 0.5, 0.25, 5, 8, **k), [{}, {"bias": rpe}, {"slopes": slopes}])):
        for extra in kw:
            probs, dropped = fwd(**extra)
            keep = rng.keep_mask(probs.numel(), 0.25, 5, 8, device).view(probs.shape)
            assert torch.equal(dropped, R.dropout_with_mask(probs, keep, 0.25))
    probs, _ = masked_ext.forward_dropout(x, mask, 0.5, 0.25, 5, 8)
    keep = rng.keep_mask(probs.numel(), 0.25, 5, 8, device).view(probs.shape)
    want_d = R.softmax_dropout_backward_fp32(g, probs, keep, 0.25, 0.5)
    assert max_err(masked_ext.backward_dropout(g.clone(), probs, 0.5, 0.25, 5, 8), want_d) <= 2 * TOL[dtype]
    assert max_err(causal_ext.backward_dropout(g.clone(), probs, 0.5, 0.25, 5, 8),
                   R.softmax_dropout_backward_fp32(g, probs.masked_fill(causal, 0), keep, 0.25, 0.5)) <= 2 * TOL[dtype]


def test_mask_and_bias_tensors_beyond_4_gib(device):
    # short rows whose mask / bias tensor no longer fits a 32-bit buffer: the several-rows-per-wave
    # kernels step aside for the row kernels, which address every row through its own buffer
    if torch.cuda.get_device_properties(device).total_memory < 80 << 30:
        pytest.skip("needs about 40 GiB of device memory")
    dtype, sk = torch.float16, 512
    sq = (1 << 23) + 8                      # mask: sq * 512 bytes > 4 GiB; bias: twice that
    x = torch.empty(1, 1, sq, sk, dtype=dtype, device=device)
    for lo in range(0, sq, 1 << 20):        # filled in pieces: no full-size fp32 temporary
        x[0, 0, lo : lo + (1 << 20)] = scores((min(1 << 20, sq - lo), sk), dtype, device, lo)
    mask = torch.zeros(1, 1, sq, sk, dtype=torch.bool, device=device)
    rows = torch.tensor([0, 1, 12345, (1 << 22) + 3, (1 << 23) - 1, 1 << 23, sq - 2, sq - 1], device=device)
    pattern = torch.rand(rows.numel(), sk, device=device, generator=gen(device, 1)) < 0.4
    pattern[:, 0] = False
    mask[0, 0, rows] = pattern
    assert mask.numel() > (1 << 32)
    y = masked_ext.forward(x, mask, 0.25)
    assert max_err(y[0, 0, rows], R.softmax_fp32(x[0, 0, rows], pattern, 0.25)) <= TOL[dtype]
    assert (y[0, 0, rows][pattern] == 0).all()
    assert torch.allclose(y[0, 0, -4096:].float().sum(-1), torch.ones(4096, device=device), atol=2e-2)
    bias = torch.zeros(1, 1, sq, sk, dtype=dtype, device=device)
    bias[0, 0, rows] = normal((rows.numel(), sk), dtype, device, 2)
    yb = masked_ext.forward_bias(x, mask, bias, 0.25)
    want = R.softmax_fp32(x[0, 0, rows].float() + bias[0, 0, rows].float(), pattern, 0.25)
    assert max_err(yb[0, 0, rows], want) <= TOL[dtype]
    other = torch.tensor([5, (1 << 23) + 5], device=device)  # rows with a zero bias and an empty mask
    assert torch.equal(yb[0, 0, other], y[0, 0, other])
    del yb, bias
    torch.cuda.empty_cache()
    from gpt_neox_amd.fused_kernels import attention_dropout as rng
    probs, dropped = masked_ext.forward_dropout(x, mask, 0.25, 0.25, 3, 4)
    assert torch.equal(probs[0, 0, rows], y[0, 0, rows])
    keep = rng.keep_mask(probs.numel(), 0.25, 3, 4, device).view(probs.shape)
    assert torch.equal(dropped[0, 0, rows], R.dropout_with_mask(probs[0, 0, rows], keep[0, 0, rows], 0.25))
