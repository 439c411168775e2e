"""The ``rope_fusion`` drop-in (gpt-neox_amd/fused_rope.py) against the oracle, on the GPU.

The reference calls ``fused_apply_rotary_pos_emb_cached(rot, cos, sin)`` on the query and the key
slices at megatron/model/transformer.py:844-848; ``fused_apply_rotary_pos_emb(t, freqs)`` is the
variant that evaluates cos/sin of the angles in its kernel (megatron/model/fused_rope.py:18-141).
Both are driven here through their autograd Functions: forward and backward, both values of
``transpose_output_memory``, fp16 and bf16, fp32 and same-dtype tables, contiguous inputs and
views into a fused QKV buffer, at a toy shape and at the rotary shapes of BASELINE configs[2]
and configs[4].

Bars.  Cached variant: bit-equal to the oracle's fp32 expression rounded once to the storage type
(forward: ``partial_rotary``; backward: ``rotary_autograd_fp32`` with the pass-through dims of the
gradient copied).  Angle variant: the kernel's sincosf and torch's cos/sin are two fp32
evaluations of the same functions that may differ in the last bit, so the bar is 1 ulp of the
storage type (2^-7 relative for bf16, 2^-10 for fp16, plus 1e-6 absolute where the two products
cancel) with at most 0.1 % of the elements differing at all; the pass-through dims are bit-identical.
"""
import pytest
import torch

from gpt_neox_amd.fused_kernels import fused_rotary_positional_embedding as rope_ext
from gpt_neox_amd.fused_rope import (
    FusedRoPECachedFunc,
    FusedRoPEFunc,
    fused_apply_rotary_pos_emb,
    fused_apply_rotary_pos_emb_cached,
)
from oracle import torch_ref as R

pytestmark = pytest.mark.gpu

DTYPES = [torch.float16, torch.bfloat16]
ULP = {torch.float16: 2.0 ** -10, torch.bfloat16: 2.0 ** -7}


def normal(shape, dtype, device, seed):
    g = torch.Generator(device=device).manual_seed(seed)
    return torch.randn(shape, device=device, generator=g).to(dtype)


def angles(s, d2, device, base=10000):
    inv = 1.0 / (base ** (torch.arange(0, d2, 2, device=device).float() / d2))
    f = torch.outer(torch.arange(s, device=device).float(), inv)
    return torch.cat((f, f), -1)[:, None, None, :].contiguous()


def expected(t, g, cos, sin, d2):
    """Oracle forward and backward for input t, output gradient g (fp32 tables)."""
    dtype = t.dtype
    fwd, _ = R.partial_rotary(t.float(), t.float(), cos.float(), sin.float(), d2)
    dq, _ = R.rotary_autograd_fp32(t[..., :d2], t[..., :d2], cos.float(), sin.float(), g[..., :d2], g[..., :d2])
    bwd = torch.cat((dq.to(dtype), g[..., d2:]), dim=-1)
    return fwd.to(dtype), bwd


def run(fn, t, tables, transpose, g):
    tin = t.detach().clone().requires_grad_(True) if t.is_contiguous() else t.detach().requires_grad_(True)
    out = fn(tin, *tables, transpose)
    out.backward(g)
    return out.detach(), tin.grad


def assert_within_one_ulp(got, want, dtype):
    diff = (got.float() - want.float()).abs()
    assert (diff <= ULP[dtype] * want.float().abs() + 1e-6).all(), diff.max().item()
    assert (got != want).float().mean().item() <= 1e-3


def check_both_variants(t, d2, transpose, device, table_dtype=torch.float32, seed=11):
    s, b, h, d = t.shape
    dtype = t.dtype
    g = normal((s, b, h, d), dtype, device, seed)
    freqs = angles(s, d2, device)
    cos, sin = R.rotary_tables_from_freqs(freqs)
    cos_t, sin_t = cos.to(table_dtype), sin.to(table_dtype)
    want_f, want_b = expected(t, g, cos_t, sin_t, d2)

    out, grad = run(fused_apply_rotary_pos_emb_cached, t, (cos_t, sin_t), transpose, g)
    assert out.shape == (s, b, h, d) and out.dtype == dtype
    assert torch.equal(out, want_f), "cached forward"
    assert torch.equal(grad, want_b), "cached backward"
    assert out.transpose(0, 1).is_contiguous() == (transpose or s == 1 or b == 1)

    if table_dtype == torch.float32:
        want_f, want_b = expected(t, g, cos, sin, d2)
        out, grad = run(fused_apply_rotary_pos_emb, t, (freqs,), transpose, g)
        assert_within_one_ulp(out, want_f, dtype)
        assert_within_one_ulp(grad, want_b, dtype)
        assert torch.equal(out[..., d2:], t[..., d2:]) and torch.equal(grad[..., d2:], g[..., d2:])


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("transpose", [False, True])
@pytest.mark.parametrize("half_tables", [False, True])
def test_toy_shape(device, dtype, transpose, half_tables):
    t = normal((12, 2, 3, 64), dtype, device, 5)
    check_both_variants(t, 16, transpose, device, dtype if half_tables else torch.float32)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("shape,d2", [
    ((33, 3, 5, 128), 128),   # full rotary, nothing to copy
    ((33, 3, 5, 96), 24),     # 20B head: 48-byte spans, 4-dim slots
    ((17, 2, 4, 256), 64),    # whole head = 32 lanes
    ((9, 2, 3, 200), 20),     # 2-dim slots, head too wide for one lane group: element-wise copy loop
    ((9, 2, 3, 10), 6),       # odd d2/2: one dim per lane, element-wise copy
    ((5, 1, 2, 1024), 1024),  # spans of more than 64 slots
    ((7, 2, 3, 72), 36),
])
def test_head_shapes(device, dtype, shape, d2):
    t = normal(shape, dtype, device, 21)
    check_both_variants(t, d2, False, device)
    check_both_variants(t, d2, True, device, seed=12)


@pytest.mark.parametrize("dtype", DTYPES)
def test_views_into_a_fused_qkv_buffer(device, dtype):
    # megatron/model/transformer.py:798-833: [sq, b, np, 3*hn] split into q, k, v, then the first
    # rotary_ndims dims of q and k are sliced off -- the inputs of the fused call are such views
    s, b, h, hn, d2 = 40, 2, 6, 64, 16
    qkv = normal((s, b, h, 3 * hn), dtype, device, 31)
    before = qkv.clone()
    for view in (qkv[..., :hn], qkv[..., hn : 2 * hn], qkv[..., :d2], qkv[..., hn : hn + d2]):
        assert not view.is_contiguous()
        check_both_variants(view, d2, False, device)
        check_both_variants(view, d2, True, device)
    assert torch.equal(qkv, before)  # out of place: the inputs are untouched
    # 2-byte aligned view: one dim per lane
    odd = qkv[..., 1 : 1 + hn]
    check_both_variants(odd, d2, False, device)


def test_partial_rotary_shape_of_configs_2(device):
    # BASELINE configs[2]: q [2048, 4, 32, 128] bf16, rotary_pct 0.25 -> d2 = 32
    t = normal((2048, 4, 32, 128), torch.bfloat16, device, 41)
    check_both_variants(t, 32, False, device)
    # as the attention layer calls it: on the sliced-off rotary dims only
    check_both_variants(t[..., :32], 32, False, device)
    check_both_variants(t, 32, True, device, table_dtype=torch.bfloat16)


def test_full_rotary_shape_of_configs_4(device):
    # BASELINE configs[4]: q [8192, 1, 32, 128] bf16, rotary_pct 1.0, positions to 8191
    t = normal((8192, 1, 32, 128), torch.bfloat16, device, 42)
    check_both_variants(t, 128, False, device)
    th = normal((8192, 1, 32, 128), torch.float16, device, 43)
    check_both_variants(th, 128, True, device)


@pytest.mark.parametrize("dtype", DTYPES)
def test_kernel_sincos_at_large_angles(device, dtype):
    # x = (1, 0) in every rotation pair: the output is (cos, sin) of the angle rounded to the
    # storage type.  Against float64 cos/sin of the same fp32 angles, for angles up to 1e5 rad
    # (range reduction) and negative ones: within 1 ulp of the storage type.
    s, d2 = 4096, 8
    freqs = torch.empty(s, 1, 1, d2, device=device)
    base = torch.linspace(-100000.0, 100000.0, s, device=device)
    for j in range(d2):
        freqs[:, 0, 0, j] = base * (0.37 + 0.21 * j)
    t = torch.zeros(s, 1, 2, d2, device=device, dtype=dtype)
    t[..., : d2 // 2] = 1.0
    out = fused_apply_rotary_pos_emb(t, freqs)
    f64 = freqs.double()
    want = torch.cat((f64.cos()[..., : d2 // 2], f64.sin()[..., d2 // 2 :]), -1).expand(s, 1, 2, d2)
    assert ((out.double() - want).abs() <= ULP[dtype] * (want.abs() + 2.0 ** -10)).all()


def test_functions_save_tables_and_return_no_table_gradients(device):
    t = normal((6, 2, 2, 32), torch.float16, device, 51).requires_grad_(True)
    freqs = angles(6, 32, device).requires_grad_(True)
    out = FusedRoPEFunc.apply(t, freqs, False)
    out.sum().backward()
    assert freqs.grad is None and t.grad is not None
    cos, sin = (x.requires_grad_(True) for x in R.rotary_tables_from_freqs(freqs.detach()))
    t2 = t.detach().clone().requires_grad_(True)
    out2 = FusedRoPECachedFunc.apply(t2, cos, sin)  # transpose_output_memory defaults to False
    out2.sum().backward()
    assert cos.grad is None and sin.grad is None
    assert torch.equal(out2, out) or (out2.float() - out.float()).abs().max().item() <= 2.0 ** -10 * 4


def test_argument_checks_follow_the_extension(device):
    # megatron/fused_kernels/fused_rotary_positional_embedding.cpp:38-127
    t = normal((6, 2, 2, 32), torch.float16, device, 61)
    f = angles(6, 32, device)
    with pytest.raises(RuntimeError, match="expected 4D tensor"):
        rope_ext.forward(t[0], f)
    with pytest.raises(RuntimeError, match="same sequence length"):
        rope_ext.forward(t, f[:5])
    with pytest.raises(RuntimeError, match="equal 1"):
        rope_ext.forward(t, f.expand(6, 2, 1, 32))
    with pytest.raises(RuntimeError, match="greater than the freqs"):
        rope_ext.forward(t[..., :16], f)
    with pytest.raises(RuntimeError, match="must be float"):
        rope_ext.forward(t, f.half())
    with pytest.raises(RuntimeError, match="same dtype"):
        rope_ext.forward_cached(t, f.cos(), f.sin().half())
    with pytest.raises(RuntimeError, match="Only fp16 and bf16"):
        rope_ext.forward(t.float(), f)
    with pytest.raises(RuntimeError, match="GPU tensors"):
        rope_ext.forward(t.cpu(), f.cpu())
    empty = rope_ext.forward(t[:0], f[:0])
    assert empty.shape == (0, 2, 2, 32)


@pytest.mark.parametrize("dtype", DTYPES)
def test_angles_for_q_and_k_in_one_launch(device, dtype):
    # the C-ABI's angle entry point takes q and k together (the Python extension API passes one
    # tensor per call, as the reference does): in place over the first d2 dims, k with fewer heads
    s, b, hq, hk, d, d2 = 70, 2, 8, 2, 64, 32
    q, k = normal((s, b, hq, d), dtype, device, 71), normal((s, b, hk, d), dtype, device, 72)
    freqs = angles(s + 3, d2, device)
    cos, sin = R.rotary_tables_from_freqs(freqs)
    want_q, want_k = R.partial_rotary(q.float(), k.float(), cos, sin, d2, offset=3)
    q1, k1 = q.clone(), k.clone()
    rope_ext.rope_launch(q1, k1, q1, k1, freqs.view(s + 3, d2), None, d2, 3, backward=False)
    assert_within_one_ulp(q1, want_q.to(dtype), dtype)
    assert_within_one_ulp(k1, want_k.to(dtype), dtype)
    assert torch.equal(q1[..., d2:], q[..., d2:]) and torch.equal(k1[..., d2:], k[..., d2:])
    # backward = the inverse rotation: applying it to the rotated tensors returns the inputs to 2 ulp
    rope_ext.rope_launch(q1, k1, q1, k1, freqs.view(s + 3, d2), None, d2, 3, backward=True)
    rot = q.float()[..., :d2]
    pair = (rot[..., : d2 // 2] ** 2 + rot[..., d2 // 2 :] ** 2).sqrt()  # a rotation mixes the two dims of a pair
    assert ((q1.float()[..., :d2] - rot).abs() <= 3 * ULP[dtype] * torch.cat((pair, pair), -1) + 1e-6).all()
