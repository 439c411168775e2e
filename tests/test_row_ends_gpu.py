"""The hint that tells the mask-tensor kernels where every row's visible keys end
(neox_mask_scan, neox_masked_softmax_ends_fwd, neox_masked_softmax_ends_bwd), through the C-ABI.

What is pinned: the scan against plain torch (last visible key + 1 per mask row, the number of
keys behind those points, the causal verdict in the first four words); the hinted forward and
backward passes bit-equal to the plain ones for every kernel family, mask pattern and feature set --
they compute the same numbers in the same order and only fetch less --, so they inherit the plain
passes' parity with the oracle (checked once more here against the fp32 expression); ends given by the caller instead of
the scan; and the Python module passing the hint along by itself, without
a host synchronisation, once it has seen that a mask hides enough.
"""
import pytest
import torch

from gpt_neox_amd.fused_kernels import scaled_masked_softmax_cuda as masked_ext
from gpt_neox_amd.fused_softmax import FusedScaleMaskSoftmax, SoftmaxFusionTypes
from oracle import torch_ref as R

pytestmark = pytest.mark.gpu

TOL = {torch.bfloat16: 2e-3, torch.float16: 1e-3}
DTYPES = [torch.float16, torch.bfloat16]


def gen(device, seed):
    return torch.Generator(device=device).manual_seed(seed)


def max_err(a, b):
    return (a.float() - b.float()).abs().max().item()


def ends_by_torch(mask):
    """last visible key + 1 per mask row (0 without a visible key), int32 [mask_b * sq]"""
    visible = (mask == 0)[:, 0]  # [mask_b, sq, sk]
    sk = mask.shape[-1]
    pos = torch.arange(1, sk + 1, device=mask.device)
    return (visible * pos).amax(-1).reshape(-1).to(torch.int32)


def masks(kind, b, sq, sk, device, seed):
    g = gen(device, seed)
    if kind == "padding":
        lens = torch.randint(1, sk + 1, (b,), device=device, generator=g)
        lens[0] = sk  # one sample without padding
        m = (torch.arange(sk, device=device).view(1, 1, 1, sk) >= lens.view(b, 1, 1, 1)).expand(b, 1, sq, sk).contiguous()
    elif kind == "causal":
        m = (torch.arange(sk, device=device).view(1, sk) > torch.arange(sq, device=device).view(sq, 1) + (sk - sq))
        m = m.view(1, 1, sq, sk).expand(b, 1, sq, sk).contiguous()
    elif kind == "random tail":  # hidden keys scattered in front of a hidden tail of random length
        lens = torch.randint(1, sk + 1, (b, 1, sq, 1), device=device, generator=g)
        m = (torch.rand(b, 1, sq, sk, device=device, generator=g) < 0.2) | (torch.arange(sk, device=device).view(1, 1, 1, sk) >= lens)
    else:
        m = torch.rand(b, 1, sq, sk, device=device, generator=g) < 0.3
    if sq > 2:
        m[0, 0, 1, :] = True   # a row without a visible key
        m[-1, 0, 2, :] = False  # and one that hides nothing
    return m


SHAPES = [(2, 2, 5, 8), (2, 3, 9, 40), (2, 2, 16, 512), (2, 2, 8, 640), (3, 2, 8, 1024), (2, 2, 6, 1280),
          (2, 2, 8, 2048), (1, 2, 6, 4096), (2, 1, 4, 8192), (1, 2, 3, 20000), (2, 1, 3, 33000), (1, 1, 3, 50008),
          (2, 2, 5, 1001), (1, 2, 3, 9001), (1, 1, 3, 36865), (2, 2, 4, 5)]


@pytest.mark.parametrize("kind", ["padding", "causal", "random tail", "random"])
@pytest.mark.parametrize("shape", SHAPES)
def test_scan_finds_the_ends_and_the_hinted_forward_equals_the_plain_one(device, shape, kind):
    b, heads, sq, sk = shape
    dtype = DTYPES[(sk + len(kind)) % 2]
    mask = masks(kind, b, sq, sk, device, sk + sq)
    record, row_end = masked_ext.scan_mask(mask)
    want = ends_by_torch(mask)
    assert torch.equal(row_end, want)
    tail = (sk - want.long())[want > 0].sum().item()
    assert masked_ext.hidden_tail_keys(record.tolist()) == tail
    if sq == sk:
        assert record[:4].tolist() == masked_ext.classify_mask(mask).tolist()
    else:
        assert record[0].item() == 1 and masked_ext.decode_mask_record(record.tolist()) is False
    assert record[6:].tolist() == [0, 0]

    x = torch.empty(shape, dtype=dtype, device=device).normal_(0.0, 4.0, generator=gen(device, sk))
    plain = masked_ext.forward(x, mask, 0.25)
    hinted = masked_ext.forward(x, mask, 0.25, row_end=row_end)
    assert torch.equal(hinted, plain)
    assert max_err(hinted, R.softmax_fp32(x, mask, 0.25)) <= TOL[dtype]
    hidden = mask.expand(shape) & ~mask.all(-1, keepdim=True).expand(shape)
    assert (hinted[hidden] == 0).all()
    # the mask of the first sample for all of them
    rec1, end1 = masked_ext.scan_mask(mask[:1])
    assert torch.equal(end1, want[:sq])
    assert torch.equal(masked_ext.forward(x, mask[:1], 0.25, row_end=end1), masked_ext.forward(x, mask[:1], 0.25))


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("shape", [(2, 3, 8, 1024), (2, 2, 4, 2048), (1, 2, 4, 8192), (2, 2, 5, 1001), (1, 2, 3, 36864), (2, 2, 8, 384)])
def test_every_feature_set_takes_the_hint(device, shape, dtype):
    b, heads, sq, sk = shape
    mask = masks("padding", b, sq, sk, device, 5 * sk)
    _, row_end = masked_ext.scan_mask(mask)
    x = torch.empty(shape, dtype=dtype, device=device).normal_(0.0, 4.0, generator=gen(device, sk + 1))
    bias = torch.empty(shape, dtype=dtype, device=device).normal_(0.0, 1.0, generator=gen(device, sk + 2))
    slopes = torch.rand(heads, device=device, generator=gen(device, sk + 3))
    scale, p, seed, offset = 0.125, 0.25, 31, 8
    assert torch.equal(masked_ext.forward_alibi(x, mask, slopes, scale, row_end=row_end),
                       masked_ext.forward_alibi(x, mask, slopes, scale))
    assert torch.equal(masked_ext.forward_bias(x, mask, bias, scale, row_end=row_end),
                       masked_ext.forward_bias(x, mask, bias, scale))
    assert torch.equal(masked_ext.forward_bias(x, mask, bias[:1], scale, slopes, row_end=row_end),
                       masked_ext.forward_bias(x, mask, bias[:1], scale, slopes))
    for extra in ({}, {"bias": bias}, {"slopes": slopes}, {"bias": bias, "slopes": slopes}):
        y, dropped = masked_ext.forward_dropout(x, mask, scale, p, seed, offset, row_end=row_end, **extra)
        y0, dropped0 = masked_ext.forward_dropout(x, mask, scale, p, seed, offset, **extra)
        assert torch.equal(y, y0) and torch.equal(dropped, dropped0)


BWD_SHAPES = [(2, 3, 9, 40), (2, 2, 8, 384), (2, 2, 16, 512), (3, 2, 8, 1024), (2, 2, 6, 1536), (2, 2, 8, 2048),
              (1, 2, 6, 4096), (2, 1, 4, 8192), (1, 2, 3, 20000), (2, 1, 3, 33000), (1, 1, 3, 50008), (2, 2, 5, 1001),
              (1, 2, 3, 9001), (1, 1, 3, 36865), (2, 2, 4, 5)]


@pytest.mark.parametrize("kind", ["padding", "random tail"])
@pytest.mark.parametrize("shape", BWD_SHAPES)
def test_hinted_backward_equals_the_plain_one(device, shape, kind):
    b, heads, sq, sk = shape
    dtype = DTYPES[(sk + len(kind)) % 2]
    mask = masks(kind, b, sq, sk, device, 3 * sk + sq)
    _, row_end = masked_ext.scan_mask(mask)
    x = torch.empty(shape, dtype=dtype, device=device).normal_(0.0, 4.0, generator=gen(device, sk))
    g = torch.empty(shape, dtype=dtype, device=device).normal_(0.0, 1.0, generator=gen(device, sk + 1))
    y = masked_ext.forward(x, mask, 0.25)
    plain = masked_ext.backward(g.clone(), y, 0.25)
    buf = g.clone()
    hinted = masked_ext.backward(buf, y, 0.25, row_end=row_end)
    assert hinted.data_ptr() == buf.data_ptr()  # in place, like the plain pass
    assert torch.equal(hinted, plain)
    hidden = mask.expand(shape) & ~mask.all(-1, keepdim=True).expand(shape)
    assert (hinted[hidden] == 0).all()
    p, seed, offset = 0.25, 17, 8
    yd, _ = masked_ext.forward_dropout(x, mask, 0.25, p, seed, offset)
    assert torch.equal(masked_ext.backward_dropout(g.clone(), yd, 0.25, p, seed, offset, row_end=row_end),
                       masked_ext.backward_dropout(g.clone(), yd, 0.25, p, seed, offset))
    # the mask of the first sample for all of them
    _, end1 = masked_ext.scan_mask(mask[:1])
    y1 = masked_ext.forward(x, mask[:1], 0.25)
    assert torch.equal(masked_ext.backward(g.clone(), y1, 0.25, row_end=end1), masked_ext.backward(g.clone(), y1, 0.25))
    with pytest.raises(RuntimeError, match="row_end"):
        masked_ext.backward(g.clone(), y, 0.25, row_end=row_end[:-1])


def test_row_ends_given_by_the_caller(device):
    # the hint is a promise of the caller -- every key at or behind a row's end is masked in the mask
    # tensor too -- which a kernel may use or not: ends that the caller knows (here: the lengths a padding
    # mask was built from) serve like those of the scan, and 0 or a value beyond sk promises nothing
    b, heads, sq = 2, 2, 6
    for sk in (1024, 2048, 8192):
        x = torch.empty((b, heads, sq, sk), dtype=torch.bfloat16, device=device).normal_(0.0, 4.0, generator=gen(device, 1))
        ends = torch.tensor([sk, 1000, 513, 512, 8, 1] * b, dtype=torch.int32, device=device)
        hidden = torch.arange(sk, device=device).view(1, 1, 1, sk) >= ends.view(b, 1, sq, 1)
        want = masked_ext.forward(x, hidden, 0.5)
        assert torch.equal(masked_ext.forward(x, hidden, 0.5, row_end=ends), want)
        longer = (ends + 3).clamp(max=sk)  # a weaker promise is still a true one
        assert torch.equal(masked_ext.forward(x, hidden, 0.5, row_end=longer), want)
        none = torch.tensor([0, sk, sk + 5, -3, 0, 2**31 - 1] * b, dtype=torch.int32, device=device)
        assert torch.equal(masked_ext.forward(x, hidden, 0.5, row_end=none), want)
        g = torch.randn_like(x)
        assert torch.equal(masked_ext.backward(g.clone(), want, 0.5, row_end=longer), masked_ext.backward(g.clone(), want, 0.5))


def test_row_end_of_the_wrong_kind_is_refused(device):
    x = torch.zeros(2, 2, 4, 64, dtype=torch.float16, device=device)
    mask = torch.zeros(2, 1, 4, 64, dtype=torch.bool, device=device)
    _, row_end = masked_ext.scan_mask(mask)
    for bad in (row_end[:-1], row_end.long(), row_end.cpu(), row_end.view(2, 4)):
        with pytest.raises(RuntimeError, match="row_end"):
            masked_ext.forward(x, mask, 1.0, row_end=bad)
    with pytest.raises(RuntimeError, match="mask must have shape"):
        masked_ext.scan_mask(mask[:, 0])


# ---------------------------------------------------------------------------------
# the module passes the hint along by itself
# ---------------------------------------------------------------------------------
def module(fusion, check="lazy", **kw):
    return FusedScaleMaskSoftmax(False, True, fusion, R.gpt2_attention_mask_func, True, 0.5, causal_mask_check=check, **kw)


def calls_with_hint(monkeypatch):
    """Counts the forward calls of the extension that carry a hint."""
    seen = {"hinted": 0, "plain": 0}
    real = masked_ext._forward_ends

    def spy(*a, **k):
        seen["hinted"] += 1
        return real(*a, **k)

    monkeypatch.setattr(masked_ext, "_forward_ends", spy)
    return seen


@pytest.mark.parametrize("check", ["lazy", "verify"])
def test_module_skips_hidden_tails_once_it_knows_the_mask(device, monkeypatch, check):
    b, heads, sq, sk = 4, 2, 1024, 1024
    x = torch.randn(b, heads, sq, sk, device=device).bfloat16().requires_grad_(True)
    mask = masks("padding", b, sq, sk, device, 7)
    m = module(SoftmaxFusionTypes.general, check)
    seen = calls_with_hint(monkeypatch)
    want = R.softmax_fp32(x.detach(), mask, 0.5)
    y = m(x, mask)
    assert max_err(y, want) <= TOL[torch.bfloat16]
    first = seen["hinted"]  # lazy: 0 if the scan was still on its way, which nobody waits for
    assert first == 1 if check == "verify" else first in (0, 1)
    torch.cuda.synchronize()
    y2 = m(x, mask)
    assert seen["hinted"] == first + 1
    assert torch.equal(y2, y)
    g = torch.randn_like(y2)
    y2.backward(g.clone())  # (the gradient kernel writes into the buffer it is given)
    _, auto = R.softmax_autograd_fp32(x.detach(), mask, 0.5, g)
    assert max_err(x.grad, auto) <= 4 * TOL[torch.bfloat16]
    # features take it too
    slopes = torch.rand(heads, device=device)
    ya = m(x, mask, alibi_slopes=slopes)
    assert seen["hinted"] == first + 2
    assert torch.equal(ya, masked_ext.forward_alibi(x.detach(), mask, slopes, 0.5))
    # a write to the mask makes it a new mask
    mask[0, 0, :, :] = False
    torch.cuda.synchronize()
    before = seen["hinted"]
    y3 = m(x, mask)
    assert max_err(y3, R.softmax_fp32(x.detach(), mask, 0.5)) <= TOL[torch.bfloat16]
    assert seen["hinted"] == before + 1 if check == "verify" else seen["hinted"] in (before, before + 1)


def test_module_passes_no_hint_for_a_mask_that_hides_little_or_when_told_not_to(device, monkeypatch):
    b, heads, sq, sk = 2, 2, 128, 1024
    x = torch.randn(b, heads, sq, sk, device=device).bfloat16()
    seen = calls_with_hint(monkeypatch)
    dense = torch.rand(b, 1, sq, sk, device=device) < 0.3  # the last visible key lies near the row end
    m = module(SoftmaxFusionTypes.general, "verify")
    for _ in range(2):
        assert max_err(m(x, dense), R.softmax_fp32(x, dense, 0.5)) <= TOL[torch.bfloat16]
    assert seen["hinted"] == 0
    padded = masks("padding", b, sq, sk, device, 9)
    padded[1, 0, :, 300:] = True
    off = module(SoftmaxFusionTypes.general, "verify", skip_hidden_tails=False)
    trusting = module(SoftmaxFusionTypes.general, "trust")
    for mod in (off, trusting):
        for _ in range(2):
            assert max_err(mod(x, padded), R.softmax_fp32(x, padded, 0.5)) <= TOL[torch.bfloat16]
    assert seen["hinted"] == 0
    assert max_err(m(x, padded), R.softmax_fp32(x, padded, 0.5)) <= TOL[torch.bfloat16]
    assert seen["hinted"] == 1


def test_causal_fusion_uses_the_hint_for_masks_that_are_not_causal(device, monkeypatch):
    # a causal mask combined with padding: neither the causal nor the window kernel may take it, the
    # mask-tensor kernel does, and it stops at every row's last visible key
    b, heads, s = 2, 2, 1024
    x = torch.randn(b, heads, s, s, device=device).bfloat16()
    mask = R.get_attn_mask(s, device).expand(b, 1, s, s).clone()
    mask[1, 0, :, 700:] = True
    seen = calls_with_hint(monkeypatch)
    m = module(SoftmaxFusionTypes.upper_triang, "verify")
    y = m(x, mask)
    assert seen["hinted"] == 1
    assert max_err(y, R.softmax_fp32(x, mask, 0.5)) <= TOL[torch.bfloat16]
    assert (y[mask.expand_as(y)] == 0).all()
    # the plain causal mask still goes to the kernel that reads no mask at all
    causal = R.get_attn_mask(s, device)
    assert m.mask_kind(causal, s, s) == "causal"
    m(x, causal)
    assert seen["hinted"] == 1


def test_launches_recorded_into_a_hip_graph_go_without_the_hint(device, monkeypatch):
    # the hint lives in the module's memo and a graph could outlive it: captured launches use the plain pass
    b, heads, s = 2, 2, 1024
    x = torch.randn(b, heads, s, s, device=device).bfloat16()
    mask = masks("padding", b, s, s, device, 11)
    m = module(SoftmaxFusionTypes.general, "verify")
    seen = calls_with_hint(monkeypatch)
    want = m(x, mask)
    assert seen["hinted"] == 1 and m.hidden_tails(mask, b, s, s) is not None
    graph = torch.cuda.CUDAGraph()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        with torch.cuda.graph(graph, stream=side):
            assert m.hidden_tails(mask, b, s, s) is None
            out = m(x, mask)
    torch.cuda.synchronize()
    assert seen["hinted"] == 1
    for _ in range(3):
        out.fill_(7.0)
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(out, want)
    assert torch.equal(m(x, mask), want) and seen["hinted"] == 2


def test_first_call_with_a_fresh_mask_uses_the_scan_that_is_still_on_its_way(device, monkeypatch):
    # lazy: nobody waits for the scan's record, but a launch on the scan's stream follows it and finds
    # the rows' ends in device memory -- a fresh causal mask costs its upper triangle not even once
    b, heads, s = 1, 2, 1024  # (a length at which the causal and the mask-tensor kernels sum a row in the same order)
    x = torch.randn(b, heads, s, s, device=device).bfloat16()
    m = module(SoftmaxFusionTypes.upper_triang, "lazy")
    seen = calls_with_hint(monkeypatch)
    want = masked_ext.forward(x, R.get_attn_mask(s, device), 0.5)
    for _ in range(3):
        fresh = R.get_attn_mask(s, device)
        before = seen["hinted"]
        y = m(x, fresh)
        kind = m.mask_kind(fresh, s, s)
        assert seen["hinted"] == before + 1 or kind == "causal"  # (unless the record has arrived already)
        assert torch.equal(y, want)
    # on another stream the scan's array may not be ready: no hint there until the record has arrived
    fresh = R.get_attn_mask(s, device)
    m(x, fresh)
    side = torch.cuda.Stream()
    with torch.cuda.stream(side):
        assert m.hidden_tails(fresh, b, s, s) is None or m.mask_kind(fresh, s, s) is not None
    torch.cuda.synchronize()


def test_hint_on_another_stream_than_the_scans(device, monkeypatch):
    b, heads, s = 2, 2, 1024
    x = torch.randn(b, heads, s, s, device=device).bfloat16()
    mask = masks("padding", b, s, s, device, 13)
    m = module(SoftmaxFusionTypes.general, "verify")
    seen = calls_with_hint(monkeypatch)
    want = m(x, mask)  # scanned on the default stream
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        for _ in range(3):
            assert torch.equal(m(x, mask), want)
    side.synchronize()
    assert seen["hinted"] == 4
