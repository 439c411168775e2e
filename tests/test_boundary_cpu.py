"""The C-ABI boundary and the Python drop-in surface, checked without a GPU.

Covers: the shared library loads and exports every symbol that
include/neox_fused.h declares; argument errors come back as status codes before
any HIP call; the dispatcher predicate; the error behaviour of the
extension-level modules; the names and signatures the reference's callers import.
"""
import ctypes
import inspect
import os
import re
import sys

import pytest
import torch

import gpt_neox_amd
from gpt_neox_amd import _lib, fused_softmax, positional_embeddings
from gpt_neox_amd.fused_kernels import (
    fused_rotary_positional_embedding,
    load_fused_kernels,
    scaled_masked_softmax_cuda,
    scaled_upper_triang_masked_softmax_cuda,
)
from gpt_neox_amd.fused_softmax import FusedScaleMaskSoftmax, SoftmaxFusionTypes

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "neox_fused.h")


def declared_functions():
    text = open(HEADER).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    decls = re.findall(r"\b(?:int|const char\*)\s+(neox_\w+)\s*\(([^)]*)\)\s*;", text)
    out = {}
    for name, args in decls:
        args = args.strip()
        out[name] = 0 if args in ("", "void") else len(args.split(","))
    return out


def test_header_declares_the_expected_entry_points():
    names = set(declared_functions())
    assert {
        "neox_causal_softmax_fwd", "neox_causal_softmax_bwd", "neox_masked_softmax_fwd",
        "neox_masked_softmax_bwd", "neox_rope_apply", "neox_get_batch_per_block",
        "neox_fused_abi_version", "neox_fused_strerror", "neox_fused_last_error",
    } <= names


def test_library_exports_every_declared_symbol_with_matching_arity():
    handle = ctypes.CDLL(_lib.LIB_PATH)
    for name, nargs in declared_functions().items():
        assert hasattr(handle, name), f"{name} declared in the header but not exported"
        assert name in _lib.SIGNATURES, f"{name} has no ctypes signature"
        assert len(_lib.SIGNATURES[name][1]) == nargs, name
    assert set(_lib.SIGNATURES) == set(declared_functions())


def test_abi_version_and_error_strings():
    lib = _lib.lib()
    assert lib.neox_fused_abi_version() == _lib.ABI_VERSION
    for code in range(0, -7, -1):
        assert lib.neox_fused_strerror(code)
    assert lib.neox_fused_strerror(-99) == b"unknown status"


def test_argument_errors_are_reported_without_touching_the_gpu():
    lib = _lib.lib()
    buf = ctypes.create_string_buffer(4096)
    p = ctypes.addressof(buf)
    p = (p + 255) & ~255  # aligned fake "device" pointer: never dereferenced on these paths
    F16, BF16, F32 = _lib.NEOX_F16, _lib.NEOX_BF16, _lib.NEOX_F32
    assert lib.neox_causal_softmax_fwd(None, p, 1.0, 1, 8, 8, F16, None) == -1
    assert b"null" in lib.neox_fused_last_error()
    assert lib.neox_causal_softmax_fwd(p, p, 1.0, 1, 8, 8, F32, None) == -2
    assert b"Only fp16 and bf16 are supported" in lib.neox_fused_last_error()
    assert lib.neox_causal_softmax_fwd(p, p, 1.0, 0, 8, 8, F16, None) == -3
    assert lib.neox_causal_softmax_fwd(p, p, 1.0, 1, 0, 8, F16, None) == -3
    assert lib.neox_causal_softmax_fwd(p, p, 1.0, 1 << 40, 8, 8, F16, None) == -3
    assert lib.neox_causal_softmax_fwd(p + 1, p, 1.0, 1, 8, 8, F16, None) == -5
    assert lib.neox_causal_softmax_bwd(p, None, p, 1.0, 1, 8, 8, BF16, None) == -1
    assert lib.neox_causal_softmax_bwd(p, p, p, 1.0, 1, 8, -1, BF16, None) == -3
    assert lib.neox_masked_softmax_fwd(p, p, None, 1.0, 2, 2, 8, 8, 2, F16, None) == -1
    assert lib.neox_masked_softmax_fwd(p, p, p, 1.0, 4, 2, 8, 8, 3, F16, None) == -3
    assert b"mask batch dim" in lib.neox_fused_last_error()
    assert lib.neox_masked_softmax_bwd(p, p, p, 1.0, 0, 8, F16, None) == -3
    assert lib.neox_masked_softmax_bwd(p, p, p, 1.0, 8, 8, 7, None) == -2
    # the mask scan and the forward pass that takes its row ends
    assert lib.neox_mask_scan(None, p, p, 1, 8, 8, None) == -1
    assert lib.neox_mask_scan(p, None, p, 1, 8, 8, None) == -1
    assert lib.neox_mask_scan(p, p, p, 0, 8, 8, None) == -3
    assert lib.neox_mask_scan(p, p, p, 1, 8, 0, None) == -3
    assert lib.neox_mask_scan(p + 4, p, p, 1, 8, 8, None) == -5  # the record holds a 64-bit count
    assert lib.neox_mask_scan(p, p + 2, p, 1, 8, 8, None) == -5
    ends = lib.neox_masked_softmax_ends_fwd
    assert ends(None, None, p, p, p, None, None, 0, 1.0, 0.0, 0, 0, None, 2, 2, 8, 8, 2, F16, None) == -1
    assert ends(None, p, p, None, p, None, None, 0, 1.0, 0.0, 0, 0, None, 2, 2, 8, 8, 2, F16, None) == -1
    assert ends(None, p, p, p, p + 2, None, None, 0, 1.0, 0.0, 0, 0, None, 2, 2, 8, 8, 2, F16, None) == -5
    assert ends(None, p, p, p, p, None, None, 0, 1.0, 0.0, 0, 0, None, 2, 2, 8, 8, 3, F16, None) == -3
    assert ends(None, p, p, p, p, None, None, 0, 1.0, 0.0, 0, 0, None, 2, 2, 8, 8, 2, F32, None) == -2
    assert ends(p, p, p, p, p, None, None, 0, 1.0, 0.5, 0, 0, None, 2, 2, 8, 8, 2, F16, None) == -4  # y_drop aliases y
    assert ends(p + 256, p, p, p, p, None, None, 0, 1.0, 1.5, 0, 0, None, 2, 2, 8, 8, 2, F16, None) == -3
    assert b"dropout probability" in lib.neox_fused_last_error()
    # without y_drop the dropout arguments are not looked at
    assert ends(None, p, p, p, p, None, p, 3, 1.0, 1.5, 0, 0, None, 2, 2, 8, 8, 2, F16, None) == -3
    assert b"bias batch dim" in lib.neox_fused_last_error()
    endsb = lib.neox_masked_softmax_ends_bwd
    assert endsb(p, None, p, p, 1.0, 0, 0.0, 0, 0, None, 2, 2, 8, 8, 2, F16, None) == -1
    assert endsb(p, p, p, p + 2, 1.0, 0, 0.0, 0, 0, None, 2, 2, 8, 8, 2, F16, None) == -5
    assert endsb(p, p, p, p, 1.0, 0, 0.0, 0, 0, None, 2, 2, 8, 8, 3, F16, None) == -3
    assert b"mask batch dim" in lib.neox_fused_last_error()
    assert endsb(p, p, p, p, 1.0, 0, 7.0, 0, 0, None, 2, 2, 8, 0, 2, F16, None) == -3  # p is not looked at
    assert b"sk=0" in lib.neox_fused_last_error()
    assert endsb(p, p, p, p, 1.0, 1, 7.0, 0, 0, None, 2, 2, 8, 8, 2, F16, None) == -3
    assert b"dropout probability" in lib.neox_fused_last_error()
    st = (ctypes.c_int64 * 3)(64, 32, 8)
    neg = (ctypes.c_int64 * 3)(64, -32, 8)
    rope = lib.neox_rope_apply
    assert rope(p, None, p, None, None, p, 4, 1, 2, 0, 8, 8, st, None, st, None, 8, 0, F16, F32, 0, None) == -1
    assert rope(p, p, p, None, p, p, 4, 1, 2, 2, 8, 8, st, st, st, st, 8, 0, F16, F32, 0, None) == -1
    assert rope(p, None, p, None, p, p, 4, 1, 2, 0, 7, 8, st, None, st, None, 8, 0, F16, F32, 0, None) == -3
    assert rope(p, None, p, None, p, p, 4, 1, 2, 0, 8, 8, neg, None, st, None, 8, 0, F16, F32, 0, None) == -4
    assert rope(p, None, p, None, p, p, 4, 1, 2, 0, 8, 8, st, None, st, None, 4, 0, F16, F32, 0, None) == -4
    assert rope(p, None, p, None, p, p, 4, 1, 2, 0, 8, 8, st, None, st, None, 8, 0, F16, BF16, 0, None) == -2
    assert rope(p, None, p, None, p, p, 4, 1, 2, 0, 8, 8, st, None, st, None, 8, -1, F16, F32, 0, None) == -3
    assert rope(p, None, p, None, p, p, 4, 1, 2, 0, 8, 6, st, None, st, None, 8, 0, F16, F32, 0, None) == -3
    assert b"smaller than d_rot" in lib.neox_fused_last_error()
    assert rope(p, None, p, None, p, p, 4, 1, 2, 0, 8, 8, st, None, st, None, 8, 0, F16, 9, 0, None) == -2
    # the d dims a call delivers per head must fit the head stride of every tensor with several heads:
    # a full 16-dim head given with a narrower output view would run into the next head
    wide = (ctypes.c_int64 * 3)(64, 32, 16)
    assert rope(p, None, p, None, p, p, 4, 1, 2, 0, 8, 16, wide, None, st, None, 8, 0, F16, F32, 0, None) == -4
    assert b"out_q head stride 8 is smaller than d=16" in lib.neox_fused_last_error()
    assert rope(p, None, p, None, p, p, 4, 1, 2, 0, 8, 16, st, None, wide, None, 8, 0, F16, F32, 0, None) == -4
    assert b"q head stride 8 is smaller than d=16" in lib.neox_fused_last_error()
    assert rope(p, p, p, p, p, p, 4, 1, 1, 2, 8, 16, st, st, wide, wide, 8, 0, F16, F32, 0, None) == -4
    assert b"k head stride" in lib.neox_fused_last_error()
    freqs = lib.neox_rope_apply_freqs
    assert freqs(p, None, p, None, None, 4, 1, 2, 0, 8, 8, st, None, st, None, 8, 0, F16, 0, None) == -1
    assert freqs(p, None, p, None, p, 4, 1, 2, 0, 8, 8, st, None, st, None, 4, 0, F16, 0, None) == -4
    assert b"freqs row stride" in lib.neox_fused_last_error()
    assert freqs(p, None, p, None, p, 4, 1, 2, 0, 8, 8, st, None, st, None, 8, 0, F32, 0, None) == -2


def test_last_error_is_kept_per_thread():
    import threading

    lib = _lib.lib()
    seen = {}

    def worker(name, bad_sk):
        buf = ctypes.create_string_buffer(64)
        p = (ctypes.addressof(buf) + 15) & ~15
        for _ in range(200):
            assert lib.neox_masked_softmax_bwd(p, p, p, 1.0, 4, bad_sk, _lib.NEOX_F16, None) == -3
            msg = lib.neox_fused_last_error().decode()
            assert f"sk={bad_sk}" in msg, msg
        seen[name] = True

    threads = [threading.Thread(target=worker, args=(i, -1 - i)) for i in range(4)]
    for t in threads:
        t.start()
    for t in threads:
        t.join()
    assert len(seen) == 4


def test_get_batch_per_block_matches_the_reference_formula_on_wave64():
    # megatron/fused_kernels/scaled_masked_softmax.h:338-352 with a 64-wide wavefront:
    # wave = min(pow2(sk), 64); rows/wave = 2 if pow2(sk) <= 128 else 1; waves/block = 128/wave
    table = {1: 256, 2: 128, 4: 64, 8: 32, 16: 16, 17: 8, 32: 8, 33: 4, 64: 4, 65: 4, 128: 4,
             129: 2, 256: 2, 1000: 2, 1024: 2, 2048: 2, 8192: 2}
    for sk, want in table.items():
        assert FusedScaleMaskSoftmax.get_batch_per_block(1024, sk, 2, 4) == want, sk
        assert scaled_masked_softmax_cuda.get_batch_per_block(8, sk, 1, 1) == want


def test_missing_library_raises_import_error(monkeypatch):
    monkeypatch.setattr(_lib, "_lib", None)
    monkeypatch.setattr(_lib, "LIB_PATH", "/nonexistent/libneox_fused.so")
    with pytest.raises(ImportError, match="not built"):
        _lib.lib()
    with pytest.raises(ImportError):
        FusedScaleMaskSoftmax(True, False, SoftmaxFusionTypes.general, None, True, None)
    # no fusion requested: the library is not needed
    FusedScaleMaskSoftmax(True, False, SoftmaxFusionTypes.none, None, True, None)


def test_fused_calls_refuse_cpu_tensors_loudly():
    x = torch.zeros(2, 8, 8, dtype=torch.float16)
    with pytest.raises(RuntimeError, match="no CPU fallback"):
        fused_softmax.ScaledUpperTriangMaskedSoftmax.apply(x, 1.0)
    x4 = torch.zeros(1, 2, 8, 8, dtype=torch.bfloat16)
    m = torch.zeros(1, 1, 8, 8, dtype=torch.bool)
    with pytest.raises(RuntimeError, match="no CPU fallback"):
        fused_softmax.ScaledMaskedSoftmax.apply(x4, m, 1.0)
    mod = FusedScaleMaskSoftmax(False, True, SoftmaxFusionTypes.upper_triang, None, True, None)
    with pytest.raises(RuntimeError, match="no CPU fallback"):
        mod(x4, m)
    with pytest.raises(RuntimeError, match="no CPU fallback"):
        fused_rotary_positional_embedding.forward_cached(
            torch.zeros(4, 1, 2, 8, dtype=torch.float16), torch.zeros(4, 1, 1, 8), torch.zeros(4, 1, 1, 8)
        )


def test_extension_level_checks_mirror_the_reference_messages():
    causal, masked = scaled_upper_triang_masked_softmax_cuda, scaled_masked_softmax_cuda
    with pytest.raises(RuntimeError, match="expected 3D tensor"):
        causal.forward(torch.zeros(1, 2, 8, 8, dtype=torch.float16), 1.0)
    with pytest.raises(RuntimeError, match="Only fp16 and bf16 are supported"):
        causal.forward(torch.zeros(2, 8, 8), 1.0)
    with pytest.raises(RuntimeError, match="expected 3D tensor"):
        causal.backward(torch.zeros(8, 8, dtype=torch.float16), torch.zeros(8, 8, dtype=torch.float16), 1.0)
    with pytest.raises(RuntimeError, match="expected 4D tensor"):
        masked.forward(torch.zeros(2, 8, 8, dtype=torch.float16), torch.zeros(1, 1, 8, 8, dtype=torch.bool), 1.0)
    with pytest.raises(RuntimeError, match="Only fp16 and bf16 are supported"):
        masked.forward(torch.zeros(1, 2, 8, 8), torch.zeros(1, 1, 8, 8, dtype=torch.bool), 1.0)
    with pytest.raises(RuntimeError, match="expected 4D tensor"):
        masked.forward(torch.zeros(1, 2, 8, 8, dtype=torch.float16), torch.zeros(8, 8, dtype=torch.bool), 1.0)
    with pytest.raises(RuntimeError, match="mask"):
        masked.forward(torch.zeros(4, 2, 8, 8, dtype=torch.float16), torch.zeros(3, 1, 8, 8, dtype=torch.bool), 1.0)
    rope = fused_rotary_positional_embedding
    t = torch.zeros(4, 1, 2, 8, dtype=torch.float16)
    with pytest.raises(RuntimeError, match="same sequence length"):
        rope.forward_cached(t, torch.zeros(5, 1, 1, 8), torch.zeros(5, 1, 1, 8))
    with pytest.raises(RuntimeError, match="second and third dims"):
        rope.forward_cached(t, torch.zeros(4, 2, 1, 8), torch.zeros(4, 2, 1, 8))
    with pytest.raises(RuntimeError, match="greater than"):
        rope.forward_cached(t, torch.zeros(4, 1, 1, 16), torch.zeros(4, 1, 1, 16))
    with pytest.raises(RuntimeError, match="same dtype"):
        rope.forward_cached(t, torch.zeros(4, 1, 1, 8), torch.zeros(4, 1, 1, 8, dtype=torch.float16))
    with pytest.raises(RuntimeError, match="must be float"):
        rope.forward(t, torch.zeros(4, 1, 1, 8, dtype=torch.float16))


def test_load_fused_kernels_registers_the_reference_module_names():
    mods = load_fused_kernels()
    for name in ("scaled_upper_triang_masked_softmax_cuda", "scaled_masked_softmax_cuda",
                 "fused_rotary_positional_embedding"):
        assert name in sys.modules
    import scaled_masked_softmax_cuda as top  # the import statement the reference uses

    assert top is mods[1] and callable(top.forward) and callable(top.backward)
    assert callable(top.get_batch_per_block)


# ---- dispatcher ---------------------------------------------------------------------


def make(fusion, fp16=True, bf16=False, scale=None):
    return FusedScaleMaskSoftmax(fp16, bf16, fusion, lambda s, m: s, True, scale)


def test_is_kernel_available_table():
    mask = torch.zeros(1, 1, 4, 4, dtype=torch.bool)
    causal, general, none = (make(t) for t in (SoftmaxFusionTypes.upper_triang,
                                                SoftmaxFusionTypes.general, SoftmaxFusionTypes.none))
    # every benchmark shape takes the fused branch, including the 8192 one
    for b, np_, sq, sk in [(4, 12, 2048, 2048), (1, 64, 2048, 2048), (1, 32, 8192, 8192), (3, 5, 7, 7)]:
        assert causal.is_kernel_available(mask, b, np_, sq, sk)
    assert general.is_kernel_available(mask, 8, 16, 1024, 1024)
    assert general.is_kernel_available(mask, 1, 3, 1, 77)  # decode step, odd sizes
    # causal fusion with sq != sk (a step against a key/value cache): fused through the mask-tensor
    # kernel when the mask has that kernel's layout, otherwise the torch branch
    assert not causal.is_kernel_available(mask, 1, 4, 1, 77)
    assert causal.is_kernel_available(torch.zeros(1, 1, 1, 77, dtype=torch.bool), 1, 4, 1, 77)
    assert causal.is_kernel_available(torch.zeros(2, 1, 5, 77, dtype=torch.uint8), 2, 4, 5, 77)
    assert not causal.is_kernel_available(torch.zeros(3, 1, 5, 77, dtype=torch.bool), 2, 4, 5, 77)
    assert not causal.is_kernel_available(torch.zeros(1, 1, 5, 77), 2, 4, 5, 77)  # float mask
    assert not causal.is_kernel_available(None, 4, 12, 64, 64)  # no mask tensor
    assert not general.is_kernel_available(None, 4, 12, 64, 64)
    assert not none.is_kernel_available(mask, 4, 12, 64, 64)  # fusion not requested
    fp32 = FusedScaleMaskSoftmax(False, False, SoftmaxFusionTypes.general, None, True, None)
    assert not fp32.is_kernel_available(mask, 4, 12, 64, 64)  # fp32 input
    assert not general.is_kernel_available(mask, 0, 12, 64, 64)  # empty


def test_plain_causal_mask_detection_and_memo():
    from oracle import torch_ref as R

    mod = FusedScaleMaskSoftmax(True, False, SoftmaxFusionTypes.none, None, True, None)
    f = mod.mask_is_plain_causal
    plain = R.get_attn_mask(9)
    assert f(plain) and f(plain)
    assert f(plain.expand(3, 1, 9, 9).contiguous()) and f(plain.to(torch.uint8))
    assert not f(R.get_attn_mask(9, sliding_window_width=2))
    assert mod.classify_mask(R.get_attn_mask(9, sliding_window_width=2)) == 2
    assert mod.classify_mask(R.get_attn_mask(9, sliding_window_width=0)) == 0
    assert mod.classify_mask(R.get_attn_mask(9, sliding_window_width=8)) == "causal"  # the window hides nothing
    ragged = R.get_attn_mask(9, sliding_window_width=2).clone()
    ragged[0, 0, 7, 5] = True  # one row with a narrower window: no single width
    assert mod.classify_mask(ragged) is None
    assert not f(torch.zeros(1, 1, 9, 9, dtype=torch.bool))
    assert not f(plain[0])  # not 4-D
    per_sample = plain.expand(2, 1, 9, 9).clone()
    assert f(per_sample)
    per_sample[1, 0, 8, 0] = True  # version bump: the remembered verdict is dropped
    assert not f(per_sample)
    for _ in range(100):  # the memo stays bounded and correct under churn
        assert f(R.get_attn_mask(5))


def test_aliases_of_a_mask_share_its_verdict():
    # activation checkpointing detach()es its inputs for every recomputed segment: each layer
    # then sees a new tensor object over the same storage, which must not cost a new comparison
    from gpt_neox_amd import fused_softmax as fs
    from oracle import torch_ref as R

    mod = FusedScaleMaskSoftmax(True, False, SoftmaxFusionTypes.none, None, True, None)
    memo = fs._causal_memo
    plain = R.get_attn_mask(12)
    assert memo.lookup(plain) is None  # never asked
    assert mod.mask_is_plain_causal(plain)
    for alias in (plain.detach(), plain.view(1, 1, 12, 12), plain[:], plain.detach().detach()):
        assert alias is not plain and memo.lookup(alias) == "causal"
    assert memo.lookup(plain[..., :11, :11]) is None  # another region of the same storage
    assert memo.lookup(plain.clone()) is None          # another storage
    window = R.get_attn_mask(12, sliding_window_width=3)
    assert not mod.mask_is_plain_causal(window) and memo.lookup(window.detach()) == 3
    alias = plain.detach()
    alias[0, 0, 11, 0] = True  # a write through an alias bumps the shared version counter
    assert memo.lookup(plain) is None and not mod.mask_is_plain_causal(plain)
    # a recycled allocation is another storage object: no verdict is inherited
    addr = window.untyped_storage().data_ptr()
    del window, alias
    for _ in range(20):
        fresh = torch.zeros(1, 1, 12, 12, dtype=torch.bool)
        if fresh.untyped_storage().data_ptr() == addr:
            assert memo.lookup(fresh) is None
            break


def test_causal_mask_check_modes():
    from oracle import torch_ref as R

    def module(mode):
        return FusedScaleMaskSoftmax(True, False, SoftmaxFusionTypes.none, None, True, None, causal_mask_check=mode)

    window = R.get_attn_mask(7, sliding_window_width=2)
    assert not module("verify").mask_is_plain_causal(window)
    assert not module("lazy").mask_is_plain_causal(window)  # CPU masks are decided at once
    assert module("lazy").mask_is_plain_causal(R.get_attn_mask(7))
    assert module("trust").mask_is_plain_causal(window)  # the reference never reads the mask
    # the default never synchronises the host: the reference's causal branch does not either
    # (megatron/model/fused_softmax.py:173-179), and GPT-NeoX builds a fresh mask per micro-batch
    assert FusedScaleMaskSoftmax(True, False, SoftmaxFusionTypes.none, None, True, None).causal_mask_check == "lazy"
    with pytest.raises(AssertionError):
        module("sometimes")


def test_reference_predicate_restated():
    # megatron/model/fused_softmax.py:148-168 with wave64 batch_per_block (= 2 for sk > 128)
    ref = FusedScaleMaskSoftmax.reference_is_kernel_available
    m = object()
    assert ref(True, True, True, m, 4, 12, 2048, 2048)
    assert not ref(True, True, True, m, 1, 32, 8192, 8192)  # the 2048 cap
    assert not ref(True, True, True, m, 4, 12, 16, 16)  # sk must exceed 16
    assert not ref(True, True, True, m, 4, 12, 2046, 2046)  # sq % 4
    assert not ref(True, True, True, m, 1, 3, 64, 64)  # (b*np) % 4
    assert not ref(True, True, True, None, 4, 12, 64, 64)
    assert not ref(False, True, True, m, 4, 12, 64, 64)
    assert not ref(True, True, False, m, 4, 12, 64, 64)
    assert ref(True, False, True, m, 8, 16, 1024, 1024)
    assert ref(True, False, True, m, 1, 4, 4, 32) is False  # sq=4, batch_per_block=8 at sk=32


def test_constructor_contract():
    with pytest.raises(AssertionError, match="Invalid fusion type"):
        FusedScaleMaskSoftmax(True, False, "general", None, True, None)
    with pytest.raises(AssertionError, match="softmax should be in fp32 when scaled"):
        FusedScaleMaskSoftmax(True, False, SoftmaxFusionTypes.none, None, False, 2.0)
    m = make(SoftmaxFusionTypes.upper_triang, fp16=False, bf16=True, scale=3.0)
    assert m.input_in_float16 and m.upper_triang_mask_fusion and not m.general_mask_fusion
    assert m.fusion and m.scale == 3.0
    with pytest.raises(AssertionError):
        m(torch.zeros(2, 8, 8), None)  # input must be 4-D


def test_public_names_and_signatures_match_the_reference_modules():
    def params(fn):
        return list(inspect.signature(fn).parameters)

    # the reference's positional parameters, plus two optional keywords: checking without waiting, and
    # not fetching what lies behind a row's last visible key (which changes no result)
    assert params(FusedScaleMaskSoftmax.__init__) == [
        "self", "input_in_fp16", "input_in_bf16", "fusion_type", "mask_func", "softmax_in_fp32", "scale",
        "causal_mask_check", "skip_hidden_tails"]
    assert inspect.signature(FusedScaleMaskSoftmax.__init__).parameters["causal_mask_check"].default == "lazy"
    assert inspect.signature(FusedScaleMaskSoftmax.__init__).parameters["skip_hidden_tails"].default is True
    # the reference's positional parameters, plus three optional additions that default to "off"
    assert params(FusedScaleMaskSoftmax.forward) == ["self", "input", "mask", "alibi_slopes", "dropout_p", "bias"]
    assert inspect.signature(FusedScaleMaskSoftmax.forward).parameters["bias"].default is None
    assert inspect.signature(FusedScaleMaskSoftmax.forward).parameters["alibi_slopes"].default is None
    assert inspect.signature(FusedScaleMaskSoftmax.forward).parameters["dropout_p"].default == 0.0
    assert params(FusedScaleMaskSoftmax.is_kernel_available) == ["self", "mask", "b", "np", "sq", "sk"]
    assert params(FusedScaleMaskSoftmax.get_batch_per_block) == ["sq", "sk", "b", "np"]
    assert params(fused_softmax.ScaledUpperTriangMaskedSoftmax.forward) == ["ctx", "inputs", "scale"]
    assert params(fused_softmax.ScaledMaskedSoftmax.forward) == ["ctx", "inputs", "mask", "scale", "row_end"]
    assert inspect.signature(fused_softmax.ScaledMaskedSoftmax.forward).parameters["row_end"].default is None
    assert [e.name for e in SoftmaxFusionTypes] == ["upper_triang", "general", "none"]
    assert [e.value for e in SoftmaxFusionTypes] == [1, 2, 3]
    pe = positional_embeddings
    assert params(pe.RotaryEmbedding.__init__) == [
        "self", "dim", "max_seq_len", "base", "precision", "save_inv_freqs"]
    assert params(pe.RotaryEmbedding.forward) == ["self", "x", "seq_dim", "seq_len"]
    assert params(pe.apply_rotary_pos_emb) == ["q", "k", "cos", "sin", "offset"]
    assert params(pe.apply_rotary_pos_emb_torch) == ["q", "k", "cos", "sin", "offset"]
    assert params(pe.rotate_half) == ["x"]
    assert params(pe.SinusoidalPositionalEmbedding.__init__) == ["self", "dim", "base", "precision"]
    assert params(pe.AliBi.__init__) == ["self", "num_heads", "mp_size", "mp_rank"]
    for name in ("FusedScaleMaskSoftmax", "RotaryEmbedding", "apply_rotary_pos_emb_torch",
                 "apply_rotary_pos_emb", "AliBi", "SoftmaxFusionTypes", "SinusoidalPositionalEmbedding"):
        assert hasattr(gpt_neox_amd, name)


def test_header_is_plain_c_and_links_from_a_c_program(tmp_path):
    """The boundary is a C ABI: the header compiles as C99 on its own, and a C program that
    includes it links against the library and gets status codes back (argument errors are
    reported without a GPU)."""
    import shutil
    import subprocess

    gcc = shutil.which("gcc")
    if gcc is None:
        pytest.skip("no C compiler")
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    header = os.path.join(root, "include", "neox_fused.h")
    subprocess.run([gcc, "-std=c99", "-Wall", "-Wextra", "-Werror", "-pedantic", "-fsyntax-only", "-x", "c", header],
                   check=True)
    src = tmp_path / "abi.c"
    src.write_text(
        '#include <stdio.h>\n#include <string.h>\n#include "neox_fused.h"\n'
        "int main(void) {\n"
        "    unsigned short buf[64];\n"
        "    if (neox_fused_abi_version() != NEOX_FUSED_ABI_VERSION) return 1;\n"
        "    if (neox_causal_softmax_fwd(NULL, buf, 1.0f, 1, 8, 8, NEOX_F16, NULL) != NEOX_ERR_NULL_POINTER) return 2;\n"
        "    if (neox_masked_softmax_bwd(buf, buf, buf, 1.0f, 4, 8, 7, NULL) != NEOX_ERR_BAD_DTYPE) return 3;\n"
        '    if (strstr(neox_fused_last_error(), "fp16 and bf16") == NULL) return 4;\n'
        "    if (neox_get_batch_per_block(1024, 1024, 8, 16) != 2) return 5;\n"
        '    puts("c abi ok");\n'
        "    return 0;\n}\n"
    )
    exe = tmp_path / "abi"
    libdir = os.path.dirname(_lib.LIB_PATH)
    subprocess.run([gcc, "-std=c99", "-Wall", "-Werror", "-I", os.path.dirname(header), str(src), "-o", str(exe),
                    "-L", libdir, "-lneox_fused", f"-Wl,-rpath,{libdir}", "-Wl,-rpath,/opt/rocm/lib"], check=True)
    res = subprocess.run([str(exe)], stdout=subprocess.PIPE, text=True)
    assert res.returncode == 0 and "c abi ok" in res.stdout, (res.returncode, res.stdout)
