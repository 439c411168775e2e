"""ctypes binding of ``libneox_fused.so`` (the C-ABI declared in ``include/neox_fused.h``).

The library is built in-tree by ``make -C gpt-neox_amd/csrc`` (see :func:`build`).
There is no CPU or eager fallback behind these calls: if the shared object is
missing or cannot be loaded, :func:`lib` raises ``ImportError``; if a tensor is
not on the GPU, the wrappers raise ``RuntimeError``.
"""
import ctypes
import os
import subprocess
import threading

import torch

_CSRC = os.path.join(os.path.dirname(os.path.abspath(__file__)), "csrc")
LIB_PATH = os.path.join(_CSRC, "libneox_fused.so")
ABI_VERSION = 4

NEOX_F16, NEOX_BF16, NEOX_F32 = 0, 1, 2
_DTYPE_CODE = {torch.float16: NEOX_F16, torch.bfloat16: NEOX_BF16, torch.float32: NEOX_F32}

_c_i64p = ctypes.POINTER(ctypes.c_int64)
_vp, _i32, _i64, _f32 = ctypes.c_void_p, ctypes.c_int32, ctypes.c_int64, ctypes.c_float
_u64 = ctypes.c_uint64

# name -> (restype, argtypes); one entry per declaration of include/neox_fused.h
SIGNATURES = {
    "neox_fused_abi_version": (ctypes.c_int, []),
    "neox_fused_strerror": (ctypes.c_char_p, [ctypes.c_int]),
    "neox_fused_last_error": (ctypes.c_char_p, []),
    "neox_causal_softmax_fwd": (ctypes.c_int, [_vp, _vp, _f32, _i64, _i32, _i32, _i32, _vp]),
    "neox_causal_softmax_alibi_fwd": (
        ctypes.c_int, [_vp, _vp, _vp, _f32, _i32, _i32, _i32, _i32, _i32, _vp]
    ),
    "neox_causal_softmax_bwd": (ctypes.c_int, [_vp, _vp, _vp, _f32, _i64, _i32, _i32, _i32, _vp]),
    "neox_masked_softmax_fwd": (
        ctypes.c_int,
        [_vp, _vp, _vp, _f32, _i32, _i32, _i32, _i32, _i32, _i32, _vp],
    ),
    "neox_masked_softmax_bwd": (ctypes.c_int, [_vp, _vp, _vp, _f32, _i64, _i32, _i32, _vp]),
    "neox_masked_softmax_alibi_fwd": (
        ctypes.c_int, [_vp, _vp, _vp, _vp, _f32, _i32, _i32, _i32, _i32, _i32, _i32, _vp]
    ),
    "neox_causal_softmax_bias_fwd": (
        ctypes.c_int, [_vp, _vp, _vp, _vp, _f32, _i32, _i32, _i32, _i32, _i32, _i32, _vp]
    ),
    "neox_masked_softmax_bias_fwd": (
        ctypes.c_int,
        [_vp, _vp, _vp, _vp, _vp, _f32, _i32, _i32, _i32, _i32, _i32, _i32, _i32, _vp],
    ),
    "neox_sliding_window_softmax_fwd": (ctypes.c_int, [_vp, _vp, _f32, _i64, _i32, _i32, _i32, _i32, _vp]),
    "neox_sliding_window_softmax_bwd": (ctypes.c_int, [_vp, _vp, _vp, _f32, _i64, _i32, _i32, _i32, _i32, _vp]),
    "neox_mask_classify": (ctypes.c_int, [_vp, _vp, _i32, _i32, _i32, _vp]),
    "neox_causal_softmax_dropout_fwd": (
        ctypes.c_int,
        [_vp, _vp, _vp, _vp, _vp, _i32, _f32, _f32, _u64, _u64, _vp, _i32, _i32, _i32, _i32, _i32, _vp],
    ),
    "neox_causal_softmax_dropout_bwd": (
        ctypes.c_int, [_vp, _vp, _vp, _f32, _f32, _u64, _u64, _vp, _i64, _i32, _i32, _i32, _vp]
    ),
    "neox_masked_softmax_dropout_fwd": (
        ctypes.c_int,
        [_vp, _vp, _vp, _vp, _vp, _vp, _i32, _f32, _f32, _u64, _u64, _vp, _i32, _i32, _i32, _i32, _i32, _i32,
         _vp],
    ),
    "neox_masked_softmax_ends_fwd": (
        ctypes.c_int,
        [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _i32, _f32, _f32, _u64, _u64, _vp, _i32, _i32, _i32, _i32, _i32, _i32,
         _vp],
    ),
    "neox_masked_softmax_ends_bwd": (
        ctypes.c_int,
        [_vp, _vp, _vp, _vp, _f32, _i32, _f32, _u64, _u64, _vp, _i32, _i32, _i32, _i32, _i32, _i32, _vp],
    ),
    "neox_mask_scan": (ctypes.c_int, [_vp, _vp, _vp, _i32, _i32, _i32, _vp]),
    "neox_masked_softmax_dropout_bwd": (
        ctypes.c_int, [_vp, _vp, _vp, _f32, _f32, _u64, _u64, _vp, _i64, _i32, _i32, _vp]
    ),
    "neox_dropout_keep_mask": (ctypes.c_int, [_vp, _f32, _u64, _u64, _vp, _i64, _vp]),
    "neox_get_batch_per_block": (ctypes.c_int, [_i32, _i32, _i32, _i32]),
    "neox_rope_apply": (
        ctypes.c_int,
        [_vp, _vp, _vp, _vp, _vp, _vp, _i32, _i32, _i32, _i32, _i32, _i32, _c_i64p, _c_i64p, _c_i64p,
         _c_i64p, _i64, _i32, _i32, _i32, _i32, _vp],
    ),
    "neox_rope_apply_freqs": (
        ctypes.c_int,
        [_vp, _vp, _vp, _vp, _vp, _i32, _i32, _i32, _i32, _i32, _i32, _c_i64p, _c_i64p, _c_i64p,
         _c_i64p, _i64, _i32, _i32, _i32, _vp],
    ),
}

_lock = threading.Lock()
_lib = None


def build(verbose=False, targets=("all",)):
    """Compile ``libneox_fused.so`` for gfx950 with hipcc (works without a GPU).  ``targets``:
    make targets; ``"probes"`` is the benchmark's copy kernel, a library of its own."""
    cmd = ["make", "-C", _CSRC, "-j8", "-B", *targets]
    res = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    if verbose or res.returncode != 0:
        print(res.stdout)
    if res.returncode != 0:
        raise RuntimeError("building libneox_fused.so failed (see output above)")
    return LIB_PATH


def lib():
    """Return the loaded library, loading it on first use."""
    global _lib
    if _lib is not None:
        return _lib
    with _lock:
        if _lib is not None:
            return _lib
        if not os.path.exists(LIB_PATH):
            raise ImportError(
                f"{LIB_PATH} not found: the fused kernels are not built. "
                "Run `make -C gpt-neox_amd/csrc` (or __graft_entry__.build())."
            )
        try:
            handle = ctypes.CDLL(LIB_PATH)
        except OSError as exc:  # unresolved HIP runtime, wrong arch, ...
            raise ImportError(f"cannot load {LIB_PATH}: {exc}") from exc
        for name, (restype, argtypes) in SIGNATURES.items():
            try:
                fn = getattr(handle, name)
            except AttributeError as exc:
                raise ImportError(f"{LIB_PATH} does not export {name}") from exc
            fn.restype = restype
            fn.argtypes = argtypes
        got = handle.neox_fused_abi_version()
        if got != ABI_VERSION:
            raise ImportError(f"{LIB_PATH}: ABI version {got}, expected {ABI_VERSION}")
        _lib = handle
    return _lib


def check(status):
    """Turn a negative neox_status into ``RuntimeError`` (as torch's checks do)."""
    if status != 0:
        handle = lib()
        msg = handle.neox_fused_last_error().decode() or handle.neox_fused_strerror(status).decode()
        raise RuntimeError(msg)


def dtype_code(dtype):
    try:
        return _DTYPE_CODE[dtype]
    except KeyError:
        raise RuntimeError("Only fp16 and bf16 are supported") from None


def require_gpu(*tensors):
    for t in tensors:
        if t is not None and not t.is_cuda:
            raise RuntimeError(
                "fused kernels need GPU tensors (got a tensor on %s); there is no CPU fallback"
                % t.device
            )


class _NoGuard:
    def __enter__(self):
        return None

    def __exit__(self, *exc):
        return False


_no_guard = _NoGuard()


def device_guard(tensor):
    """Context that makes the tensor's device current for the launch; a no-op object when it
    already is (the usual case: one process per GPU), which saves a few microseconds per call."""
    if tensor.device.index == torch.cuda.current_device():
        return _no_guard
    return torch.cuda.device(tensor.device)


try:  # the raw handle of torch's current stream without building a Stream object (a few us less)
    _raw_stream = torch._C._cuda_getCurrentRawStream
except AttributeError:  # pragma: no cover - older/newer torch without the private accessor
    _raw_stream = None


def current_stream(tensor):
    """hipStream_t of torch's current stream on the tensor's device, as an integer."""
    if _raw_stream is not None:
        return _raw_stream(tensor.device.index)
    return torch.cuda.current_stream(tensor.device).cuda_stream


_strides3_cache = {}


def strides3(t):
    """First three element strides of a 4-D tensor as a C int64[3] (read-only for the callee, so
    one array per distinct stride triple is kept and reused)."""
    s = t.stride()
    key = (s[0], s[1], s[2])
    arr = _strides3_cache.get(key)
    if arr is None:
        if len(_strides3_cache) > 4096:
            _strides3_cache.clear()
        arr = _strides3_cache[key] = (ctypes.c_int64 * 3)(*key)
    return arr
