"""Loader of the fused kernels, with the reference loader's entry points.

Reference: megatron/fused_kernels/__init__.py:35-192 JIT-builds three pybind
extensions with torch's cpp_extension (hipifying the CUDA sources on ROCm) and
``load_fused_kernels()`` verifies that they import, calling ``exit()`` if not.
Here the three extension APIs are thin Python modules over ONE prebuilt C-ABI
library of hand-written gfx950 kernels, so

* ``load()`` compiles that library with hipcc if it is not built yet and registers the
  extension-named modules, as the reference's JIT load leaves them importable;
* ``load_fused_kernels()`` loads it, raises ``ImportError`` if that fails (no
  ``exit()``), and registers the modules under the reference's top-level names
  so that code doing ``import scaled_masked_softmax_cuda`` finds them.
"""
import os
import sys

from .. import _lib

_EXTENSION_NAMES = (
    "scaled_upper_triang_masked_softmax_cuda",
    "scaled_masked_softmax_cuda",
    "fused_rotary_positional_embedding",
)


def load(neox_args=None):
    """Make sure the shared library exists; build it in-tree if it does not.

    ``neox_args`` is accepted for signature compatibility; its
    ``fused_kernels_build_path`` is not used because the library lives next to its sources.
    """
    if not os.path.exists(_lib.LIB_PATH):
        rank = getattr(neox_args, "rank", 0) if neox_args is not None else 0
        if rank == 0:
            _lib.build()
    if os.path.exists(_lib.LIB_PATH):
        # the reference's JIT load leaves the three extensions importable by name; so does this
        load_fused_kernels()
    return _lib.LIB_PATH


def load_fused_kernels():
    """Check that the kernels are usable; register the extension-named modules."""
    _lib.lib()  # ImportError if the library is absent or broken
    from . import fused_rotary_positional_embedding as rope
    from . import scaled_masked_softmax_cuda as masked
    from . import scaled_upper_triang_masked_softmax_cuda as causal

    for name, mod in zip(_EXTENSION_NAMES, (causal, masked, rope)):
        sys.modules.setdefault(name, mod)
    return causal, masked, rope
