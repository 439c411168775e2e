"""MI355X-native fused softmax and rotary-embedding path of GPT-NeoX.

``fused_softmax`` and ``positional_embeddings`` are drop-ins for the reference
modules of the same names under ``megatron/model``; ``fused_rope`` mirrors
``megatron/model/fused_rope.py``; ``fused_kernels`` mirrors the loader and the three
extension-module APIs of ``megatron/fused_kernels``.  All of them call ONE C-ABI
library, ``csrc/libneox_fused.so`` (declared in ``include/neox_fused.h``), through
``_lib``; there is no CPU or eager fallback for the fused calls.

The directory is named ``gpt-neox_amd``; import it as ``gpt_neox_amd`` (the module
``gpt_neox_amd.py`` at the repository root registers the alias).
"""
from . import _lib  # noqa: F401
from .fused_softmax import (  # noqa: F401
    FusedScaleMaskSoftmax,
    ScaledMaskedSoftmax,
    ScaledUpperTriangMaskedSoftmax,
    SoftmaxFusionTypes,
)
from .positional_embeddings import (  # noqa: F401
    AliBi,
    RotaryEmbedding,
    SinusoidalPositionalEmbedding,
    apply_rotary_pos_emb,
    apply_rotary_pos_emb_,
    apply_rotary_pos_emb_qkv_,
    apply_rotary_pos_emb_torch,
    rotate_half,
)

__all__ = [
    "FusedScaleMaskSoftmax",
    "ScaledMaskedSoftmax",
    "ScaledUpperTriangMaskedSoftmax",
    "SoftmaxFusionTypes",
    "AliBi",
    "RotaryEmbedding",
    "SinusoidalPositionalEmbedding",
    "apply_rotary_pos_emb",
    "apply_rotary_pos_emb_",
    "apply_rotary_pos_emb_qkv_",
    "apply_rotary_pos_emb_torch",
    "rotate_half",
]
