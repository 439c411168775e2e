"""Random-number plumbing of the fused softmax + attention-dropout kernels.

The reference applies ``torch.nn.Dropout`` to the attention probabilities inside
``mpu.get_cuda_rng_tracker().fork()`` (megatron/model/transformer.py:536-539,
megatron/mpu/random.py:20-37): the tracker swaps the model-parallel RNG state into the
device's default generator for the duration of the block.  The fused kernels draw their
keep pattern from that same generator: :func:`take_philox_state` reads its
``(seed, offset)`` and advances the offset, exactly as a torch random kernel would, so the
call composes with the tracker, with ``torch.manual_seed`` and with checkpointed RNG
states, and never reuses random bits of another consumer.
"""
import torch

from .. import _lib

# One Philox counter value per group of 8 elements is consumed at the offset taken;
# torch keeps generator offsets at multiples of 4.
OFFSET_STEP = 4


def take_philox_state(device):
    """``(seed, offset)`` of ``device``'s default generator; the generator moves on by
    ``OFFSET_STEP``.  Not usable while a HIP graph is being captured (the state would be
    frozen into the graph): the caller falls back to softmax followed by torch's dropout."""
    device = torch.device(device)
    index = device.index if device.index is not None else torch.cuda.current_device()
    gen = torch.cuda.default_generators[index]
    seed = gen.initial_seed()
    offset = gen.get_offset()
    gen.set_offset(offset + OFFSET_STEP)
    return seed, offset


def keep_mask(n, p, seed, offset, device):
    """The keep pattern the dropout kernels use for a tensor of ``n`` elements (row-major),
    as a bool tensor ``[n]`` on ``device`` (True = kept)."""
    device = torch.device(device)
    if device.type != "cuda":
        raise RuntimeError("fused kernels need a GPU device; there is no CPU fallback")
    out = torch.empty(n, dtype=torch.uint8, device=device)
    if n == 0:
        return out.bool()
    with torch.cuda.device(device):
        _lib.check(
            _lib.lib().neox_dropout_keep_mask(
                out.data_ptr(), float(p), int(seed), int(offset), n,
                torch.cuda.current_stream(device).cuda_stream,
            )
        )
    return out.bool()
