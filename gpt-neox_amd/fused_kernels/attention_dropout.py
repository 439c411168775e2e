"""Random-number plumbing of the fused softmax + attention-dropout kernels.

The reference applies ``torch.nn.Dropout`` to the attention probabilities inside
``mpu.get_cuda_rng_tracker().fork()`` (megatron/model/transformer.py:536-539,
megatron/mpu/random.py:20-37): the tracker swaps the model-parallel RNG state into the
device's default generator for the duration of the block.  The fused kernels draw their
keep pattern from that same generator: :func:`take_philox_state` reads its
``(seed, offset)`` and advances the offset, exactly as a torch random kernel would, so the
call composes with the tracker, with ``torch.manual_seed`` and with checkpointed RNG
states, and never reuses random bits of another consumer.  Launches recorded into a HIP
graph follow a device-resident copy of that state instead (:func:`graph_state`).
"""
import torch

from .. import _lib

# A generator offset counts 32-bit outputs, four to a Philox counter value; a fused call draws
# every group's block at the one counter value offset / 4 and so owns the offsets
# [offset, offset + 4).  torch keeps generator offsets at multiples of 4.
OFFSET_STEP = 4
# Offsets drawn from the device-resident state (HIP graphs) start far above anything the
# host-side generator reaches, so the two never draw from the same counter.
GRAPH_OFFSET_BASE = 1 << 62

_graph_states = {}  # device index -> int64 tensor [seed, offset] on that device


def _index(device):
    device = torch.device(device)
    return device.index if device.index is not None else torch.cuda.current_device()


def graph_state(device, reseed=False):
    """The device-resident ``[seed, offset]`` that dropout launches recorded into a HIP graph
    follow.  Call it once *before* capturing (creating it needs a host-to-device copy); it is
    seeded from ``device``'s default generator -- ``reseed=True`` does that again, e.g. after
    ``torch.manual_seed``.  Every captured call snapshots the state and advances the stored
    offset with two small device operations that become part of the graph, so each replay draws
    a fresh pattern and a captured backward pass sees its forward pass's pattern."""
    index = _index(device)
    state = _graph_states.get(index)
    if state is None or reseed:
        if torch.cuda.is_current_stream_capturing():
            raise RuntimeError(
                "attention_dropout.graph_state(device) must be called once before a HIP graph "
                "with fused softmax+dropout is captured"
            )
        gen = torch.cuda.default_generators[index]
        # int64 holds the low 63 bits of the seed; the kernels use them as an unsigned key
        values = [gen.initial_seed() & ((1 << 63) - 1), GRAPH_OFFSET_BASE + gen.get_offset()]
        fresh = torch.tensor(values, dtype=torch.int64, device=torch.device("cuda", index))
        if state is None:
            _graph_states[index] = state = fresh
        else:
            state.copy_(fresh)  # graphs captured earlier keep following the same tensor
    return state


def take_philox_state(device):
    """``(seed, offset, state)`` for one fused dropout call on ``device``.

    Eagerly: ``(seed, offset)`` of the device's default generator, which moves on by
    ``OFFSET_STEP``, and ``state = None``.  While a HIP graph is being captured the numbers
    would be frozen into the graph, so the call gets ``state``, a snapshot (device tensor) of
    :func:`graph_state` taken by the graph itself, and the stored offset moves on inside the
    graph; ``seed`` and ``offset`` are then 0 and unused."""
    index = _index(device)
    if torch.cuda.is_current_stream_capturing():
        live = graph_state(index)
        snapshot = live.clone()
        live[1:].add_(OFFSET_STEP)
        return 0, 0, snapshot
    gen = torch.cuda.default_generators[index]
    seed = gen.initial_seed()
    offset = gen.get_offset()
    gen.set_offset(offset + OFFSET_STEP)
    return seed, offset, None


def state_pointer(state):
    """Device address of a ``[seed, offset]`` tensor for the C-ABI, or None."""
    if state is None:
        return None
    if not (state.is_cuda and state.dtype == torch.int64 and state.numel() == 2 and state.is_contiguous()):
        raise RuntimeError("dropout state must be a contiguous int64 device tensor [seed, offset]")
    return state.data_ptr()


def keep_mask(n, p, seed, offset, device, state=None):
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
                out.data_ptr(), float(p), int(seed), int(offset), state_pointer(state), n,
                torch.cuda.current_stream(device).cuda_stream,
            )
        )
    return out.bool()
