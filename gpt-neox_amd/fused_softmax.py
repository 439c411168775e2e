"""Drop-in for ``megatron/model/fused_softmax.py`` on MI355X.

Public names, constructor arguments, call signatures and tensor layouts are those
of the reference module (megatron/model/fused_softmax.py:24-205):

* ``ScaledUpperTriangMaskedSoftmax.apply(inputs[B, sq, sk], scale)``
* ``ScaledMaskedSoftmax.apply(inputs[b, np, sq, sk], mask[1|b, 1, sq, sk], scale)``
* ``SoftmaxFusionTypes``
* ``FusedScaleMaskSoftmax(input_in_fp16, input_in_bf16, fusion_type, mask_func,
  softmax_in_fp32, scale)`` with ``forward(input, mask)``, ``is_kernel_available``,
  ``forward_fused_softmax``, ``forward_torch_softmax``, ``get_batch_per_block``.

The fused branches run hand-written gfx950 kernels through the C-ABI library; the
unfused branch evaluates the same torch expression as the reference.

Deliberate differences from the reference:

* the fused kernels take any ``sk`` (the reference stops at 2048 and silently
  runs the torch path beyond it) and need none of the ``sq % 4``,
  ``attn_batches % 4`` or ``% batch_per_block`` divisibility rules, which were
  artefacts of the CUDA launch shape -- see :meth:`is_kernel_available`;
* by default the causal branch finds out once per mask (per storage region, so ``detach()``ed
  aliases share the verdict) whether the mask really is the plain upper-triangular one, the
  causal mask with a sliding window (served by a kernel that skips everything outside the
  band) or something else (packed-sequence masks, ...: the mask-tensor kernel with the mask it
  was given) -- the reference's causal kernel ignores the mask's contents, so above its 2048
  limit (torch path) and below it (fused kernel) the reference computes two different things
  for such masks; here both agree with the torch path.  The constructor's
  ``causal_mask_check`` selects how: ``"lazy"`` (default) never synchronises -- one small
  kernel reads the mask the first time it is seen, and calls made while its answer is in flight
  run the mask-tensor kernel, which is right for any mask --, ``"verify"`` waits for that answer
  (one host synchronisation per new mask), and ``"trust"`` restores the reference's behaviour of
  never reading the mask (megatron/model/fused_softmax.py:173-179).  A causal-fusion call with ``sq != sk`` (a step
  against a key/value cache, where the reference asserts) also runs the mask-tensor kernel.  The
  general fusion uses the same verdicts for square masks (never on trust), and whatever call the
  mask-tensor kernel serves tells it where every mask row's visible keys end once the same scan has
  found that worthwhile (``skip_hidden_tails``): the padding of a batch is then neither fetched nor
  computed, with the same bits as before;
* masked scores are excluded, so their probability is exactly 0 as in the torch
  path (the reference's padded kernel fills -10000), and a fully masked row is
  uniform ``1/sk`` as in the torch path;
* ``scale`` is applied in fp32 (the reference's forward narrows it to fp16/bf16);
* a missing kernel library raises ``ImportError`` instead of calling ``exit()``.

Additions (all optional, off by default): ``FusedScaleMaskSoftmax.forward`` also takes
``alibi_slopes``, ``bias`` and ``dropout_p``, which fold the ALiBi bias, an additive bias
tensor (relative-position bias) and the attention dropout that follows the softmax
(megatron/model/transformer.py:526-539) into the softmax kernels; the autograd Functions
``ScaledUpperTriangMaskedSoftmaxAlibi``, ``Scaled*SoftmaxBias`` and ``Scaled*SoftmaxDropout``
are their building blocks.
"""
import ctypes
import enum
import weakref

import torch

from .fused_kernels import attention_dropout as _rng
from .fused_kernels import load_fused_kernels
from .fused_kernels import scaled_masked_softmax_cuda as _masked_ext
from .fused_kernels import scaled_upper_triang_masked_softmax_cuda as _causal_ext


def alibi_bias(slopes, sq, sk, device, dtype):
    """The ALiBi bias ``[np, sq, sk]`` (``[np, 1, sk]`` for a one-query decode step) as the
    reference's ``AliBi`` module builds it, in ``dtype``: ``-slope_h * (i - j)`` for ``j <= i``,
    0 above the diagonal (megatron/model/positional_embeddings.py:161-206)."""
    rows = torch.arange(sk, device=device).view(sk, 1)
    cols = torch.arange(sk, device=device).view(1, sk)
    dist = (-torch.tril(rows - cols)).to(dtype)
    bias = dist * slopes.to(device=device, dtype=dtype).view(-1, 1, 1)
    if sq != sk:
        assert sq == 1, "assumption sq == sk unless at inference time with cache in layer_past with sq == 1"
        bias = bias[:, sk - 1, :].view(bias.shape[0], 1, sk)
    return bias


def _fp32(scale):
    """``scale`` rounded to fp32, as a Python float: the value the kernels receive in both
    passes.  (The reference keeps it as a one-element fp32 CPU tensor next to the saved
    probabilities, megatron/model/fused_softmax.py:36-41; a float on ``ctx`` costs the host a
    few microseconds less per call.)"""
    return ctypes.c_float(scale).value


def _remember(ctx, probs, scale):
    ctx.save_for_backward(probs)
    ctx.scale = scale
    return probs


def _recall(ctx):
    (probs,) = ctx.saved_tensors
    return probs, ctx.scale


class _MaskVerdict:
    """One remembered mask region: the storage it lives in (weakly), the version counter it had,
    and what is known about it -- ``verdict``: ``"causal"``, a sliding-window width (int) or False for
    any other mask; ``ends``: where every row's visible keys end (the ``row_end`` hint of the
    mask-tensor kernels, a device tensor) if that saves a sixteenth of the keys or more, else None.
    Both are None while the device-side scan is still running (then ``pending`` holds the pinned
    result slot, the event that follows the copy, the hint, the number of keys of the mask and the
    stream the scan runs on)."""

    __slots__ = ("storage", "version", "verdict", "ends", "stream", "pending")

    def __init__(self, storage, version, verdict=None, pending=None):
        self.storage = weakref.ref(storage)
        self.version = version
        self.verdict = verdict
        self.ends = None
        self.stream = None  # the stream the scan ran on, whose allocator pool holds ``ends``
        self.pending = pending

    def poll(self, wait):
        """The verdict if it is known by now.  ``wait``: True blocks until it is, False asks the
        event, None does not touch the event at all (for use while a HIP graph is captured)."""
        if self.verdict is None and self.pending is not None and wait is not None:
            slot, event, ends, keys, self.stream = self.pending
            if wait:
                event.synchronize()
            if wait or event.query():
                # host memory, the copy has finished: no synchronisation
                record = slot.tolist()
                self.verdict = _masked_ext.decode_mask_record(record)
                # the kernels that read no mask serve the causal kinds; for the others the hint is
                # kept when it spares the forward pass a sixteenth of its keys or more
                if self.verdict is False and 16 * _masked_ext.hidden_tail_keys(record) >= keys:
                    self.ends = ends
                self.pending = None
        return self.verdict

    def facts(self, wait):
        """``(verdict, ends, stream of the scan)``, or None while they are on their way."""
        return None if self.poll(wait) is None else (self.verdict, self.ends, self.stream)

    def early_ends(self, stream):
        """The hint of a scan that is still on its way, for a launch on the stream the scan runs on: the
        launch follows the scan there and finds the array filled, whatever the host knows by then."""
        if self.pending is None or self.pending[4] != stream:
            return None
        return self.pending[2]


class _CausalMaskMemo:
    """Remembers, per mask region, whether it is the causal mask ``triu(ones, 1)``, the causal mask
    with a sliding window, or something else.

    A region is (storage address, offset, shape, strides); an entry is valid while the storage
    object it was decided for is alive (weak reference -- a recycled allocation is another
    storage object and cannot inherit a verdict) and the tensor's version counter is unchanged
    (in-place writes bump it).  Aliases of one mask -- ``mask.detach()``, which activation
    checkpointing applies to its inputs for every recomputed segment, or an equal view --
    share the storage, the region and the version counter, hence the verdict.  (A write through
    ``.data`` or from outside torch bumps no counter and is not seen.)

    The classification is one kernel on the mask's device and stream that reads the mask once
    (``neox_mask_scan``; it also notes where every row's visible keys end, the hint that spares the
    mask-tensor kernels the hidden tail of a padded row), followed by a 32-byte copy into pinned
    memory and an event.
    ``classify(mask, wait=True)`` waits for it (one host synchronisation per new mask); with
    ``wait=False`` it returns None while the result is on its way and the caller uses a kernel
    that is right for any mask in the meantime."""

    def __init__(self, limit=64):
        self._entries = {}
        self._limit = limit
        self._slots = None  # pinned result slots, handed out in turn
        self._slot_owner = None  # per slot: the entry whose verdict it holds or will hold
        self._next_slot = 0

    @staticmethod
    def _key(mask):
        storage = mask.untyped_storage()
        return (storage.data_ptr(), mask.storage_offset(), tuple(mask.shape), mask.stride()), storage

    def _entry(self, mask):
        key, storage = self._key(mask)
        hit = self._entries.get(key)
        if hit is not None and hit.storage() is storage and hit.version == mask._version:
            return hit
        return None

    def lookup(self, mask, wait=False):
        """The verdict for this region in its current version, or None if it is unknown (never
        asked, or still being computed and ``wait`` is not True; see ``_MaskVerdict.poll``)."""
        hit = self._entry(mask)
        return None if hit is None else hit.poll(wait)

    def lookup_facts(self, mask, wait=False):
        """``(verdict, ends, stream)`` likewise."""
        hit = self._entry(mask)
        return None if hit is None else hit.facts(wait)

    def early_ends(self, mask):
        """See ``_MaskVerdict.early_ends``; None for a mask without a scan on its way."""
        hit = self._entry(mask)
        return None if hit is None else hit.early_ends(_masked_ext.launch_stream(mask))

    def _result_slot(self, entry):
        """Eight pinned host words for the record of ``entry``.  The slots are handed out in turn; an
        entry that still waits for the slot's previous content reads it first (its copy finished
        long ago), so a slot is never overwritten under an entry that has not looked yet."""
        if self._slots is None:
            self._slots = torch.zeros(256, 8, dtype=torch.int32, pin_memory=True)
            self._slot_owner = [None] * self._slots.shape[0]
        self._next_slot = (self._next_slot + 1) % self._slots.shape[0]
        owner = self._slot_owner[self._next_slot]
        if owner is not None:
            owner.poll(wait=True)
        self._slot_owner[self._next_slot] = entry
        return self._slots[self._next_slot]

    @staticmethod
    def _classify_on_host(mask):
        """The same verdict for a mask in host memory (plain torch)."""
        s = mask.shape[-1]
        hidden = mask.reshape(-1, s, s) != 0
        rows = torch.arange(s).view(s, 1)
        cols = torch.arange(s).view(1, s)
        if bool((hidden == (cols > rows)).all()):
            return "causal"
        first = (~hidden[0]).float().argmax(-1)  # first visible key of every row of the first sample
        widths = (torch.arange(s) - first)[first > 0]
        if widths.numel() and bool((widths == widths[0]).all()):
            w = int(widths[0])
            if bool((hidden == ((cols > rows) | (cols < rows - w))).all()):
                return w
        return False

    def classify(self, mask, wait=True):
        """``"causal"``, a window width, False, or None (still running and ``wait`` is False)."""
        return self._scan(mask).poll(wait)

    def facts(self, mask, wait=True):
        """``(verdict, ends, stream)`` of ``_MaskVerdict``, or None (still running and ``wait`` is False)."""
        return self._scan(mask).facts(wait)

    def _scan(self, mask):
        """The entry of ``mask`` ``[mask_b, 1, sq, sk]``, started now if there is none."""
        hit = self._entry(mask)
        if hit is not None:
            return hit
        key, storage = self._key(mask)
        if mask.is_cuda:
            record, ends = _masked_ext.scan_mask(mask)
            entry = _MaskVerdict(storage, mask._version)
            slot = self._result_slot(entry)
            with torch.cuda.device(mask.device):  # copy and event on the mask's device and stream
                slot.copy_(record, non_blocking=True)
                event = torch.cuda.Event()
                event.record()
            entry.pending = (slot, event, ends, mask.numel(), _masked_ext.launch_stream(mask))
        else:
            square = mask.shape[-1] == mask.shape[-2]
            entry = _MaskVerdict(storage, mask._version, verdict=self._classify_on_host(mask) if square else False)
        if len(self._entries) >= self._limit:
            self._entries = {k: v for k, v in self._entries.items() if v.storage() is not None}
            if len(self._entries) >= self._limit:
                self._entries.clear()
        self._entries[key] = entry
        return entry

    def is_plain_causal(self, mask, wait=True):
        verdict = self.classify(mask, wait)
        return None if verdict is None else verdict == "causal"


_causal_memo = _CausalMaskMemo()


class ScaledUpperTriangMaskedSoftmax(torch.autograd.Function):
    """scale -> causal (upper-triangular) mask -> softmax, in one kernel.

    ``inputs``: ``[attn_batches, sq, sk]`` fp16/bf16 on the GPU; returns probabilities
    of the same shape and dtype with exact zeros above the diagonal.  The gradient
    kernel writes into the incoming gradient buffer when it is contiguous, as the
    reference does.  Reference: megatron/model/fused_softmax.py:24-53.
    """

    @staticmethod
    def forward(ctx, inputs, scale):
        scale = _fp32(scale)
        return _remember(ctx, _causal_ext.forward(inputs, scale), scale)

    @staticmethod
    def backward(ctx, output_grads):
        probs, scale = _recall(ctx)
        return _causal_ext.backward(output_grads, probs, scale), None


class _CausalSoftmax4D(torch.autograd.Function):
    """``ScaledUpperTriangMaskedSoftmax`` on ``[b, np, sq, sk]`` as the module holds it.  The
    reference views the scores to three dims and the probabilities back
    (megatron/model/fused_softmax.py:173-179); here the leading dims simply count as batches, which
    spares the autograd graph two view nodes -- about 15 us of host time per forward + backward."""

    @staticmethod
    def forward(ctx, inputs, scale):
        if not inputs.is_contiguous():
            inputs = inputs.contiguous()
        return _remember(ctx, _causal_ext.forward_nd(inputs, scale), scale)

    @staticmethod
    def backward(ctx, output_grads):
        probs, scale = _recall(ctx)
        if not output_grads.is_contiguous():
            output_grads = output_grads.contiguous()
        return _causal_ext.backward_nd(output_grads, probs, scale), None


class ScaledUpperTriangMaskedSoftmaxAlibi(torch.autograd.Function):
    """Causal softmax of ``scale * (inputs + alibi_bias(slopes))`` in one kernel; the bias is
    computed from the per-head slopes inside the kernel instead of being added to the scores
    in a pass of its own (megatron/model/transformer.py:529-534).

    ``inputs``: ``[b, np, sq, sk]`` fp16/bf16; ``slopes``: ``[np]``.  Gradient with respect to
    ``inputs`` only (the bias is a constant)."""

    @staticmethod
    def forward(ctx, inputs, slopes, scale):
        scale = _fp32(scale)
        return _remember(ctx, _causal_ext.forward_alibi(inputs, slopes, scale), scale)

    @staticmethod
    def backward(ctx, output_grads):
        probs, scale = _recall(ctx)
        if not output_grads.is_contiguous():
            output_grads = output_grads.contiguous()
        return _causal_ext.backward_nd(output_grads, probs, scale), None, None


def _bias_gradient(grads, bias_shape):
    """Gradient of an additive bias from the gradient of the scores: the bias is broadcast
    over the batch dimension when its first dimension is 1."""
    if bias_shape[0] == 1 and grads.shape[0] != 1:
        return grads.sum(dim=0, keepdim=True)
    return grads


class ScaledUpperTriangMaskedSoftmaxBias(torch.autograd.Function):
    """Causal softmax of ``scale * (inputs + bias)`` in one kernel, the bias being a tensor
    ``[1 or b, np, sq, sk]`` such as the relative-position bias that the reference adds to the
    scores in a pass of its own (megatron/model/transformer.py:526-534).  Differentiable with
    respect to ``inputs`` and ``bias``.  ``slopes`` (optional, ``[np]``) adds the ALiBi bias as well."""

    @staticmethod
    def forward(ctx, inputs, bias, scale, slopes=None):
        scale = _fp32(scale)
        ctx.bias_shape = bias.shape
        return _remember(ctx, _causal_ext.forward_bias(inputs, bias, scale, slopes), scale)

    @staticmethod
    def backward(ctx, output_grads):
        probs, scale = _recall(ctx)
        if not output_grads.is_contiguous():
            output_grads = output_grads.contiguous()
        grads = _causal_ext.backward_nd(output_grads, probs, scale)
        return grads, (_bias_gradient(grads, ctx.bias_shape) if ctx.needs_input_grad[1] else None), None, None


class ScaledMaskedSoftmaxBias(torch.autograd.Function):
    """Mask-tensor softmax of ``scale * (inputs + bias)`` in one kernel; see
    ``ScaledUpperTriangMaskedSoftmaxBias``."""

    @staticmethod
    def forward(ctx, inputs, mask, bias, scale, slopes=None, row_end=None):
        scale = _fp32(scale)
        ctx.bias_shape = bias.shape
        ctx.row_end = row_end
        return _remember(ctx, _masked_ext.forward_bias(inputs, mask, bias, scale, slopes, row_end=row_end), scale)

    @staticmethod
    def backward(ctx, output_grads):
        probs, scale = _recall(ctx)
        grads = _masked_ext.backward(output_grads, probs, scale, row_end=ctx.row_end)
        return grads, None, (_bias_gradient(grads, ctx.bias_shape) if ctx.needs_input_grad[2] else None), None, None, None


class ScaledMaskedSoftmaxAlibi(torch.autograd.Function):
    """Mask-tensor softmax of ``scale * (inputs + alibi_bias(slopes))`` in one kernel: what the
    reference computes with ``AliBi.forward`` followed by the softmax when the fused causal kernel
    does not serve the call -- general fusion, a sliding-window or other mask, or a one-query
    step against a key/value cache (megatron/model/positional_embeddings.py:210-257,
    megatron/model/transformer.py:529-534).  Gradient with respect to ``inputs`` only."""

    @staticmethod
    def forward(ctx, inputs, mask, slopes, scale, row_end=None):
        scale = _fp32(scale)
        ctx.row_end = row_end
        return _remember(ctx, _masked_ext.forward_alibi(inputs, mask, slopes, scale, row_end=row_end), scale)

    @staticmethod
    def backward(ctx, output_grads):
        probs, scale = _recall(ctx)
        return _masked_ext.backward(output_grads, probs, scale, row_end=ctx.row_end), None, None, None, None


class ScaledSlidingWindowSoftmax(torch.autograd.Function):
    """scale -> causal mask with a sliding window -> softmax, in one kernel that reads no mask
    and no score outside the band: row i sees the keys ``max(0, i - window) .. i``, as under
    ``get_attn_mask(seq_length, device, sliding_window_width=window)`` (megatron/utils.py:67-80).
    ``inputs``: ``[attn_batches, sq, sk]`` or ``[b, np, sq, sk]`` as ``_causal_ext.window_kernel_takes``
    describes."""

    @staticmethod
    def forward(ctx, inputs, scale, window):
        scale = _fp32(scale)
        ctx.window = window
        return _remember(ctx, _causal_ext.forward_window(inputs, scale, window), scale)

    @staticmethod
    def backward(ctx, output_grads):
        probs, scale = _recall(ctx)
        return _causal_ext.backward_window(output_grads, probs, scale, ctx.window), None, None


class ScaledMaskedSoftmax(torch.autograd.Function):
    """scale -> mask tensor -> softmax, in one kernel.

    ``inputs``: ``[b, np, sq, sk]`` fp16/bf16; ``mask``: ``[1 or b, 1, sq, sk]`` bool or
    uint8, non-zero = masked, shared by all heads.  Reference:
    megatron/model/fused_softmax.py:56-83.  ``row_end`` (optional, an addition): where every mask
    row's visible keys end, as ``scaled_masked_softmax_cuda.scan_mask`` finds it -- the forward
    kernel then fetches nothing behind that point.
    """

    @staticmethod
    def forward(ctx, inputs, mask, scale, row_end=None):
        scale = _fp32(scale)
        ctx.row_end = row_end
        return _remember(ctx, _masked_ext.forward(inputs, mask, scale, row_end=row_end), scale)

    @staticmethod
    def backward(ctx, output_grads):
        probs, scale = _recall(ctx)
        return _masked_ext.backward(output_grads, probs, scale, row_end=ctx.row_end), None, None, None


class ScaledUpperTriangMaskedSoftmaxDropout(torch.autograd.Function):
    """Causal softmax followed by dropout with probability ``p``, in one kernel per pass.

    Returns ``dropout(softmax(scale * inputs))`` -- what the reference obtains from the
    softmax and ``self.attention_dropout`` (megatron/model/transformer.py:533-539).  The keep
    pattern comes from the device's default generator (see ``fused_kernels.attention_dropout``),
    so call it where the reference calls the dropout: inside the RNG tracker's ``fork()``.
    The undropped probabilities are kept for the backward pass; the pattern is regenerated
    there from the saved generator state instead of being stored.

    ``inputs``: ``[attn_batches, sq, sk]``, or ``[b, np, sq, sk]`` -- required with ``slopes``
    (ALiBi slopes ``[np]``) and ``bias`` (``[1 or b, np, sq, sk]``, differentiable), which add to
    the scores as in ``ScaledUpperTriangMaskedSoftmaxAlibi`` / ``...Bias``."""

    @staticmethod
    def forward(ctx, inputs, scale, p, slopes=None, bias=None):
        scale = _fp32(scale)
        seed, offset, state = _rng.take_philox_state(inputs.device)
        probs, dropped = _causal_ext.forward_dropout(
            inputs, scale, p, seed, offset, state, slopes=slopes, bias=bias)
        _remember(ctx, probs, scale)
        ctx.dropout = (p, seed, offset, state)
        ctx.bias_shape = None if bias is None else bias.shape
        return dropped

    @staticmethod
    def backward(ctx, output_grads):
        probs, scale = _recall(ctx)
        grads = _causal_ext.backward_dropout(output_grads, probs, scale, *ctx.dropout)
        wants_bias = ctx.bias_shape is not None and ctx.needs_input_grad[4]
        return grads, None, None, None, (_bias_gradient(grads, ctx.bias_shape) if wants_bias else None)


class ScaledMaskedSoftmaxDropout(torch.autograd.Function):
    """Mask-tensor softmax followed by dropout with probability ``p``, in one kernel per
    pass; see ``ScaledUpperTriangMaskedSoftmaxDropout``.  ``bias`` (optional,
    ``[1 or b, np, sq, sk]``, differentiable) and ``slopes`` (optional, ALiBi) add to the scores."""

    @staticmethod
    def forward(ctx, inputs, mask, scale, p, bias=None, slopes=None, row_end=None):
        scale = _fp32(scale)
        seed, offset, state = _rng.take_philox_state(inputs.device)
        probs, dropped = _masked_ext.forward_dropout(
            inputs, mask, scale, p, seed, offset, state, bias=bias, slopes=slopes, row_end=row_end)
        _remember(ctx, probs, scale)
        ctx.dropout = (p, seed, offset, state)
        ctx.bias_shape = None if bias is None else bias.shape
        ctx.row_end = row_end
        return dropped

    @staticmethod
    def backward(ctx, output_grads):
        probs, scale = _recall(ctx)
        grads = _masked_ext.backward_dropout(output_grads, probs, scale, *ctx.dropout, row_end=ctx.row_end)
        wants_bias = ctx.bias_shape is not None and ctx.needs_input_grad[4]
        return grads, None, None, None, (_bias_gradient(grads, ctx.bias_shape) if wants_bias else None), None, None


class SoftmaxFusionTypes(enum.Enum):
    upper_triang = 1  # causal mask
    general = 2  # general mask
    none = 3  # no fusion


class FusedScaleMaskSoftmax(torch.nn.Module):
    """Scaling + masking + softmax of attention scores ``[b, np, sq, sk]``.

    input_in_fp16 / input_in_bf16: storage type of the scores.
    fusion_type: a ``SoftmaxFusionTypes``; ``none`` always takes the torch branch.
    mask_func: ``mask_func(scores, mask) -> scores`` used by the torch branch.
    softmax_in_fp32: torch branch computes in fp32 (the kernels always do).
    scale: multiplier applied before the softmax, or None.
    causal_mask_check (not in the reference): ``"lazy"`` (default) | ``"verify"`` | ``"trust"`` -- how
        the upper_triang fusion treats the mask it is given; see the module text.
    skip_hidden_tails (not in the reference, default True): a call that the mask-tensor kernel serves
        tells it where every row's visible keys end, unless the scan of the mask has found that this
        spares less than a sixteenth of the keys (the padding of a batch of sequences of different
        lengths is more): the kernel then fetches nothing behind those points.  The scan is the one of
        ``causal_mask_check`` -- once per mask, never waited for under ``"lazy"``, never made under
        ``"trust"`` --, and the result is the same bit for bit.

    Reference: megatron/model/fused_softmax.py:92-205.
    """

    def __init__(self, input_in_fp16, input_in_bf16, fusion_type, mask_func, softmax_in_fp32, scale,
                 causal_mask_check="lazy", skip_hidden_tails=True):
        super().__init__()
        assert fusion_type in list(SoftmaxFusionTypes), f"Invalid fusion type {fusion_type}"
        assert scale is None or softmax_in_fp32, "softmax should be in fp32 when scaled"
        assert causal_mask_check in ("verify", "lazy", "trust"), f"Invalid causal_mask_check {causal_mask_check}"
        # how upper_triang fusion makes sure that the mask is the plain triangle (see the module text)
        self.causal_mask_check = causal_mask_check
        self.skip_hidden_tails = skip_hidden_tails

        self.input_in_fp16 = input_in_fp16
        self.input_in_bf16 = input_in_bf16
        self.input_in_float16 = input_in_fp16 or input_in_bf16
        self.fusion = fusion_type is not SoftmaxFusionTypes.none
        self.upper_triang_mask_fusion = fusion_type is SoftmaxFusionTypes.upper_triang
        self.general_mask_fusion = fusion_type is SoftmaxFusionTypes.general
        self.mask_func = mask_func
        self.softmax_in_fp32 = softmax_in_fp32
        self.scale = scale
        self._last_mask = None  # (weak reference to the mask of the previous call, its version, (verdict, ends))
        if self.fusion:
            load_fused_kernels()  # ImportError here, not at the first forward

    def forward(self, input, mask, alibi_slopes=None, dropout_p=0.0, bias=None):
        """``alibi_slopes`` (optional, ``[np]``) is an addition to the reference signature:
        ``forward(scores, mask, alibi_slopes=alibi.slopes)`` equals
        ``forward(alibi(scores), mask)`` (megatron/model/transformer.py:529-534) with the bias
        evaluated in fp32 inside the softmax kernel instead of a separate pass in half precision.

        ``dropout_p`` (optional, training only) is the second addition:
        ``forward(scores, mask, dropout_p=p)`` equals ``dropout(forward(scores, mask), p)``
        (megatron/model/transformer.py:533-539) and is to be called where the reference calls
        the dropout, inside the RNG tracker's ``fork()``.

        ``bias`` (optional, ``[1 or b, np, sq, sk]``) is the third:
        ``forward(scores, mask, bias=rpe)`` equals ``forward(scores + rpe, mask)``
        (megatron/model/transformer.py:526-534) with the bias read inside the softmax kernel and
        the sum taken in fp32.

        Every combination of the three runs in one kernel per pass whenever the fused softmax
        serves the call."""
        assert input.dim() == 4  # [b, np, sq, sk]
        b, np, sq, sk = input.size()
        if self.is_kernel_available(mask, b, np, sq, sk):
            if alibi_slopes is None and bias is None and not dropout_p:
                return self.forward_fused_softmax(input, mask)
            return self.forward_fused_features(input, mask, alibi_slopes, dropout_p, bias)
        # the unfused sequence of the reference: bias, ALiBi, softmax, dropout
        if bias is not None:
            input = input + bias
        if alibi_slopes is not None:
            input = input + alibi_bias(alibi_slopes, sq, sk, input.device, input.dtype)
        probs = self.forward_torch_softmax(input, mask)
        return torch.nn.functional.dropout(probs, dropout_p, True) if dropout_p else probs

    def forward_fused_features(self, input, mask, alibi_slopes, dropout_p, bias):
        """The fused branch with ALiBi slopes, a bias tensor and/or dropout folded in."""
        b, np, sq, sk = input.size()
        scale = 1.0 if self.scale is None else self.scale
        if alibi_slopes is not None:
            assert sq == sk or sq == 1, "assumption sq == sk unless at inference time with cache in layer_past with sq == 1"
        causal = self.mask_kind(mask, sq, sk) == "causal"
        ends = None if causal else self.hidden_tails(mask, b, sq, sk)
        if dropout_p:
            if causal:
                return ScaledUpperTriangMaskedSoftmaxDropout.apply(input, scale, dropout_p, alibi_slopes, bias)
            return ScaledMaskedSoftmaxDropout.apply(input, mask, scale, dropout_p, bias, alibi_slopes, ends)
        if bias is not None:
            if causal:
                return ScaledUpperTriangMaskedSoftmaxBias.apply(input, bias, scale, alibi_slopes)
            return ScaledMaskedSoftmaxBias.apply(input, mask, bias, scale, alibi_slopes, ends)
        if causal:
            return ScaledUpperTriangMaskedSoftmaxAlibi.apply(input, alibi_slopes, scale)
        return ScaledMaskedSoftmaxAlibi.apply(input, mask, alibi_slopes, scale, ends)

    def is_kernel_available(self, mask, b, np, sq, sk):
        """Whether the fused branch serves this call.

        Kept from the reference predicate (megatron/model/fused_softmax.py:148-168):
        the user asked for fusion, the input is fp16/bf16, a mask tensor is given.
        Dropped: ``16 < sk <= 2048``, ``sq % 4``, ``(b*np) % 4`` and the
        ``batch_per_block`` rules.  Added: the tensor must not be empty, and a causal-fusion call
        with ``sq != sk`` (a decode or prefill step against a key/value cache; the reference
        asserts ``sq == sk`` and never gets there) is served by the mask-tensor kernel with the
        mask it was given, provided that mask has the kernel's layout ``[1 or b, 1, sq, sk]``.
        """
        if not (self.fusion and self.input_in_float16 and mask is not None):
            return False
        if b * np * sq * sk == 0:
            return False
        if self.upper_triang_mask_fusion and sq != sk:
            return self._mask_fits_the_mask_kernel(mask, b, sq, sk)
        return True

    @staticmethod
    def _mask_fits_the_mask_kernel(mask, b, sq, sk):
        return (
            mask.dim() == 4
            and mask.dtype in (torch.bool, torch.uint8)
            and mask.shape[0] in (1, b)
            and tuple(mask.shape[1:]) == (1, sq, sk)
        )

    @staticmethod
    def reference_is_kernel_available(fusion, upper_triang, input_in_float16, mask, b, np, sq, sk):
        """The reference's own predicate (megatron/model/fused_softmax.py:148-168),
        evaluated with wave64 ``get_batch_per_block`` values; for comparison only."""
        shape_ok = 16 < sk <= 2048 and sq % 4 == 0 and (b * np) % 4 == 0
        if not (fusion and input_in_float16 and mask is not None and shape_ok):
            return False
        per_block = FusedScaleMaskSoftmax.get_batch_per_block(sq, sk, b, np)
        return ((b * np) if upper_triang else sq) % per_block == 0

    def forward_fused_softmax(self, input, mask):
        b, np, sq, sk = input.size()
        scale = 1.0 if self.scale is None else self.scale
        kind = self.mask_kind(mask, sq, sk)
        records = torch.is_grad_enabled() and input.requires_grad
        if kind == "causal":
            # the causal kernel works on [attn_batches, sq, sk] and never reads `mask`
            if not input.is_contiguous():
                input = input.contiguous()
            if not records:
                # nothing to record: straight to the extension (the autograd Function costs the host
                # several microseconds per call)
                return _causal_ext.forward_nd(input, _fp32(scale))
            return _CausalSoftmax4D.apply(input, _fp32(scale))
        if kind is not None and _causal_ext.window_kernel_takes(input, kind):
            # the causal mask with a sliding window: the band kernel reads neither the mask nor
            # the scores outside the band
            if not records:
                return _causal_ext.forward_window(input, _fp32(scale), kind)
            return ScaledSlidingWindowSoftmax.apply(input, scale, kind)
        # general fusion, or a causal-fusion call whose mask is not (known to be) a causal one -- some
        # other pattern, a step against a key/value cache, a verdict still on its way: what the torch
        # path computes, from the mask itself (and not from the hidden tails of its rows, if it has any)
        ends = self.hidden_tails(mask, b, sq, sk)
        if not records:
            return _masked_ext.forward(input, mask, _fp32(scale), row_end=ends)
        return ScaledMaskedSoftmax.apply(input, mask, scale, ends)

    def mask_kind(self, mask, sq, sk):
        """What the module knows about ``mask``: ``"causal"``, a sliding-window width, or None -- use
        the mask tensor (``sq != sk``, any other pattern, or a classification that has not arrived
        yet).  See ``classify_mask``.  The general fusion asks too: GPT-NeoX hands it the same causal
        masks (``scaled_masked_softmax_fusion``), and a mask that has been read and found causal is
        served by the kernels that read no mask -- but nothing is taken on trust there, since its
        masks may be anything."""
        if sq != sk:
            return None
        if self.upper_triang_mask_fusion:
            return self.classify_mask(mask)
        if self.general_mask_fusion and self.causal_mask_check != "trust":
            return self.classify_mask(mask)
        return None

    def classify_mask(self, mask):
        """``"causal"`` -- the mask hides exactly the keys ``j > i``, or ``causal_mask_check`` is
        ``"trust"`` --, an int ``w`` -- the causal mask with a sliding window of that width --, or
        None: not (known to be) either.

        ``"verify"`` and ``"lazy"`` decide once per mask region (see ``_CausalMaskMemo``);
        ``"lazy"`` never waits and answers None until the verdict has arrived.  While a HIP graph
        is being captured nothing can be classified and no event may be asked: a mask decided
        before the capture keeps its verdict, any other is None."""
        if self.causal_mask_check == "trust":
            return "causal"
        facts = self._mask_facts(mask)
        verdict = None if facts is None else facts[0]
        return None if verdict is False else verdict  # (a window of width 0 is a verdict too)

    def hidden_tails(self, mask, b, sq, sk):
        """The ``row_end`` hint for a call that the mask-tensor kernel serves, or None: switched off,
        ``"trust"`` (the mask is never read), a mask in another layout than ``[1 or b, 1, sq, sk]``
        on the GPU, a mask known to hide less than a sixteenth of its keys behind its rows' last
        visible ones, or a HIP graph being captured.  While the scan of a mask is still on its way
        the hint is passed already, to launches on the scan's stream."""
        if not self.skip_hidden_tails or self.causal_mask_check == "trust":
            return None
        if not (mask.is_cuda and self._mask_fits_the_mask_kernel(mask, b, sq, sk)):
            return None
        facts = self._mask_facts(mask)
        if facts is not None and facts[1] is None:
            return None
        # the hint lives in the memo, which may drop it when many masks have passed: a HIP graph that
        # recorded its address could outlive it, so captured launches go without
        if torch.cuda.is_current_stream_capturing():
            return None
        if facts is None:
            # the scan is still on its way: a launch on its stream comes after it and may use what it
            # writes -- the first call with a fresh mask skips the hidden tails already
            return _causal_memo.early_ends(mask)
        ends = facts[1]
        if facts[2] != _masked_ext.launch_stream(mask):
            # a launch on another stream than the one whose pool the array came from: the allocator
            # must not hand the block on before this launch is through, should the memo drop it
            ends.record_stream(torch.cuda.current_stream(mask.device))
        return ends

    def _mask_facts(self, mask):
        """The memo's answer: ``(verdict, ends, stream)`` -- the verdict False for a mask that is not a
        causal one --, or None while it is on its way."""
        last = self._last_mask
        if last is not None and last[0]() is mask and last[1] == mask._version:
            return last[2]  # the tensor object of the previous call, unchanged: no lookup
        if mask.dim() != 4 or mask.shape[1] != 1 or mask.dtype not in (torch.bool, torch.uint8):
            return (False, None, None)
        if mask.is_cuda and torch.cuda.is_current_stream_capturing():
            facts = _causal_memo.lookup_facts(mask, wait=None)
        else:
            facts = _causal_memo.facts(mask, wait=self.causal_mask_check == "verify")
        if facts is not None:
            self._last_mask = (weakref.ref(mask), mask._version, facts)
        return facts

    def mask_is_plain_causal(self, mask):
        """True if the causal kernel may serve ``mask``; see ``classify_mask``."""
        return self.classify_mask(mask) == "causal"

    def forward_torch_softmax(self, input, mask):
        """The unfused path: optional upcast, scale, ``mask_func``, softmax, cast back."""
        upcast = self.input_in_float16 and self.softmax_in_fp32
        scores = input.float() if upcast else input
        if self.scale is not None:
            scores = scores * self.scale
        if mask is not None:
            scores = self.mask_func(scores, mask)
        probs = torch.softmax(scores, dim=-1)
        if upcast:
            probs = probs.half() if self.input_in_fp16 else probs.bfloat16()
        return probs

    @staticmethod
    def get_batch_per_block(sq, sk, b, np):
        return _masked_ext.get_batch_per_block(sq, sk, b, np)
