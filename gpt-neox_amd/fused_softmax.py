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
* by default the causal branch checks once per mask (per storage region, so ``detach()``ed
  aliases share the verdict) that the mask really is the plain upper-triangular one and
  otherwise (sliding-window masks, packed-sequence masks) runs the mask-tensor kernel with
  the mask it was given -- the reference's causal kernel ignores the mask's contents, so
  above its 2048 limit (torch path) and below it (fused kernel) the reference computes two
  different things for such masks; here both agree with the torch path.  The constructor's
  ``causal_mask_check`` selects how: ``"verify"`` (default) waits for the device-side
  comparison the first time a mask is seen (one host synchronisation per new mask),
  ``"lazy"`` never synchronises -- calls made while the comparison is in flight run the
  mask-tensor kernel, which is right for any mask -- and ``"trust"`` restores the
  reference's behaviour of never reading the mask
  (megatron/model/fused_softmax.py:173-179).  A causal-fusion call with ``sq != sk`` (a step
  against a key/value cache, where the reference asserts) also runs the mask-tensor kernel;
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
    and the verdict -- True / False, or None while the device-side comparison is still running
    (then ``pending`` holds the pinned result slot and the event that follows the copy)."""

    __slots__ = ("storage", "version", "verdict", "pending")

    def __init__(self, storage, version, verdict=None, pending=None):
        self.storage = weakref.ref(storage)
        self.version = version
        self.verdict = verdict
        self.pending = pending

    def poll(self, wait):
        if self.verdict is None and self.pending is not None:
            slot, event = self.pending
            if wait:
                event.synchronize()
            if wait or event.query():
                self.verdict = bool(slot.item())  # host memory, the copy has finished: no sync
                self.pending = None
        return self.verdict


class _CausalMaskMemo:
    """Remembers, per mask region, whether it equals ``triu(ones, 1)``.

    A region is (storage address, offset, shape, strides); an entry is valid while the storage
    object it was decided for is alive (weak reference -- a recycled allocation is another
    storage object and cannot inherit a verdict) and the tensor's version counter is unchanged
    (in-place writes bump it).  Aliases of one mask -- ``mask.detach()``, which activation
    checkpointing applies to its inputs for every recomputed segment, or an equal view --
    share the storage, the region and the version counter, hence the verdict.  (A write through
    ``.data`` or from outside torch bumps no counter and is not seen.)

    The comparison runs on the device.  ``is_plain_causal(mask, wait=True)`` waits for it (one
    host synchronisation per new mask); with ``wait=False`` it returns None while the result is
    on its way and the caller uses a kernel that is right for any mask in the meantime."""

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
        """The verdict for this region in its current version: True, False, or None if it is
        unknown (never asked, or still being computed and ``wait`` is False)."""
        hit = self._entry(mask)
        return None if hit is None else hit.poll(wait)

    def _result_slot(self, entry):
        """A pinned host byte for the verdict of ``entry``.  The slots are handed out in turn; an
        entry that still waits for the slot's previous content reads it first (its copy finished
        long ago), so a slot is never overwritten under an entry that has not looked yet."""
        if self._slots is None:
            self._slots = torch.zeros(256, dtype=torch.bool, pin_memory=True)
            self._slot_owner = [None] * self._slots.numel()
        self._next_slot = (self._next_slot + 1) % self._slots.numel()
        owner = self._slot_owner[self._next_slot]
        if owner is not None:
            owner.poll(wait=True)
        self._slot_owner[self._next_slot] = entry
        return self._slots[self._next_slot : self._next_slot + 1]

    def is_plain_causal(self, mask, wait=True):
        hit = self._entry(mask)
        if hit is not None:
            return hit.poll(wait)
        sq, sk = mask.shape[-2], mask.shape[-1]
        expected = torch.ones(sq, sk, dtype=torch.bool, device=mask.device).triu_(1)
        same = (mask.bool() == expected).all()  # a 0-dim tensor on the mask's device
        key, storage = self._key(mask)
        if mask.is_cuda:
            entry = _MaskVerdict(storage, mask._version)
            slot = self._result_slot(entry)
            with torch.cuda.device(mask.device):  # copy and event on the mask's device and stream
                slot.copy_(same.view(1), non_blocking=True)
                event = torch.cuda.Event()
                event.record()
            entry.pending = (slot, event)
        else:
            entry = _MaskVerdict(storage, mask._version, verdict=bool(same))
        if len(self._entries) >= self._limit:
            self._entries = {k: v for k, v in self._entries.items() if v.storage() is not None}
            if len(self._entries) >= self._limit:
                self._entries.clear()
        self._entries[key] = entry
        return entry.poll(wait)


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
        b, np, sq, sk = probs.shape
        grads = _causal_ext.backward(output_grads.reshape(-1, sq, sk), probs.view(-1, sq, sk), scale)
        return grads.view(b, np, sq, sk), None, None


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
    respect to ``inputs`` and ``bias``."""

    @staticmethod
    def forward(ctx, inputs, bias, scale):
        scale = _fp32(scale)
        ctx.bias_shape = bias.shape
        return _remember(ctx, _causal_ext.forward_bias(inputs, bias, scale), scale)

    @staticmethod
    def backward(ctx, output_grads):
        probs, scale = _recall(ctx)
        b, np, sq, sk = probs.shape
        grads = _causal_ext.backward(output_grads.reshape(-1, sq, sk), probs.view(-1, sq, sk), scale)
        grads = grads.view(b, np, sq, sk)
        return grads, (_bias_gradient(grads, ctx.bias_shape) if ctx.needs_input_grad[1] else None), None


class ScaledMaskedSoftmaxBias(torch.autograd.Function):
    """Mask-tensor softmax of ``scale * (inputs + bias)`` in one kernel; see
    ``ScaledUpperTriangMaskedSoftmaxBias``."""

    @staticmethod
    def forward(ctx, inputs, mask, bias, scale):
        scale = _fp32(scale)
        ctx.bias_shape = bias.shape
        return _remember(ctx, _masked_ext.forward_bias(inputs, mask, bias, scale), scale)

    @staticmethod
    def backward(ctx, output_grads):
        probs, scale = _recall(ctx)
        grads = _masked_ext.backward(output_grads, probs, scale)
        return grads, None, (_bias_gradient(grads, ctx.bias_shape) if ctx.needs_input_grad[2] else None), None


class ScaledMaskedSoftmax(torch.autograd.Function):
    """scale -> mask tensor -> softmax, in one kernel.

    ``inputs``: ``[b, np, sq, sk]`` fp16/bf16; ``mask``: ``[1 or b, 1, sq, sk]`` bool or
    uint8, non-zero = masked, shared by all heads.  Reference:
    megatron/model/fused_softmax.py:56-83.
    """

    @staticmethod
    def forward(ctx, inputs, mask, scale):
        scale = _fp32(scale)
        return _remember(ctx, _masked_ext.forward(inputs, mask, scale), scale)

    @staticmethod
    def backward(ctx, output_grads):
        probs, scale = _recall(ctx)
        return _masked_ext.backward(output_grads, probs, scale), None, None


class ScaledUpperTriangMaskedSoftmaxDropout(torch.autograd.Function):
    """Causal softmax followed by dropout with probability ``p``, in one kernel per pass.

    Returns ``dropout(softmax(scale * inputs))`` -- what the reference obtains from the
    softmax and ``self.attention_dropout`` (megatron/model/transformer.py:533-539).  The keep
    pattern comes from the device's default generator (see ``fused_kernels.attention_dropout``),
    so call it where the reference calls the dropout: inside the RNG tracker's ``fork()``.
    The undropped probabilities are kept for the backward pass; the pattern is regenerated
    there from the saved generator state instead of being stored.

    ``inputs``: ``[attn_batches, sq, sk]``, or ``[b, np, sq, sk]`` -- required with ``slopes``
    (ALiBi slopes ``[np]``) or ``bias`` (``[1 or b, np, sq, sk]``, differentiable), which add to
    the scores as in ``ScaledUpperTriangMaskedSoftmaxAlibi`` / ``...Bias``; at most one of them."""

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
    ``[1 or b, np, sq, sk]``, differentiable) adds to the scores."""

    @staticmethod
    def forward(ctx, inputs, mask, scale, p, bias=None):
        scale = _fp32(scale)
        seed, offset, state = _rng.take_philox_state(inputs.device)
        probs, dropped = _masked_ext.forward_dropout(
            inputs, mask, scale, p, seed, offset, state, bias=bias)
        _remember(ctx, probs, scale)
        ctx.dropout = (p, seed, offset, state)
        ctx.bias_shape = None if bias is None else bias.shape
        return dropped

    @staticmethod
    def backward(ctx, output_grads):
        probs, scale = _recall(ctx)
        grads = _masked_ext.backward_dropout(output_grads, probs, scale, *ctx.dropout)
        wants_bias = ctx.bias_shape is not None and ctx.needs_input_grad[4]
        return grads, None, None, None, (_bias_gradient(grads, ctx.bias_shape) if wants_bias else None)


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
    causal_mask_check (not in the reference): ``"verify"`` | ``"lazy"`` | ``"trust"`` -- how the
        upper_triang fusion treats the mask it is given; see the module text.

    Reference: megatron/model/fused_softmax.py:92-205.
    """

    def __init__(self, input_in_fp16, input_in_bf16, fusion_type, mask_func, softmax_in_fp32, scale,
                 causal_mask_check="verify"):
        super().__init__()
        assert fusion_type in list(SoftmaxFusionTypes), f"Invalid fusion type {fusion_type}"
        assert scale is None or softmax_in_fp32, "softmax should be in fp32 when scaled"
        assert causal_mask_check in ("verify", "lazy", "trust"), f"Invalid causal_mask_check {causal_mask_check}"
        # how upper_triang fusion makes sure that the mask is the plain triangle (see the module text)
        self.causal_mask_check = causal_mask_check

        self.input_in_fp16 = input_in_fp16
        self.input_in_bf16 = input_in_bf16
        self.input_in_float16 = input_in_fp16 or input_in_bf16
        self.fusion = fusion_type is not SoftmaxFusionTypes.none
        self.upper_triang_mask_fusion = fusion_type is SoftmaxFusionTypes.upper_triang
        self.general_mask_fusion = fusion_type is SoftmaxFusionTypes.general
        self.mask_func = mask_func
        self.softmax_in_fp32 = softmax_in_fp32
        self.scale = scale
        if self.fusion:
            load_fused_kernels()  # ImportError here, not at the first forward

    def forward(self, input, mask, alibi_slopes=None, dropout_p=0.0, bias=None):
        """``alibi_slopes`` (optional, ``[np]``) is an addition to the reference signature:
        ``forward(scores, mask, alibi_slopes=alibi.slopes)`` equals
        ``forward(alibi(scores), mask)`` (megatron/model/transformer.py:529-534) with the bias
        evaluated in fp32 inside the causal kernel instead of a separate pass in half precision.

        ``dropout_p`` (optional, training only) is the second addition:
        ``forward(scores, mask, dropout_p=p)`` equals ``dropout(forward(scores, mask), p)``
        (megatron/model/transformer.py:533-539) and is to be called where the reference calls
        the dropout, inside the RNG tracker's ``fork()``.

        ``bias`` (optional, ``[1 or b, np, sq, sk]``) is the third:
        ``forward(scores, mask, bias=rpe)`` equals ``forward(scores + rpe, mask)``
        (megatron/model/transformer.py:526-534) with the bias read inside the softmax kernel and
        the sum taken in fp32."""
        assert input.dim() == 4  # [b, np, sq, sk]
        if dropout_p:
            return self.forward_with_dropout(input, mask, alibi_slopes, dropout_p, bias)
        fused = self.is_kernel_available(mask, *input.size())
        if bias is not None:
            if fused and alibi_slopes is None:
                return self.forward_fused_softmax(input, mask, bias)
            input = input + bias
        if alibi_slopes is not None:
            b, np, sq, sk = input.size()
            if fused and self.upper_triang_mask_fusion and sq == sk and self.mask_is_plain_causal(mask):
                scale = 1.0 if self.scale is None else self.scale
                return ScaledUpperTriangMaskedSoftmaxAlibi.apply(input, alibi_slopes, scale)
            input = input + alibi_bias(alibi_slopes, sq, sk, input.device, input.dtype)
        return self.forward_fused_softmax(input, mask) if fused else self.forward_torch_softmax(input, mask)

    def forward_with_dropout(self, input, mask, alibi_slopes, dropout_p, bias=None):
        """Softmax and dropout in one kernel per pass when the fused softmax serves the call --
        with the ALiBi slopes (plain causal mask only) or a bias tensor folded in as well, though
        not both at once; otherwise the softmax above followed by torch's dropout.  Under HIP
        graph capture the fused kernels follow ``attention_dropout.graph_state(device)``, which
        has to exist before the capture starts."""
        b, np, sq, sk = input.size()
        fusable = self.is_kernel_available(mask, b, np, sq, sk) and (alibi_slopes is None or bias is None)
        causal = fusable and self.upper_triang_mask_fusion and sq == sk and self.mask_is_plain_causal(mask)
        if fusable and alibi_slopes is not None and not causal:
            fusable = False  # the mask-tensor kernels have no ALiBi variant
        if not fusable:
            return torch.nn.functional.dropout(self.forward(input, mask, alibi_slopes, 0.0, bias), dropout_p, True)
        scale = 1.0 if self.scale is None else self.scale
        if causal:
            return ScaledUpperTriangMaskedSoftmaxDropout.apply(input, scale, dropout_p, alibi_slopes, bias)
        return ScaledMaskedSoftmaxDropout.apply(input, mask, scale, dropout_p, bias)

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

    def forward_fused_softmax(self, input, mask, bias=None):
        b, np, sq, sk = input.size()
        scale = 1.0 if self.scale is None else self.scale
        if not (self.upper_triang_mask_fusion and sq == sk and self.mask_is_plain_causal(mask)):
            # general fusion, or a causal-fusion call whose mask is not the plain square triangle (a
            # sliding-window mask, a step against a key/value cache): what the torch path computes,
            # from the mask itself
            if bias is not None:
                return ScaledMaskedSoftmaxBias.apply(input, mask, bias, scale)
            if not (torch.is_grad_enabled() and input.requires_grad):
                return _masked_ext.forward(input, mask, _fp32(scale))
            return ScaledMaskedSoftmax.apply(input, mask, scale)
        if bias is not None:
            return ScaledUpperTriangMaskedSoftmaxBias.apply(input, bias, scale)
        # the causal kernel works on [attn_batches, sq, sk] and never reads `mask`
        if not (torch.is_grad_enabled() and input.requires_grad):
            # nothing to record: straight to the extension (the autograd Function costs the host
            # several microseconds per call)
            return _causal_ext.forward(input.view(-1, sq, sk), _fp32(scale)).view(b, np, sq, sk)
        probs = ScaledUpperTriangMaskedSoftmax.apply(input.view(-1, sq, sk), scale)
        return probs.view(b, np, sq, sk)

    def mask_is_plain_causal(self, mask):
        """True if the causal kernel may serve ``mask``: it hides exactly the keys ``j > i``
        (``"verify"``, ``"lazy"``; decided once per mask region, see ``_CausalMaskMemo``), or
        without looking (``"trust"``).  ``"lazy"`` answers False while the comparison is still
        running.  While a HIP graph is being captured nothing can be compared: a mask decided
        before the capture keeps its verdict, for any other the answer is False and the
        mask-tensor kernel is used."""
        if self.causal_mask_check == "trust":
            return True
        if mask.dim() != 4 or mask.shape[1] != 1 or mask.dtype not in (torch.bool, torch.uint8):
            return False
        if mask.is_cuda and torch.cuda.is_current_stream_capturing():
            return bool(_causal_memo.lookup(mask))
        return bool(_causal_memo.is_plain_causal(mask, wait=self.causal_mask_check == "verify"))

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
