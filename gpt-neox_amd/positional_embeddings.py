"""Drop-in for ``megatron/model/positional_embeddings.py`` on MI355X.

Exports the reference module's names (megatron/model/positional_embeddings.py:19-257):
``SinusoidalPositionalEmbedding``, ``RotaryEmbedding``, ``rotate_half``,
``apply_rotary_pos_emb``, ``apply_rotary_pos_emb_torch``, ``AliBi``.

The rotary apply is the accelerated part: for fp16/bf16 GPU tensors both
``apply_rotary_pos_emb`` and ``apply_rotary_pos_emb_torch`` run ONE gfx950 kernel
launch that rotates q and k together (forward), and one more for both gradients
(backward).  q and k may be strided views (e.g. the ``[..., :rotary_ndims]``
slices of a fused QKV projection); only the last dim must be dense.

What differs from the reference, on purpose:

* arithmetic is fp32 from the raw fp16/bf16 values with a single rounding of the
  result, whatever the dtype of cos/sin; the torch expression rounds three times
  when the tables are half precision;
* the result has the dtype of q/k also when cos/sin are fp32 (torch would
  promote the whole result to fp32);
* ``RotaryEmbedding.forward`` keeps a per-device copy of its tables instead of
  copying them to ``x.device`` on every call.

Other dtypes and CPU tensors evaluate the reference's torch expression.
``apply_rotary_pos_emb_`` is an in-place variant over whole heads (partial
rotary without the slice/concatenate round trip) and ``apply_rotary_pos_emb_qkv_``
does the same directly on the fused QKV projection of the attention layer.
"""
import math

import torch

from .fused_kernels import fused_rotary_positional_embedding as _rope_ext

_HALF = (torch.float16, torch.bfloat16)


class SinusoidalPositionalEmbedding(torch.nn.Module):
    """Sin/cos absolute position features ``[1, seq, dim]``
    (megatron/model/positional_embeddings.py:19-35); plain torch."""

    def __init__(self, dim, base=10000, precision=torch.half):
        super().__init__()
        exponents = torch.arange(0, dim, 2).float() / dim
        self.register_buffer("inv_freq", 1.0 / (base**exponents))
        self.precision = precision

    def forward(self, x, seq_dim=1):
        positions = torch.arange(x.shape[seq_dim], device=x.device).type_as(self.inv_freq)
        angles = torch.outer(positions, self.inv_freq)
        via_fp32 = self.precision == torch.bfloat16
        if via_fp32:
            angles = angles.float()
        sin, cos = angles.sin(), angles.cos()
        if via_fp32:
            sin, cos = sin.bfloat16(), cos.bfloat16()
        return torch.cat((sin, cos), dim=-1).unsqueeze(0)


class RotaryEmbedding(torch.nn.Module):
    """cos/sin tables ``[max_seq_len, 1, 1, dim]`` of the rotary embedding
    (megatron/model/positional_embeddings.py:38-97).

    ``inv_freq_i = base^(-2i/dim)``; the angle of position ``t`` and dim ``j`` is
    ``t * inv_freq[j mod dim/2]``.  Tables are computed in fp32 and stored in
    ``precision``.  ``forward`` returns ``(cos[:seq_len], sin[:seq_len])`` on the
    device of ``x``.
    """

    def __init__(self, dim, max_seq_len, base=10000, precision=torch.half, save_inv_freqs=False):
        super().__init__()
        self.seq_len_cached = None
        self.precision = precision
        self.max_seq_len = max_seq_len
        self.base = base
        self.dim = dim
        cos_cached, sin_cached, inv_freq = self._prepare_cache(max_seq_len, precision, base)
        # same buffer name and persistence rule as the reference, so state dicts round-trip
        self.register_buffer("inv_freq", inv_freq, persistent=save_inv_freqs)
        self.cos_cached = cos_cached
        self.sin_cached = sin_cached
        self._per_device = {}

    def _prepare_cache(self, seq_len, precision, base):
        inv_freq = 1.0 / (base ** (torch.arange(0, self.dim, 2).float() / self.dim))
        t = torch.arange(seq_len).type_as(inv_freq)
        freqs = torch.outer(t, inv_freq)
        emb = torch.cat((freqs, freqs), dim=-1)  # [seq, dim], fp32
        self.emb = emb.reshape(emb.size(0), 1, 1, emb.size(1))
        cos_cached = emb.cos()[:, None, None, :]
        sin_cached = emb.sin()[:, None, None, :]
        return cos_cached.to(precision), sin_cached.to(precision), inv_freq.to(precision)

    def get_emb(self):
        return self.emb.to(self.precision).cuda()

    def _tables_on(self, device):
        device = torch.device(device)
        if device == self.cos_cached.device:
            return self.cos_cached, self.sin_cached
        hit = self._per_device.get(device)
        if hit is None:
            hit = (self.cos_cached.to(device), self.sin_cached.to(device))
            self._per_device[device] = hit
        return hit

    def forward(self, x, seq_dim=0, seq_len=None):
        if seq_len is None:
            seq_len = x.shape[seq_dim]
        assert seq_len <= self.max_seq_len
        cos, sin = self._tables_on(x.device)
        if seq_len != self.max_seq_len:
            return cos[:seq_len, ...], sin[:seq_len, ...]
        return cos, sin


# rotary pos emb helpers:


def rotate_half(x):
    """``cat(-x[d/2:], x[:d/2])`` (megatron/model/positional_embeddings.py:103-107)."""
    half = x.shape[-1] // 2
    return torch.cat((-x[..., half:], x[..., :half]), dim=x.ndim - 1)


def _rotary_torch(q, k, cos, sin, offset):
    cos = cos[offset : q.shape[0] + offset, ...]
    sin = sin[offset : q.shape[0] + offset, ...]
    return (q * cos) + (rotate_half(q) * sin), (k * cos) + (rotate_half(k) * sin)


def _as_table(t, d_rot, need_rows):
    """View a ``[seq, 1, 1, d]`` (or ``[seq, d]``) table as rows the kernel can index."""
    if t.dim() == 2 and t.shape[1] == d_rot and t.shape[0] >= need_rows and t.stride(1) == 1 and t.stride(0) >= d_rot:
        return t  # already rows (the tables the autograd Functions keep for their backward pass)
    if t.shape[-1] != d_rot or t.numel() != t.shape[0] * d_rot:
        raise RuntimeError(
            f"cos/sin must have shape [seq, 1, 1, {d_rot}], got {tuple(t.shape)}"
        )
    if t.shape[0] < need_rows:
        raise RuntimeError(
            f"cos/sin hold {t.shape[0]} positions, offset + seq_len = {need_rows} needed"
        )
    t2 = t.reshape(t.shape[0], d_rot)
    if t2.stride(1) != 1 or (t2.shape[0] > 1 and t2.stride(0) < d_rot):
        t2 = t2.contiguous()
    return t2


def _dense_last(t):
    return t if t.stride(-1) == 1 else t.contiguous()


def _on(t, device):
    """``t`` on ``device``; the tensor itself when it is already there (the usual case, and
    cheaper than asking ``Tensor.to`` to find that out)."""
    return t if t.device == device else t.to(device)


def _needs_grad(*tensors):
    """Whether autograd has to record the call (else the autograd Function, which costs the host
    several microseconds per call, is bypassed)."""
    return torch.is_grad_enabled() and any(t.requires_grad for t in tensors)


def _rotary_out_of_place(q, k, cos, sin, offset):
    """New tensors ``rotary(q), rotary(k)`` in one launch; returns them and the table rows used."""
    d_rot = q.shape[-1]
    cos2 = _as_table(cos, d_rot, offset + q.shape[0])
    sin2 = _as_table(sin, d_rot, offset + q.shape[0])
    q, k = _dense_last(q), _dense_last(k)
    out_q = torch.empty(q.shape, dtype=q.dtype, device=q.device)
    out_k = torch.empty(k.shape, dtype=k.dtype, device=k.device)
    if q.numel() or k.numel():
        _rope_ext.rope_launch(out_q, out_k, q, k, cos2, sin2, d_rot, offset, backward=False)
    return out_q, out_k, cos2, sin2


class _FusedRotary(torch.autograd.Function):
    """q' , k' = rotary(q), rotary(k) in one launch; gradients in one launch."""

    @staticmethod
    def forward(ctx, q, k, cos, sin, offset):
        out_q, out_k, cos2, sin2 = _rotary_out_of_place(q, k, cos, sin, offset)
        ctx.save_for_backward(cos2, sin2)
        ctx.offset = offset
        return out_q, out_k

    @staticmethod
    def backward(ctx, grad_q, grad_k):
        cos2, sin2 = ctx.saved_tensors
        grad_q, grad_k = _dense_last(grad_q), _dense_last(grad_k)
        dq = torch.empty(grad_q.shape, dtype=grad_q.dtype, device=grad_q.device)
        dk = torch.empty(grad_k.shape, dtype=grad_k.dtype, device=grad_k.device)
        if dq.numel() or dk.numel():
            _rope_ext.rope_launch(
                dq, dk, grad_q, grad_k, cos2, sin2, grad_q.shape[-1], ctx.offset, backward=True
            )
        return dq, dk, None, None, None


def _fusable(q, k, cos, sin):
    return (
        q.is_cuda
        and k.is_cuda
        and q.dtype in _HALF
        and k.dtype == q.dtype
        and q.dim() == 4
        and k.dim() == 4
        and q.shape[:2] == k.shape[:2]
        and q.shape[-1] == k.shape[-1]
        and q.shape[-1] % 2 == 0
        and cos.dtype == sin.dtype
        and cos.dtype in (torch.float32, q.dtype)
    )


def apply_rotary_pos_emb(q, k, cos, sin, offset: int = 0):
    """``(q*cos + rotate_half(q)*sin, k*cos + rotate_half(k)*sin)`` with cos/sin rows
    ``offset .. offset+sq`` (megatron/model/positional_embeddings.py:110-116).
    q, k: ``[sq, b, heads, d_rot]``; cos, sin: ``[seq, 1, 1, d_rot]``."""
    if _fusable(q, k, cos, sin):
        if not _needs_grad(q, k):
            return _rotary_out_of_place(q, k, _on(cos, q.device), _on(sin, q.device), offset)[:2]
        return _FusedRotary.apply(q, k, _on(cos, q.device), _on(sin, q.device), offset)
    return _rotary_torch(q, k, cos, sin, offset)


def apply_rotary_pos_emb_torch(q, k, cos, sin, offset: int = 0):
    """Same contract as :func:`apply_rotary_pos_emb`; the reference keeps two copies
    because its TorchScript one cannot take bf16
    (megatron/model/positional_embeddings.py:119-126)."""
    return apply_rotary_pos_emb(q, k, cos, sin, offset)


# Writes made through raw pointers are invisible to autograd: the tensors' version counters have to be
# bumped by hand, or a tensor that another op saved for its backward pass could be rotated in place
# without the error autograd raises for such a change.
_increment_version = getattr(torch.autograd.graph, "increment_version", None)


def _may_bypass_autograd(*tensors):
    """The in-place rotation may skip the autograd Function: nothing needs a gradient and the
    version counters can still be bumped (or no graph is being recorded at all)."""
    return not _needs_grad(*tensors) and (_increment_version is not None or not torch.is_grad_enabled())


def _written_in_place(*tensors):
    if _increment_version is not None:
        _increment_version(tensors)


def _rotary_in_place(q, k, cos, sin, offset, d_rot):
    cos2 = _as_table(cos, d_rot, offset + q.shape[0])
    sin2 = _as_table(sin, d_rot, offset + q.shape[0])
    if q.numel() or k.numel():
        _rope_ext.rope_launch(q, k, q, k, cos2, sin2, d_rot, offset, backward=False)
    return cos2, sin2


class _FusedRotaryInplace(torch.autograd.Function):
    @staticmethod
    def forward(ctx, q, k, cos, sin, offset, d_rot):
        cos2, sin2 = _rotary_in_place(q, k, cos, sin, offset, d_rot)
        ctx.mark_dirty(q, k)
        ctx.save_for_backward(cos2, sin2)
        ctx.offset, ctx.d_rot = offset, d_rot
        return q, k

    @staticmethod
    def backward(ctx, grad_q, grad_k):
        cos2, sin2 = ctx.saved_tensors
        dq, dk = grad_q.clone(), grad_k.clone()
        dq, dk = _dense_last(dq), _dense_last(dk)
        if dq.numel() or dk.numel():
            _rope_ext.rope_launch(dq, dk, dq, dk, cos2, sin2, ctx.d_rot, ctx.offset, backward=True)
        return dq, dk, None, None, None, None


def apply_rotary_pos_emb_(q, k, cos, sin, offset: int = 0, rotary_ndims=None):
    """In-place rotary over the first ``rotary_ndims`` dims of whole heads.

    q, k: ``[sq, b, heads, hn]`` fp16/bf16 GPU tensors with a dense last dim; dims
    ``>= rotary_ndims`` are left untouched, so a partial rotary
    (megatron/model/transformer.py:823-860: slice, rotate, concatenate) becomes one
    pass that reads and writes only the rotated span.  Returns ``(q, k)``.
    """
    d_rot = q.shape[-1] if rotary_ndims is None else int(rotary_ndims)
    if not _fusable(q, k, cos, sin) or q.stride(-1) != 1 or k.stride(-1) != 1:
        raise RuntimeError(
            "apply_rotary_pos_emb_ needs fp16/bf16 GPU tensors [sq, b, heads, hn] with a dense last dim"
        )
    if d_rot > q.shape[-1] or d_rot % 2:
        raise RuntimeError(f"rotary_ndims={d_rot} must be even and <= head size {q.shape[-1]}")
    if _may_bypass_autograd(q, k):
        _rotary_in_place(q, k, _on(cos, q.device), _on(sin, q.device), offset, d_rot)
        _written_in_place(q, k)
        return q, k
    return _FusedRotaryInplace.apply(q, k, _on(cos, q.device), _on(sin, q.device), offset, d_rot)


class _FusedQKVRotary(torch.autograd.Function):
    @staticmethod
    def forward(ctx, mixed, cos, sin, offset, d_rot):
        hn = mixed.shape[-1] // 3
        cos2 = _as_table(cos, d_rot, offset + mixed.shape[0])
        sin2 = _as_table(sin, d_rot, offset + mixed.shape[0])
        if mixed.numel():
            q, k = mixed[..., :hn], mixed[..., hn : 2 * hn]
            _rope_ext.rope_launch(q, k, q, k, cos2, sin2, d_rot, offset, backward=False)
        ctx.mark_dirty(mixed)
        ctx.save_for_backward(cos2, sin2)
        ctx.offset, ctx.d_rot, ctx.hn = offset, d_rot, hn
        return mixed

    @staticmethod
    def backward(ctx, grad_mixed):
        cos2, sin2 = ctx.saved_tensors
        dm = grad_mixed.clone(memory_format=torch.contiguous_format)  # v and pass-through dims: identity
        if dm.numel():
            dq, dk = dm[..., : ctx.hn], dm[..., ctx.hn : 2 * ctx.hn]
            _rope_ext.rope_launch(dq, dk, dq, dk, cos2, sin2, ctx.d_rot, ctx.offset, backward=True)
        return dm, None, None, None, None


def apply_rotary_pos_emb_qkv_(mixed_x_layer, cos, sin, offset: int = 0, rotary_ndims=None):
    """Rotary at the call site of the attention layer, without its slice / concatenate copies.

    ``mixed_x_layer`` is the fused projection ``[sq, b, np, 3*hn]``
    (megatron/model/transformer.py:798-809).  The q and k thirds are rotated in place over
    their first ``rotary_ndims`` dims (all ``hn`` when None) in one launch; v and the
    pass-through dims are not touched.  Returns the views ``(query, key, value)``, each
    ``[sq, b, np, hn]`` -- what megatron/model/transformer.py:807-860 produces with two
    ``torch.cat`` and four slices.  Differentiable with respect to ``mixed_x_layer``.
    """
    if mixed_x_layer.dim() != 4 or mixed_x_layer.shape[-1] % 3:
        raise RuntimeError("mixed_x_layer must be [sq, b, np, 3*hn]")
    hn = mixed_x_layer.shape[-1] // 3
    d_rot = hn if rotary_ndims is None else int(rotary_ndims)
    if d_rot > hn or d_rot % 2:
        raise RuntimeError(f"rotary_ndims={d_rot} must be even and <= head size {hn}")
    if (
        not mixed_x_layer.is_cuda
        or mixed_x_layer.dtype not in _HALF
        or mixed_x_layer.stride(-1) != 1
        or cos.dtype != sin.dtype
        or cos.dtype not in (torch.float32, mixed_x_layer.dtype)
    ):
        raise RuntimeError(
            "apply_rotary_pos_emb_qkv_ needs an fp16/bf16 GPU tensor with a dense last dim and "
            "cos/sin in fp32 or its dtype"
        )
    dev = mixed_x_layer.device
    if _may_bypass_autograd(mixed_x_layer):
        mixed = mixed_x_layer
        if mixed.numel():
            _rotary_in_place(mixed[..., :hn], mixed[..., hn : 2 * hn], _on(cos, dev), _on(sin, dev), offset, d_rot)
            _written_in_place(mixed)
        return mixed[..., :hn], mixed[..., hn : 2 * hn], mixed[..., 2 * hn :]
    mixed = _FusedQKVRotary.apply(mixed_x_layer, _on(cos, dev), _on(sin, dev), offset, d_rot)
    return mixed[..., :hn], mixed[..., hn : 2 * hn], mixed[..., 2 * hn :]


class AliBi(torch.nn.Module):
    """Attention with linear biases: adds ``-slope_h * (i - j)`` for ``j <= i`` to the
    scores ``[b, np, sq, sk]`` (megatron/model/positional_embeddings.py:129-257); plain
    torch.  ``mp_rank`` selects this rank's slice of the head slopes."""

    def __init__(self, num_heads, mp_size=1, mp_rank=1):
        super().__init__()
        assert mp_size <= num_heads and mp_rank <= mp_size
        self.mp_size = mp_size
        self.mp_rank = mp_rank
        self.num_heads = num_heads
        self.slice_size = num_heads // mp_size
        self.cached_matrix = None
        self.cached_seq_len = None
        lo = mp_rank * self.slice_size
        slopes = torch.Tensor(self._get_slopes(num_heads))[lo : lo + self.slice_size]
        self.register_buffer("slopes", slopes)

    def _get_slopes(self, n):
        """Geometric slopes 2^(-8/n * (i+1)) for a power-of-two head count; other counts
        take the slopes of the power of two below and every second slope of the one above."""

        def pow2_slopes(m):
            first = 2.0 ** (-(2.0 ** -(math.log2(m) - 3)))
            return [first * first**i for i in range(m)]

        if math.log2(n).is_integer():
            return pow2_slopes(n)
        below = 2 ** math.floor(math.log2(n))
        return pow2_slopes(below) + self._get_slopes(2 * below)[0::2][: n - below]

    def _matrix(self, seq_len_q, seq_len_k, device, dtype):
        # build for the first key length seen, grow 4x when a longer one arrives
        if self.cached_seq_len is None or self.cached_seq_len < seq_len_k:
            n = seq_len_k if self.cached_seq_len is None else self.cached_seq_len * 4
            rows = torch.arange(n).view(n, 1)
            cols = torch.arange(n).view(1, n)
            dist = -torch.tril(rows - cols)
            dist = dist.to(device).to(dtype)
            slopes = self.slopes.to(dist.device).to(dist.dtype)
            self.cached_matrix = dist * slopes.view(self.slopes.shape[0], 1, 1)
            self.cached_seq_len = n
        a = self.cached_matrix
        if self.cached_seq_len > seq_len_k:
            a = a[:, :seq_len_k, :seq_len_k]
        if seq_len_q != seq_len_k:
            # decoding with a key/value cache: one query, the last row of the bias
            assert (
                seq_len_q == 1
            ), "assumption sq == sk unless at inference time with cache in layer_past with sq == 1"
            a = a[:, seq_len_k - 1, :].view(a.shape[0], 1, a.shape[2])
        return a

    def bias(self, seq_len_q, seq_len_k, device, dtype):
        return self._matrix(seq_len_q, seq_len_k, device, dtype)

    def forward(self, x):
        return x + self._matrix(x.shape[-2], x.shape[-1], x.device, x.dtype)
