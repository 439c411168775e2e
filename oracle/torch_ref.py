"""The reference's unfused path, restated in plain torch (runs on any device).

Each function names the reference lines it follows (paths relative to the
GPT-NeoX source tree).  Test infrastructure: never imported by the product.
"""
import torch


# --- masks -------------------------------------------------------------------------


def get_attn_mask(seq_length, device="cpu", sliding_window_width=None):
    """Boolean ``[1, 1, s, s]`` mask, True = hidden: everything above the diagonal,
    and (optionally) everything more than ``sliding_window_width`` below it.
    Follows megatron/utils.py:67-80."""
    visible = torch.tril(torch.ones((1, seq_length, seq_length), device=device))
    visible = visible.view(1, 1, seq_length, seq_length)
    if sliding_window_width is not None:
        visible = torch.triu(visible, diagonal=-sliding_window_width)
    return visible < 0.5


def gpt2_attention_mask_func(attention_scores, ltor_mask):
    """Fill hidden positions with the most negative finite value of the score dtype,
    in place.  Follows megatron/model/gpt2_model.py:49-57."""
    lowest = torch.tensor(
        torch.finfo(attention_scores.dtype).min,
        dtype=attention_scores.dtype,
        device=attention_scores.device,
    )
    attention_scores.masked_fill_(ltor_mask, lowest)
    return attention_scores


def padding_mask(lengths, sq, sk, device="cpu"):
    """``[b, 1, sq, sk]`` bool mask hiding keys ``j >= lengths[b]``."""
    lengths = torch.as_tensor(lengths, device=device)
    hide = torch.arange(sk, device=device)[None, None, None, :] >= lengths[:, None, None, None]
    return hide.expand(lengths.numel(), 1, sq, sk).contiguous()


# --- softmax -----------------------------------------------------------------------


def forward_torch_softmax(
    input,
    mask,
    scale,
    input_in_fp16=False,
    input_in_bf16=False,
    softmax_in_fp32=True,
    mask_func=gpt2_attention_mask_func,
):
    """scale -> mask -> softmax over the last dim -> cast back.
    Follows FusedScaleMaskSoftmax.forward_torch_softmax,
    megatron/model/fused_softmax.py:184-199."""
    half_in = input_in_fp16 or input_in_bf16
    if half_in and softmax_in_fp32:
        input = input.float()
    if scale is not None:
        input = input * scale
    if mask is not None:
        input = mask_func(input, mask)
    probs = torch.nn.Softmax(dim=-1)(input)
    if half_in and softmax_in_fp32:
        probs = probs.half() if input_in_fp16 else probs.bfloat16()
    return probs


def softmax_fp32(x, mask, scale):
    """The fp32 probabilities of the unfused path *before* the final cast: the value
    the |err| <= 2e-3 (bf16) / 1e-3 (fp16) bars are measured against."""
    t = x.float()
    t = t * scale if scale is not None else t.clone()
    if mask is not None:
        t = gpt2_attention_mask_func(t, mask)
    return torch.softmax(t, dim=-1)


def softmax_backward_fp32(grad_out, probs, scale):
    """d/dx of softmax(scale*x): ``scale * y * (g - sum_j g_j y_j)`` in fp32.
    This is what the reference's fused backward evaluates
    (megatron/fused_kernels/scaled_masked_softmax.h:240-335) and what autograd
    gives for the unfused path wherever y > 0."""
    g = grad_out.float()
    y = probs.float()
    dot = (g * y).sum(dim=-1, keepdim=True)
    s = 1.0 if scale is None else scale
    return s * (y * (g - dot))


def softmax_autograd_fp32(x, mask, scale, grad_out):
    """Forward + autograd backward of the unfused path in fp32; returns (probs, dx)."""
    xf = x.detach().float().requires_grad_(True)
    t = xf * scale if scale is not None else xf * 1.0
    if mask is not None:
        t = gpt2_attention_mask_func(t, mask)
    y = torch.softmax(t, dim=-1)
    y.backward(grad_out.float())
    return y.detach(), xf.grad


# --- attention dropout ----------------------------------------------------------------


def dropout_scale(p):
    """``1/(1-p)`` as torch's device dropout kernel forms it: the keep probability is
    narrowed to fp32 and the quotient is taken from that (0 for ``p == 1``)."""
    if p >= 1.0:
        return 0.0
    keep = torch.tensor(1.0 - p, dtype=torch.float32)
    return float((1.0 / keep.double()).float())


def dropout_with_mask(probs, keep, p):
    """``torch.nn.Dropout(p)`` on ``probs`` for a given keep pattern, as the attention
    dropout of megatron/model/transformer.py:536-539 computes it on the device:
    ``probs * keep * 1/(1-p)`` in fp32, rounded once to the dtype of ``probs``."""
    scale = torch.tensor(dropout_scale(p), dtype=torch.float32, device=probs.device)
    return torch.where(keep, probs.float() * scale, torch.zeros((), device=probs.device)).to(probs.dtype)


def softmax_dropout_backward_fp32(grad_out, probs, keep, p, scale):
    """Gradient of ``dropout(softmax(scale * x))`` with respect to ``x`` in fp32:
    the dropout's backward ``g = grad_out * keep / (1-p)`` followed by
    ``softmax_backward_fp32`` (autograd of transformer.py:533-539)."""
    g = torch.where(keep, grad_out.float() * dropout_scale(p), torch.zeros((), device=grad_out.device))
    return softmax_backward_fp32(g, probs, scale)


def alibi_slopes(n):
    """Head slopes of ALiBi: 2^(-8/n * (k+1)) for a power-of-two n, otherwise the slopes of the
    power of two below plus every second slope of the one above.
    Follows AliBi._get_slopes, megatron/model/positional_embeddings.py:147-170."""
    import math

    def power_of_two(m):
        start = 2 ** (-(2 ** -(math.log2(m) - 3)))
        return [start * start**k for k in range(m)]

    if math.log2(n).is_integer():
        return power_of_two(n)
    below = 2 ** math.floor(math.log2(n))
    return power_of_two(below) + alibi_slopes(2 * below)[0::2][: n - below]


def alibi_bias_fp32(slopes, sq, sk, device="cpu"):
    """fp32 ALiBi bias [np, sq, sk]: -slope_h * (i - j) on j <= i, 0 above the diagonal; with
    sq == 1 (a decode step against a key/value cache) the last row of the [sk, sk] matrix.
    Follows AliBi.forward, megatron/model/positional_embeddings.py:210-257 (sq != sk: 236-250)."""
    j = torch.arange(sk, device=device, dtype=torch.int32).view(1, sk)
    if sq != sk:
        assert sq == 1, "assumption sq == sk unless at inference time with cache in layer_past with sq == 1"
        dist = -((sk - 1) - j).float()  # row sk - 1 of the [sk, sk] matrix, without building it
    else:
        i = torch.arange(sk, device=device, dtype=torch.int32).view(sk, 1)
        dist = -torch.tril(i - j).float()
    return dist * torch.as_tensor(slopes, dtype=torch.float32, device=device).view(-1, 1, 1)


# --- rotary ------------------------------------------------------------------------


def rotary_tables(dim, seq_len, base=10000, precision=torch.float):
    """cos/sin ``[seq, 1, 1, dim]``: angle(t, j) = t * base^(-2 (j mod dim/2) / dim),
    evaluated in fp32, then cast.  Follows RotaryEmbedding._prepare_cache,
    megatron/model/positional_embeddings.py:60-80."""
    inv_freq = 1.0 / (base ** (torch.arange(0, dim, 2).float() / dim))
    t = torch.arange(seq_len).type_as(inv_freq)
    freqs = torch.einsum("i,j->ij", t, inv_freq)
    emb = torch.cat((freqs, freqs), dim=-1)
    cos = emb.cos()[:, None, None, :]
    sin = emb.sin()[:, None, None, :]
    return cos.to(precision), sin.to(precision)


def rotary_tables_from_freqs(freqs):
    """cos/sin of fp32 angles ``[s, 1, 1, d2]``, evaluated in fp32: what the ``freqs`` variant of
    the fused rotary evaluates per element inside its kernel.
    Follows megatron/fused_kernels/fused_rotary_positional_embedding.h:47-49, 95-98."""
    freqs = freqs.float()
    return freqs.cos(), freqs.sin()


def rotate_half(x):
    """Follows megatron/model/positional_embeddings.py:103-107."""
    x1, x2 = x[..., : x.shape[-1] // 2], x[..., x.shape[-1] // 2 :]
    return torch.cat((-x2, x1), dim=x1.ndim - 1)


def apply_rotary_pos_emb(q, k, cos, sin, offset=0):
    """Follows apply_rotary_pos_emb_torch, megatron/model/positional_embeddings.py:119-126."""
    cos = cos[offset : q.shape[0] + offset, ...]
    sin = sin[offset : q.shape[0] + offset, ...]
    return (q * cos) + (rotate_half(q) * sin), (k * cos) + (rotate_half(k) * sin)


def rotary_fp32(q, k, cos, sin, offset=0):
    """The unfused expression evaluated in fp32 from the stored q/k values."""
    return apply_rotary_pos_emb(q.float(), k.float(), cos.float(), sin.float(), offset)


def rotary_autograd_fp32(q, k, cos, sin, grad_q, grad_k, offset=0):
    """Autograd gradients of the unfused expression in fp32; returns (dq, dk)."""
    qf = q.detach().float().requires_grad_(True)
    kf = k.detach().float().requires_grad_(True)
    oq, ok = apply_rotary_pos_emb(qf, kf, cos.float(), sin.float(), offset)
    torch.autograd.backward([oq, ok], [grad_q.float(), grad_k.float()])
    return qf.grad, kf.grad


def partial_rotary(q, k, cos, sin, rotary_ndims, offset=0):
    """Slice the first ``rotary_ndims`` dims, rotate, concatenate the rest back.
    Follows megatron/model/transformer.py:823-860."""
    q_rot, q_pass = q[..., :rotary_ndims], q[..., rotary_ndims:]
    k_rot, k_pass = k[..., :rotary_ndims], k[..., rotary_ndims:]
    q_rot, k_rot = apply_rotary_pos_emb(q_rot, k_rot, cos, sin, offset)
    return torch.cat((q_rot, q_pass), dim=-1), torch.cat((k_rot, k_pass), dim=-1)
