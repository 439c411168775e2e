"""Independent float64 evaluation of the softmax and rotary formulas with explicit
loops (``math`` / numpy scalars, no torch ops).  Small inputs only; used to pin
``oracle.torch_ref``.  Test infrastructure: never imported by the product.
"""
import math

import numpy as np


def softmax_rows(x, scale, hidden=None):
    """x: [rows, cols] float array; hidden: same-shape bool (True = excluded) or None.
    A row with every entry hidden comes out uniform, as filling all its scores with
    one constant does (megatron/model/gpt2_model.py:49-57 followed by softmax)."""
    x = np.asarray(x, dtype=np.float64)
    rows, cols = x.shape
    out = np.zeros((rows, cols), dtype=np.float64)
    for r in range(rows):
        keep = [c for c in range(cols) if hidden is None or not hidden[r][c]]
        if not keep:
            for c in range(cols):
                out[r, c] = 1.0 / cols
            continue
        top = max(scale * x[r, c] for c in keep)
        total = 0.0
        for c in keep:
            total += math.exp(scale * x[r, c] - top)
        for c in keep:
            out[r, c] = math.exp(scale * x[r, c] - top) / total
    return out


def causal_hidden(sq, sk):
    return [[c > r for c in range(sk)] for r in range(sq)]


def softmax_rows_backward(g, y, scale):
    """dx[r, c] = scale * y[r, c] * (g[r, c] - sum_j g[r, j] y[r, j])."""
    g = np.asarray(g, dtype=np.float64)
    y = np.asarray(y, dtype=np.float64)
    rows, cols = y.shape
    dx = np.zeros_like(y)
    for r in range(rows):
        dot = 0.0
        for c in range(cols):
            dot += g[r, c] * y[r, c]
        for c in range(cols):
            dx[r, c] = scale * y[r, c] * (g[r, c] - dot)
    return dx


def rotary_angle(pos, j, dim, base=10000.0):
    """Angle of position ``pos`` for dim ``j``: pairs (j, j + dim/2) share a frequency
    (megatron/model/positional_embeddings.py:60-73)."""
    return pos * base ** (-2.0 * (j % (dim // 2)) / dim)


def rotary_vec(x, pos, base=10000.0):
    """Rotate one head vector x[dim] at position ``pos``: each pair (j, j+dim/2) turns by
    its angle, i.e. out_j = x_j cos - x_{j+h} sin, out_{j+h} = x_{j+h} cos + x_j sin."""
    x = np.asarray(x, dtype=np.float64)
    dim = x.shape[0]
    h = dim // 2
    out = np.zeros(dim, dtype=np.float64)
    for j in range(h):
        a = rotary_angle(pos, j, dim, base)
        c, s = math.cos(a), math.sin(a)
        out[j] = x[j] * c - x[j + h] * s
        out[j + h] = x[j + h] * c + x[j] * s
    return out


def rotary_vec_backward(g, pos, base=10000.0):
    """Transpose (= inverse rotation) applied to the output gradient."""
    g = np.asarray(g, dtype=np.float64)
    dim = g.shape[0]
    h = dim // 2
    out = np.zeros(dim, dtype=np.float64)
    for j in range(h):
        a = rotary_angle(pos, j, dim, base)
        c, s = math.cos(a), math.sin(a)
        out[j] = g[j] * c + g[j + h] * s
        out[j + h] = g[j + h] * c - g[j] * s
    return out


# --- attention dropout: Philox4x32-10 on Python integers -----------------------------------


def philox4x32_10(counter, key):
    """One Philox4x32-10 block (Salmon et al., SC'11) on Python integers: ``counter`` four and
    ``key`` two 32-bit words; ten rounds of two 32x32->64 bit multiplications, the key bumped
    by the Weyl constants between rounds."""
    c = [int(v) for v in counter]
    k = [int(v) for v in key]
    for _ in range(10):
        p0 = 0xD2511F53 * c[0]
        p1 = 0xCD9E8D57 * c[2]
        c = [(p1 >> 32) ^ c[1] ^ k[0], p1 & 0xFFFFFFFF, (p0 >> 32) ^ c[3] ^ k[1], p0 & 0xFFFFFFFF]
        k = [(k[0] + 0x9E3779B9) & 0xFFFFFFFF, (k[1] + 0xBB67AE85) & 0xFFFFFFFF]
    return c


def keep_element(e, p, seed, offset):
    """Whether the element with row-major index ``e`` survives a dropout of probability ``p``
    drawn from Philox state ``(seed, offset)``: its group of 8 shares the block with counter
    ``(offset // 4, e // 8)``; the element owns 16 bits of it and is kept iff they are not below
    ``round(p * 65536)``."""
    group = e // 8
    block = offset // 4
    words = philox4x32_10(
        [block & 0xFFFFFFFF, block >> 32, group & 0xFFFFFFFF, group >> 32],
        [seed & 0xFFFFFFFF, seed >> 32],
    )
    field = (words[(e % 8) // 2] >> (16 * (e % 2))) & 0xFFFF
    return field >= int(round(p * 65536))
