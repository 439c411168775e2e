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
