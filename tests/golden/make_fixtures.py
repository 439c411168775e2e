"""Writes the golden vectors tests/golden/*.npz.

The reference holds no vectors for this path, so these come from the float64
loop evaluation in ``oracle/brute.py`` (no torch op takes part).  Inputs are
multiples of 1/8 of magnitude < 32, exactly representable in fp16 and bf16, so
the same files serve both storage types.  Run from the repository root:

    python tests/golden/make_fixtures.py
"""
import os
import sys

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)
from oracle import brute  # noqa: E402

HERE = os.path.dirname(os.path.abspath(__file__))


def grid_values(rng, shape, span=200):
    return (rng.integers(-span, span + 1, size=shape) / 8.0).astype(np.float32)


def causal_case(rng, name, batches, s, scale):
    x = grid_values(rng, (batches, s, s))
    g = grid_values(rng, (batches, s, s), span=16)
    hidden = brute.causal_hidden(s, s)
    y = np.stack([brute.softmax_rows(x[b], scale, hidden) for b in range(batches)])
    dx = np.stack([brute.softmax_rows_backward(g[b], y[b], scale) for b in range(batches)])
    np.savez(os.path.join(HERE, name), x=x, g=g, y=y, dx=dx, scale=np.float64(scale))


def masked_case(rng, name, b, heads, sq, sk, scale, lengths):
    x = grid_values(rng, (b, heads, sq, sk))
    g = grid_values(rng, (b, heads, sq, sk), span=16)
    mask = np.zeros((b, 1, sq, sk), dtype=np.uint8)
    for i, n in enumerate(lengths):
        mask[i, 0, :, n:] = 1
    mask[0, 0, 1, :] = 1       # a row with every key hidden
    mask[b - 1, 0, 0, 0] = 1   # a hidden key in the middle of visible ones
    mask[b - 1, 0, 0, 3] = 1
    y = np.zeros(x.shape, dtype=np.float64)
    dx = np.zeros(x.shape, dtype=np.float64)
    for i in range(b):
        for h in range(heads):
            y[i, h] = brute.softmax_rows(x[i, h], scale, mask[i, 0].astype(bool))
            dx[i, h] = brute.softmax_rows_backward(g[i, h], y[i, h], scale)
    np.savez(os.path.join(HERE, name), x=x, g=g, mask=mask, y=y, dx=dx, scale=np.float64(scale))


def rotary_case(rng, name, s, b, heads, dim, offset, base=10000.0):
    q = grid_values(rng, (s, b, heads, dim), span=24)
    k = grid_values(rng, (s, b, heads, dim), span=24)
    gq = grid_values(rng, (s, b, heads, dim), span=24)
    gk = grid_values(rng, (s, b, heads, dim), span=24)
    oq, ok, dq, dk = (np.zeros(q.shape, dtype=np.float64) for _ in range(4))
    for t in range(s):
        for i in range(b):
            for h in range(heads):
                oq[t, i, h] = brute.rotary_vec(q[t, i, h], t + offset, base)
                ok[t, i, h] = brute.rotary_vec(k[t, i, h], t + offset, base)
                dq[t, i, h] = brute.rotary_vec_backward(gq[t, i, h], t + offset, base)
                dk[t, i, h] = brute.rotary_vec_backward(gk[t, i, h], t + offset, base)
    np.savez(os.path.join(HERE, name), q=q, k=k, gq=gq, gk=gk, oq=oq, ok=ok, dq=dq, dk=dk,
             offset=np.int64(offset), base=np.float64(base))


def dropout_case(rng, name, batches, s, scale, p, seed, offset):
    """Causal softmax followed by dropout: the keep pattern from the integer Philox of
    oracle/brute.py, everything else in float64 (no rounding of the probabilities)."""
    x = grid_values(rng, (batches, s, s))
    g = grid_values(rng, (batches, s, s), span=16)
    hidden = brute.causal_hidden(s, s)
    keep = np.array([brute.keep_element(e, p, seed, offset) for e in range(x.size)]).reshape(x.shape)
    y = np.stack([brute.softmax_rows(x[b], scale, hidden) for b in range(batches)])
    y_drop = y * keep / (1.0 - p)
    dx = np.stack([brute.softmax_rows_backward(g[b] * keep[b] / (1.0 - p), y[b], scale) for b in range(batches)])
    np.savez(os.path.join(HERE, name), x=x, g=g, y=y, keep=keep.astype(np.uint8), y_drop=y_drop, dx=dx,
             scale=np.float64(scale), p=np.float64(p), seed=np.uint64(seed), offset=np.uint64(offset))


def main():
    rng = np.random.default_rng(20240521)
    causal_case(rng, "causal_8", batches=2, s=8, scale=0.125)
    causal_case(rng, "causal_40", batches=1, s=40, scale=0.5)
    masked_case(rng, "masked_4x16", b=2, heads=2, sq=4, sk=16, scale=0.25, lengths=[16, 9])
    masked_case(rng, "masked_3x37", b=2, heads=1, sq=3, sk=37, scale=0.125, lengths=[20, 37])
    rotary_case(rng, "rotary_d8", s=5, b=2, heads=2, dim=8, offset=3)
    rotary_case(rng, "rotary_d32", s=6, b=1, heads=3, dim=32, offset=0)
    rotary_case(rng, "rotary_d24", s=4, b=2, heads=1, dim=24, offset=1)
    # drawn after all earlier cases, so their files do not change
    dropout_case(rng, "dropout_causal_16", batches=2, s=16, scale=0.25, p=0.25, seed=2**40 + 77, offset=2**33 + 8)
    dropout_case(rng, "dropout_causal_37", batches=1, s=37, scale=0.125, p=0.1, seed=1234, offset=0)


if __name__ == "__main__":
    main()
