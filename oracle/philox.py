"""TEST INFRASTRUCTURE ONLY: CPU restatement of the attention-dropout keep mask.

The reference draws the mask with ``torch.nn.Dropout`` inside the model-parallel RNG
tracker (megatron/model/transformer.py:536-539, megatron/mpu/random.py:20-37), i.e. from
the device generator's Philox4x32-10 stream selected by (seed, offset).  The fused
softmax+dropout kernels draw from the same generator family with their own, documented,
element-to-counter assignment; this file restates that assignment in numpy so that tests
can compare the kernels' keep pattern bit for bit.

* ``philox4x32_10``: the Philox4x32-10 block function of Salmon et al., "Parallel random
  numbers: as easy as 1, 2, 3" (SC'11).  Pinned in tests/test_oracle_dropout.py against
  the known-answer vectors published with Random123 (kat_vectors, three philox4x32 10
  lines) and against this image's ``torch.rand`` on the GPU, which consumes the same block
  function.
* ``keep_mask``: element ``e`` (row-major index into the score tensor) belongs to group
  ``e // 8``; the group's 128-bit block is ``philox(counter=(c_lo, c_hi, group_lo,
  group_hi), key=(seed_lo, seed_hi))`` with ``c = offset // 4`` (a generator offset counts
  32-bit outputs, four to a block, as in torch's device generator); element ``e`` owns the 16-bit field
  ``(word[(e % 8) // 2] >> (16 * (e % 2))) & 0xffff`` and is kept iff
  ``field >= threshold(p)``, ``threshold = round(p * 65536)``.
"""
import numpy as np

_M0 = np.uint64(0xD2511F53)
_M1 = np.uint64(0xCD9E8D57)
_W0 = 0x9E3779B9
_W1 = 0xBB67AE85
_LO = np.uint64(0xFFFFFFFF)
_S32 = np.uint64(32)


def philox4x32_10(counter, key):
    """counter: uint32 array [..., 4]; key: (k0, k1) python ints.  Returns uint32 [..., 4]."""
    c = np.asarray(counter, dtype=np.uint64)
    c0, c1, c2, c3 = (c[..., i].copy() for i in range(4))
    k0, k1 = int(key[0]) & 0xFFFFFFFF, int(key[1]) & 0xFFFFFFFF
    for _ in range(10):
        p0 = _M0 * c0  # 32x32 -> 64 bit products (operands < 2^32, so no overflow)
        p1 = _M1 * c2
        hi0, lo0 = p0 >> _S32, p0 & _LO
        hi1, lo1 = p1 >> _S32, p1 & _LO
        c0, c1, c2, c3 = hi1 ^ c1 ^ np.uint64(k0), lo1, hi0 ^ c3 ^ np.uint64(k1), lo0
        k0 = (k0 + _W0) & 0xFFFFFFFF
        k1 = (k1 + _W1) & 0xFFFFFFFF
    return np.stack([c0, c1, c2, c3], axis=-1).astype(np.uint32)


def threshold(p):
    """16-bit drop threshold: a field below it drops the element.  0 keeps all, 65536 none."""
    if not 0.0 <= p <= 1.0:
        raise ValueError("dropout probability has to be between 0 and 1, but got %r" % (p,))
    return int(round(p * 65536.0))


def dropout_scale(p):
    """1/(1-p) as torch's dropout kernel forms it: fp32 keep probability, fp32 quotient."""
    if p >= 1.0:
        return np.float32(0.0)
    keep = np.float32(1.0 - p)
    return np.float32(1.0 / np.float64(keep))


def keep_mask(n, p, seed, offset):
    """bool [n]: True where the element with row-major index 0..n-1 is kept."""
    groups = (n + 7) // 8
    g = np.arange(groups, dtype=np.uint64)
    ctr = np.empty((groups, 4), dtype=np.uint64)
    block = offset >> 2  # the Philox block the generator offset lies in
    ctr[:, 0] = np.uint64(block & 0xFFFFFFFF)
    ctr[:, 1] = np.uint64((block >> 32) & 0xFFFFFFFF)
    ctr[:, 2] = g & _LO
    ctr[:, 3] = g >> _S32
    words = philox4x32_10(ctr, (seed & 0xFFFFFFFF, (seed >> 32) & 0xFFFFFFFF))  # [groups, 4]
    fields = np.empty((groups, 8), dtype=np.uint32)
    fields[:, 0::2] = words & np.uint32(0xFFFF)
    fields[:, 1::2] = words >> np.uint32(16)
    return (fields.reshape(-1)[:n] >= np.uint32(threshold(p))) if threshold(p) <= 0xFFFF else np.zeros(n, bool)
