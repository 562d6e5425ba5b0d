"""Philox4x32-10 and the attention-dropout keep-mask (numpy). TEST INFRASTRUCTURE ONLY.

The reference draws its dropout numbers from ``tl.rand`` (Triton's Philox4x32,
10 rounds, Random123 constants; call sites trident/kernel/attention.py:159 and
trident/kernel/dropout.py:70-71) with a non-deterministic seed
(trident/operation/attention.py:125) and no test pins the stream
(tests/test_dropout.py:22-43 only uses p in {0, 1}).  The generator itself is
the published Random123 algorithm (Salmon et al., SC'11); it is pinned here by
the Random123 known-answer vectors (tests/golden/philox_kat.json).

Dropout convention of this build (what the HIP kernels implement bit for bit):

    key  = (seed & 0xffffffff, seed >> 32)
    ctr  = (j >> 2, i >> 2, bh, offset & 0xffffffff)
           i = query row, j = key column, bh = b * H + h
    r    = philox4x32_10(ctr, key)            # 4 x uint32, one 4x4 block of P
    u8   = (r[i & 3] >> (8 * (j & 3))) & 0xff
    keep = u8 >= thr8,   thr8 = clamp(rint(p * 256), 0, 256)
    Z    = keep / (1 - thr8 / 256)            # 0 everywhere when thr8 == 256

so the drop probability is quantised to multiples of 1/256 (the same 8-bit
granularity FlashAttention-2 uses) and the rescale uses the quantised value,
which keeps E[Z] == 1 exactly.  The layout does not depend on any tile shape.
"""
import numpy as np

PHILOX_M0 = np.uint64(0xD2511F53)
PHILOX_M1 = np.uint64(0xCD9E8D57)
PHILOX_W0 = 0x9E3779B9
PHILOX_W1 = 0xBB67AE85
MASK32 = np.uint64(0xFFFFFFFF)


def philox4x32_10(c0, c1, c2, c3, k0, k1, rounds=10):
    """Vectorised Philox4x32-R. Counter words are broadcastable uint32 arrays,
    key words are Python ints. Returns four uint32 arrays."""
    c0, c1, c2, c3 = np.broadcast_arrays(
        *[np.asarray(c, dtype=np.uint32) for c in (c0, c1, c2, c3)]
    )
    c0 = c0.astype(np.uint64)
    c1 = c1.astype(np.uint64)
    c2 = c2.astype(np.uint64)
    c3 = c3.astype(np.uint64)
    k0 = int(k0) & 0xFFFFFFFF
    k1 = int(k1) & 0xFFFFFFFF
    for _ in range(rounds):
        p0 = PHILOX_M0 * c0
        p1 = PHILOX_M1 * c2
        hi0, lo0 = p0 >> np.uint64(32), p0 & MASK32
        hi1, lo1 = p1 >> np.uint64(32), p1 & MASK32
        c0, c1, c2, c3 = (
            hi1 ^ c1 ^ np.uint64(k0),
            lo1,
            hi0 ^ c3 ^ np.uint64(k1),
            lo0,
        )
        k0 = (k0 + PHILOX_W0) & 0xFFFFFFFF
        k1 = (k1 + PHILOX_W1) & 0xFFFFFFFF
    return tuple(c.astype(np.uint32) for c in (c0, c1, c2, c3))


def philox4x32_10_scalar(ctr, key, rounds=10):
    """Pure-Python-int restatement of one Philox4x32-R call (cross-check for the
    vectorised one). ctr: 4 ints, key: 2 ints -> 4 ints."""
    c = [int(x) & 0xFFFFFFFF for x in ctr]
    k = [int(x) & 0xFFFFFFFF for x in key]
    for _ in range(rounds):
        p0 = 0xD2511F53 * c[0]
        p1 = 0xCD9E8D57 * c[2]
        c = [
            ((p1 >> 32) ^ c[1] ^ k[0]) & 0xFFFFFFFF,
            p1 & 0xFFFFFFFF,
            ((p0 >> 32) ^ c[3] ^ k[1]) & 0xFFFFFFFF,
            p0 & 0xFFFFFFFF,
        ]
        k = [(k[0] + PHILOX_W0) & 0xFFFFFFFF, (k[1] + PHILOX_W1) & 0xFFFFFFFF]
    return c


def dropout_threshold(p):
    """thr8 in [0, 256]: a decision byte u8 is kept iff u8 >= thr8."""
    p32 = float(np.float32(p))
    return int(min(256, max(0, int(np.rint(p32 * 256.0)))))


def dropout_scale(p):
    """1 / (1 - thr8/256), or 0 when everything is dropped."""
    thr = dropout_threshold(p)
    return 0.0 if thr >= 256 else 256.0 / (256.0 - thr)


def dropout_keep_mask(seed, offset, bh, rows, cols, p):
    """Boolean keep-mask [len(rows), len(cols)] for head index ``bh``.
    rows / cols are integer arrays of absolute query-row / key-column indices."""
    rows = np.asarray(rows, dtype=np.int64)
    cols = np.asarray(cols, dtype=np.int64)
    thr = dropout_threshold(p)
    i = rows[:, None]
    j = cols[None, :]
    r = philox4x32_10(
        (j >> 2).astype(np.uint32),
        (i >> 2).astype(np.uint32),
        np.uint32(bh),
        np.uint32(int(offset) & 0xFFFFFFFF),
        int(seed) & 0xFFFFFFFF,
        (int(seed) >> 32) & 0xFFFFFFFF,
    )
    words = np.stack(r, axis=0)  # [4, R, C]
    sel = np.broadcast_to((i & 3), words.shape[1:])
    word = np.take_along_axis(words, sel[None].astype(np.int64), axis=0)[0]
    u8 = (word >> ((j & 3) * 8).astype(np.uint32)) & np.uint32(0xFF)
    return u8.astype(np.int64) >= thr
