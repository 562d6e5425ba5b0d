"""Writes the committed fixtures of this directory from the CPU oracle.

    python tests/golden/make_fixtures.py

The reference stores no golden vectors for attention (its tests compare against PyTorch at run
time with unseeded inputs, tests/test_attention.py:26-28,47-50), so these files pin this build's
own oracle: attention_small.npz (inputs and fp64 outputs/gradients for three variants) and
dropout_mask.json (keep bits of the documented Philox layout). philox_kat.json holds the
Random123 known-answer vectors and is not generated here.
"""
import json
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(os.path.dirname(HERE)))

from oracle import attention as oracle  # noqa: E402
from oracle import philox  # noqa: E402


def main():
    rng = np.random.default_rng(20240607)
    B, H, S, D = 1, 2, 16, 16
    q, k, v, d_o = [rng.standard_normal((B, H, S, D)).astype(np.float32).astype(np.float64) for _ in range(4)]
    mask = rng.standard_normal((B, 1, S, S)).astype(np.float32).astype(np.float64)
    mask[0, 0, :, 13:] = -np.inf
    out = {"q": q, "k": k, "v": v, "d_o": d_o, "mask": mask}
    variants = {
        "plain": dict(),
        "causal": dict(is_causal=True),
        "mask_dropout": dict(mask=mask, dropout_p=0.25, seed=0x5EED, offset=2),
    }
    for name, kw in variants.items():
        o, lse2 = oracle.attention_forward(q, k, v, **kw)
        dq, dk, dv, dmask, delta = oracle.attention_backward(q, k, v, d_o, want_dmask=True, **kw)
        out[f"{name}.o"], out[f"{name}.lse2"] = o, lse2
        out[f"{name}.dq"], out[f"{name}.dk"], out[f"{name}.dv"], out[f"{name}.delta"] = dq, dk, dv, delta
        if dmask is not None:
            out[f"{name}.dmask"] = dmask
    np.savez_compressed(os.path.join(HERE, "attention_small.npz"), **out)

    cases = []
    for seed, offset, bh, p in [(0x5EED, 0, 3, 0.1), (0xDEADBEEFCAFE, 7, 31, 0.5), (1, 0xFFFFFFFF, 0, 0.9)]:
        keep = philox.dropout_keep_mask(seed, offset, bh, np.arange(32), np.arange(40, 72), p)
        bits = np.packbits(keep.astype(np.uint8), axis=None).tobytes().hex()
        cases.append({"seed": seed, "offset": offset, "bh": bh, "p": p, "row0": 0, "rows": 32, "col0": 40, "cols": 32,
                      "thr8": philox.dropout_threshold(p), "keep_bits_hex": bits})
    with open(os.path.join(HERE, "dropout_mask.json"), "w") as f:
        json.dump({"layout": "row-major keep bits, numpy.packbits order", "cases": cases}, f, indent=1)


if __name__ == "__main__":
    main()
