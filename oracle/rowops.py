"""fp64 CPU restatement of the attention path's sibling operations. TEST INFRASTRUCTURE ONLY.

* softmax along a dimension (trident/kernel/softmax.py:34-121): exp(x - max) / sum exp(x - max);
* masked softmax (trident/kernel/masked_softmax.py:25-88): positions with mask > eps count as -inf
  (the reference's own test states it as torch.where(mask.bool(), -inf, input), tests/test_masked_softmax.py:22-26);
* their gradient (trident/kernel/softmax.py:123-238): delta = sum(dO * O), dX = O * (dO - delta);
* dropout on this build's documented Philox stream (the reference's stream is unpinned, tests/test_dropout.py:22-43
  use p in {0, 1} only): element i takes byte (i & 3) of word ((i >> 2) & 3) of
  philox4x32_10(ctr = (lo32(i >> 4), hi32(i >> 4), 0x44524F50, offset), key = seed); keep iff byte >= thr8;
  kept elements are scaled by 256 / (256 - thr8); the gradient is masked and scaled the same way.

Pinned by tests/test_rowops_oracle.py: torch.softmax and torch autograd in fp64, the reference's masked-softmax
test formula, a pure-Python-int Philox restatement for the dropout layout, keep rates, p in {0, 1} against
torch.nn.functional.dropout.
"""
import numpy as np

from . import philox

EPS = 2.220446049250313e-16  # trident/language/constant.py:17-20
DROPOUT_STREAM = 0x44524F50


def softmax_forward(x, dim, mask=None):
    x = np.asarray(x, dtype=np.float64)
    if mask is not None:
        x = np.where(np.asarray(mask, dtype=np.float64) > EPS, -np.inf, x)
    m = np.max(x, axis=dim, keepdims=True)
    m = np.where(np.isfinite(m), m, 0.0)
    e = np.exp(x - m)
    with np.errstate(divide="ignore", invalid="ignore"):
        return e / np.sum(e, axis=dim, keepdims=True)


def softmax_backward(out, grad_out, dim):
    out = np.asarray(out, dtype=np.float64)
    grad_out = np.asarray(grad_out, dtype=np.float64)
    delta = np.sum(out * grad_out, axis=dim, keepdims=True)
    return out * (grad_out - delta)


def dropout_keep(seed, offset, n, p):
    """Boolean keep decisions of elements 0..n-1."""
    i = np.arange(n, dtype=np.int64)
    blk = i >> 4
    r = philox.philox4x32_10((blk & 0xFFFFFFFF).astype(np.uint32), (blk >> 32).astype(np.uint32), np.uint32(DROPOUT_STREAM),
                             np.uint32(int(offset) & 0xFFFFFFFF), int(seed) & 0xFFFFFFFF, (int(seed) >> 32) & 0xFFFFFFFF)
    words = np.stack(r, axis=0)  # [4, n]
    word = np.take_along_axis(words, ((i >> 2) & 3)[None], axis=0)[0]
    u8 = (word >> ((i & 3) * 8).astype(np.uint32)) & np.uint32(0xFF)
    return u8.astype(np.int64) >= philox.dropout_threshold(p)


def dropout_apply(x, p, seed, offset):
    """Forward on the input, or backward on the incoming gradient: the same masked scaling."""
    x = np.asarray(x, dtype=np.float64)
    keep = dropout_keep(seed, offset, x.size, p).reshape(x.shape)
    return np.where(keep, x * philox.dropout_scale(p), 0.0)
