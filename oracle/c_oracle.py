"""ctypes view of oracle/attention_oracle.c (the plain-C restatement). TEST INFRASTRUCTURE ONLY."""
import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_SO = os.path.join(_HERE, "liboracle_attn.so")
_lib = None

_dp = ctypes.POINTER(ctypes.c_double)


def build():
    subprocess.check_call(["make", "-s", "-C", _HERE, "liboracle_attn.so"])


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(_SO):
            build()
        _lib = ctypes.CDLL(_SO)
        _lib.oracle_dropout_keep.restype = ctypes.c_int
        _lib.oracle_dropout_keep.argtypes = [ctypes.c_uint64, ctypes.c_uint32, ctypes.c_uint32, ctypes.c_uint32,
                                             ctypes.c_uint32, ctypes.c_int]
    return _lib


def _p(a):
    return None if a is None else a.ctypes.data_as(_dp)


def philox(ctr, key):
    c = (ctypes.c_uint32 * 4)(*ctr)
    k = (ctypes.c_uint32 * 2)(*key)
    o = (ctypes.c_uint32 * 4)()
    lib().oracle_philox4x32_10(c, k, o)
    return list(o)


def dropout_mask(seed, offset, bh, S, thr8):
    keep = np.empty((S, S), dtype=np.uint8)
    lib().oracle_dropout_mask(ctypes.c_uint64(seed), ctypes.c_uint32(offset), ctypes.c_uint32(bh), S, thr8,
                              keep.ctypes.data_as(ctypes.POINTER(ctypes.c_uint8)))
    return keep.astype(bool)


def fwd_head(q, k, v, mask, causal, scale, seed=0, offset=0, bh=0, thr8=0):
    S, D = q.shape
    q, k, v = [np.ascontiguousarray(x, dtype=np.float64) for x in (q, k, v)]
    mask = None if mask is None else np.ascontiguousarray(mask, dtype=np.float64)
    o = np.empty((S, D))
    lse2 = np.empty(S)
    lib().oracle_attn_fwd_head(_p(q), _p(k), _p(v), _p(mask), S, D, int(causal), ctypes.c_double(scale),
                               ctypes.c_uint64(seed), ctypes.c_uint32(offset), ctypes.c_uint32(bh), thr8,
                               _p(o), _p(lse2))
    return o, lse2


def bwd_head(q, k, v, mask, o, d_o, causal, scale, seed=0, offset=0, bh=0, thr8=0, want_dmask=False):
    S, D = q.shape
    q, k, v, o, d_o = [np.ascontiguousarray(x, dtype=np.float64) for x in (q, k, v, o, d_o)]
    mask = None if mask is None else np.ascontiguousarray(mask, dtype=np.float64)
    dq, dk, dv = np.empty((S, D)), np.empty((S, D)), np.empty((S, D))
    dmask = np.empty((S, S)) if want_dmask else None
    delta = np.empty(S)
    lib().oracle_attn_bwd_head(_p(q), _p(k), _p(v), _p(mask), _p(o), _p(d_o), S, D, int(causal),
                               ctypes.c_double(scale), ctypes.c_uint64(seed), ctypes.c_uint32(offset),
                               ctypes.c_uint32(bh), thr8, _p(dq), _p(dk), _p(dv), _p(dmask), _p(delta))
    return dq, dk, dv, dmask, delta
