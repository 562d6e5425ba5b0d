"""Host glue of the attention path (reference: trident/util/util.py:48-62,93-100)."""
import ctypes

import torch

from . import config

_DTYPE_CODES = {torch.float32: 0, torch.float16: 1, torch.bfloat16: 2}
_roctx = None


def dtype(input):
    """torch dtype -> element-type code of the C ABI (reference maps to Triton dtypes and
    raises the same error for anything else, trident/util/util.py:48-58)."""
    try:
        return _DTYPE_CODES[input]
    except KeyError:
        raise ValueError(f"Unable to convert the given input: '{input}'.") from None


def is_pow2(value):
    return False if value == 0 else (value & (value - 1)) == 0


def _load_roctx():
    global _roctx
    if _roctx is None:
        for name in ("libroctx64.so", "/opt/rocm/lib/libroctx64.so", "libroctx64.so.4"):
            try:
                _roctx = ctypes.CDLL(name)
                break
            except OSError:
                continue
        else:
            _roctx = False
        if _roctx:
            _roctx.roctxRangePushA.argtypes = [ctypes.c_char_p]
            _roctx.roctxRangePushA.restype = ctypes.c_int
            _roctx.roctxRangePop.restype = ctypes.c_int
    return _roctx


def push_trace(message: str):
    if config.use_trace:
        lib = _load_roctx()
        if lib:
            lib.roctxRangePushA(("Trident/" + message).encode())


def pop_trace():
    if config.use_trace:
        lib = _load_roctx()
        if lib:
            lib.roctxRangePop()
