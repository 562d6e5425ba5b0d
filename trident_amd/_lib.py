"""ctypes binding of libtrident_attn.so (declarations: include/tri_attn.h)."""
import ctypes
import os
import struct

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.environ.get("TRIDENT_AMD_LIB") or os.path.join(_HERE, "libtrident_attn.so")  # (another build of the library)
EALIGN = -8
ENOFUSE = -9  # tri_attn_bwd_dq_delta: no fused kernel for this problem, nothing launched
ABI_VERSION = 3
ESCRATCH = -10  # tri_attn_bwd_noalloc: B*H*S above NOALLOC_MAX_ROWS, nothing launched
NOALLOC_MAX_ROWS = 1 << 20

_i64x4 = ctypes.c_int64 * 4


class TriAttnArgs(ctypes.Structure):
    _fields_ = [
        ("struct_size", ctypes.c_uint32),
        ("dtype", ctypes.c_int32),
        ("B", ctypes.c_int32),
        ("H", ctypes.c_int32),
        ("S", ctypes.c_int32),
        ("D", ctypes.c_int32),
        ("is_causal", ctypes.c_int32),
        ("mask_dtype", ctypes.c_int32),
        ("softmax_scale", ctypes.c_float),
        ("dropout_p", ctypes.c_float),
        ("seed", ctypes.c_uint64),
        ("offset", ctypes.c_uint64),
        ("q", ctypes.c_void_p),
        ("k", ctypes.c_void_p),
        ("v", ctypes.c_void_p),
        ("o", ctypes.c_void_p),
        ("lse", ctypes.c_void_p),
        ("mask", ctypes.c_void_p),
        ("d_o", ctypes.c_void_p),
        ("dq", ctypes.c_void_p),
        ("dk", ctypes.c_void_p),
        ("dv", ctypes.c_void_p),
        ("dmask", ctypes.c_void_p),
        ("delta", ctypes.c_void_p),
        ("q_stride", _i64x4),
        ("k_stride", _i64x4),
        ("v_stride", _i64x4),
        ("o_stride", _i64x4),
        ("do_stride", _i64x4),
        ("dq_stride", _i64x4),
        ("dk_stride", _i64x4),
        ("dv_stride", _i64x4),
        ("mask_stride", _i64x4),
        ("dmask_stride", _i64x4),
        ("stream", ctypes.c_void_p),
        ("mask_classes", ctypes.c_void_p),
    ]


# TriAttnArgs as one struct.pack_into call (an argument structure filled field by field costs a small call several
# microseconds): scalars, the twelve pointers, the ten stride arrays, stream and mask_classes, in declaration order.
ARGS_PACKER = struct.Struct("@Iiiiiiiiff" "QQ" "12P" "40q" "PP")
assert ARGS_PACKER.size == ctypes.sizeof(TriAttnArgs)


class TriRowArgs(ctypes.Structure):
    """include/tri_rowops.h"""
    _fields_ = [
        ("struct_size", ctypes.c_uint32),
        ("dtype", ctypes.c_int32),
        ("y_size", ctypes.c_int64),
        ("x_size", ctypes.c_int64),
        ("y_stride", ctypes.c_int64),
        ("x_stride", ctypes.c_int64),
        ("input", ctypes.c_void_p),
        ("output", ctypes.c_void_p),
        ("mask", ctypes.c_void_p),
        ("mask_dtype", ctypes.c_int32),
        ("p", ctypes.c_float),
        ("grad_output", ctypes.c_void_p),
        ("grad_input", ctypes.c_void_p),
        ("seed", ctypes.c_uint64),
        ("offset", ctypes.c_uint64),
        ("stream", ctypes.c_void_p),
    ]


ROW_EXPORTS = ("tri_softmax_fwd", "tri_softmax_bwd", "tri_dropout_fwd", "tri_dropout_bwd")

EXPORTS = (
    "tri_attn_version",
    "tri_attn_strerror",
    "tri_attn_fwd",
    "tri_attn_bwd_delta",
    "tri_attn_bwd_dkdv",
    "tri_attn_bwd_dq",
    "tri_attn_bwd_dq_delta",
    "tri_attn_bwd",
    "tri_attn_bwd_noalloc",
    "tri_attn_dropout_mask",
    "tri_attn_uses_matrix_cores",
    "tri_attn_classify_mask",
    "tri_attn_mask_classes_size",
)

_lib = None


def lib():
    """The loaded library. Raises if it has not been built: there is no fallback path."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise RuntimeError(
                f"{LIB_PATH} is missing: build it with `python -m trident_amd.build` "
                "(hipcc, gfx950). trident_amd has no CPU or PyTorch fallback."
            )
        cdll = ctypes.CDLL(LIB_PATH)
        for name in EXPORTS:
            getattr(cdll, name)  # AttributeError if a declared symbol is not exported
        cdll.tri_attn_version.restype = ctypes.c_int
        cdll.tri_attn_strerror.restype = ctypes.c_char_p
        cdll.tri_attn_strerror.argtypes = [ctypes.c_int]
        for name in ("tri_attn_fwd", "tri_attn_bwd_delta", "tri_attn_bwd_dkdv", "tri_attn_bwd_dq",
                     "tri_attn_bwd_dq_delta", "tri_attn_bwd", "tri_attn_bwd_noalloc", "tri_attn_classify_mask"):
            fn = getattr(cdll, name)
            fn.restype = ctypes.c_int
            fn.argtypes = [ctypes.POINTER(TriAttnArgs)]
        cdll.tri_attn_mask_classes_size.restype = ctypes.c_int64
        cdll.tri_attn_mask_classes_size.argtypes = [ctypes.POINTER(TriAttnArgs)]
        cdll.tri_attn_uses_matrix_cores.restype = ctypes.c_int
        cdll.tri_attn_uses_matrix_cores.argtypes = [ctypes.POINTER(TriAttnArgs), ctypes.c_int]
        cdll.tri_attn_dropout_mask.restype = ctypes.c_int
        cdll.tri_attn_dropout_mask.argtypes = [
            ctypes.c_uint64, ctypes.c_uint64, ctypes.c_float, ctypes.c_uint32,
            ctypes.c_int32, ctypes.c_int32, ctypes.c_int32, ctypes.c_int32,
            ctypes.c_void_p, ctypes.c_void_p,
        ]
        for name in ROW_EXPORTS:
            fn = getattr(cdll, name)  # AttributeError if a declared symbol is not exported
            fn.restype = ctypes.c_int
            fn.argtypes = [ctypes.POINTER(TriRowArgs)]
        if cdll.tri_attn_version() != ABI_VERSION:
            raise RuntimeError("libtrident_attn.so ABI version mismatch: rebuild it")
        _lib = cdll
    return _lib


PROBE_LIB_PATH = os.path.join(_HERE, "libtri_probe.so")
PROBE_EXPORTS = ("tri_probe_mfma", "tri_probe_coexec")
_probe = None


def probe_lib():
    """The calibration kernels of include/tri_probe.h (a library of their own; only bench.py --ceiling loads it)."""
    global _probe
    if _probe is None:
        if not os.path.exists(PROBE_LIB_PATH):
            raise RuntimeError(f"{PROBE_LIB_PATH} is missing: build it with `python -m trident_amd.build`")
        cdll = ctypes.CDLL(PROBE_LIB_PATH)
        cdll.tri_probe_mfma.restype = ctypes.c_int
        cdll.tri_probe_mfma.argtypes = [ctypes.c_int, ctypes.c_int, ctypes.c_int, ctypes.c_void_p, ctypes.c_void_p,
                                        ctypes.c_void_p]
        cdll.tri_probe_coexec.restype = ctypes.c_int
        cdll.tri_probe_coexec.argtypes = [ctypes.c_int, ctypes.c_int, ctypes.c_int, ctypes.c_int, ctypes.c_int,
                                          ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p]
        _probe = cdll
    return _probe


def check(status):
    if status != 0:
        raise RuntimeError("tri_attn: " + lib().tri_attn_strerror(status).decode())
