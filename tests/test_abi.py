"""Boundary checks that need no GPU: the library loads, exports what include/tri_attn.h declares,
the ctypes struct matches the C one, and argument errors surface as the reference's errors."""
import ctypes
import os
import re
import subprocess

import pytest
import torch

import trident_amd as trident
from trident_amd import _lib

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "tri_attn.h")


def test_library_exports_every_declared_symbol():
    text = open(HEADER).read()
    declared = set(re.findall(r"\b(tri_attn_\w+)\s*\(", text))
    assert declared == set(_lib.EXPORTS)
    lib = _lib.lib()
    for name in declared:
        assert hasattr(lib, name)
    assert lib.tri_attn_version() == _lib.ABI_VERSION


def test_probe_library_exports_its_header():
    """The calibration kernels live in a library and header of their own, outside the operator's boundary."""
    text = open(os.path.join(ROOT, "include", "tri_probe.h")).read()
    declared = set(re.findall(r"\b(tri_probe_\w+)\s*\(", text))
    assert declared == set(_lib.PROBE_EXPORTS)
    assert not re.search(r"tri_\w*probe", open(HEADER).read())
    lib = _lib.probe_lib()
    for name in declared:
        assert hasattr(lib, name)


def test_struct_layout_matches_header(tmp_path):
    src = tmp_path / "sz.c"
    src.write_text(
        '#include <stdio.h>\n#include <stddef.h>\n#include "tri_attn.h"\n'
        'int main(){printf("%zu %zu %zu %zu %zu", sizeof(TriAttnArgs), offsetof(TriAttnArgs,seed),'
        ' offsetof(TriAttnArgs,q), offsetof(TriAttnArgs,mask_stride), offsetof(TriAttnArgs,stream));}'
    )
    exe = tmp_path / "sz"
    subprocess.check_call(["gcc", "-I", os.path.dirname(HEADER), str(src), "-o", str(exe)])
    got = [int(x) for x in subprocess.check_output([str(exe)]).split()]
    T = _lib.TriAttnArgs
    assert got == [ctypes.sizeof(T), T.seed.offset, T.q.offset, T.mask_stride.offset, T.stream.offset]


def test_status_codes_without_gpu():
    lib = _lib.lib()
    assert lib.tri_attn_fwd(None) == -1
    args = _lib.TriAttnArgs()
    assert lib.tri_attn_fwd(ctypes.byref(args)) == -7  # struct_size unset
    args.struct_size = ctypes.sizeof(args)
    args.dtype = 9
    assert lib.tri_attn_fwd(ctypes.byref(args)) == -3
    args.dtype = 2
    args.B, args.H, args.S, args.D = 1, 1, 128, 48
    assert lib.tri_attn_fwd(ctypes.byref(args)) == -2
    args.D = 64
    args.dropout_p = 1.5
    assert lib.tri_attn_bwd(ctypes.byref(args)) == -6
    args.dropout_p = 0.0
    assert lib.tri_attn_fwd(ctypes.byref(args)) == -1  # pointers missing
    args.mask = 64
    args.is_causal = 1
    assert lib.tri_attn_fwd(ctypes.byref(args)) == -5
    assert b"mask and is_causal" in lib.tri_attn_strerror(-5)
    assert lib.tri_attn_dropout_mask(0, 0, 0.1, 0, 0, 4, 0, 4, None, None) == -1
    # the entry point that allocates nothing refuses problems beyond its buffer before it touches the GPU
    big = _lib.TriAttnArgs()
    big.struct_size = ctypes.sizeof(big)
    big.dtype = 2
    big.B, big.H, big.S, big.D = 1, 64, _lib.NOALLOC_MAX_ROWS // 64 + 128, 64
    assert lib.tri_attn_bwd_noalloc(ctypes.byref(big)) == _lib.ESCRATCH
    assert lib.tri_attn_bwd_noalloc(None) == -1
    # the combined backward checks the arguments of all three launches before the first one: a call without dK
    # is refused as a whole, not after dQ and delta have been written (the pointers below are never followed)
    part = _lib.TriAttnArgs()
    part.struct_size = ctypes.sizeof(part)
    part.dtype = 2
    part.B, part.H, part.S, part.D = 1, 1, 256, 64
    for name in ("q", "k", "v", "o", "lse", "d_o", "delta", "dq", "dv"):
        setattr(part, name, 4096)
    for name in ("q_stride", "k_stride", "v_stride", "o_stride", "do_stride", "dq_stride", "dk_stride", "dv_stride"):
        getattr(part, name)[:] = [256 * 64, 256 * 64, 64, 1]
    assert lib.tri_attn_bwd(ctypes.byref(part)) == -1  # dk missing


def test_reference_value_errors():
    """Same texts as trident/operation/attention.py:28-45."""
    f = trident.function.scaled_dot_product_attention
    x = torch.zeros(2, 4, 8, 16)
    with pytest.raises(ValueError, match="The dimension of query, key and value should be 4."):
        f(x[0], x[0], x[0])
    y = torch.zeros(2, 4, 12, 16)
    with pytest.raises(ValueError, match="Attention supports only for power of 2 size tensors."):
        f(y, y, y)
    m = torch.zeros(2, 4, 8, 8)
    with pytest.raises(ValueError, match="Error because both attn_mask and is_causal are set."):
        f(x, x, x, attn_mask=m, is_causal=True)
    with pytest.raises(ValueError, match="Boolean mask is not supported yet."):
        f(x, x, x, attn_mask=m.bool())
    with pytest.raises(AssertionError):
        z = torch.zeros(1, 1, 8, 256)
        f(z, z, z)
    with pytest.raises(ValueError, match="Unable to convert the given input"):
        trident.util.dtype(torch.int8)


def test_value_errors_with_and_without_a_graph():
    """function.scaled_dot_product_attention runs operation.Attention.forward directly when nothing asks for a
    gradient, and through autograd otherwise: the argument checks are the same code on both ways."""
    f = trident.function.scaled_dot_product_attention
    for grad in (False, True):
        y = torch.zeros(2, 4, 12, 16, requires_grad=grad)
        with pytest.raises(ValueError, match="Attention supports only for power of 2 size tensors."):
            f(y, y, y)
        x = torch.zeros(1, 1, 8, 16, requires_grad=grad)
        with pytest.raises(RuntimeError, match="GPU only"):
            f(x, x, x)
        with torch.no_grad(), pytest.raises(RuntimeError, match="GPU only"):
            f(x, x, x)


def test_argument_packer_matches_the_structure():
    """_lib.ARGS_PACKER writes TriAttnArgs in one call: every field must land where the ctypes structure (and the
    header) has it."""
    from trident_amd import _lib
    args = _lib.TriAttnArgs()
    values = [_lib.ARGS_PACKER.size, 2, 3, 5, 7, 11, 1, 0, 0.25, 0.5, 2**63 + 5, 2**40 + 1]
    values += [1000 + i for i in range(12)] + [2000 + i for i in range(40)] + [77, 88]
    _lib.ARGS_PACKER.pack_into(args, 0, *values)
    assert (args.struct_size, args.dtype, args.B, args.H, args.S, args.D, args.is_causal, args.mask_dtype) == tuple(values[:8])
    assert (args.softmax_scale, args.dropout_p, args.seed, args.offset) == (0.25, 0.5, 2**63 + 5, 2**40 + 1)
    pointers = ["q", "k", "v", "o", "lse", "mask", "d_o", "dq", "dk", "dv", "dmask", "delta"]
    assert [getattr(args, n) for n in pointers] == [1000 + i for i in range(12)]
    strides = ["q_stride", "k_stride", "v_stride", "o_stride", "do_stride", "dq_stride", "dk_stride", "dv_stride",
               "mask_stride", "dmask_stride"]
    assert [x for n in strides for x in getattr(args, n)] == [2000 + i for i in range(40)]
    assert (args.stream, args.mask_classes) == (77, 88)


def test_reference_limits_can_be_lifted():
    """config.reference_limits = False: any sequence length and boolean masks get past the argument checks
    (and then stop at the GPU-only check on this host); head sizes stay powers of two."""
    f = trident.function.scaled_dot_product_attention
    y = torch.zeros(2, 4, 12, 16)
    m = torch.ones(2, 4, 12, 12, dtype=torch.bool)
    trident.config.reference_limits = False
    try:
        with pytest.raises(RuntimeError, match="GPU only"):
            f(y, y, y)
        with pytest.raises(RuntimeError, match="GPU only"):
            f(y, y, y, attn_mask=m)
        with pytest.raises(ValueError, match="both attn_mask and is_causal"):
            f(y, y, y, attn_mask=m, is_causal=True)
        z = torch.zeros(2, 4, 16, 24)
        with pytest.raises(ValueError, match="power of 2"):
            f(z, z, z)
    finally:
        trident.config.reference_limits = True
    with pytest.raises(ValueError, match="power of 2"):
        f(y, y, y)


def test_no_cpu_fallback():
    x = torch.zeros(1, 1, 8, 16)
    with pytest.raises(RuntimeError, match="GPU only"):
        trident.function.scaled_dot_product_attention(x, x, x)


def test_mixed_devices_raise_before_the_library_is_called():
    """A host (or other-device) key, value, mask, grad_output, output or LSE must raise in Python: the
    kernels would dereference its pointer on the GPU."""
    from trident_amd import operation

    cpu = torch.zeros(1, 1, 8, 16)
    gpu0, gpu1 = torch.device("cuda:0"), torch.device("cuda:1")
    for name in ("key", "value", "mask", "grad_output", "output", "log_sum_exp"):
        with pytest.raises(RuntimeError, match=name + " is on cpu"):
            operation._require_same_gpu(gpu0, **{name: cpu})
    meta = torch.zeros(1, 1, 8, 16, device="meta")
    with pytest.raises(RuntimeError, match="GPU only"):
        operation._require_same_gpu(meta.device, key=meta)
    operation._require_same_gpu(gpu0, key=None, mask=None)

    class FakeCuda:  # stands for a tensor on another GPU (none exists on a CPU-only host)
        device = gpu1

    with pytest.raises(RuntimeError, match="value is on cuda:1, expected cuda:0"):
        operation._require_same_gpu(gpu0, value=FakeCuda())
    # through the operator: query on one device type, key on another
    with pytest.raises(RuntimeError):
        trident.function.scaled_dot_product_attention(meta, cpu, cpu)


def test_api_surface():
    import inspect

    sig = inspect.signature(trident.function.scaled_dot_product_attention)
    assert list(sig.parameters) == ["query", "key", "value", "attn_mask", "dropout_p", "is_causal", "use_accelerator"]
    sig = inspect.signature(trident.function.attention)
    assert list(sig.parameters) == ["query", "key", "value", "mask", "dropout_p", "is_causal", "softmax_scale"]
    assert issubclass(trident.operation.Attention, torch.autograd.Function)
    assert isinstance(trident.Attention(is_causal=True), torch.nn.Module)
    assert trident.util.is_pow2(64) and not trident.util.is_pow2(0) and not trident.util.is_pow2(48)
    assert trident.config.use_trace is False


def test_product_does_not_import_oracle():
    pkg = os.path.join(ROOT, "trident_amd")
    for dirpath, _, files in os.walk(pkg):
        for name in files:
            if name.endswith((".py", ".hip", ".hpp", ".h")):
                text = open(os.path.join(dirpath, name)).read()
                assert "oracle" not in text, os.path.join(dirpath, name)


def test_bench_refuses_more_than_one_gpu():
    """bench.py measures one GPU: --gpus N > 1 (or a launcher's WORLD_SIZE > 1) exits with a message, before touching a GPU."""
    import os
    import subprocess
    import sys
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    for extra_args, extra_env in ((["--gpus", "2"], {}), ([], {"WORLD_SIZE": "2"})):
        res = subprocess.run([sys.executable, os.path.join(root, "bench.py"), *extra_args], capture_output=True, text=True,
                             env={**os.environ, **extra_env}, cwd=root, timeout=120)
        assert res.returncode != 0
        assert "one GPU" in res.stderr and res.stdout.strip() == ""
