"""Pins oracle/rowops.py (softmax, masked softmax, dropout) and checks the sibling operations' host logic.
Runs without a GPU."""
import ctypes
import os
import re

import numpy as np
import pytest
import torch

import trident_amd as trident
from oracle import philox, rowops
from trident_amd import _lib

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _rand(shape, seed):
    return np.random.default_rng(seed).standard_normal(shape)


@pytest.mark.parametrize("shape,dim", [((2, 512), 0), ((3, 1000), 1), ((1, 32), 1), ((4, 5, 6), 2)])
def test_softmax_matches_torch(shape, dim):
    """The reference's own test shapes (tests/test_softmax.py:22,29,47) against torch in fp64, values and gradient."""
    x, g = _rand(shape, 1), _rand(shape, 2)
    tx = torch.tensor(x, requires_grad=True)
    out = torch.softmax(tx, dim)
    out.backward(torch.tensor(g))
    np.testing.assert_allclose(rowops.softmax_forward(x, dim), out.detach().numpy(), rtol=0, atol=1e-15)
    np.testing.assert_allclose(rowops.softmax_backward(out.detach().numpy(), g, dim), tx.grad.numpy(), rtol=0, atol=1e-15)
    np.testing.assert_allclose(rowops.softmax_forward(x, dim).sum(axis=dim), 1.0, rtol=0, atol=1e-14)


@pytest.mark.parametrize("shape,dim", [((2, 512), 0), ((3, 1000), 1)])
def test_masked_softmax_matches_the_references_test_formula(shape, dim):
    """tests/test_masked_softmax.py:22-33: input = where(mask.bool(), -inf, input); softmax; mask from randint(0, 2)
    with row 0 and column 0 cleared."""
    x, g = _rand(shape, 3), _rand(shape, 4)
    mask = torch.randint(0, 2, shape, generator=torch.Generator().manual_seed(5))
    mask[0, :] = mask[:, 0] = 0
    tx = torch.tensor(x, requires_grad=True)
    out = torch.softmax(torch.where(mask.bool(), float("-inf"), tx), dim)
    out.backward(torch.tensor(g))
    got = rowops.softmax_forward(x, dim, mask.numpy())
    np.testing.assert_allclose(got, out.detach().numpy(), rtol=0, atol=1e-15)
    np.testing.assert_allclose(rowops.softmax_backward(got, g, dim), tx.grad.numpy(), rtol=0, atol=1e-15)
    assert (got[mask.numpy() > 0] == 0).all()
    # a float mask counts where it exceeds eps, like the kernel's comparison
    fm = mask.numpy() * 0.5
    np.testing.assert_array_equal(rowops.softmax_forward(x, dim, fm), got)
    np.testing.assert_array_equal(rowops.softmax_forward(x, dim, fm * 1e-17), rowops.softmax_forward(x, dim))


def test_fully_masked_row_is_nan():
    x = _rand((2, 8), 6)
    mask = np.zeros((2, 8))
    mask[1] = 1
    out = rowops.softmax_forward(x, 1, mask)
    assert np.isnan(out[1]).all() and not np.isnan(out[0]).any()


def test_dropout_layout_against_scalar_philox():
    """Element i takes byte (i & 3) of word ((i >> 2) & 3) of the call with counter (i >> 4, 0, 'DROP', offset)."""
    seed, offset, p = 0x123456789ABCDEF, 7, 0.3
    keep = rowops.dropout_keep(seed, offset, 100, p)
    thr = philox.dropout_threshold(p)
    for i in (0, 1, 3, 4, 15, 16, 17, 63, 99):
        r = philox.philox4x32_10_scalar([i >> 4, 0, 0x44524F50, offset], [seed & 0xFFFFFFFF, seed >> 32])
        byte = (r[(i >> 2) & 3] >> (8 * (i & 3))) & 0xFF
        assert bool(keep[i]) == (byte >= thr), i
    assert not np.array_equal(keep, rowops.dropout_keep(seed, offset + 1, 100, p))
    assert not np.array_equal(keep, rowops.dropout_keep(seed + 1, offset, 100, p))


@pytest.mark.parametrize("p", [0.1, 0.5, 0.9])
def test_dropout_rate_and_unit_mean(p):
    n = 1 << 18
    keep = rowops.dropout_keep(99, 0, n, p)
    q = philox.dropout_threshold(p) / 256.0
    assert abs(keep.mean() - (1 - q)) < 4 * np.sqrt(q * (1 - q) / n)
    y = rowops.dropout_apply(np.ones(n), p, 99, 0)
    assert abs(y.mean() - 1.0) < 0.02 and set(np.unique(y)) <= {0.0, philox.dropout_scale(p)}


@pytest.mark.parametrize("n,p", [(256, 0.0), (512, 1.0)])
def test_dropout_extremes_match_torch(n, p):
    """tests/test_dropout.py:22-26 (p in {0, 1}): identity and zeros, for values and gradient alike."""
    x = _rand((n,), 8)
    want = torch.nn.functional.dropout(torch.tensor(x), p).numpy()
    np.testing.assert_array_equal(rowops.dropout_apply(x, p, 1, 2), want)


# ---------------------------------------------------------------- boundary (no GPU)
def test_row_abi_exports_and_struct_layout(tmp_path):
    import subprocess

    text = open(os.path.join(ROOT, "include", "tri_rowops.h")).read()
    declared = set(re.findall(r"\b(tri_(?:softmax|dropout)_\w+)\s*\(", text))
    assert declared == set(_lib.ROW_EXPORTS)
    lib = _lib.lib()
    for name in declared:
        assert hasattr(lib, name)
    src = tmp_path / "sz.c"
    src.write_text('#include <stdio.h>\n#include <stddef.h>\n#include "tri_rowops.h"\n'
                   'int main(){printf("%zu %zu %zu %zu %zu", sizeof(TriRowArgs), offsetof(TriRowArgs,input),'
                   ' offsetof(TriRowArgs,p), offsetof(TriRowArgs,seed), offsetof(TriRowArgs,stream));}')
    exe = tmp_path / "sz"
    subprocess.check_call(["gcc", "-I", os.path.join(ROOT, "include"), str(src), "-o", str(exe)])
    got = [int(v) for v in subprocess.check_output([str(exe)]).split()]
    T = _lib.TriRowArgs
    assert got == [ctypes.sizeof(T), T.input.offset, T.p.offset, T.seed.offset, T.stream.offset]


def test_row_abi_status_codes_without_gpu():
    lib = _lib.lib()
    assert lib.tri_softmax_fwd(None) == -1
    a = _lib.TriRowArgs()
    assert lib.tri_softmax_fwd(ctypes.byref(a)) == -7
    a.struct_size = ctypes.sizeof(a)
    a.dtype = 7
    assert lib.tri_softmax_bwd(ctypes.byref(a)) == -3
    a.dtype = 0
    assert lib.tri_softmax_fwd(ctypes.byref(a)) == -2      # sizes unset
    a.y_size, a.x_size, a.y_stride, a.x_stride = 4, 8, 8, 1
    assert lib.tri_softmax_fwd(ctypes.byref(a)) == -1      # pointers missing
    a.x_stride = -1
    assert lib.tri_softmax_fwd(ctypes.byref(a)) == -4
    a.x_stride, a.p = 1, 1.5
    assert lib.tri_dropout_fwd(ctypes.byref(a)) == -6
    a.p = 0.5
    assert lib.tri_dropout_bwd(ctypes.byref(a)) == -1


def test_sibling_api_surface_and_host_errors():
    import inspect

    assert list(inspect.signature(trident.function.softmax).parameters) == ["input", "dim"]
    assert list(inspect.signature(trident.function.masked_softmax).parameters) == ["input", "mask", "dim"]
    assert list(inspect.signature(trident.function.dropout).parameters) == ["input", "p", "training"]
    for cls in (trident.operation.Softmax, trident.operation.MaskedSoftmax, trident.operation.Dropout):
        assert issubclass(cls, torch.autograd.Function)
    assert "dim=1" in repr(trident.Softmax(1)) and "p=0.7" in repr(trident.Dropout(0.7))
    x = torch.zeros(3, 8)
    with pytest.raises(RuntimeError, match="GPU only"):
        trident.function.softmax(x, 1)
    with pytest.raises(RuntimeError, match="GPU only"):
        trident.function.dropout(x, 0.5)
    assert torch.equal(trident.function.dropout(x, 0.5, training=False), x)   # evaluation mode: a copy
    from trident_amd import rowops as ops
    assert ops.size_and_stride(torch.zeros(3, 8), 0) == (8, 3, 1, 8)
    assert ops.size_and_stride(torch.zeros(3, 8), 1) == (3, 8, 8, 1)
    assert ops.size_and_stride(torch.zeros(2, 3, 8), -1) == (6, 8, 8, 1)
    with pytest.raises(ValueError, match="is not supported"):
        ops.size_and_stride(torch.zeros(2, 3, 8), 0)
