"""Parity of the sibling operations (Softmax, MaskedSoftmax, Dropout) on the GPU, through the operator API and the
C ABI, against the CPU oracle. The first tests of each group are the reference's own (tests/test_softmax.py,
tests/test_masked_softmax.py, tests/test_dropout.py) with seeded inputs and the oracle in place of the run-time
PyTorch call. Tolerance: fp32 atol 1e-4 (the reference's rule is atol 1e-2), fp16/bf16 atol 1e-2 against fp64."""
import numpy as np
import pytest
import torch

import trident_amd as trident
from oracle import rowops
from tests import parity

pytestmark = pytest.mark.gpu


def _pair(shape, seed, dtype=torch.float32):
    g = torch.Generator().manual_seed(seed)
    return torch.randn(shape, generator=g).to(dtype), torch.randn(shape, generator=g).to(dtype)


def _build_mask(shape, seed):
    mask = torch.randint(0, 2, shape, generator=torch.Generator().manual_seed(seed))
    mask[0, :] = mask[:, 0] = 0
    return mask


def _softmax_case(device, x, g, dim, dtype, mask=None, tag=""):
    tx = x.to(device).requires_grad_(True)
    if mask is None:
        out = trident.function.softmax(tx, dim)
    else:
        out = trident.function.masked_softmax(tx, mask.to(device), dim)
    assert out.dtype == dtype and out.shape == x.shape
    out.backward(g.to(device))
    want = rowops.softmax_forward(parity.to64(x), dim, None if mask is None else mask.numpy())
    parity.close(out, want, dtype, tag + " out")
    # the gradient is defined on the stored (rounded) output, like delta in the attention backward
    parity.close(tx.grad, rowops.softmax_backward(parity.to64(out), parity.to64(g), dim), dtype, tag + " grad")
    return out


@pytest.mark.parametrize("y_size, x_size, dim", [(2, 512, 0), (3, 1000, 1), (3, 1000, 0), (2, 512, 1)])
def test_softmax_reference_shapes(y_size, x_size, dim, device):
    x, g = _pair((y_size, x_size), 1)
    _softmax_case(device, x, g, dim, torch.float32, tag="softmax")


@pytest.mark.parametrize("y_size, x_size, dim", [(2, 512, 0), (3, 1000, 1), (3, 1000, 0), (2, 512, 1)])
def test_masked_softmax_reference_shapes(y_size, x_size, dim, device):
    x, g = _pair((y_size, x_size), 2)
    mask = _build_mask((y_size, x_size), 3)
    out = _softmax_case(device, x, g, dim, torch.float32, mask=mask, tag="masked softmax")
    assert (out[mask.bool().to(device)] == 0).all()


@pytest.mark.parametrize("dtype", [torch.float32, torch.float16, torch.bfloat16])
def test_modules_keep_dtype(dtype, device):
    """tests/test_softmax.py:47-61, tests/test_masked_softmax.py:58-73, tests/test_dropout.py:46-58."""
    x, g = _pair((1, 32), 4, dtype)
    tx = x.to(device).requires_grad_(True)
    out = trident.Softmax(1).forward(tx)
    assert out is not None and out.dtype == dtype
    out.backward(g.to(device))
    assert tx.grad is not None and tx.grad.dtype == dtype
    tx = x.to(device).requires_grad_(True)
    out = trident.MaskedSoftmax(1).forward(tx, _build_mask((1, 32), 5).to(device))
    assert out.dtype == dtype
    out.backward(g.to(device))
    assert tx.grad.dtype == dtype
    x1, g1 = _pair((16,), 6, dtype)
    tx = x1.to(device).requires_grad_(True)
    out = trident.Dropout(0.7).forward(tx)
    assert out is not None and out.dtype == dtype
    out.backward(g1.to(device))
    assert tx.grad is not None and tx.grad.dtype == dtype


@pytest.mark.parametrize("dtype", [torch.float32, torch.float16, torch.bfloat16])
@pytest.mark.parametrize("shape,dim", [((5, 7), 1), ((64, 2048), 1), ((9, 2056), 1), ((3, 5000), 1), ((17, 4097), 1), ((3, 20000), 1),
                                       ((300, 33), 0), ((4, 6, 128), 2)])
def test_softmax_shapes_and_dtypes(shape, dim, dtype, device):
    """Wave-per-row and workgroup-per-row kernels, rows that stay in registers and rows too long for that (two sweeps),
    16-byte and per-element accesses (odd lengths), the thread-per-row kernel (dim 0), a contiguous 3-D input along
    its last dimension."""
    x, g = _pair(shape, 10 + shape[-1], dtype)
    _softmax_case(device, x * 3, g, dim, dtype, tag=f"softmax {shape} {dtype}")


@pytest.mark.parametrize("mask_dtype", [torch.int64, torch.int32, torch.bool, torch.uint8, torch.float32, torch.bfloat16])
def test_masked_softmax_mask_dtypes_and_fully_masked_row(mask_dtype, device):
    x, g = _pair((6, 300), 20, torch.bfloat16)
    mask = _build_mask((6, 300), 21)
    mask[3, :] = 1  # a fully masked row is NaN, like softmax over -inf
    tx = x.to(device)
    out = trident.function.masked_softmax(tx, mask.to(mask_dtype).to(device), 1)
    want = rowops.softmax_forward(parity.to64(x), 1, mask.numpy())
    parity.close(out, want, torch.bfloat16, f"mask {mask_dtype}")
    assert torch.isnan(out[3]).all() and not torch.isnan(out[2]).any()


def test_softmax_of_a_transposed_view_and_large_values(device):
    x, g = _pair((40, 70), 30)
    xt = (x * 30).t()  # strides (1, 70): rows are columns of the storage
    _softmax_case(device, xt, g.t(), 1, torch.float32, tag="transposed")
    big = torch.tensor([[1e4, 1e4 - 1, -1e4, 0.0]])
    out = trident.function.softmax(big.to(device), 1)
    parity.close(out, rowops.softmax_forward(parity.to64(big), 1), torch.float32, "large values")


# ------------------------------------------------------------------ dropout
@pytest.mark.parametrize("x_size, p", [(256, 0.0), (512, 1.0)])
def test_dropout_reference_cases(x_size, p, device):
    """tests/test_dropout.py:22-43: p = 0 is the identity, p = 1 gives zeros, for values and gradient."""
    x, g = _pair((x_size,), 40)
    tx = x.to(device).requires_grad_(True)
    out = trident.function.dropout(tx, p)
    out.backward(g.abs().to(device))
    want = torch.nn.functional.dropout(x, p)
    assert torch.equal(out.cpu(), want)
    assert torch.equal(tx.grad.cpu(), g.abs() if p == 0.0 else torch.zeros_like(g))


@pytest.mark.parametrize("dtype", [torch.float32, torch.float16, torch.bfloat16])
@pytest.mark.parametrize("shape,p", [((4096,), 0.1), ((33, 77), 0.5), ((1, 5), 0.9), ((8, 128, 64), 0.25)])
def test_dropout_is_bit_exact_against_the_documented_stream(shape, p, dtype, device):
    x, g = _pair(shape, 50, dtype)
    trident.config.dropout_seed = (0xD0C5EED, 11)
    try:
        tx = x.to(device).requires_grad_(True)
        out = trident.function.dropout(tx, p)
        out.backward(g.to(device))
    finally:
        trident.config.dropout_seed = None
    keep = rowops.dropout_keep(0xD0C5EED, 11, x.numel(), p).reshape(shape)
    assert np.array_equal((out != 0).cpu().numpy() | (x == 0).numpy(), keep | (x == 0).numpy())
    parity.close(out, rowops.dropout_apply(parity.to64(x), p, 0xD0C5EED, 11), dtype, "dropout out")
    parity.close(tx.grad, rowops.dropout_apply(parity.to64(g), p, 0xD0C5EED, 11), dtype, "dropout grad")


def test_dropout_seeding_and_eval_mode(device):
    x = torch.randn(1000, generator=torch.Generator().manual_seed(60)).to(device)
    torch.manual_seed(5)
    a = trident.function.dropout(x, 0.4)
    torch.manual_seed(5)
    b = trident.function.dropout(x, 0.4)
    c = trident.function.dropout(x, 0.4)
    assert torch.equal(a, b) and not torch.equal(a, c)
    layer = trident.Dropout(0.4).eval()
    assert torch.equal(layer(x), x)
