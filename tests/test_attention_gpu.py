"""Parity of the HIP path (through the C ABI, via the operator API) against the CPU oracle.

The first three tests are the reference's own (tests/test_attention.py:22-116) with seeded
inputs, the oracle in place of the run-time PyTorch call, and the tighter tolerance of this
build (fp32 atol 1e-4 instead of 1e-2)."""
import math
import os

import numpy as np
import pytest
import torch

import trident_amd as trident
from oracle import philox
from tests import parity
from trident_amd import workloads

pytestmark = pytest.mark.gpu


def _gen(shape, seed, dtype=torch.float32, uniform_q=False):
    g = torch.Generator().manual_seed(seed)
    q = (torch.rand(shape, generator=g) if uniform_q else torch.randn(shape, generator=g)).to(dtype)
    k, v, d_o = [torch.randn(shape, generator=g).to(dtype) for _ in range(3)]
    return q, k, v, d_o


def _run(device, q, k, v, d_o=None, mask=None, dropout_p=0.0, is_causal=False, scale=None, mask_grad=False):
    """Runs the product path; returns (o, dq, dk, dv, dmask) as device tensors."""
    tq, tk, tv = [x.to(device).requires_grad_(d_o is not None) for x in (q, k, v)]
    tm = None if mask is None else mask.to(device).requires_grad_(mask_grad)
    if scale is None:
        out = trident.function.scaled_dot_product_attention(tq, tk, tv, tm, dropout_p, is_causal)
    else:
        out = trident.function.attention(tq, tk, tv, tm, dropout_p, is_causal, scale)
    if d_o is None:
        return out, None, None, None, None
    out.backward(d_o.to(device))
    return out, tq.grad, tk.grad, tv.grad, (tm.grad if mask_grad else None)


def _check(device, dtype, q, k, v, d_o, mask=None, dropout_p=0.0, is_causal=False, scale=None, mask_grad=False,
           seed=None, tag=""):
    if dropout_p > 0:
        trident.config.dropout_seed = (seed, 3)
    try:
        o, dq, dk, dv, dm = _run(device, q, k, v, d_o, mask, dropout_p, is_causal, scale, mask_grad)
    finally:
        trident.config.dropout_seed = None
    kw = dict(mask=mask, dropout_p=dropout_p, is_causal=is_causal, scale=scale, seed=seed or 0, offset=3)
    o_ref, _ = parity.oracle_forward(q, k, v, **kw)
    parity.close(o, o_ref, dtype, tag + " O")
    if d_o is not None:
        dq_r, dk_r, dv_r, dm_r, _ = parity.oracle_backward(q, k, v, d_o, want_dmask=mask_grad, o=o, **kw)
        _, a_dq, a_dk, a_dv = parity.oracle_abs_sums(q, k, v, d_o, o=o, **kw)
        parity.close(dq, dq_r, dtype, tag + " dQ", a_dq)
        parity.close(dk, dk_r, dtype, tag + " dK", a_dk)
        parity.close(dv, dv_r, dtype, tag + " dV", a_dv)
        if mask_grad:
            # dS is computed from the stored (rounded) O and 16-bit operands: its error budget is
            # that of the q/k/v dtype even when the mask itself is fp32
            loose = dtype if parity.ATOL[dtype] > parity.ATOL[mask.dtype] else mask.dtype
            parity.close(dm, dm_r, loose, tag + " dMask")
    return o


# ------------------------------------------------------------------ the reference's tests
@pytest.mark.parametrize("num_batches, num_heads, y_size, x_size, is_causal",
                         [(4, 8, 128, 64, True), (4, 8, 256, 32, False)])
def test_forward(num_batches, num_heads, y_size, x_size, is_causal, device):
    q, k, v, _ = _gen((num_batches, num_heads, y_size, x_size), 11)
    _check(device, torch.float32, q, k, v, None, is_causal=is_causal, tag="forward")
    mask = torch.randn(num_batches, num_heads, y_size, y_size, generator=torch.Generator().manual_seed(12))
    _check(device, torch.float32, q, k, v, None, mask=mask, tag="forward+mask")


@pytest.mark.parametrize("num_batches, num_heads, y_size, x_size, is_causal",
                         [(4, 8, 128, 64, True), (4, 8, 256, 32, False)])
def test_backward(num_batches, num_heads, y_size, x_size, is_causal, device):
    q, k, v, d_o = _gen((num_batches, num_heads, y_size, x_size), 13, uniform_q=True)
    _check(device, torch.float32, q, k, v, d_o, is_causal=is_causal, tag="backward")
    mask = torch.randn(num_batches, num_heads, y_size, y_size, generator=torch.Generator().manual_seed(14))
    _check(device, torch.float32, q, k, v, d_o, mask=mask, mask_grad=True, tag="backward+mask")


@pytest.mark.parametrize("dtype", [torch.float32, torch.float16, torch.bfloat16])
@pytest.mark.parametrize("is_causal", [True, False])
def test_attention(is_causal, dtype, device):
    q, k, v, d_o = _gen((1, 1, 1, 16), 15, dtype, uniform_q=True)
    o, dq, dk, dv, _ = _run(device, q, k, v, d_o, is_causal=is_causal)
    assert o is not None and o.dtype == dtype
    for g in (dq, dk, dv):
        assert g is not None and g.dtype == dtype
    parity.close(o, parity.to64(v), dtype, "S=1 O")          # softmax over one key is 1
    parity.close(dv, parity.to64(d_o), dtype, "S=1 dV")
    parity.close(dq, np.zeros((1, 1, 1, 16)), dtype, "S=1 dQ")
    parity.close(dk, np.zeros((1, 1, 1, 16)), dtype, "S=1 dK")
    mask = torch.randn(1, 1, 1, 1, generator=torch.Generator().manual_seed(16)).to(dtype)
    _, _, _, _, dm = _run(device, q, k, v, d_o, mask=mask, mask_grad=True)
    assert dm is not None and dm.dtype == dtype


# ------------------------------------------------------------------ the five benchmark configs
def _config_case(device, name, **override):
    w = workloads.WORKLOADS[name]
    q, k, v, d_o, mask = workloads.make_inputs(w, **override)
    return _check(device, w.dtype, q, k, v, d_o if w.backward else None, mask=mask, dropout_p=w.dropout_p,
                  is_causal=w.is_causal, seed=w.dropout_seed if w.dropout_p > 0 else None, tag=name)


def test_config1_fp32_plumbing(device):
    _config_case(device, "C1")


def test_config2_fp16_forward(device):
    _config_case(device, "C2", B=1, H=4)


def test_config3_bf16_causal_reduced(device):
    _config_case(device, "C3", B=1, H=2, S=1024)


def test_config4_bf16_length_mask_reduced(device):
    _config_case(device, "C4", B=2, H=3, S=512)


def test_config5_bf16_causal_dropout_reduced(device):
    _config_case(device, "C5", B=1, H=2, S=1024)


# ------------------------------------------------------------------ shapes, layouts, edge cases
@pytest.mark.parametrize("dtype", [torch.float32, torch.float16, torch.bfloat16])
@pytest.mark.parametrize("S,D", [(1, 16), (2, 32), (8, 16), (32, 64), (64, 128), (128, 16), (256, 128), (512, 64)])
@pytest.mark.parametrize("variant", ["plain", "causal", "mask"])
def test_shapes(dtype, S, D, variant, device):
    q, k, v, d_o = _gen((2, 3, S, D), 100 + S + D, dtype)
    mask = None
    if variant == "mask":
        mask = torch.randn(2, 3, S, S, generator=torch.Generator().manual_seed(5)).to(dtype)
    _check(device, dtype, q, k, v, d_o, mask=mask, is_causal=variant == "causal", mask_grad=mask is not None,
           tag=f"{dtype} S={S} D={D} {variant}")


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("S,D,causal", [(256, 64, True), (512, 128, False), (200, 128, True), (333, 32, False)])
def test_strided_inputs(dtype, S, D, causal, device):
    """[B,S,H,D] storage viewed as [B,H,S,D]: rows of one head are H*D apart. Through the phased 16-bit kernels, their
    variants for other lengths, and the 32-row-tile kernels (fp32)."""
    B, H = 2, 4
    g = torch.Generator().manual_seed(21)
    q, k, v, d_o = [torch.randn(B, S, H, D, generator=g).to(dtype).transpose(1, 2) for _ in range(4)]
    assert not q.is_contiguous()
    trident.config.reference_limits = S in (256, 512)
    try:
        _check(device, dtype, q, k, v, d_o, is_causal=causal, tag=f"strided S={S} D={D}")
    finally:
        trident.config.reference_limits = True


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("mshape", [(1, 1), (2, 1), (1, 3), (2, 3)])
def test_broadcast_masks_and_their_gradient(dtype, mshape, device):
    B, H, S, D = 2, 3, 128, 64
    q, k, v, d_o = _gen((B, H, S, D), 31, dtype)
    mask = torch.randn(*mshape, S, S, generator=torch.Generator().manual_seed(32))
    mask[..., :, 100:] = float("-inf")
    _check(device, dtype, q, k, v, d_o, mask=mask, mask_grad=True, tag=f"bmask{mshape}")


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("D,S,p", [(64, 256, 0.0), (128, 256, 0.0), (128, 512, 0.0), (128, 512, 0.2)])
def test_key_padding_mask_row_broadcast(dtype, D, S, p, device):
    """[B,1,1,S] additive mask (one row for all queries, row stride 0), as a key-padding mask is given. At D = 128 the
    16-bit dK/dV pass then runs the phased kernel with the mask as one value per key."""
    B, H = 2, 3
    q, k, v, d_o = _gen((B, H, S, D), 33, dtype)
    mask = torch.zeros(B, 1, 1, S)
    mask[0, ..., S - 56:] = float("-inf")
    mask[1, ..., S // 2 + 3:] = float("-inf")
    mask += 0.25 * torch.randn(B, 1, 1, S, generator=torch.Generator().manual_seed(34))
    _check(device, dtype, q, k, v, d_o, mask=mask, dropout_p=p, seed=35 if p else None, tag="key-padding")
    if dtype == torch.bfloat16:   # the same mask in the operand type
        _check(device, dtype, q, k, v, d_o, mask=mask.to(dtype), dropout_p=p, seed=35 if p else None, tag="key-padding 16-bit")


@pytest.mark.parametrize("dtype,mask_dtype,mshape", [(torch.bfloat16, torch.bfloat16, (2, 3, 256, 256)),
                                                     (torch.bfloat16, torch.float32, (2, 1, 256, 256)),
                                                     (torch.float16, torch.float16, (1, 3, 256, 256)),
                                                     (torch.bfloat16, torch.float32, (2, 1, 1, 256)),
                                                     (torch.float32, torch.float32, (1, 1, 1, 256))])
@pytest.mark.parametrize("D", [16, 32, 64, 128])
def test_mask_gradient_on_the_matrix_cores(dtype, mask_dtype, mshape, D, device):
    """The mask gradient from the matrix-core dQ kernel (16-bit problems): written in place for a full mask, added
    atomically into the mask's own shape for masks broadcast over batch, heads or rows (a key-padding mask with a
    gradient among them), in the mask's dtype. The fp32 problem runs the general kernels on the same contract."""
    import ctypes
    from trident_amd import _lib, operation
    B, H, S = 2, 3, 256
    q, k, v, d_o = _gen((B, H, S, D), 37 + D, dtype)
    mask = (0.5 * torch.randn(*mshape, generator=torch.Generator().manual_seed(38))).to(mask_dtype)
    _check(device, dtype, q, k, v, d_o, mask=mask, mask_grad=True, tag=f"dmask {mshape} {mask_dtype}")
    # which kernel family writes it
    tq = q.to(device)
    buf = torch.zeros(mshape, device=device, dtype=torch.float32 if mshape != (B, H, S, S) else mask_dtype)
    mview = operation._expand_mask(mask.to(device).to(buf.dtype), (B, H, S, S))
    lse = torch.empty(B, H, S, device=device)
    args = operation._make_args(tq, tq, tq, tq, lse, mview, 0.0, False, 0.125, 0, 0, grad_output=tq, grad_query=tq,
                                grad_mask=buf.expand(B, H, S, S), delta=lse)
    assert _lib.lib().tri_attn_uses_matrix_cores(ctypes.byref(args), 2) == (2 if dtype == torch.float32 else 1)


@pytest.mark.parametrize("D", [32, 64, 128])
def test_fp32_mask_many_tiles(D, device):
    """fp32 mask shared by the heads over 8 key tiles and 2 workgroups per head: the staged mask path (D=64)
    refills its LDS region every tile; D=128 takes the direct loads."""
    B, H, S = 2, 2, 512
    q, k, v, d_o = _gen((B, H, S, D), 35, torch.bfloat16)
    mask = torch.randn(B, 1, S, S, generator=torch.Generator().manual_seed(36))
    mask[..., 300:420] = float("-inf")
    _check(device, torch.bfloat16, q, k, v, d_o, mask=mask, tag=f"fp32 mask D={D}")


def test_mask_with_fully_masked_leading_tiles(device):
    """Keys [0, 192) masked for every row: the running max stays -inf over whole tiles."""
    B, H, S, D = 1, 2, 256, 64
    q, k, v, d_o = _gen((B, H, S, D), 41, torch.bfloat16)
    mask = torch.zeros(B, 1, S, S)
    mask[..., :192] = float("-inf")
    _check(device, torch.bfloat16, q, k, v, d_o, mask=mask, tag="lead-masked")


def test_fully_masked_row_gives_nan_like_softmax(device):
    B, H, S, D = 1, 1, 128, 64
    q, k, v, _ = _gen((B, H, S, D), 42, torch.float32)
    mask = torch.zeros(B, H, S, S)
    mask[0, 0, 5, :] = float("-inf")
    o, *_ = _run(device, q, k, v, mask=mask)
    assert torch.isnan(o[0, 0, 5]).all() and not torch.isnan(o[0, 0, 6]).any()


def test_explicit_softmax_scale_and_module(device):
    q, k, v, d_o = _gen((1, 2, 128, 64), 51, torch.float16)
    _check(device, torch.float16, q, k, v, d_o, scale=0.05, tag="scale")
    mod = trident.Attention(is_causal=True).to(device)
    o = mod(q.to(device), k.to(device), v.to(device))
    o_ref, _ = parity.oracle_forward(q, k, v, is_causal=True)
    parity.close(o, o_ref, torch.float16, "module")


def test_forward_without_a_graph_is_the_same_forward(device):
    """Inputs that ask for no gradient (and torch.no_grad) skip autograd's bookkeeping: same kernel, same bits, no
    grad_fn; with a gradient asked for the result carries one."""
    q, k, v, _ = [x.to(device) for x in _gen((2, 2, 128, 64), 52, torch.bfloat16)]
    f = trident.function.scaled_dot_product_attention
    plain = f(q, k, v, is_causal=True)
    assert plain.grad_fn is None and not plain.requires_grad
    qg = q.clone().requires_grad_()
    tracked = f(qg, k, v, is_causal=True)
    assert tracked.grad_fn is not None
    with torch.no_grad():
        quiet = f(qg, k, v, is_causal=True)
    assert quiet.grad_fn is None
    assert torch.equal(plain, tracked.detach()) and torch.equal(plain, quiet)


# ------------------------------------------------------------------ dropout
def test_dropout_mask_bits_match_oracle(device):
    from trident_amd import _lib

    lib = _lib.lib()
    for seed, offset, bh, p, row0, rows, col0, cols in [(0x5EED, 0, 3, 0.1, 0, 64, 0, 64),
                                                         (2**63 + 99, 0xFFFFFFFF, 255, 0.5, 1021, 70, 16383 - 64, 65)]:
        keep = torch.empty(rows * cols, dtype=torch.uint8, device=device)
        _lib.check(lib.tri_attn_dropout_mask(seed, offset, p, bh, row0, rows, col0, cols, keep.data_ptr(), None))
        torch.cuda.synchronize()
        want = philox.dropout_keep_mask(seed, offset, bh, np.arange(row0, row0 + rows), np.arange(col0, col0 + cols), p)
        assert (keep.cpu().numpy().reshape(rows, cols).astype(bool) == want).all()


@pytest.mark.parametrize("dtype,S,D", [(torch.float32, 64, 32), (torch.bfloat16, 256, 128), (torch.float16, 128, 64),
                                       (torch.bfloat16, 512, 64), (torch.float16, 512, 128), (torch.bfloat16, 512, 32),
                                       (torch.float16, 128, 32)])
@pytest.mark.parametrize("p", [0.1, 0.5])
def test_dropout_forward_backward(dtype, S, D, p, device):
    q, k, v, d_o = _gen((2, 2, S, D), 61, dtype)
    _check(device, dtype, q, k, v, d_o, dropout_p=p, is_causal=True, seed=0xC0FFEE, tag=f"dropout p={p}")
    mask = torch.randn(2, 1, S, S, generator=torch.Generator().manual_seed(62))
    _check(device, dtype, q, k, v, d_o, mask=mask, dropout_p=p, seed=12345, tag=f"dropout+mask p={p}")


def test_dropout_extremes_and_determinism(device):
    q, k, v, d_o = _gen((1, 2, 128, 64), 71, torch.bfloat16)
    o0, *_ = _run(device, q, k, v)
    trident.config.dropout_seed = (5, 0)
    o_tiny, *_ = _run(device, q, k, v, dropout_p=0.001)     # thr8 == 0: nothing dropped
    trident.config.dropout_seed = (5, 0)
    o_all, dq, dk, dv, _ = _run(device, q, k, v, d_o, dropout_p=1.0)
    trident.config.dropout_seed = None
    assert torch.equal(o0, o_tiny)
    assert (o_all == 0).all() and (dq == 0).all() and (dk == 0).all() and (dv == 0).all()
    torch.manual_seed(77)
    a, *_ = _run(device, q, k, v, dropout_p=0.3)
    torch.manual_seed(77)
    b, *_ = _run(device, q, k, v, dropout_p=0.3)
    c, *_ = _run(device, q, k, v, dropout_p=0.3)
    assert torch.equal(a, b) and not torch.equal(a, c)


# ------------------------------------------------------------------ lengths the operator API rejects
def _assert_kernel_family(q, mask, p, causal, scale, expected):
    """tri_attn_uses_matrix_cores on the arguments of a call (forward, dK/dV, dQ)."""
    import ctypes
    from trident_amd import _lib, operation
    lse = torch.empty(q.shape[:3], device=q.device, dtype=torch.float32)
    mview = None if mask is None else operation._expand_mask(mask, (*q.shape[:3], q.shape[2]))
    # (only the pointers' alignment and the strides matter)
    args = operation._make_args(q, q, q, q, lse, mview, p, causal, scale, 0, 0, grad_output=q, grad_query=q, grad_key=q,
                                grad_value=q, delta=lse)
    got = [_lib.lib().tri_attn_uses_matrix_cores(ctypes.byref(args), which) for which in (0, 1, 2)]
    want = list(expected) if isinstance(expected, (list, tuple)) else [1 if expected else 0] * 3
    assert got == want, (got, want)


def _abi_case(device, dtype, S, D, variant, seed, batches=1, heads=2, matrix_cores=None):
    """The operator API accepts power-of-two lengths only (reference rule); the C ABI takes any
    length.  This calls the ABI wrappers directly: a multiple of 128 that is not one of 256 runs the
    4-wave matrix-core kernels over several tiles, other lengths run the general kernels."""
    from trident_amd.operation import Attention
    q, k, v, d_o = _gen((batches, heads, S, D), seed, dtype)
    mask, causal, p = None, False, 0.0
    if variant == "causal":
        causal = True
    elif variant == "mask":
        mask = torch.randn(batches, heads, S, S, generator=torch.Generator().manual_seed(seed + 1))
    elif variant == "mask16":
        mask = torch.randn(1, 1, S, S, generator=torch.Generator().manual_seed(seed + 1)).to(dtype)
    elif variant == "causal+dropout":
        causal, p = True, 0.2
    elif variant == "dropout":
        p = 0.2
    scale = 1.0 / math.sqrt(D)
    rng = (977, 3) if p > 0 else (0, 0)
    tq, tk, tv, tdo = [x.to(device) for x in (q, k, v, d_o)]
    tm = None if mask is None else mask.to(device)
    if matrix_cores is not None:
        _assert_kernel_family(tq, tm, p, causal, scale, matrix_cores)
    o, lse = Attention._forward(tq, tk, tv, tm, p, causal, scale, *rng)
    delta = torch.full_like(lse, float("nan"))
    dq, dk, dv, _ = Attention._backward(tdo, tq, tk, tv, o, lse, tm, scale, p, causal, *rng, False, delta_out=delta)
    kw = dict(mask=mask, dropout_p=p, is_causal=causal, scale=scale, seed=rng[0], offset=rng[1])
    tag = f"abi S={S} D={D} {variant}"
    o_ref, lse_ref = parity.oracle_forward(q, k, v, **kw)
    parity.close(o, o_ref, dtype, tag + " O")
    dq_r, dk_r, dv_r, _, delta_ref = parity.oracle_backward(q, k, v, d_o, o=o, **kw)
    # the two fp32 statistics the ABI hands over: lse2 = log2 sum exp(s), delta = rowsum(dO * O)
    parity.lse_delta_close(lse, lse_ref, tag + " LSE", dtype)
    parity.lse_delta_close(delta, delta_ref, tag + " delta")
    _, a_dq, a_dk, a_dv = parity.oracle_abs_sums(q, k, v, d_o, o=o, **kw)
    parity.close(dq, dq_r, dtype, tag + " dQ", a_dq)
    parity.close(dk, dk_r, dtype, tag + " dK", a_dk)
    parity.close(dv, dv_r, dtype, tag + " dV", a_dv)


@pytest.mark.parametrize("variant", ["plain", "causal", "mask", "mask16", "causal+dropout"])
@pytest.mark.parametrize("S,D", [(384, 64), (384, 128), (640, 64), (640, 128), (384, 32), (640, 32), (384, 16), (1024, 16)])
def test_four_wave_kernels_over_several_tiles(S, D, variant, device):
    _abi_case(device, torch.bfloat16, S, D, variant, 200 + S + D)


@pytest.mark.parametrize("variant", ["plain", "causal", "mask", "causal+dropout"])
@pytest.mark.parametrize("dtype,S,D", [(torch.float32, 100, 32), (torch.bfloat16, 200, 64), (torch.float16, 72, 128),
                                       (torch.float32, 384, 64)])
def test_lengths_that_are_not_powers_of_two(dtype, S, D, variant, device):
    _abi_case(device, dtype, S, D, variant, 300 + S + D)


@pytest.mark.parametrize("S,D", [(256, 64), (256, 128), (512, 64), (512, 128), (384, 128), (512, 32), (384, 32)])
def test_dropout_without_causal_or_mask(S, D, device):
    """Dropout alone: the persistent forward kernel, the D = 128 unphased dQ kernel, the phased dQ kernel at
    D = 64, the unphased one at D = 32 and the D = 128 pair dK/dV kernel in their non-causal dropout instantiations."""
    _abi_case(device, torch.bfloat16, S, D, "dropout", 250 + S + D)


@pytest.mark.parametrize("dtype,S,D", [(torch.bfloat16, 200, 64), (torch.float32, 100, 32), (torch.float16, 384, 128)])
def test_operator_without_the_reference_limits(dtype, S, D, device):
    """config.reference_limits = False: a length that is no power of two and a boolean mask (True = the key takes
    part, as torch.nn.functional.scaled_dot_product_attention reads it) go through the operator API."""
    q, k, v, d_o = _gen((2, 2, S, D), 320 + S, dtype)
    keep = torch.rand(2, 1, S, S, generator=torch.Generator().manual_seed(9)) > 0.3
    keep[..., 0] = True  # no fully masked row
    additive = torch.zeros(2, 1, S, S).masked_fill(~keep, float("-inf"))
    trident.config.reference_limits = False
    try:
        _check(device, dtype, q, k, v, d_o, is_causal=True, tag=f"any length S={S}")
        o, dq, dk, dv, _ = _run(device, q, k, v, d_o, mask=keep)
    finally:
        trident.config.reference_limits = True
    o_ref, _ = parity.oracle_forward(q, k, v, mask=additive)
    parity.close(o, o_ref, dtype, "bool mask O")
    dq_r, dk_r, dv_r, _, _ = parity.oracle_backward(q, k, v, d_o, mask=additive, o=o)
    _, a_dq, a_dk, a_dv = parity.oracle_abs_sums(q, k, v, d_o, mask=additive, o=o)
    parity.close(dq, dq_r, dtype, "bool mask dQ", a_dq)
    parity.close(dk, dk_r, dtype, "bool mask dK", a_dk)
    parity.close(dv, dv_r, dtype, "bool mask dV", a_dv)


@pytest.mark.parametrize("variant", ["plain", "causal", "dropout", "causal+dropout"])
@pytest.mark.parametrize("dtype,S,D", [(torch.float16, 32, 64), (torch.bfloat16, 64, 64), (torch.bfloat16, 32, 128),
                                       (torch.float16, 72, 64), (torch.bfloat16, 200, 128), (torch.bfloat16, 129, 64),
                                       (torch.float16, 255, 128), (torch.bfloat16, 1000, 64), (torch.bfloat16, 1, 64),
                                       (torch.float16, 833, 128), (torch.bfloat16, 32, 32), (torch.float16, 333, 32),
                                       (torch.bfloat16, 1, 32), (torch.float16, 70, 16), (torch.bfloat16, 333, 16)])
def test_any_length_runs_on_the_matrix_cores(dtype, S, D, variant, device):
    """Lengths that are not multiples of 128 (the reference's benchmark regime S = 32, 64 among them): the 128-row
    matrix-core kernels with boundary handling (clamped loads, masked keys and rows, guarded stores), not the
    vector-ALU kernels. Three heads, so that a head's last rows are followed by another head's first ones."""
    _abi_case(device, dtype, S, D, variant, 600 + S + D, batches=1, heads=3, matrix_cores=True)


def test_what_the_16_bit_kernels_leave_runs_on_the_32_row_tile_kernels(device):
    """Masked problems of other lengths and fp32 problems: family 2 (v_mfma_f32_32x32x2_f32 for fp32 data, the 16-bit
    32x32x8 instruction for 16-bit data) in all three passes; 16-bit heads of 16 and 32 are family 1."""
    _abi_case(device, torch.bfloat16, 200, 64, "mask", 650, matrix_cores=[2, 2, 2])
    _abi_case(device, torch.float32, 256, 64, "plain", 651, matrix_cores=[2, 2, 2])
    _abi_case(device, torch.bfloat16, 200, 16, "mask", 654, matrix_cores=[2, 2, 2])
    _abi_case(device, torch.bfloat16, 256, 16, "causal", 652, matrix_cores=[1, 1, 1])
    _abi_case(device, torch.bfloat16, 256, 32, "causal", 653, matrix_cores=[1, 1, 1])


@pytest.mark.parametrize("variant", ["plain", "causal", "mask", "mask16", "dropout", "causal+dropout"])
@pytest.mark.parametrize("dtype,S,D", [(torch.float32, 333, 128), (torch.float32, 200, 64), (torch.float32, 97, 32),
                                       (torch.float32, 70, 16), (torch.float32, 1, 128), (torch.float32, 512, 128),
                                       (torch.bfloat16, 130, 16), (torch.float16, 260, 32), (torch.float16, 70, 16),
                                       (torch.bfloat16, 333, 32)])
def test_32_row_tile_kernels(dtype, S, D, variant, device):
    """The 32-row-tile kernels (forward, dQ, dK/dV; the split dK/dV kernel at D = 128; fp32 data on
    v_mfma_f32_32x32x2_f32, 16-bit data on the 32x32x8 instruction of its type) at every head
    size, over lengths with a ragged last tile (and one of a single row), three heads, every mask mode and dropout."""
    if variant == "mask16" and dtype == torch.float32:
        pytest.skip("a 16-bit mask is a mask of the operand type")
    # (16-bit heads of 16 and 32 without a mask are the 64-key-tile kernels' at any length)
    family = 1 if dtype != torch.float32 and D <= 32 and "mask" not in variant else 2
    _abi_case(device, dtype, S, D, variant, 700 + S + D, batches=2 if S < 300 else 1, heads=3, matrix_cores=[family] * 3)


def test_32_row_tile_kernels_masked_16_bit_lengths(device):
    """16-bit problems the 16-bit kernels leave: a masked length that is no multiple of 128, at D = 64 and 128."""
    _abi_case(device, torch.bfloat16, 200, 128, "mask", 760, heads=3, matrix_cores=[2, 2, 2])
    _abi_case(device, torch.float16, 72, 64, "mask16", 761, heads=3, matrix_cores=[2, 2, 2])


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_views_that_are_not_four_element_aligned_take_the_vector_alu_kernels(dtype, device):
    """Rows D + 1 elements apart (and a pointer one element into its buffer): neither matrix-core family reads such
    rows (16-byte / four-element accesses), the element-wise kernels do."""
    from trident_amd.operation import Attention
    B, H, S, D = 1, 3, 150, 64
    q, k, v, d_o = _gen((B, H, S, D), 790, dtype)

    def odd_view(x):
        buf = torch.zeros(B, H, S, D + 1, dtype=dtype, device=device).flatten()
        buf = torch.cat([buf, buf.new_zeros(1)])[1:]          # one element past an aligned address
        view = buf.view(B, H, S, D + 1)[..., :D]
        view.copy_(x)
        return view

    tq, tk, tv, tdo = [odd_view(x) for x in (q, k, v, d_o)]
    assert tq.stride(2) == D + 1 and tq.stride(3) == 1
    scale = 1.0 / math.sqrt(D)
    _assert_kernel_family(tq, None, 0.0, True, scale, [0, 0, 0])
    o, lse = Attention._forward(tq, tk, tv, None, 0.0, True, scale, 0, 0)
    dq, dk, dv, _ = Attention._backward(tdo, tq, tk, tv, o, lse, None, scale, 0.0, True, 0, 0, False)
    kw = dict(is_causal=True, scale=scale)
    o_ref, _ = parity.oracle_forward(q, k, v, **kw)
    parity.close(o, o_ref, dtype, "odd view O")
    dq_r, dk_r, dv_r, _, _ = parity.oracle_backward(q, k, v, d_o, o=o, **kw)
    _, a_dq, a_dk, a_dv = parity.oracle_abs_sums(q, k, v, d_o, o=o, **kw)
    parity.close(dq, dq_r, dtype, "odd view dQ", a_dq)
    parity.close(dk, dk_r, dtype, "odd view dK", a_dk)
    parity.close(dv, dv_r, dtype, "odd view dV", a_dv)


def _random_cases(count, seed):
    rng = np.random.RandomState(seed)
    cases = []
    for i in range(count):
        dtype = [torch.float32, torch.bfloat16, torch.float16][rng.randint(3)]
        D = [16, 32, 64, 128][rng.randint(4)]
        S = int(rng.choice([rng.randint(1, 40), rng.randint(40, 300), rng.randint(300, 700), 128 * rng.randint(1, 6)]))
        variant = ["plain", "causal", "mask", "mask16", "dropout", "causal+dropout"][rng.randint(6)]
        if variant == "mask16" and dtype == torch.float32:
            variant = "mask"
        cases.append((dtype, S, D, variant, int(rng.randint(1, 3)), int(rng.randint(1, 4)), 9000 + i))
    return cases


@pytest.mark.parametrize("dtype,S,D,variant,batches,heads,seed",
                         _random_cases(int(os.environ.get("TRI_RANDOM_CASES", "48")),
                                       int(os.environ.get("TRI_RANDOM_SEED", "20240611"))))
def test_random_problems(dtype, S, D, variant, batches, heads, seed, device):
    """A fixed pseudo-random sample of (dtype, length, head size, mask mode, dropout, batch, heads): whatever kernel
    family the dispatch picks, forward, LSE, delta and the three gradients match the oracle. TRI_RANDOM_CASES and
    TRI_RANDOM_SEED in the environment draw a larger or another sample."""
    _abi_case(device, dtype, S, D, variant, seed, batches=batches, heads=heads)


# ------------------------------------------------------------------ tile counts of the phased kernels
@pytest.mark.parametrize("variant", ["plain", "causal", "causal+dropout"])
@pytest.mark.parametrize("S,D", [(256, 128), (768, 128), (1280, 128), (768, 64), (1024, 64), (256, 32), (1280, 32)])
def test_phased_kernels_over_tile_counts(S, D, variant, device):
    """Multiples of 256 that are not powers of two included (the operator API cannot pass those): 4 to 20
    streamed tiles, so the prologue, the steady state and the drain of the load pipeline of the forward
    and dQ kernels, and the waves that stop early under the causal mask, are all exercised."""
    _abi_case(device, torch.bfloat16 if D == 128 else torch.float16, S, D, variant, 500 + S + D)


@pytest.mark.parametrize("variant", ["plain", "causal", "causal+dropout"])
@pytest.mark.parametrize("batches,heads,S,D", [(4, 40, 512, 128), (3, 31, 768, 64), (8, 8, 1280, 128), (5, 31, 768, 32)])
def test_more_items_than_compute_units(batches, heads, S, D, variant, device):
    """More (head, row tile) items than the GPU has compute units (320, 279 and 320 against 256): the
    persistent forward workgroups each walk two items, with the items dealt per XCD when the head count is a
    multiple of 8 (a partly filled, reversed second round) and in launch order otherwise."""
    _abi_case(device, torch.bfloat16 if D == 128 else torch.float16, S, D, variant, 700 + S + D, batches, heads)


@pytest.mark.parametrize("B,H,S,D,causal", [(8, 16, 896, 32, False), (8, 16, 2176, 32, True), (8, 16, 1024, 32, True),
                                            (6, 16, 1152, 64, True), (8, 12, 896, 32, "mask"), (8, 12, 640, 64, "mask"),
                                            (8, 16, 1152, 16, True), (8, 12, 896, 16, "mask"),
                                            (8, 12, 1024, 128, "mask"), (6, 12, 768, 128, True)])
def test_a_head_does_not_depend_on_its_company(B, H, S, D, causal, device):
    """Several workgroups resident per compute unit (small heads: four 4-wave workgroups): every head of a launch with a
    thousand workgroups gets bit for bit what it gets in a launch of its batch alone, and two heads match the oracle.
    (A fragment of a tile requested before the barrier that publishes the tile shows up here, and only here: in small
    launches the tile has always landed.)"""
    from trident_amd.operation import Attention
    dtype = torch.bfloat16
    q, k, v, d_o = _gen((B, H, S, D), 4100 + S + D, dtype)
    scale = 1.0 / math.sqrt(D)
    tq, tk, tv, tdo = [x.to(device) for x in (q, k, v, d_o)]
    mask = tm = None
    if causal == "mask":  # (a dense fp32 mask shared by the heads of a batch)
        causal = False
        mask = torch.randn(B, 1, S, S, generator=torch.Generator().manual_seed(4099))
        tm = mask.to(device)
    o, lse = Attention._forward(tq, tk, tv, tm, 0.0, causal, scale, 0, 0)
    dq, dk, dv, _ = Attention._backward(tdo, tq, tk, tv, o, lse, tm, scale, 0.0, causal, 0, 0, False)
    for b in range(B):
        sl = slice(b, b + 1)
        m1 = None if tm is None else tm[sl]
        o1, lse1 = Attention._forward(tq[sl], tk[sl], tv[sl], m1, 0.0, causal, scale, 0, 0)
        dq1, dk1, dv1, _ = Attention._backward(tdo[sl], tq[sl], tk[sl], tv[sl], o1, lse1, m1, scale, 0.0, causal, 0, 0, False)
        for name, whole, part in (("O", o, o1), ("LSE", lse, lse1), ("dQ", dq, dq1), ("dK", dk, dk1), ("dV", dv, dv1)):
            assert torch.equal(whole[sl], part), f"{name} of batch {b} differs between the launches"
    hs = slice(H - 2, H)
    kw = dict(is_causal=causal, scale=scale, mask=None if mask is None else mask[B - 1:])
    qs, ks, vs, gs = [x[B - 1:, hs] for x in (q, k, v, d_o)]
    o_ref, _ = parity.oracle_forward(qs, ks, vs, **kw)
    parity.close(o[B - 1:, hs], o_ref, dtype, "company O")
    dq_r, dk_r, dv_r, _, _ = parity.oracle_backward(qs, ks, vs, gs, o=o[B - 1:, hs], **kw)
    _, a_dq, a_dk, a_dv = parity.oracle_abs_sums(qs, ks, vs, gs, o=o[B - 1:, hs], **kw)
    parity.close(dq[B - 1:, hs], dq_r, dtype, "company dQ", a_dq)
    parity.close(dk[B - 1:, hs], dk_r, dtype, "company dK", a_dk)
    parity.close(dv[B - 1:, hs], dv_r, dtype, "company dV", a_dv)


# ------------------------------------------------------------------ the combined backward entry point
@pytest.mark.parametrize("S,D,causal,p", [(512, 128, True, 0.0), (256, 64, False, 0.0), (512, 64, True, 0.25),
                                          (256, 128, True, 0.25), (384, 128, True, 0.0), (512, 32, True, 0.0),
                                          (384, 32, False, 0.25)])
def test_combined_backward_matches_the_three_calls(S, D, causal, p, device):
    """tri_attn_bwd may fold the delta pre-pass into the dQ kernel and reorder the launches; its
    results must be those of delta, dK/dV and dQ called one after the other."""
    import ctypes
    from trident_amd import _lib, operation
    lib = _lib.lib()
    q, k, v, d_o = [x.to(device) for x in _gen((2, 2, S, D), 400 + S + D, torch.bfloat16)]
    o = torch.empty_like(q)
    lse = torch.empty(2, 2, S, device=device, dtype=torch.float32)
    outs = []
    for combined in (False, True):
        delta = torch.full_like(lse, float("nan"))
        dq, dk, dv = [torch.full_like(q, float("nan")) for _ in range(3)]
        args = operation._make_args(q, k, v, o, lse, None, p, causal, 1.0 / math.sqrt(D), 99 if p > 0 else 0, 0,
                                    d_o, dq, dk, dv, None, delta)
        ref = ctypes.byref(args)
        _lib.check(lib.tri_attn_fwd(ref))
        if combined:
            _lib.check(lib.tri_attn_bwd(ref))
        else:
            _lib.check(lib.tri_attn_bwd_delta(ref))
            _lib.check(lib.tri_attn_bwd_dkdv(ref))
            _lib.check(lib.tri_attn_bwd_dq(ref))
        torch.cuda.synchronize()
        outs.append((delta.clone(), dq.clone(), dk.clone(), dv.clone()))
    (d0, q0, k0, v0), (d1, q1, k1, v1) = outs
    assert not torch.isnan(d1).any()
    # delta: the same fp32 products summed in another order
    assert (d0 - d1).abs().max().item() <= 1e-4 * max(1.0, d0.abs().max().item())
    for a, b_ in ((q0, q1), (k0, k1), (v0, v1)):
        assert not torch.isnan(b_.float()).any()
        assert (a.float() - b_.float()).abs().max().item() <= 2.0 ** -7 * max(1.0, a.float().abs().max().item())


# ------------------------------------------------------------------ head-shared masks dealt per XCD
@pytest.mark.parametrize("B,H,S", [(8, 2, 512), (4, 3, 1024)])
def test_shared_mask_units_multiple_of_eight(B, H, S, device):
    """A [B,1,S,S] mask with B * S/256 a multiple of 8: the workgroup mapping for head-shared masks deals
    whole (batch, tile) units to the 8 XCDs (the branch the full-size C4 workload takes)."""
    w = workloads.WORKLOADS["C4"]
    q, k, v, d_o, mask = workloads.make_inputs(w, B=B, H=H, S=S)
    assert mask.shape == (B, 1, S, S) and (B * (S // 256)) % 8 == 0
    _check(device, w.dtype, q, k, v, d_o, mask=mask, tag=f"C4 B={B} H={H} S={S}")


def test_backward_through_a_fully_masked_row(device):
    """A row with every key masked has lse = -inf: softmax gives NaN there, and so do the gradients that the row
    touches (all of dK and dV, its own dQ row), exactly as in the oracle; other dQ rows stay finite."""
    B, H, S, D = 1, 2, 256, 64
    q, k, v, d_o = _gen((B, H, S, D), 43, torch.bfloat16)
    mask = torch.zeros(B, 1, S, S)
    mask[0, 0, 77, :] = float("-inf")
    o, dq, dk, dv, _ = _run(device, q, k, v, d_o, mask=mask)
    dq_r, dk_r, dv_r, _, _ = parity.oracle_backward(q, k, v, d_o, mask=mask, o=o)
    assert torch.isnan(o[0, :, 77]).all() and np.isnan(dq_r[0, :, 77]).all()
    rows = [r for r in range(S) if r != 77]
    assert not torch.isnan(dq[0, :, rows].float()).any()
    parity.close(dq[:, :, rows], dq_r[:, :, rows], torch.bfloat16, "masked-row dQ")
    assert torch.isnan(dq[0, :, 77].float()).all()
    assert torch.isnan(dk.float()).all() == bool(np.isnan(dk_r).all())
    assert torch.isnan(dv.float()).all() == bool(np.isnan(dv_r).all())


def test_trace_ranges_switch_on(device):
    """config.use_trace = True: the roctx range calls around the operation and every launch really execute."""
    q, k, v, d_o = _gen((1, 2, 128, 64), 52, torch.bfloat16)
    trident.config.use_trace = True
    try:
        o, dq, dk, dv, _ = _run(device, q, k, v, d_o, is_causal=True)
        assert trident.util._roctx, "the roctx library was not found"
    finally:
        trident.config.use_trace = False
    o_ref, _ = parity.oracle_forward(q, k, v, is_causal=True)
    parity.close(o, o_ref, torch.bfloat16, "traced O")


# ------------------------------------------------------------------ mask block classes
def _block_masks(B, H, S, seed):
    """Masks made of 64 x 64 blocks of different kinds, and the kinds: 0 all zero, 1 all -inf, 2 mixed."""
    g = torch.Generator().manual_seed(seed)
    n = S // 64
    kinds = torch.randint(0, 3, (B, H, n, n), generator=g)
    kinds[..., 0] = 2  # (no fully masked row)
    mask = torch.zeros(B, H, S, S)
    for idx in torch.nonzero(kinds).tolist():
        b, h, r, c = idx
        blk = mask[b, h, 64 * r:64 * r + 64, 64 * c:64 * c + 64]
        if kinds[b, h, r, c] == 1:
            blk.fill_(float("-inf"))
        else:
            blk.copy_(torch.randn(64, 64, generator=g))
            blk[::7, ::5] = float("-inf")
    return mask, kinds


def _classes_of(device, mask_view, B, H, S, dtype_code=2):
    import ctypes
    from trident_amd import _lib
    args = _lib.TriAttnArgs()
    args.struct_size = ctypes.sizeof(args)
    args.dtype, args.B, args.H, args.S, args.D = dtype_code, B, H, S, 64
    args.mask, args.mask_dtype = mask_view.data_ptr(), trident.util.dtype(mask_view.dtype)
    args.mask_stride[:] = list(mask_view.stride())
    size = _lib.lib().tri_attn_mask_classes_size(ctypes.byref(args))
    out = torch.full((max(size, 1),), 77, dtype=torch.uint8, device=device)
    args.mask_classes = out.data_ptr()
    _lib.check(_lib.lib().tri_attn_classify_mask(ctypes.byref(args)))
    torch.cuda.synchronize()
    return out.cpu(), size


@pytest.mark.parametrize("mask_dtype", [torch.float32, torch.bfloat16, torch.float16])
@pytest.mark.parametrize("mshape", [(2, 3, 384, 384), (2, 1, 384, 384), (1, 1, 1, 384), (1, 3, 384, 384)])
def test_mask_block_classes(mshape, mask_dtype, device):
    B, H, S = 2, 3, 384
    mask, kinds = _block_masks(mshape[0], mshape[1], S, 81)
    if mshape[2] == 1:
        mask, kinds = mask[:, :, :1].clone(), kinds[:, :, :1]
        kinds = torch.where(kinds == 2, torch.tensor(2), kinds)
        # one row of a mixed block is mixed or, by chance, uniform: recompute from the row itself
        row = mask[:, :, 0].reshape(mshape[0], mshape[1], S // 64, 64)
        kinds = torch.where((row == 0).all(-1), 0, torch.where((row == float("-inf")).all(-1), 1, 2))[:, :, None]
    from trident_amd import operation
    view = operation._expand_mask(mask.to(mask_dtype).to(device), (B, H, S, S))
    got, size = _classes_of(device, view, B, H, S)
    assert size == kinds.numel()
    assert torch.equal(got[:size].reshape(kinds.shape).long(), kinds)


@pytest.mark.parametrize("D,p", [(64, 0.0), (128, 0.0), (64, 0.3), (32, 0.0)])
def test_classes_do_not_change_results(D, p, device):
    """The same calls with and without mask_classes give the same results: skipped tiles only ever added zeros."""
    import ctypes
    from trident_amd import _lib, operation
    lib = _lib.lib()
    B, H, S = 2, 2, 512
    for kind in ("blocks", "lengths"):
        if kind == "blocks":
            mask = _block_masks(B, 1, S, 82)[0]
        else:
            mask = workloads.length_mask(B, S, torch.Generator().manual_seed(83))[0]
            mask[1, 0, :, 100:] = float("-inf")   # a batch whose keys stop inside the first 128-key workgroup
        q, k, v, d_o = [x.to(device) for x in _gen((B, H, S, D), 84, torch.bfloat16)]
        tm = mask.to(device)
        outs = []
        for with_classes in (False, True):
            o = torch.empty_like(q)
            lse = torch.empty(B, H, S, device=device)
            delta = torch.empty_like(lse)
            dq, dk, dv = [torch.full_like(q, float("nan")) for _ in range(3)]
            args = operation._make_args(q, k, v, o, lse, operation._expand_mask(tm, (B, H, S, S)), p, False,
                                        1.0 / math.sqrt(D), 5, 0, d_o, dq, dk, dv, None, delta)
            if with_classes:
                classes = torch.empty(lib.tri_attn_mask_classes_size(ctypes.byref(args)), dtype=torch.uint8, device=device)
                args.mask_classes = classes.data_ptr()
                _lib.check(lib.tri_attn_classify_mask(ctypes.byref(args)))
            _lib.check(lib.tri_attn_fwd(ctypes.byref(args)))
            _lib.check(lib.tri_attn_bwd(ctypes.byref(args)))
            torch.cuda.synchronize()
            outs.append((o, lse, dq, dk, dv))
        # a tile whose mask is all zero takes the arithmetic of a tile without a mask (one fused multiply-add per score
        # instead of product, sum and difference): the same results up to that fp32 rounding of the exponents
        for name, a, b_ in zip(("O", "LSE", "dQ", "dK", "dV"), *outs):
            assert not torch.isnan(a.float()).any(), (kind, name)
            a32, b32 = a.float(), b_.float()
            if name == "LSE":
                assert (a32 - b32).abs().max().item() <= 2e-5, (kind, name)
            else:
                # within a bf16 ulp of the tensor's scale (sums with cancellation move by an ulp of their terms), and
                # nearly all elements equal
                assert (a32 - b32).abs().max().item() <= 2.0**-8 * a32.abs().max().item(), (kind, name)
                assert (a32 != b32).float().mean().item() < 0.2, (kind, name)


@pytest.mark.parametrize("D", [32, 64, 128])
def test_dense_mask_gradient_behind_the_last_active_tile(D, device):
    """A full-shape mask whose trailing key blocks are all -inf, with a gradient: the block classes let the kernels
    stop streaming behind the last active tile, but the mask gradient written in place must still cover every tile
    (zeros there). The buffer starts as NaN; results with and without classes are the same bits."""
    import ctypes
    from trident_amd import _lib, operation
    lib = _lib.lib()
    B, H, S = 1, 2, 512
    dtype = torch.bfloat16
    q, k, v, d_o = _gen((B, H, S, D), 91 + D, dtype)
    mask = (0.5 * torch.randn(B, H, S, S, generator=torch.Generator().manual_seed(92))).to(dtype)
    mask[..., 300:] = float("-inf")        # (key blocks from 320 on are -inf over every row)
    mask[:, 1, 128:, 200:] = float("-inf")  # (and, for the lower rows of head 1, from 256 on)
    tq, tk, tv, tdo, tm = [x.to(device) for x in (q, k, v, d_o, mask)]
    scale = 1.0 / math.sqrt(D)
    outs = []
    for with_classes in (False, True):
        o = torch.empty_like(tq)
        lse = torch.empty(B, H, S, device=device)
        delta = torch.empty_like(lse)
        dq, dk, dv = [torch.full_like(tq, float("nan")) for _ in range(3)]
        dmask = torch.full_like(tm, float("nan"))
        args = operation._make_args(tq, tk, tv, o, lse, tm, 0.0, False, scale, 0, 0, tdo, dq, dk, dv, dmask, delta)
        assert lib.tri_attn_uses_matrix_cores(ctypes.byref(args), 2) == 1
        if with_classes:
            classes = torch.empty(lib.tri_attn_mask_classes_size(ctypes.byref(args)), dtype=torch.uint8, device=device)
            args.mask_classes = classes.data_ptr()
            _lib.check(lib.tri_attn_classify_mask(ctypes.byref(args)))
        _lib.check(lib.tri_attn_fwd(ctypes.byref(args)))
        _lib.check(lib.tri_attn_bwd(ctypes.byref(args)))
        torch.cuda.synchronize()
        assert not torch.isnan(dmask.float()).any(), f"classes={with_classes}: part of the mask gradient was not written"
        outs.append((o, dq, dk, dv, dmask))
    for name, a, b_ in zip(("O", "dQ", "dK", "dV", "dMask"), *outs):
        assert torch.equal(a, b_), name
    o, dq, dk, dv, dmask = outs[1]
    kw = dict(mask=mask, scale=scale)
    o_ref, _ = parity.oracle_forward(q, k, v, **kw)
    parity.close(o, o_ref, dtype, "O")
    dq_r, dk_r, dv_r, dm_r, _ = parity.oracle_backward(q, k, v, d_o, want_dmask=True, o=o, **kw)
    _, a_dq, a_dk, a_dv = parity.oracle_abs_sums(q, k, v, d_o, o=o, **kw)
    parity.close(dq, dq_r, dtype, "dQ", a_dq)
    parity.close(dk, dk_r, dtype, "dK", a_dk)
    parity.close(dv, dv_r, dtype, "dV", a_dv)
    parity.close(dmask, dm_r, dtype, "dMask")
    # the same through the operator, which computes and passes the classes itself
    _check(device, dtype, q, k, v, d_o, mask=mask, mask_grad=True, tag="operator dmask")


@pytest.mark.parametrize("D", [32, 64, 128])
def test_mask_written_between_two_calls(D, device):
    """The operator keeps the block classes of a mask tensor between calls; writing to the tensor (version counter)
    must bring fresh ones: the second mask opens keys the first one had masked out."""
    B, H, S = 2, 2, 512
    dtype = torch.bfloat16
    q, k, v, _ = _gen((B, H, S, D), 93, dtype)
    g = torch.Generator().manual_seed(94)
    first = workloads.length_mask(B, S, g)[0]
    second = torch.zeros_like(first)
    second[:, :, :, :64] = float("-inf")
    second[:, :, 256:, 200:330] = torch.randn(S - 256, 130, generator=g)
    tq, tk, tv = [x.to(device) for x in (q, k, v)]
    tm = first.to(device)
    o1 = trident.function.scaled_dot_product_attention(tq, tk, tv, tm)
    parity.close(o1, parity.oracle_forward(q, k, v, mask=first)[0], dtype, "first mask")
    tm.copy_(second.to(device))
    o2 = trident.function.scaled_dot_product_attention(tq, tk, tv, tm)
    parity.close(o2, parity.oracle_forward(q, k, v, mask=second)[0], dtype, "second mask, same tensor")
    # a write torch does not see needs forget_mask_classes() (or config.cache_mask_classes = False)
    tm.data.copy_(first.to(device))
    trident.operation.forget_mask_classes()
    o3 = trident.function.scaled_dot_product_attention(tq, tk, tv, tm)
    assert torch.equal(o3, o1)
    trident.config.cache_mask_classes = False
    try:
        tm.data.copy_(second.to(device))
        o4 = trident.function.scaled_dot_product_attention(tq, tk, tv, tm)
        assert torch.equal(o4, o2)
    finally:
        trident.config.cache_mask_classes = True


@pytest.mark.parametrize("dtype,S,D", [(torch.float32, 64, 32), (torch.bfloat16, 128, 32), (torch.bfloat16, 256, 64),
                                       (torch.float32, 100, 128)])
@pytest.mark.parametrize("scale", [-0.25, 0.0])
def test_scales_that_are_not_positive(dtype, S, D, scale, device):
    """softmax_scale <= 0 (function.attention accepts any value): the matrix-core kernels take row maxima before
    scaling, so these problems run the element-wise kernels, which scale first."""
    q, k, v, d_o = _gen((1, 2, S, D), 95, dtype)
    for causal in (False, True):
        _assert_kernel_family(q.to(device), None, 0.0, causal, scale, 0)
        trident.config.reference_limits = False
        try:
            _check(device, dtype, q, k, v, d_o, is_causal=causal, scale=scale, tag=f"scale {scale}")
        finally:
            trident.config.reference_limits = True


@pytest.mark.parametrize("mask_dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("mask_grad", [False, True])
def test_mask_with_dropout_at_the_large_head(mask_dtype, mask_grad, device):
    """D = 128 with a mask and dropout together (and a mask gradient on top): the variants that do not fit the 8-wave
    kernels' registers take a smaller fragment ring (forward) or 128-row workgroups (dQ); no kernel of the library uses
    scratch memory."""
    B, H, S, D = 1, 2, 512, 128
    q, k, v, d_o = _gen((B, H, S, D), 96, torch.bfloat16)
    mask = (0.5 * torch.randn(B, H, S, S, generator=torch.Generator().manual_seed(97))).to(mask_dtype)
    _assert_kernel_family(q.to(device), mask.to(device), 0.2, False, 1.0 / math.sqrt(D), 1)
    _check(device, torch.bfloat16, q, k, v, d_o, mask=mask, dropout_p=0.2, mask_grad=mask_grad, seed=98,
           tag=f"mask {mask_dtype} + dropout, D=128")


def test_config2_full_size(device):
    """C2 at its full size (B=4, H=16: 256 items, one per compute unit through the persistent forward's item map):
    two heads against the oracle, and V = 1 gives O = 1 everywhere."""
    w = workloads.WORKLOADS["C2"]
    q, k, v, _, _ = workloads.make_inputs(w)
    tq, tk, tv = [x.to(device) for x in (q, k, v)]
    out = trident.function.scaled_dot_product_attention(tq, tk, tv)
    for (b, h) in [(0, 0), (3, 15), (2, 7)]:
        sl = (slice(b, b + 1), slice(h, h + 1))
        o_ref, _ = parity.oracle_forward(q[sl], k[sl], v[sl])
        parity.close(out[sl], o_ref, w.dtype, f"C2 head {b},{h} O")
    o1 = trident.function.scaled_dot_product_attention(tq, tk, torch.ones_like(tv))
    assert (o1.float() - 1).abs().max().item() <= 2.0**-10
    perm = torch.randperm(w.H, generator=torch.Generator().manual_seed(2)).to(device)
    o_p = trident.function.scaled_dot_product_attention(tq[:, perm], tk[:, perm], tv[:, perm])
    assert torch.equal(o_p, out[:, perm])


# ------------------------------------------------------------------ full-size properties
def _abi_full(device, w, q, k, v, d_o, mask):
    """Forward + backward of a whole workload through the operator's two ABI wrappers; returns device tensors."""
    from trident_amd.operation import Attention
    tq, tk, tv, tdo = [x.to(device) for x in (q, k, v, d_o)]
    tm = None if mask is None else mask.to(device)
    rng = (w.dropout_seed, 0) if w.dropout_p > 0 else (0, 0)
    o, lse = Attention._forward(tq, tk, tv, tm, w.dropout_p, w.is_causal, w.scale, *rng)
    delta = torch.empty_like(lse)
    dq, dk, dv, _ = Attention._backward(tdo, tq, tk, tv, o, lse, tm, w.scale, w.dropout_p, w.is_causal, *rng, False,
                                        delta_out=delta)
    torch.cuda.synchronize()
    return o, lse, delta, dq, dk, dv


def test_config4_full_size(device):
    """C4 at B=8, H=12, S=2048, D=64 with its [B,1,S,S] length mask: two whole heads against the oracle
    (O, LSE, delta, dQ, dK, dV), and V = 1 gives O = 1 everywhere."""
    w = workloads.WORKLOADS["C4"]
    q, k, v, d_o, mask = workloads.make_inputs(w)
    o, lse, delta, dq, dk, dv = _abi_full(device, w, q, k, v, d_o, mask)
    for (b, h) in [(0, 0), (7, 11)]:
        sl = (slice(b, b + 1), slice(h, h + 1))
        m = mask[b:b + 1]
        kw = dict(mask=m, scale=w.scale)
        o_ref, lse_ref = parity.oracle_forward(q[sl], k[sl], v[sl], **kw)
        parity.close(o[sl], o_ref, w.dtype, f"C4 head {b},{h} O")
        parity.lse_delta_close(lse[sl], lse_ref, f"C4 head {b},{h} LSE", w.dtype)
        dq_r, dk_r, dv_r, _, delta_r = parity.oracle_backward(q[sl], k[sl], v[sl], d_o[sl], o=o[sl], **kw)
        _, a_dq, a_dk, a_dv = parity.oracle_abs_sums(q[sl], k[sl], v[sl], d_o[sl], o=o[sl], **kw)
        parity.lse_delta_close(delta[sl], delta_r, f"C4 head {b},{h} delta")
        parity.close(dq[sl], dq_r, w.dtype, f"C4 head {b},{h} dQ", a_dq)
        parity.close(dk[sl], dk_r, w.dtype, f"C4 head {b},{h} dK", a_dk)
        parity.close(dv[sl], dv_r, w.dtype, f"C4 head {b},{h} dV", a_dv)
    ones = torch.ones_like(v).to(device)
    o1 = trident.function.scaled_dot_product_attention(q.to(device), k.to(device), ones, attn_mask=mask.to(device))
    assert (o1.float() - 1).abs().max().item() <= 2.0**-8


def test_config5_full_size_row_blocks(device):
    """C5 at B=1, H=32, S=16384, D=128, causal, dropout 0.1: the first and the last 256 query rows of two heads
    against the oracle with the Philox mask (O, LSE, delta, dQ; from the last block also dK and dV of the last
    256 keys, which only those rows see), and with p = 0, V = 1 gives O = 1."""
    w = workloads.WORKLOADS["C5"]
    q, k, v, d_o, _ = workloads.make_inputs(w)
    o, lse, delta, dq, dk, dv = _abi_full(device, w, q, k, v, d_o, None)
    R = 256
    for h in (0, 31):
        for row0 in (0, w.S - R):
            ref = parity.oracle_rows(q, k, v, d_o, 0, h, row0, R, w.H, o=o, dropout_p=w.dropout_p, is_causal=True,
                                     scale=w.scale, seed=w.dropout_seed, offset=0)
            sl = slice(row0, row0 + R)
            tag = f"C5 head {h} rows {row0}+{R}"
            parity.close(o[0, h, sl], ref["o"], w.dtype, tag + " O")
            parity.lse_delta_close(lse[0, h, sl], ref["lse2"], tag + " LSE", w.dtype)
            parity.lse_delta_close(delta[0, h, sl], ref["delta"], tag + " delta")
            parity.close(dq[0, h, sl], ref["dq"], w.dtype, tag + " dQ", ref["a_dq"])
            if row0 + R == w.S:
                parity.close(dk[0, h, sl], ref["dk_part"][sl], w.dtype, tag + " dK", ref["a_dk_part"][sl])
                parity.close(dv[0, h, sl], ref["dv_part"][sl], w.dtype, tag + " dV", ref["a_dv_part"][sl])
    ones = torch.ones_like(v).to(device)
    o1 = trident.function.scaled_dot_product_attention(q.to(device), k.to(device), ones, is_causal=True)
    assert (o1.float() - 1).abs().max().item() <= 2.0**-8



def test_config3_full_size_properties(device):
    """At B=2,H=16,S=4096,D=128 the oracle is too slow for the whole tensor; check it on a few
    heads' worth of rows and use size-independent properties for the rest."""
    w = workloads.WORKLOADS["C3"]
    q, k, v, d_o, _ = workloads.make_inputs(w)
    tq, tk, tv = [x.to(device).requires_grad_(True) for x in (q, k, v)]
    out = trident.function.scaled_dot_product_attention(tq, tk, tv, is_causal=True)
    out.backward(d_o.to(device))
    # causal row 0 copies V row 0; dV is exact where only one query sees the key (last key)
    assert torch.equal(out[:, :, 0], tv[:, :, 0])
    # one head against the oracle
    for (b, h) in [(0, 0), (1, 15)]:
        sl = (slice(b, b + 1), slice(h, h + 1))
        o_ref, _ = parity.oracle_forward(q[sl], k[sl], v[sl], is_causal=True)
        dq_r, dk_r, dv_r, _, _ = parity.oracle_backward(q[sl], k[sl], v[sl], d_o[sl], is_causal=True, o=out[sl])
        parity.close(out[sl], o_ref, w.dtype, f"C3 head {b},{h} O")
        _, a_dq, a_dk, a_dv = parity.oracle_abs_sums(q[sl], k[sl], v[sl], d_o[sl], is_causal=True, o=out[sl])
        for name, got, want, a in (("dQ", tq.grad, dq_r, a_dq), ("dK", tk.grad, dk_r, a_dk), ("dV", tv.grad, dv_r, a_dv)):
            st = {}
            parity.close(got[sl], want, w.dtype, "C3 " + name, a, stats=st)
            # how much the two documented additions to the plain atol (output rounding, 16-bit operand) were used
            print(f"C3 head {b},{h} {name}: max err {st['max_err']:.2e}; {st['over_atol']} of {st['elements']} elements "
                  f"above the plain atol, worst {st['max_over_atol']:.2f} x atol")
    # V == 1 gives O == 1 at full size (softmax rows sum to one)
    ones = torch.ones_like(tv)
    o1 = trident.function.scaled_dot_product_attention(tq.detach(), tk.detach(), ones, is_causal=True)
    assert (o1.float() - 1).abs().max().item() <= 2.0**-8
    # heads are independent: permuting heads permutes outputs bit for bit
    perm = torch.randperm(w.H, generator=torch.Generator().manual_seed(1)).to(device)
    o_p = trident.function.scaled_dot_product_attention(tq.detach()[:, perm], tk.detach()[:, perm],
                                                        tv.detach()[:, perm], is_causal=True)
    assert torch.equal(o_p, out.detach()[:, perm])
