"""Pins the CPU oracle (oracle/) before anything is compared against it. Runs without a GPU."""
import json
import math
import os

import numpy as np
import pytest
import torch

from oracle import attention as oracle
from oracle import c_oracle, philox

GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")


def _rand(shape, seed):
    return np.random.default_rng(seed).standard_normal(shape)


# ---------------------------------------------------------------- Philox / dropout layout
def test_philox_known_answers():
    kat = json.load(open(os.path.join(GOLDEN, "philox_kat.json")))
    for vec in kat["vectors"]:
        ctr = [int(x, 16) for x in vec["ctr"]]
        key = [int(x, 16) for x in vec["key"]]
        out = [int(x, 16) for x in vec["out"]]
        assert philox.philox4x32_10_scalar(ctr, key) == out
        assert [int(x) for x in philox.philox4x32_10(*ctr, *key)] == out
        assert c_oracle.philox(ctr, key) == out


def test_philox_vectorised_matches_scalar():
    rng = np.random.default_rng(5)
    ctr = rng.integers(0, 2**32, size=(50, 4), dtype=np.uint64)
    key = [0x12345678, 0x9ABCDEF0]
    vec = philox.philox4x32_10(ctr[:, 0], ctr[:, 1], ctr[:, 2], ctr[:, 3], *key)
    for n in range(50):
        assert [int(w[n]) for w in vec] == philox.philox4x32_10_scalar(ctr[n], key)


@pytest.mark.parametrize("p,thr", [(0.0, 0), (0.001, 0), (0.1, 26), (0.25, 64), (0.5, 128), (0.999, 256), (1.0, 256)])
def test_dropout_threshold(p, thr):
    assert philox.dropout_threshold(p) == thr


def test_dropout_mask_numpy_vs_c_and_rate():
    for seed, offset, bh, p in [(0x5EED, 0, 0, 0.1), (2**63 + 12345, 9, 77, 0.5)]:
        a = philox.dropout_keep_mask(seed, offset, bh, np.arange(128), np.arange(128), p)
        b = c_oracle.dropout_mask(seed, offset, bh, 128, philox.dropout_threshold(p))
        assert (a == b).all()
        p_eff = philox.dropout_threshold(p) / 256
        assert abs(a.mean() - (1 - p_eff)) < 4 * math.sqrt(p_eff * (1 - p_eff) / a.size)
    assert philox.dropout_keep_mask(1, 0, 0, np.arange(16), np.arange(16), 0.0).all()
    assert not philox.dropout_keep_mask(1, 0, 0, np.arange(16), np.arange(16), 1.0).any()


def test_dropout_mask_layout_is_tile_independent():
    full = philox.dropout_keep_mask(42, 3, 5, np.arange(64), np.arange(64), 0.3)
    part = philox.dropout_keep_mask(42, 3, 5, np.arange(17, 40), np.arange(9, 50), 0.3)
    assert (full[17:40, 9:50] == part).all()
    other_head = philox.dropout_keep_mask(42, 3, 6, np.arange(64), np.arange(64), 0.3)
    other_call = philox.dropout_keep_mask(42, 4, 5, np.arange(64), np.arange(64), 0.3)
    assert (full != other_head).any() and (full != other_call).any()


def test_dropout_mask_golden():
    data = json.load(open(os.path.join(GOLDEN, "dropout_mask.json")))
    for c in data["cases"]:
        keep = philox.dropout_keep_mask(c["seed"], c["offset"], c["bh"], np.arange(c["row0"], c["row0"] + c["rows"]),
                                        np.arange(c["col0"], c["col0"] + c["cols"]), c["p"])
        assert np.packbits(keep.astype(np.uint8), axis=None).tobytes().hex() == c["keep_bits_hex"]
        assert philox.dropout_threshold(c["p"]) == c["thr8"]


# ---------------------------------------------------------------- forward
@pytest.mark.parametrize("variant", ["plain", "causal", "mask", "bmask", "dropout"])
def test_forward_vs_bruteforce(variant):
    B, H, S, D = 2, 2, 9, 4
    q, k, v = _rand((B, H, S, D), 1), _rand((B, H, S, D), 2), _rand((B, H, S, D), 3)
    kw, bf = {}, {}
    if variant == "causal":
        kw["is_causal"] = bf["is_causal"] = True
    if variant == "mask":
        kw["mask"] = bf["mask"] = _rand((B, H, S, S), 4)
    if variant == "bmask":
        m = _rand((1, H, S, S), 4)
        m[0, :, :, 7:] = -np.inf
        kw["mask"] = bf["mask"] = m
    if variant == "dropout":
        kw.update(dropout_p=0.4, seed=99, offset=1)
        z = np.stack([[philox.dropout_keep_mask(99, 1, b * H + h, np.arange(S), np.arange(S), 0.4)
                       for h in range(H)] for b in range(B)]) * philox.dropout_scale(0.4)
        bf["keep_scale"] = z
    o, lse2 = oracle.attention_forward(q, k, v, scale=0.37, **kw)
    o_bf, lse_bf = oracle.attention_bruteforce(q, k, v, scale=0.37, **bf)
    np.testing.assert_allclose(o, o_bf, rtol=0, atol=1e-12)
    np.testing.assert_allclose(lse2, lse_bf * oracle.LOG2E, rtol=0, atol=1e-12)


def _torch_sdpa(q, k, v, d_o, mask=None, is_causal=False):
    tq, tk, tv = [torch.tensor(x, requires_grad=True) for x in (q, k, v)]
    tm = None if mask is None else torch.tensor(mask, requires_grad=True)
    out = torch.nn.functional.scaled_dot_product_attention(tq, tk, tv, attn_mask=tm, is_causal=is_causal)
    out.backward(torch.tensor(d_o))
    return out.detach().numpy(), tq.grad.numpy(), tk.grad.numpy(), tv.grad.numpy(), None if tm is None else tm.grad.numpy()


@pytest.mark.parametrize("shape,causal", [((4, 8, 128, 64), True), ((4, 8, 256, 32), False), ((1, 1, 1, 16), True)])
def test_against_torch_sdpa_reference_shapes(shape, causal):
    """The shapes and checks of the reference's tests/test_attention.py:22-84 in fp64."""
    B, H, S, D = shape
    q = np.random.default_rng(1).random(shape)  # the reference's backward test draws q uniform
    k, v, d_o = _rand(shape, 2), _rand(shape, 3), _rand(shape, 4)
    o_t, dq_t, dk_t, dv_t, _ = _torch_sdpa(q, k, v, d_o, is_causal=causal)
    o, _ = oracle.attention_forward(q, k, v, is_causal=causal)
    dq, dk, dv, _, _ = oracle.attention_backward(q, k, v, d_o, is_causal=causal)
    for a, b in [(o, o_t), (dq, dq_t), (dk, dk_t), (dv, dv_t)]:
        np.testing.assert_allclose(a, b, rtol=0, atol=1e-10)
    mask = _rand((B, H, S, S), 5)
    o_t, dq_t, dk_t, dv_t, dm_t = _torch_sdpa(q, k, v, d_o, mask=mask)
    o, _ = oracle.attention_forward(q, k, v, mask=mask)
    dq, dk, dv, dm, _ = oracle.attention_backward(q, k, v, d_o, mask=mask, want_dmask=True)
    for a, b in [(o, o_t), (dq, dq_t), (dk, dk_t), (dv, dv_t), (dm, dm_t)]:
        np.testing.assert_allclose(a, b, rtol=0, atol=1e-10)


@pytest.mark.parametrize("mshape", [(3, 1, 16, 16), (1, 4, 16, 16), (3, 1, 1, 16), (1, 1, 1, 16)])
def test_broadcast_mask_gradient_matches_autograd(mshape):
    shape = (3, 4, 16, 8)
    q, k, v, d_o = [_rand(shape, s) for s in (1, 2, 3, 4)]
    mask = _rand(mshape, 5)
    _, _, _, _, dm_t = _torch_sdpa(q, k, v, d_o, mask=mask)
    _, _, _, dm, _ = oracle.attention_backward(q, k, v, d_o, mask=mask, want_dmask=True)
    np.testing.assert_allclose(dm, dm_t, rtol=0, atol=1e-10)


def test_lse_matches_logsumexp():
    shape = (1, 2, 32, 8)
    q, k, v = [_rand(shape, s) for s in (1, 2, 3)]
    mask = _rand((1, 2, 32, 32), 9)
    _, lse2 = oracle.attention_forward(q, k, v, mask=mask, scale=0.5)
    s = torch.tensor(q) @ torch.tensor(k).transpose(-1, -2) * 0.5 + torch.tensor(mask)
    np.testing.assert_allclose(lse2, torch.logsumexp(s, -1).numpy() * oracle.LOG2E, rtol=0, atol=1e-12)


def test_dropout_gradients_match_autograd_of_explicit_formula():
    B, H, S, D = 1, 3, 24, 8
    q, k, v, d_o = [_rand((B, H, S, D), s) for s in (1, 2, 3, 4)]
    p, seed, offset = 0.3, 1234567, 5
    z = np.stack([[philox.dropout_keep_mask(seed, offset, b * H + h, np.arange(S), np.arange(S), p)
                   for h in range(H)] for b in range(B)]) * philox.dropout_scale(p)
    tq, tk, tv = [torch.tensor(x, requires_grad=True) for x in (q, k, v)]
    s = tq @ tk.transpose(-1, -2) / math.sqrt(D)
    s = s.masked_fill(~torch.ones(S, S, dtype=torch.bool).tril(), float("-inf"))
    out = (torch.softmax(s, -1) * torch.tensor(z)) @ tv
    out.backward(torch.tensor(d_o))
    o, _ = oracle.attention_forward(q, k, v, dropout_p=p, is_causal=True, seed=seed, offset=offset)
    dq, dk, dv, _, delta = oracle.attention_backward(q, k, v, d_o, dropout_p=p, is_causal=True, seed=seed, offset=offset)
    np.testing.assert_allclose(o, out.detach().numpy(), rtol=0, atol=1e-12)
    np.testing.assert_allclose(dq, tq.grad.numpy(), rtol=0, atol=1e-11)
    np.testing.assert_allclose(dk, tk.grad.numpy(), rtol=0, atol=1e-11)
    np.testing.assert_allclose(dv, tv.grad.numpy(), rtol=0, atol=1e-11)
    np.testing.assert_allclose(delta, (d_o * o).sum(-1), rtol=0, atol=1e-12)


# ---------------------------------------------------------------- C restatement vs numpy
@pytest.mark.parametrize("variant", ["plain", "causal", "mask_dropout"])
def test_c_restatement_matches_numpy(variant):
    S, D = 40, 16
    q, k, v, d_o = [_rand((1, 1, S, D), s) for s in (1, 2, 3, 4)]
    mask = None
    kw = {}
    thr8, seed, offset, bh = 0, 0, 0, 0
    if variant == "causal":
        kw["is_causal"] = True
    if variant == "mask_dropout":
        mask = _rand((1, 1, S, S), 5)
        mask[..., 33:] = -np.inf
        seed, offset = 0xABCDEF0123, 4
        kw.update(mask=mask, dropout_p=0.2, seed=seed, offset=offset)
        thr8 = philox.dropout_threshold(0.2)
    o, lse2 = oracle.attention_forward(q, k, v, scale=0.3, **kw)
    dq, dk, dv, dm, delta = oracle.attention_backward(q, k, v, d_o, scale=0.3, want_dmask=True, **kw)
    m2 = None if mask is None else mask[0, 0]
    causal = kw.get("is_causal", False)
    o_c, lse_c = c_oracle.fwd_head(q[0, 0], k[0, 0], v[0, 0], m2, causal, 0.3, seed, offset, bh, thr8)
    dq_c, dk_c, dv_c, dm_c, delta_c = c_oracle.bwd_head(q[0, 0], k[0, 0], v[0, 0], m2, o_c, d_o[0, 0], causal, 0.3,
                                                        seed, offset, bh, thr8, want_dmask=True)
    for a, b in [(o[0, 0], o_c), (lse2[0, 0], lse_c), (dq[0, 0], dq_c), (dk[0, 0], dk_c), (dv[0, 0], dv_c),
                 (delta[0, 0], delta_c)]:
        np.testing.assert_allclose(a, b, rtol=0, atol=1e-11)
    if dm is not None:
        np.testing.assert_allclose(dm[0, 0], dm_c, rtol=0, atol=1e-11)


# ---------------------------------------------------------------- what the mathematics fixes
def test_special_cases():
    shape = (2, 2, 16, 8)
    q, k, v, d_o = [_rand(shape, s) for s in (1, 2, 3, 4)]
    # V == 1 -> O == 1
    o, _ = oracle.attention_forward(q, k, np.ones(shape), is_causal=True)
    np.testing.assert_allclose(o, 1.0, atol=1e-13)
    # Q == 0 -> uniform weights: mean of V (prefix mean when causal)
    o, lse2 = oracle.attention_forward(np.zeros(shape), k, v)
    np.testing.assert_allclose(o, np.broadcast_to(v.mean(-2, keepdims=True), shape), atol=1e-13)
    np.testing.assert_allclose(lse2, math.log2(16), atol=1e-13)
    o, _ = oracle.attention_forward(np.zeros(shape), k, v, is_causal=True)
    prefix = np.cumsum(v, -2) / np.arange(1, 17)[:, None]
    np.testing.assert_allclose(o, prefix, atol=1e-13)
    # causal row 0 sees only key 0
    o, _ = oracle.attention_forward(q, k, v, is_causal=True)
    np.testing.assert_allclose(o[..., 0, :], v[..., 0, :], atol=1e-13)
    # causal == additive upper-triangular -inf mask
    tri = np.where(np.tril(np.ones((16, 16), bool)), 0.0, -np.inf)[None, None]
    o2, _ = oracle.attention_forward(q, k, v, mask=tri)
    np.testing.assert_allclose(o, o2, atol=1e-13)
    g1 = oracle.attention_backward(q, k, v, d_o, is_causal=True)
    g2 = oracle.attention_backward(q, k, v, d_o, mask=tri)
    for a, b in zip(g1[:3], g2[:3]):
        np.testing.assert_allclose(a, b, atol=1e-13)
    # a per-row constant in the mask leaves O unchanged and shifts the LSE
    c = _rand((2, 2, 16, 1), 7)
    oa, la = oracle.attention_forward(q, k, v, mask=np.zeros((2, 2, 16, 16)))
    ob, lb = oracle.attention_forward(q, k, v, mask=np.broadcast_to(c, (2, 2, 16, 16)).copy())
    np.testing.assert_allclose(oa, ob, atol=1e-12)
    np.testing.assert_allclose(lb - la, c[..., 0] * oracle.LOG2E, atol=1e-12)
    # rows of dS (the mask gradient) sum to zero
    mask = _rand((2, 2, 16, 16), 8)
    _, _, _, dm, _ = oracle.attention_backward(q, k, v, d_o, mask=mask, want_dmask=True)
    np.testing.assert_allclose(dm.sum(-1), 0.0, atol=1e-13)
    # key permutation invariance (non-causal)
    perm = np.random.default_rng(3).permutation(16)
    o3, _ = oracle.attention_forward(q, k[..., perm, :], v[..., perm, :])
    np.testing.assert_allclose(oa, o3, atol=1e-13)
    # a length mask equals truncating K and V
    lm = np.zeros((2, 1, 16, 16))
    lm[..., 11:] = -np.inf
    o4, _ = oracle.attention_forward(q, k, v, mask=lm)
    for b in range(2):
        for h in range(2):
            s = q[b, h] @ k[b, h, :11].T / math.sqrt(8)
            pr = np.exp(s - s.max(-1, keepdims=True))
            pr /= pr.sum(-1, keepdims=True)
            np.testing.assert_allclose(o4[b, h], pr @ v[b, h, :11], atol=1e-13)


def test_single_position_smoke_shape():
    """S == 1 (the reference's smoke shape, tests/test_attention.py:88): O = V, dV = dO, dQ = dK = 0."""
    shape = (1, 1, 1, 16)
    q, k, v, d_o = [_rand(shape, s) for s in (1, 2, 3, 4)]
    for causal in (True, False):
        o, lse2 = oracle.attention_forward(q, k, v, is_causal=causal)
        dq, dk, dv, _, _ = oracle.attention_backward(q, k, v, d_o, is_causal=causal)
        np.testing.assert_allclose(o, v, atol=1e-14)
        np.testing.assert_allclose(dv, d_o, atol=1e-14)
        np.testing.assert_allclose(dq, 0, atol=1e-14)
        np.testing.assert_allclose(dk, 0, atol=1e-14)


def test_finite_differences():
    shape = (1, 1, 6, 4)
    q, k, v, d_o = [_rand(shape, s) for s in (1, 2, 3, 4)]
    mask = _rand((1, 1, 6, 6), 5)
    kw = dict(mask=mask, dropout_p=0.3, seed=7, offset=0)
    dq, dk, dv, dm, _ = oracle.attention_backward(q, k, v, d_o, want_dmask=True, **kw)

    def loss(q_, k_, v_, m_):
        kw2 = dict(kw, mask=m_)
        return float((oracle.attention_forward(q_, k_, v_, **kw2)[0] * d_o).sum())

    eps = 1e-6
    for grad, which in [(dq, 0), (dk, 1), (dv, 2), (dm, 3)]:
        args = [q, k, v, mask]
        for idx in [(0, 0, 1, 2), (0, 0, 5, 3), (0, 0, 3, 0)]:
            hi = [a.copy() for a in args]
            lo = [a.copy() for a in args]
            hi[which][idx] += eps
            lo[which][idx] -= eps
            fd = (loss(*hi) - loss(*lo)) / (2 * eps)
            assert abs(fd - grad[idx]) < 1e-7


def test_mask_and_causal_rejected():
    x = _rand((1, 1, 4, 4), 1)
    with pytest.raises(ValueError, match="both attn_mask and is_causal"):
        oracle.attention_forward(x, x, x, mask=np.zeros((1, 1, 4, 4)), is_causal=True)


def test_golden_fixture():
    data = np.load(os.path.join(GOLDEN, "attention_small.npz"))
    q, k, v, d_o, mask = [data[n] for n in ("q", "k", "v", "d_o", "mask")]
    variants = {
        "plain": dict(),
        "causal": dict(is_causal=True),
        "mask_dropout": dict(mask=mask, dropout_p=0.25, seed=0x5EED, offset=2),
    }
    for name, kw in variants.items():
        o, lse2 = oracle.attention_forward(q, k, v, **kw)
        dq, dk, dv, dm, delta = oracle.attention_backward(q, k, v, d_o, want_dmask=True, **kw)
        for key, val in [("o", o), ("lse2", lse2), ("dq", dq), ("dk", dk), ("dv", dv), ("delta", delta)]:
            np.testing.assert_allclose(val, data[f"{name}.{key}"], rtol=0, atol=1e-13)
        if dm is not None:
            np.testing.assert_allclose(dm, data[f"{name}.dmask"], rtol=0, atol=1e-13)


def test_backward_with_saved_output_and_abs_sums():
    """delta is defined on the output tensor handed to the backward; abs sums bound the gradients."""
    shape = (1, 2, 12, 4)
    q, k, v, d_o = [_rand(shape, s) for s in (1, 2, 3, 4)]
    o, _ = oracle.attention_forward(q, k, v, is_causal=True)
    base = oracle.attention_backward(q, k, v, d_o, is_causal=True)
    same = oracle.attention_backward(q, k, v, d_o, is_causal=True, o=o)
    for a, b in zip(base[:3], same[:3]):
        np.testing.assert_allclose(a, b, atol=1e-13)
    o2 = o + 0.5
    dq2, dk2, dv2, _, delta2 = oracle.attention_backward(q, k, v, d_o, is_causal=True, o=o2)
    np.testing.assert_allclose(delta2, (d_o * o2).sum(-1), atol=1e-13)
    np.testing.assert_allclose(dv2, base[2], atol=1e-13)  # dV does not depend on delta
    assert np.abs(dq2 - base[0]).max() > 1e-3
    a_o, a_dq, a_dk, a_dv = oracle.operand_abs_sums(q, k, v, d_o, is_causal=True)
    assert (np.abs(o) <= a_o + 1e-12).all() and (np.abs(base[0]) <= a_dq + 1e-12).all()
    assert (np.abs(base[1]) <= a_dk + 1e-12).all() and (np.abs(base[2]) <= a_dv + 1e-12).all()
    # non-negative inputs make the bound tight for O
    o_pos, _ = oracle.attention_forward(q, k, np.abs(v), is_causal=True)
    np.testing.assert_allclose(o_pos, a_o, atol=1e-13)


# ---------------------------------------------------------------- row-block form (full-size checks)
@pytest.mark.parametrize("variant", ["causal+dropout", "mask", "plain"])
def test_row_blocks_reassemble_to_autograd_of_the_explicit_formula(variant):
    """oracle.attention_rows against torch autograd of softmax(QK^T*scale + mask) * Z @ V: O, LSE, delta and dQ of
    a block are the rows of the whole result; the dK/dV parts of all blocks add up to dK/dV; and under the
    causal mask the LAST block alone gives dK/dV of its own keys."""
    H, S, D, R = 2, 48, 8, 16
    q, k, v, d_o = [_rand((1, H, S, D), s) for s in (11, 12, 13, 14)]
    causal = variant.startswith("causal")
    p, seed, offset = (0.3, 99, 2) if "dropout" in variant else (0.0, 0, 0)
    mask = _rand((1, H, S, S), 15) if variant == "mask" else None
    for h in range(H):
        tq, tk, tv = [torch.tensor(x[0, h], requires_grad=True) for x in (q, k, v)]
        s = tq @ tk.T / math.sqrt(D)
        if causal:
            s = s.masked_fill(~torch.ones(S, S, dtype=torch.bool).tril(), float("-inf"))
        if mask is not None:
            s = s + torch.tensor(mask[0, h])
        pr = torch.softmax(s, -1)
        if p > 0:
            pr = pr * torch.tensor(philox.dropout_keep_mask(seed, offset, h, np.arange(S), np.arange(S), p) *
                                   philox.dropout_scale(p))
        out = pr @ tv
        out.backward(torch.tensor(d_o[0, h]))
        dk_sum, dv_sum = np.zeros((S, D)), np.zeros((S, D))
        for r0 in range(0, S, R):
            blk = oracle.attention_rows(q[0, h, r0:r0 + R], k[0, h], v[0, h], d_o[0, h, r0:r0 + R], r0, h,
                                        mask_rows=None if mask is None else mask[0, h, r0:r0 + R], dropout_p=p,
                                        is_causal=causal, seed=seed, offset=offset)
            np.testing.assert_allclose(blk["o"], out.detach().numpy()[r0:r0 + R], rtol=0, atol=1e-12)
            np.testing.assert_allclose(blk["lse2"], torch.logsumexp(s, -1).detach().numpy()[r0:r0 + R] * oracle.LOG2E,
                                       rtol=0, atol=1e-12)
            np.testing.assert_allclose(blk["delta"], (d_o[0, h] * out.detach().numpy()).sum(-1)[r0:r0 + R], rtol=0,
                                       atol=1e-12)
            np.testing.assert_allclose(blk["dq"], tq.grad.numpy()[r0:r0 + R], rtol=0, atol=1e-11)
            dk_sum += blk["dk_part"]
            dv_sum += blk["dv_part"]
        np.testing.assert_allclose(dk_sum, tk.grad.numpy(), rtol=0, atol=1e-11)
        np.testing.assert_allclose(dv_sum, tv.grad.numpy(), rtol=0, atol=1e-11)
        if causal:
            np.testing.assert_allclose(blk["dk_part"][S - R:], tk.grad.numpy()[S - R:], rtol=0, atol=1e-11)
            np.testing.assert_allclose(blk["dv_part"][S - R:], tv.grad.numpy()[S - R:], rtol=0, atol=1e-11)
