"""fp64 CPU restatement of the attention hot path. TEST INFRASTRUCTURE ONLY.

What is restated, and where the reference fixes it:

* semantics compared by the reference's own tests: softmax(Q K^T * scale + mask) V against
  torch.nn.functional.scaled_dot_product_attention, outputs and all gradients incl. the
  mask gradient (tests/test_attention.py:22-84, rule tests/util.py:18-19);
* default scale 1/sqrt(D) (trident/function/function.py:238-253);
* causal rule "row >= col is visible" (trident/kernel/attention.py:131-134, 294-296);
  the mask is additive and is not combined with causal (trident/operation/attention.py:41-45);
* saved statistic log2sum = max + log2(sum) in the log2 domain of s * log2(e)
  (trident/kernel/attention.py:115-117, 142-149, 164);
* backward closed forms: delta = rowsum(dO * O) (trident/kernel/softmax.py:223-238),
  P = exp2(s2 - log2sum), dV = P^T dO, dP = dO V^T, dS = P * (dP - delta),
  dQ = scale dS K, dK = scale dS^T Q, dMask = dS (trident/kernel/attention.py:304-333).

Deliberately NOT restated (quirks the build does not copy): fp16 accumulation for bf16
inputs (trident/language/standard.py:21-22), accumulators and log2sum in the input dtype
(trident/kernel/attention.py:120,283-284; trident/operation/attention.py:102), and the
reference's dropout-on-O with a non-deterministic seed (trident/kernel/attention.py:158-161,
309-313).  Dropout here is the standard Bernoulli keep-mask on P rescaled by 1/(1-p), driven
by the counter-based generator documented in oracle/philox.py.

Pinned by: tests/test_oracle.py (brute-force scalar loops on tiny inputs, torch CPU SDPA
forward and autograd gradients, closed-form special cases, finite differences) and the
committed fixtures under tests/golden/.
"""
import math

import numpy as np

from . import philox

LOG2E = 1.4426950408889634  # trident/language/constant.py:17-20


def _mask_slice(mask, b, h):
    if mask is None:
        return None
    mb = 0 if mask.shape[0] == 1 else b
    mh = 0 if mask.shape[1] == 1 else h
    return mask[mb, mh]


def _scores(q, k, mask_bh, is_causal, scale):
    s = (q @ k.T) * scale
    if is_causal:
        n = s.shape[0]
        s = np.where(np.tril(np.ones((n, n), dtype=bool)), s, -np.inf)
    elif mask_bh is not None:
        s = s + mask_bh
    return s


def _softmax_rows(s):
    m = np.max(s, axis=-1, keepdims=True)
    m_safe = np.where(np.isfinite(m), m, 0.0)
    e = np.exp(s - m_safe)
    l = np.sum(e, axis=-1, keepdims=True)
    with np.errstate(divide="ignore", invalid="ignore"):
        p = e / l
        lse = m_safe + np.log(l)
    return p, lse[..., 0]


def _keep_scale(seed, offset, bh, n, p):
    if p <= 0.0 or philox.dropout_threshold(p) == 0:
        return None
    keep = philox.dropout_keep_mask(seed, offset, bh, np.arange(n), np.arange(n), p)
    return keep.astype(np.float64) * philox.dropout_scale(p)


def attention_forward(q, k, v, mask=None, dropout_p=0.0, is_causal=False, scale=None, seed=0, offset=0):
    """q, k, v: float64 [B,H,S,D]; mask: float64 broadcastable [B|1, H|1, S, S] or None.
    Returns (O [B,H,S,D], lse2 [B,H,S]) with lse2 = log2(sum_j exp(s_ij)) = lse_natural * log2(e)."""
    q = np.asarray(q, dtype=np.float64)
    k = np.asarray(k, dtype=np.float64)
    v = np.asarray(v, dtype=np.float64)
    if mask is not None and is_causal:
        raise ValueError("Error because both attn_mask and is_causal are set.")
    B, H, S, D = q.shape
    if scale is None:
        scale = 1.0 / math.sqrt(D)
    out = np.empty_like(q)
    lse2 = np.empty((B, H, S), dtype=np.float64)
    for b in range(B):
        for h in range(H):
            s = _scores(q[b, h], k[b, h], _mask_slice(mask, b, h), is_causal, scale)
            p, lse = _softmax_rows(s)
            z = _keep_scale(seed, offset, b * H + h, S, dropout_p)
            if z is not None:
                p = p * z
            out[b, h] = p @ v[b, h]
            lse2[b, h] = lse * LOG2E
    return out, lse2


def attention_backward(q, k, v, d_out, mask=None, dropout_p=0.0, is_causal=False, scale=None, seed=0, offset=0,
                       want_dmask=False, o=None):
    """Closed-form gradients. Returns (dQ, dK, dV, dMask or None, delta [B,H,S]).
    dMask has the mask's own (possibly broadcast) shape: summed over broadcast dims.
    ``o``: the saved forward output the backward is handed (the reference computes delta from the
    stored output tensor, trident/operation/attention.py:139-164); None recomputes it exactly."""
    q = np.asarray(q, dtype=np.float64)
    k = np.asarray(k, dtype=np.float64)
    v = np.asarray(v, dtype=np.float64)
    d_out = np.asarray(d_out, dtype=np.float64)
    B, H, S, D = q.shape
    if scale is None:
        scale = 1.0 / math.sqrt(D)
    dq = np.empty_like(q)
    dk = np.empty_like(k)
    dv = np.empty_like(v)
    delta = np.empty((B, H, S), dtype=np.float64)
    dmask = np.zeros(mask.shape, dtype=np.float64) if (want_dmask and mask is not None) else None
    for b in range(B):
        for h in range(H):
            s = _scores(q[b, h], k[b, h], _mask_slice(mask, b, h), is_causal, scale)
            p, _ = _softmax_rows(s)
            z = _keep_scale(seed, offset, b * H + h, S, dropout_p)
            pz = p if z is None else p * z
            o_bh = pz @ v[b, h] if o is None else np.asarray(o[b, h], dtype=np.float64)
            dlt = np.sum(d_out[b, h] * o_bh, axis=-1)
            dp = d_out[b, h] @ v[b, h].T
            if z is not None:
                dp = dp * z
            ds = p * (dp - dlt[:, None])
            dv[b, h] = pz.T @ d_out[b, h]
            dq[b, h] = scale * (ds @ k[b, h])
            dk[b, h] = scale * (ds.T @ q[b, h])
            delta[b, h] = dlt
            if dmask is not None:
                mb = 0 if mask.shape[0] == 1 else b
                mh = 0 if mask.shape[1] == 1 else h
                dmask[mb, mh] += ds.sum(axis=0, keepdims=True) if mask.shape[2] == 1 else ds  # (row-broadcast mask)
    return dq, dk, dv, dmask, delta


def attention_rows(q_rows, k, v, d_out_rows, row0, bh, mask_rows=None, dropout_p=0.0, is_causal=False, scale=None,
                   seed=0, offset=0, o_rows=None):
    """One head, the block of query rows [row0, row0 + R): everything that is local to those rows, so that a
    full-size problem can be checked block by block (same formulas as attention_forward / attention_backward).
    q_rows, d_out_rows: [R,D]; k, v: [S,D]; mask_rows: [R,S] or None; bh = b * H + h (dropout counter).
    Returns dict(o [R,D], lse2 [R], delta [R], dq [R,D], dk_part [S,D], dv_part [S,D]) plus the sums of
    absolute terms a_o, a_dq, a_dk_part, a_dv_part (see operand_abs_sums); dk_part / dv_part are
    these rows' contributions to dK / dV. Under a causal mask the rows of a block that ends at S are the only
    ones that see keys >= row0, so dk_part[row0:] and dv_part[row0:] are then the complete gradients."""
    q_rows, k, v, d_out_rows = [np.asarray(x, dtype=np.float64) for x in (q_rows, k, v, d_out_rows)]
    R, D = q_rows.shape
    S = k.shape[0]
    if scale is None:
        scale = 1.0 / math.sqrt(D)
    s = (q_rows @ k.T) * scale
    rows = np.arange(row0, row0 + R)
    if is_causal:
        s = np.where(rows[:, None] >= np.arange(S)[None, :], s, -np.inf)
    elif mask_rows is not None:
        s = s + np.asarray(mask_rows, dtype=np.float64)
    p, lse = _softmax_rows(s)
    pz = p
    z = None
    if dropout_p > 0.0 and philox.dropout_threshold(dropout_p) != 0:
        z = philox.dropout_keep_mask(seed, offset, bh, rows, np.arange(S), dropout_p).astype(np.float64)
        z *= philox.dropout_scale(dropout_p)
        pz = p * z
    o = pz @ v
    o_used = o if o_rows is None else np.asarray(o_rows, dtype=np.float64)
    dlt = np.sum(d_out_rows * o_used, axis=-1)
    dp = d_out_rows @ v.T
    if z is not None:
        dp = dp * z
    ds = p * (dp - dlt[:, None])
    ads = np.abs(ds)
    return dict(o=o, lse2=lse * LOG2E, delta=dlt, dq=scale * (ds @ k), dk_part=scale * (ds.T @ q_rows),
                dv_part=pz.T @ d_out_rows, a_o=pz @ np.abs(v), a_dq=scale * (ads @ np.abs(k)),
                a_dk_part=scale * (ads.T @ np.abs(q_rows)), a_dv_part=pz.T @ np.abs(d_out_rows))


def operand_abs_sums(q, k, v, d_out, mask=None, dropout_p=0.0, is_causal=False, scale=None, seed=0, offset=0, o=None):
    """Sum of |terms| of the contractions whose left operand a 16-bit matrix-core kernel must round
    (P for O and dV, dS for dQ and dK): A_O = |PZ| |V|, A_dV = |PZ|^T |dO|, A_dQ = |scale| |dS| |K|,
    A_dK = |scale| |dS|^T |Q|.  Rounding P or dS to a type with unit roundoff u perturbs each output by
    at most u * A, whatever the kernel; the parity tests add that bound to the stated atol."""
    q, k, v, d_out = [np.asarray(x, dtype=np.float64) for x in (q, k, v, d_out)]
    B, H, S, D = q.shape
    if scale is None:
        scale = 1.0 / math.sqrt(D)
    a_o, a_dq, a_dk, a_dv = [np.empty_like(q) for _ in range(4)]
    for b in range(B):
        for h in range(H):
            s = _scores(q[b, h], k[b, h], _mask_slice(mask, b, h), is_causal, scale)
            p, _ = _softmax_rows(s)
            z = _keep_scale(seed, offset, b * H + h, S, dropout_p)
            pz = p if z is None else p * z
            o_bh = pz @ v[b, h] if o is None else np.asarray(o[b, h], dtype=np.float64)
            dlt = np.sum(d_out[b, h] * o_bh, axis=-1)
            dp = d_out[b, h] @ v[b, h].T
            if z is not None:
                dp = dp * z
            ds = np.abs(p * (dp - dlt[:, None]))
            a_o[b, h] = pz @ np.abs(v[b, h])
            a_dv[b, h] = pz.T @ np.abs(d_out[b, h])
            a_dq[b, h] = abs(scale) * (ds @ np.abs(k[b, h]))
            a_dk[b, h] = abs(scale) * (ds.T @ np.abs(q[b, h]))
    return a_o, a_dq, a_dk, a_dv


def attention_bruteforce(q, k, v, mask=None, is_causal=False, scale=None, keep_scale=None):
    """Scalar-loop forward for tiny inputs (pins the vectorised path). keep_scale: optional
    [B,H,S,S] array of Z = keep/(1-p). Returns (O, lse_natural)."""
    B, H, S, D = q.shape
    if scale is None:
        scale = 1.0 / math.sqrt(D)
    out = np.zeros((B, H, S, D))
    lse = np.zeros((B, H, S))
    for b in range(B):
        for h in range(H):
            for i in range(S):
                sc = []
                for j in range(S):
                    if is_causal and j > i:
                        sc.append(-math.inf)
                        continue
                    acc = 0.0
                    for d in range(D):
                        acc += float(q[b, h, i, d]) * float(k[b, h, j, d])
                    acc *= scale
                    if mask is not None and not is_causal:
                        acc += float(mask[0 if mask.shape[0] == 1 else b, 0 if mask.shape[1] == 1 else h, i, j])
                    sc.append(acc)
                m = max(sc)
                e = [math.exp(x - m) if x != -math.inf else 0.0 for x in sc]
                l = sum(e)
                lse[b, h, i] = m + math.log(l)
                for j in range(S):
                    w = e[j] / l
                    if keep_scale is not None:
                        w *= float(keep_scale[b, h, i, j])
                    for d in range(D):
                        out[b, h, i, d] += w * float(v[b, h, j, d])
    return out, lse


def sdpa_cpu(q, k, v, mask=None, dropout_p=0.0, is_causal=False):
    """The oracle the reference's own tests use (tests/test_attention.py:31,38,60,78):
    torch.nn.functional.scaled_dot_product_attention on CPU tensors. Also the op timed as
    the CPU baseline."""
    import torch

    return torch.nn.functional.scaled_dot_product_attention(
        q, k, v, attn_mask=mask, dropout_p=dropout_p, is_causal=is_causal
    )
