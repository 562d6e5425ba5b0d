"""Shared helpers of the parity tests: oracle calls on torch tensors and the comparison rule."""
import numpy as np
import torch

from oracle import attention as oracle

# north_star tolerances: fp32 atol 1e-4; fp16/bf16 atol 1e-2 against an fp32/fp64 reference.
ATOL = {torch.float32: 1e-4, torch.float16: 1e-2, torch.bfloat16: 1e-2}
# A correctly rounded result in a 16-bit type is itself off by up to half an ulp of the output
# (2^-9 relative for bf16, 2^-12 for fp16), which exceeds 1e-2 once |x| > 4 in bf16. That
# storage rounding is added to the tolerance; the arithmetic error budget stays atol.
RTOL = {torch.float32: 1e-5, torch.float16: 2.0**-11, torch.bfloat16: 2.0**-8}
# Unit roundoff of the 16-bit operand (P or dS) a matrix-core kernel feeds to its second MFMA:
# each output moves by at most UNIT * sum|terms| because of it (oracle.operand_abs_sums). Added
# to the tolerance where a test passes `abs_sum`; it only matters for ill-conditioned sums
# (e.g. dV of the first keys under a causal mask, which add up hundreds of probabilities).
UNIT = {torch.float32: 0.0, torch.float16: 2.0**-11, torch.bfloat16: 2.0**-8}


def to64(t):
    return None if t is None else t.detach().cpu().to(torch.float64).numpy()


def close(actual: torch.Tensor, expected: np.ndarray, dtype, what="", abs_sum=None, stats=None):
    a = actual.detach().cpu().to(torch.float64).numpy()
    e = np.asarray(expected, dtype=np.float64)
    assert a.shape == e.shape, (what, a.shape, e.shape)
    both_nan = np.isnan(a) & np.isnan(e)
    err = np.abs(a - e)
    err[both_nan] = 0.0
    tol = ATOL[dtype] + RTOL[dtype] * np.abs(e)
    if abs_sum is not None:
        tol = tol + UNIT[dtype] * np.asarray(abs_sum, dtype=np.float64)
    tol = np.where(np.isfinite(tol), tol, np.inf)
    bad = ~(err <= tol)
    bad &= ~((a == e) & ~np.isnan(a))  # equal infinities
    if stats is not None:
        # how much of the tolerance beyond the plain atol was needed (quantifies the two documented additions)
        finite = np.isfinite(err)
        over = finite & (err > ATOL[dtype])
        stats.update(elements=int(a.size), over_atol=int(over.sum()), max_err=float(np.nanmax(err)) if err.size else 0.0,
                     max_over_atol=float((err[over] / ATOL[dtype]).max()) if over.any() else 0.0)
    if bad.any():
        idx = np.unravel_index(np.argmax(np.where(bad, err, 0)), a.shape)
        raise AssertionError(
            f"{what}: {bad.sum()} of {a.size} elements off; worst at {idx}: got {a[idx]!r}, want {e[idx]!r}, "
            f"max abs err {np.nanmax(err):.3e}"
        )
    return float(np.nanmax(err)) if err.size else 0.0


# The matrix-core forward kernels take the softmax denominator over the probabilities ROUNDED to the 16-bit
# operand type (the very values that multiply V, so O = sum(p~ v) / sum(p~) is self-consistent). Each term is
# off by at most half an ulp (2^-9 relative in bf16, 2^-12 in fp16), hence so is the sum, and lse2 = m + log2(l)
# by at most that times log2(e). fp32 inputs (and delta, a plain fp32 dot product) get no such allowance.
LSE_OPERAND = {None: 0.0, torch.float32: 0.0, torch.float16: 2.0**-12 * 1.4427 * 1.05, torch.bfloat16: 2.0**-9 * 1.4427 * 1.05}


def lse_delta_close(actual: torch.Tensor, expected: np.ndarray, what, operand_dtype=None):
    """fp32 statistics (LSE, delta): |err| <= 1e-4 * max(1, |x|) (+ LSE_OPERAND[operand_dtype] for the LSE of a
    16-bit problem); -inf must match exactly."""
    a = actual.detach().cpu().to(torch.float64).numpy()
    e = np.asarray(expected, dtype=np.float64)
    assert a.shape == e.shape, (what, a.shape, e.shape)
    same = (a == e) | (np.isnan(a) & np.isnan(e))
    with np.errstate(invalid="ignore"):
        ok = same | (np.abs(a - e) <= 1e-4 * np.maximum(1.0, np.abs(e)) + LSE_OPERAND[operand_dtype])
    assert ok.all(), f"{what}: {(~ok).sum()} of {a.size} off, worst {np.nanmax(np.where(ok, 0, np.abs(a - e))):.3e}"


def oracle_rows(q, k, v, d_o, b, h, row0, rows, H, mask=None, o=None, **kw):
    """oracle.attention_rows for head (b, h), query rows [row0, row0 + rows) of [B,H,S,D] torch tensors."""
    sl = slice(row0, row0 + rows)
    mrows = None
    if mask is not None:
        mrows = to64(mask[0 if mask.shape[0] == 1 else b, 0 if mask.shape[1] == 1 else h, sl])
    return oracle.attention_rows(to64(q[b, h, sl]), to64(k[b, h]), to64(v[b, h]), to64(d_o[b, h, sl]), row0, b * H + h,
                                 mask_rows=mrows, o_rows=None if o is None else to64(o[b, h, sl]), **kw)


def oracle_forward(q, k, v, mask=None, dropout_p=0.0, is_causal=False, scale=None, seed=0, offset=0):
    return oracle.attention_forward(to64(q), to64(k), to64(v), to64(mask), dropout_p, is_causal, scale, seed, offset)


def oracle_abs_sums(q, k, v, d_o, mask=None, dropout_p=0.0, is_causal=False, scale=None, seed=0, offset=0, o=None):
    return oracle.operand_abs_sums(to64(q), to64(k), to64(v), to64(d_o), to64(mask), dropout_p, is_causal, scale,
                                   seed, offset, o=to64(o))


def oracle_backward(q, k, v, d_o, mask=None, dropout_p=0.0, is_causal=False, scale=None, seed=0, offset=0,
                    want_dmask=False, o=None):
    """``o``: the forward output the backward under test was handed (already checked against the
    oracle's forward); delta is defined on that stored tensor."""
    return oracle.attention_backward(to64(q), to64(k), to64(v), to64(d_o), to64(mask), dropout_p, is_causal, scale,
                                     seed, offset, want_dmask, o=to64(o))
