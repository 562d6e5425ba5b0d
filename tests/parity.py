"""Shared helpers of the parity tests: oracle calls on torch tensors and the comparison rule."""
import os

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


# Every comparison leaves a record here: how far beyond the plain atol the two documented additions (storage rounding
# of a 16-bit result, rounding of the 16-bit MFMA operand) had to stretch. tests/conftest.py writes the summary of a
# GPU session to parity_margins.txt in the session's output folder, and `close` itself bounds both: of a 16-bit comparison at most
# OVER_ATOL_FRACTION of the elements may lie above the plain atol, and none further than OVER_ATOL_FACTOR times
# it (fp32 comparisons: none at all above 1e-4 + 1e-5 |x|, which the rule already says). The bounds sit just above
# what a recorded session shows (profiles/parity_margins.txt: of 342 million bf16 elements six lie above the plain
# atol, the worst at 1.18 times it; worst fraction of one comparison 2.3e-5, in dV under dropout), so a defect of a few
# 1e-2 on an ill-conditioned sum no longer hides behind the operand allowance.
MARGINS = []
OVER_ATOL_FRACTION = 1e-4
OVER_ATOL_FACTOR = 2.0


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
    # how much of the tolerance beyond the plain atol was needed (quantifies the two documented additions); the
    # storage rounding of the expected value itself (half an ulp of a 16-bit result) is not counted as excess
    finite = np.isfinite(err)
    excess = np.where(finite, err - RTOL[dtype] * np.abs(np.where(np.isfinite(e), e, 0.0)), 0.0)
    over = finite & (excess > ATOL[dtype])
    record = dict(what=what, dtype=str(dtype).replace("torch.", ""), elements=int(a.size), over_atol=int(over.sum()),
                  max_err=float(np.nanmax(err[finite])) if finite.any() else 0.0,
                  max_over_atol=float((excess[over] / ATOL[dtype]).max()) if over.any() else 0.0)
    MARGINS.append(record)
    if stats is not None:
        stats.update(record)
    if bad.any():
        idx = np.unravel_index(np.argmax(np.where(bad, err, 0)), a.shape)
        raise AssertionError(
            f"{what}: {bad.sum()} of {a.size} elements off; worst at {idx}: got {a[idx]!r}, want {e[idx]!r}, "
            f"max abs err {np.nanmax(err):.3e}"
        )
    if os.environ.get("TRI_PARITY_RECORD_ONLY"):  # (a session that only gathers the margins)
        return float(np.nanmax(err)) if err.size else 0.0
    if a.size >= 4096:  # (a fraction means little on a handful of elements)
        assert record["over_atol"] <= OVER_ATOL_FRACTION * a.size, \
            f"{what}: {record['over_atol']} of {a.size} elements needed more than the plain atol {ATOL[dtype]}"
    assert record["max_over_atol"] <= OVER_ATOL_FACTOR, \
        f"{what}: an element is {record['max_over_atol']:.2f} x the plain atol {ATOL[dtype]} off (after its storage rounding)"
    return float(np.nanmax(err)) if err.size else 0.0


def margins_summary():
    """Text summary of MARGINS: per dtype the totals and the worst comparisons."""
    lines = ["# comparisons against the fp64 oracle in this session: elements whose error exceeded the plain atol",
             "# (fp32 1e-4, fp16 / bf16 1e-2) after the storage rounding of a 16-bit result was taken off",
             f"# bounds enforced by tests/parity.py: fraction <= {OVER_ATOL_FRACTION:g} per comparison of >= 4096 elements, "
             f"worst element <= {OVER_ATOL_FACTOR:g} x atol"]
    for dt in ("float32", "float16", "bfloat16"):
        rows = [r for r in MARGINS if r["dtype"] == dt]
        if not rows:
            continue
        n = sum(r["elements"] for r in rows)
        over = sum(r["over_atol"] for r in rows)
        lines.append(f"{dt}: {len(rows)} comparisons, {n} elements, {over} above the plain atol ({over / max(n, 1):.2e}); "
                     f"worst element {max(r['max_over_atol'] for r in rows):.2f} x atol; largest error {max(r['max_err'] for r in rows):.3e}")
        worst = sorted(rows, key=lambda r: (-r["over_atol"] / max(r["elements"], 1), -r["max_over_atol"]))[:8]
        for r in worst:
            if r["over_atol"]:
                lines.append(f"    {r['what'] or '(unnamed)'}: {r['over_atol']} of {r['elements']} ({r['over_atol'] / r['elements']:.2e}), "
                             f"worst {r['max_over_atol']:.2f} x atol, max err {r['max_err']:.3e}")
    return "\n".join(lines) + "\n"


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
