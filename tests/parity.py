"""Error metric and pass/fail gates shared by the parity tests.

`rel_err(a, b)` is the largest element-wise error of `a` against `b`, each
element's error divided by max(|b_i|, rms(b)): a plain element-wise relative
error is meaningless where the expected value crosses zero, a plain absolute
one hides errors in small tensors.

`check(...)` applies the gate used everywhere: the candidate must agree with the
fp32 reference restatement within `tol`; where the fp32 reference is itself
further than `tol` from the float64 evaluation of the same algorithm (long
sequential fp32 sums, E[x^2]-mean^2 cancellation), a candidate is also accepted
when it is at least as close to the float64 answer as the reference is.
"""
import numpy as np

TOL_F32 = 1e-5   # fp32 storage and arithmetic
TOL_F16 = 2e-3   # fp16 storage, fp32 accumulation
TOL_F64 = 1e-10  # binary64 storage and arithmetic, against the float64 evaluation of the reference code


def rel_err(a, b):
    a = np.asarray(a, dtype=np.float64)
    b = np.asarray(b, dtype=np.float64)
    assert a.shape == b.shape, (a.shape, b.shape)
    if a.size == 0:
        return 0.0
    bad = ~np.isfinite(a) | ~np.isfinite(b)
    if bad.any():
        # non-finite entries must match exactly (same NaN positions, same infinities)
        same = (np.isnan(a) & np.isnan(b)) | (a == b)
        if not same[bad].all():
            return float("inf")
        a = np.where(bad, 0.0, a)
        b = np.where(bad, 0.0, b)
    rms = float(np.sqrt(np.mean(b * b)))
    denom = np.maximum(np.abs(b), rms)
    denom = np.where(denom == 0.0, 1.0, denom)
    return float(np.max(np.abs(a - b) / denom))


# Every check() of the process, in call order: what the parity report is written from
# (tests/conftest.py writes it when the GPU tests end; tests/parity_report.py formats it).
REPORT = []


def check(name, got, ref32, exact64=None, tol=TOL_F32, slack=1.0, strict=False):
    """Returns the dict of measured errors; raises AssertionError when the gate fails.

    strict: only the fp32-reference leg counts (the float64 distances are still recorded).

    The dict names the leg that passed: "fp32 reference" (within `tol` of the restated
    reference) or "float64" (at least as close to the float64 evaluation as the fp32
    reference is).  With `exact64` given, all three distances are measured and recorded
    whichever leg passes."""
    e_ref = rel_err(got, ref32)
    out = {"name": name, "tol": tol, "vs_ref": e_ref, "leg": "fp32 reference" if e_ref <= tol else None}
    if exact64 is not None:
        out["vs_exact"] = rel_err(got, exact64)
        out["ref_vs_exact"] = rel_err(ref32, exact64)
    REPORT.append(out)
    if e_ref <= tol:
        return out
    assert exact64 is not None and not strict, f"{name}: err vs fp32 reference {e_ref:.3e} > {tol:.1e}"
    e_exact, e_ref_exact = out["vs_exact"], out["ref_vs_exact"]
    assert e_exact <= max(tol, slack * e_ref_exact), (
        f"{name}: err vs fp32 reference {e_ref:.3e} > {tol:.1e} and err vs float64 "
        f"{e_exact:.3e} > reference's own {e_ref_exact:.3e}")
    out["leg"] = "float64"
    return out


def record(name, got, ref32, exact64=None, tol=TOL_F32):
    """Measures and records like check() but never fails: for comparisons that are reported
    for information (a different summation formula, say) and gated elsewhere."""
    out = {"name": name, "tol": tol, "vs_ref": rel_err(got, ref32), "leg": "informational"}
    if exact64 is not None:
        out["vs_exact"] = rel_err(got, exact64)
        out["ref_vs_exact"] = rel_err(ref32, exact64)
    REPORT.append(out)
    return out
