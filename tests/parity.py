"""Float parity check shared by the GPU tests: the tolerance of the task statement, per element,
with nothing scaled by the tensor's largest value.

    |hip - reference| <= 1e-5 + 1e-4 * |reference|        for every element,

where `reference` is the fp32 CPU oracle (the restatement of the reference's fp32 path).  When the
double-precision build of the same oracle is given as well, both fp32 results are also measured
against it, which says how much of the difference is the oracle's own rounding.  Every check
leaves a line in the session's parity report (printed by conftest.py at the end of the run), so
the observed errors are part of the test output and not only their pass/fail.
"""
import numpy as np

RTOL, ATOL = 1e-4, 1e-5
REPORT = []


def _worst(err, ref):
    tol = ATOL + RTOL * np.abs(ref)
    return float(err.max()), float((err / tol).max())


def check(what, got, ref32, ref64=None, enforce=True):
    """enforce=False only records the observed errors (for comparisons whose bound is stated and
    asserted by the caller)."""
    got = np.asarray(got)
    ref32 = np.asarray(ref32)
    assert got.shape == ref32.shape, "%s: shape %s vs %s" % (what, got.shape, ref32.shape)
    err = np.abs(got.astype(np.float64) - ref32.astype(np.float64))
    e_abs, e_tol = _worst(err, ref32)
    rel = float((err / np.maximum(np.abs(ref32), 1e-3)).max())
    line = "%s: %d values, max|ref| %.3g; hip vs fp32 oracle: max abs %.3e, max rel (|ref|>=1e-3) %.3e, worst err/tol %.3f" % (
        what, got.size, float(np.abs(ref32).max()), e_abs, rel, e_tol)
    if ref64 is not None:
        ref64 = np.asarray(ref64, np.float64)
        h_abs, h_tol = _worst(np.abs(got - ref64), ref64)
        o_abs, o_tol = _worst(np.abs(ref32 - ref64), ref64)
        line += "; vs f64 oracle: hip max abs %.3e (err/tol %.3f), fp32 oracle max abs %.3e (err/tol %.3f)" % (
            h_abs, h_tol, o_abs, o_tol)
    REPORT.append(line)
    print(line)
    if enforce:
        assert e_tol <= 1.0, line
        if ref64 is not None:
            assert h_tol <= 1.0, line
    return e_abs, e_tol
