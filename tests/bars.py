"""Floating-point parity bars shared by the GPU tests.

The hot path's stated tolerance is 1e-4 relative / 1e-5 absolute.  For a contraction of many signed
terms no f32 algorithm -- the reference's BLAS included -- meets that literally next to a
cancellation, so contractions are held to three bars that an f32 implementation CAN meet and a
wrong one cannot:

  1. |got - truth64| <= 2e-6 * (|A|.|B|) element-wise, where |A|.|B| is the same contraction of
     absolute values: about 32 units in the last place of the quantity that rounding errors scale
     with.  A dropped, doubled or misplaced term is an error of order 1/K of |A|.|B|, far above it.
  2. where the f32 oracle (the reference's algorithm, OpenBLAS when it is loaded) ran on the same
     inputs: |got - truth64| <= 2 * max|oracle32 - truth64| -- the GPU is not less accurate than
     the reference's own arithmetic by more than a factor of two -- except for elements whose
     error is below 8 units of f32 roundoff (8 * 2^-24) of |A|.|B|: that close to exact, which of
     two correctly rounded algorithms came out ahead on one instance says nothing (the reference
     sums a 3x3 input gradient as nine 32-term chains, the implicit GEMM as one 288-term chain cut
     at 256);
  3. at least 99 % of the elements meet the literal bound |got - oracle32| <= 1e-5 + 1e-4*|oracle32|.
"""
import sys

import numpy as np

RTOL, ATOL = 1e-4, 1e-5
CONTRACTION_BOUND = 2e-6      # bar 1
ORACLE_ERROR_FACTOR = 2.0     # bar 2
ROUNDOFF_FLOOR = 8 * 2.0 ** -24  # bar 2 does not apply below this fraction of |A|.|B|
LITERAL_FRACTION = 0.99       # bar 3


def say(*a):
    print("[case]", *a, flush=True)
    sys.stdout.flush()


def assert_close(got, ref, what=""):
    """The literal bound, element-wise."""
    got, ref = np.asarray(got, dtype=np.float64), np.asarray(ref, dtype=np.float64)
    assert got.shape == ref.shape, f"{what}: shape {got.shape} vs {ref.shape}"
    err = np.abs(got - ref)
    tol = ATOL + RTOL * np.abs(ref)
    bad = err > tol
    assert not bad.any(), (f"{what}: {bad.sum()} of {bad.size} elements outside 1e-5 + 1e-4|ref|; "
                           f"worst err {err.max():.3e} (ref {ref.reshape(-1)[err.argmax()]:.3e})")


def assert_contraction(got, truth, absdot, what="", ref32=None, bound=CONTRACTION_BOUND):
    got, truth, absdot = (np.asarray(a, dtype=np.float64) for a in (got, truth, absdot))
    assert got.shape == truth.shape == absdot.shape, f"{what}: shapes {got.shape} {truth.shape} {absdot.shape}"
    assert np.isfinite(got).all(), f"{what}: non-finite values"
    err = np.abs(got - truth)
    # bar 1 (an element whose terms are all zero must be exactly zero)
    tol = bound * absdot
    bad = err > tol
    worst = float((err / np.maximum(absdot, 1e-300)).max()) if err.size else 0.0
    msg = f"{what}: max err/(|A|.|B|) = {worst:.2e}"
    if ref32 is not None:
        ref32 = np.asarray(ref32, dtype=np.float64)
        ref_err = np.abs(ref32 - truth)
        lit = np.abs(got - ref32) <= ATOL + RTOL * np.abs(ref32)
        msg += (f"; max err {err.max():.3e} vs oracle32's {ref_err.max():.3e}; "
                f"{100.0 * lit.mean():.3f} % within 1e-5 + 1e-4|ref32|")
    say(msg)
    assert not bad.any(), f"{what}: {bad.sum()} of {bad.size} outside {bound:g}*(|A|.|B|); worst ratio {worst:.3e}"
    if ref32 is not None and err.size:
        worse = (err > ORACLE_ERROR_FACTOR * ref_err.max()) & (err > ROUNDOFF_FLOOR * absdot)
        assert not worse.any(), (f"{what}: {worse.sum()} elements with an error above {ORACLE_ERROR_FACTOR} x the f32 "
                                 f"oracle's {ref_err.max():.3e} (worst {err[worse].max():.3e})")
        assert lit.mean() >= LITERAL_FRACTION, \
            f"{what}: only {100.0 * lit.mean():.2f} % of the elements within 1e-5 + 1e-4|ref32|"
