"""Shared checks for the parity tests: the tolerance rules written once.

Centroids: |a - b| <= rtol * |b| + rtol * rms(b), rtol = 1e-4 (float32) or
1e-9 (float64).
Labels: must be equal except on rows whose two candidate centroids are a
near-tie (see label_report). The counts of excused rows are returned so every test
reports them.
"""
import numpy as np

CENTROID_RTOL = {np.dtype(np.float32): 1e-4, np.dtype(np.float64): 1e-9}
GAP_RTOL = 1e-5
NOISE_MULT = 8.0


def centroid_err(a, b):
    """Largest |a-b| / (|b| + rms(b))."""
    a = np.asarray(a, np.float64)
    b = np.asarray(b, np.float64)
    rms = np.sqrt(np.mean(b * b)) + 1e-300
    return float(np.max(np.abs(a - b) / (np.abs(b) + rms)))


def assert_centroids_close(a, b, dtype, what="centroids"):
    tol = CENTROID_RTOL[np.dtype(dtype)]
    err = centroid_err(a, b)
    assert err <= tol, "%s differ: scaled error %.3e > %.1e" % (what, err, tol)
    return err


def label_report(oracle, X, C, got, want, gap_rtol=GAP_RTOL, noise_mult=NOISE_MULT):
    """Compares two label vectors. A differing row is excused when its two candidate
    centroids are a near-tie in exact arithmetic (float64, direct form):
        |da - db| <= gap_rtol * max(da, db)                       (the stated 1e-5 bar)
     or |da - db| <= noise_mult * eps(dtype) * (|x|^2 + max|c|^2)  (rounding floor)
    The second clause is the rounding noise of the expanded form xx + cc - 2 x.c in the
    working precision: when |x|^2 + |c|^2 is much larger than the distance itself
    (well-separated data far from the origin) two correct float32 evaluations that sum
    in a different order already differ by that much, so no implementation can be held
    to less. It is 2e-15 relative for float64 and never matters there.
    Returns counts of both kinds; raises on any other mismatch."""
    got = np.asarray(got)
    want = np.asarray(want)
    assert got.shape == want.shape
    bad = np.nonzero(got != want)[0]
    rep = {"rows": int(got.size), "mismatch": int(bad.size), "excused": 0,
           "excused_by_gap": 0, "excused_by_noise_floor": 0, "worst_gap": 0.0,
           "worst_floor_mult": 0.0}
    if bad.size == 0:
        return rep
    assert (got[bad] >= 0).all() and (got[bad] < C.shape[0]).all(), "label out of range"
    assert (want[bad] >= 0).all()
    Xb = np.ascontiguousarray(X[bad])
    da, db = oracle.pair_dist_exact(Xb, C, got[bad], want[bad], threads=4)
    diff = np.abs(da - db)
    gap = diff / np.maximum(np.maximum(da, db), 1e-300)
    xx = (Xb.astype(np.float64) ** 2).sum(1)
    C64 = C.astype(np.float64)
    cc = np.maximum((C64[got[bad]] ** 2).sum(1), (C64[want[bad]] ** 2).sum(1))
    floor = noise_mult * float(np.finfo(X.dtype).eps) * (xx + cc)
    by_gap = gap <= gap_rtol
    by_floor = ~by_gap & (diff <= floor)
    rep["worst_gap"] = float(gap.max())
    # largest |da - db| of a mismatch in units of eps * (|x|^2 + |c|^2): how much of the
    # noise-floor allowance (noise_mult of these units) is actually used
    rep["worst_floor_mult"] = float((diff / (floor / noise_mult)).max())
    rep["excused_by_gap"] = int(by_gap.sum())
    rep["excused_by_noise_floor"] = int(by_floor.sum())
    rep["excused"] = rep["excused_by_gap"] + rep["excused_by_noise_floor"]
    real = bad[~(by_gap | by_floor)]
    assert real.size == 0, (
        "%d of %d label mismatches are not near-ties (worst relative gap %.3e), first rows %s"
        % (real.size, bad.size, gap[~(by_gap | by_floor)].max(), real[:5]))
    return rep


def record(entry):
    """Appends one JSON line to the file named by the environment variable
    H2O4GPU_PARITY_REPORT (the per-configuration parity table is assembled from these);
    without the variable nothing is written. Never fails a test."""
    import json
    import os
    path = os.environ.get("H2O4GPU_PARITY_REPORT")
    if not path:
        return
    try:
        os.makedirs(os.path.dirname(os.path.abspath(path)), exist_ok=True)
        with open(path, "a") as f:
            f.write(json.dumps(entry) + "\n")
    except OSError:
        pass
