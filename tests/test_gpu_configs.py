"""The five benchmark shapes on the GPU.

Scaled-down rows (same d and k) are checked against the CPU oracle in lock-step and
end-to-end; the full shapes are checked through size-independent properties plus an
oracle check on a random sample of rows, so the CPU side stays within seconds.
"""
import numpy as np
import pytest

from h2o4gpu_amd import datasets
from parity import assert_centroids_close, centroid_err, label_report

pytestmark = pytest.mark.gpu

# name, dtype, row scale for the oracle comparison, iterations compared
SCALED = [
    ("C1", np.float32, 1.0, 20),
    ("C2", np.float32, 0.1, 50),
    ("C3", np.float32, 0.02, 30),
    ("C4", np.float32, 0.01, 20),
    ("C4", np.float64, 0.005, 10),
    ("C5", np.float32, 0.02, 5),
]


def _start(name, X, k, hip_handle=None):
    seed = datasets.SHAPES[name][3]
    if name == "C4":
        # benchmark text: k-means++ from a fixed seed, computed once by the engine's own
        # seeding code and fed identically to both sides
        hip_handle.init_plusplus(seed)
        return hip_handle.centroids()
    return datasets.seeded_row_init(X, k, seed)


@pytest.mark.parametrize("name,dtype,scale,iters", SCALED)
def test_scaled_shape_lockstep_and_end_to_end(hip, oracle, name, dtype, scale, iters):
    X, k, _ = datasets.make(name, scale, dtype)
    n, d = X.shape
    tol = 1e-5 if dtype == np.float32 else 1e-12
    with hip.Handle(n, d, k, dtype) as h:
        h.set_data(X)
        C0 = _start(name, X, k, h)
        variant = h.assign_variant()
        # lock-step: both sides start every iteration from the oracle's centroids
        C = C0.copy()
        excused = mism = 0
        for it in range(min(iters, 6)):
            h.set_centroids(C)
            h.iterate(1)
            labels = h.labels()
            rep = label_report(oracle, X, C, labels, oracle.assign(X, C, threads=8))
            excused += rep["excused"]
            mism += rep["mismatch"]
            wC, wcounts = oracle.update(X, labels, C)
            assert np.array_equal(h.counts(), wcounts)
            assert np.allclose(h.centroids(), wC, rtol=tol, atol=tol * np.abs(wC).max())
            C = wC
        # end to end, fixed iteration count, tol = 0
        h.set_centroids(C0)
        done = h.fit(iters, 0.0)
        Cg, Lg = h.centroids(), h.labels()
        inertia = h.inertia()
    assert done == iters
    wC, wL, _, _ = oracle.lloyd(X, C0, iters, 0.0, threads=8)
    err = centroid_err(Cg, wC)
    rep = label_report(oracle, X, wC, Lg, wL, gap_rtol=1.0)   # report only, see below
    w_inertia = float(oracle.assign(X, wC, threads=8, return_mindist=True)[1].astype(np.float64).sum())
    print("%s %s n=%d d=%d k=%d [%s]: lockstep mismatches %d (all excused near-ties: %d); "
          "end-to-end centroid error %.2e, label mismatches %d, inertia rel diff %.2e"
          % (name, np.dtype(dtype).name, n, d, k, variant, mism, excused, err, rep["mismatch"],
             abs(inertia - w_inertia) / w_inertia))
    # A near-tie row that flips moves its two centroids by |x-c|/cluster_size; with the
    # scaled-down rows (clusters of a few hundred points) that can exceed 1e-4 although
    # both runs are valid Lloyd trajectories, so the end-to-end bar is applied when no
    # label flipped, and the objective must agree closely in every case.
    if mism == 0 and rep["mismatch"] == 0:
        assert_centroids_close(Cg, wC, dtype)
    assert abs(inertia - w_inertia) <= 1e-4 * w_inertia


def _full_shape_checks(hip, oracle, name, dtype, iters, extra=None):
    X, k, _ = datasets.make(name, 1.0, dtype)
    n, d = X.shape
    rng = np.random.default_rng(99)
    with hip.Handle(n, d, k, dtype) as h:
        h.set_data(X)
        C0 = _start(name, X, k, h)
        h.set_centroids(C0)
        # monotone objective over the first iterations
        prev = None
        for _ in range(3):
            h.assign()
            cur = h.inertia()
            if prev is not None:
                assert cur <= prev * (1 + 1e-6), "objective went up: %r -> %r" % (prev, cur)
            prev = cur
            h.update(want_shift=False)
        h.set_centroids(C0)
        done = h.fit(iters, 0.0)
        assert done == iters
        C, L, counts = h.centroids(), h.labels(), h.counts()
        # final relabel used the final centroids: predicting the same rows gives the labels
        sub = np.sort(rng.choice(n, size=min(n, 20000), replace=False))
        assert np.array_equal(h.predict(X[sub]), L[sub])
        # oracle on a sample of rows (exact up to near-ties)
        rep = label_report(oracle, X[sub], C, L[sub], oracle.assign(X[sub], C, threads=8))
        if extra:
            extra(h, X, C, L)
    assert L.min() >= 0 and L.max() < k
    # the last update's counts describe the labelling before the final relabel; they sum to n
    assert int(counts.sum()) == n
    # centroids are means of their rows: check a handful of clusters directly
    final_counts = np.bincount(L, minlength=k)
    tol = 5e-4 if dtype == np.float32 else 1e-8
    h2 = None
    for c in rng.choice(k, size=4, replace=False):
        rows = np.nonzero(L == c)[0]
        if rows.size == 0:
            continue
        mean = X[rows].astype(np.float64).mean(0)
        # C is the mean under the previous labelling; after `iters` iterations on blob data
        # the two differ by at most the last shift, checked loosely
        scale = np.abs(mean).max() + np.sqrt(np.mean(C.astype(np.float64) ** 2))
        assert np.max(np.abs(C[c] - mean)) <= 0.05 * scale
    print("%s %s full shape: n=%d d=%d k=%d, sample label check %s, empty clusters %d"
          % (name, np.dtype(dtype).name, n, d, k, rep, int((final_counts == 0).sum())))


def test_full_shape_c3_headline(hip, oracle):
    _full_shape_checks(hip, oracle, "C3", np.float32, 30)


def test_full_shape_c3_end_to_end_against_oracle(hip, oracle):
    """The headline shape, all 10M rows, fixed iterations on both sides.

    A random-row start splits some blobs between two centroids; rows on such a boundary
    are near-ties at the rounding level of the float32 expanded form, and a flipped row
    moves the boundary a little in the next iteration. How far two CORRECT float32
    evaluations drift apart after a fixed number of iterations is measured here with the
    oracle itself (features summed ascending vs descending); the engine must stay within
    the same order of magnitude of the oracle and agree on the objective."""
    X, k, _ = datasets.make("C3", 1.0, np.float32)
    n, d = X.shape
    iters = 12
    C0 = datasets.seeded_row_init(X, k, datasets.SHAPES["C3"][3])
    with hip.Handle(n, d, k, np.float32) as h:
        h.set_data(X)
        h.set_centroids(C0)
        assert h.fit(iters, 0.0) == iters
        Cg, Lg = h.centroids(), h.labels()
        inertia = h.inertia()
    wC, wL, _, _ = oracle.lloyd(X, C0, iters, 0.0, threads=16)
    oracle.set_dot_order(True)
    try:
        rC, rL, _, _ = oracle.lloyd(X, C0, iters, 0.0, threads=16)
    finally:
        oracle.set_dot_order(False)
    err = centroid_err(Cg, wC)
    self_err = centroid_err(rC, wC)
    w_inertia = float(oracle.assign(X, wC, threads=16, return_mindist=True)[1].astype(np.float64).sum())
    print("C3 full, %d iterations: engine vs oracle centroid error %.2e (label diffs %d); "
          "oracle ascending vs descending order %.2e (label diffs %d); inertia rel diff %.2e"
          % (iters, err, int((Lg != wL).sum()), self_err, int((rL != wL).sum()),
             abs(inertia - w_inertia) / w_inertia))
    assert err <= max(1e-4, 4 * self_err)
    assert abs(inertia - w_inertia) <= 1e-5 * w_inertia


def test_full_shape_c2_with_predict(hip, oracle):
    _full_shape_checks(hip, oracle, "C2", np.float32, 50)


def test_full_shape_c4_float32(hip, oracle):
    _full_shape_checks(hip, oracle, "C4", np.float32, 20)


def test_full_shape_c4_float64(hip, oracle):
    _full_shape_checks(hip, oracle, "C4", np.float64, 20)


def test_full_shape_c5_with_transform(hip, oracle):
    def transform_check(h, X, C, L):
        H = datasets.make_holdout("C5", 100_000)
        D = h.transform(H)                      # [k][rows], squared distances
        assert D.shape == (C.shape[0], H.shape[0])
        rng = np.random.default_rng(5)
        rows = rng.choice(H.shape[0], size=64, replace=False)
        cols = rng.choice(C.shape[0], size=64, replace=False)
        want = ((H[rows][:, None, :].astype(np.float64) - C[cols][None, :, :].astype(np.float64)) ** 2).sum(-1)
        got = D[np.ix_(cols, rows)].T.astype(np.float64)
        scale = (H[rows].astype(np.float64) ** 2).sum(1).max() * 2
        assert np.max(np.abs(got - want)) <= 64 * np.finfo(np.float32).eps * scale
        # labels of the held-out rows = column argmin of the transform (up to near-ties)
        pl = h.predict(H[:5000])
        am = np.argmin(D[:, :5000], axis=0)
        bad = np.nonzero(pl != am)[0]
        for i in bad:
            a, b = D[pl[i], i], D[am[i], i]
            assert abs(a - b) <= 1e-5 * max(a, b)
    _full_shape_checks(hip, oracle, "C5", np.float32, 15, extra=transform_check)
