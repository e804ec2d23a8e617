"""Stacked restarts: several centroid sets of one fit as one model through the fused
row-stationary kernel, per-set argmin and per-set sums, against the same restarts run one
after another on ordinary handles (through the C ABI)."""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu


def blobs(n, d, k, dtype, seed):
    rng = np.random.default_rng(seed)
    centres = rng.uniform(-8, 8, size=(k, d))
    return np.ascontiguousarray((centres[rng.integers(0, k, size=n)] +
                                 1.5 * rng.standard_normal((n, d))).astype(dtype))


def serial_fit(hip, X, k, C0, iters, tol):
    n, d = X.shape
    with hip.Handle(n, d, k, X.dtype) as h:
        h.set_data(X)
        h.set_option("assign", "mfma_rowstat")  # the kernel family a stacked handle runs
        h.set_centroids(C0)
        it = h.fit(iters, tol)
        return h.centroids(), h.labels(), h.counts(), h.inertia(), it


SHAPES = [(50000, 32, 20, 3), (40000, 64, 64, 2), (60000, 16, 8, 4), (30000, 24, 33, 2), (20000, 8, 5, 6),
          (25000, 7, 9, 3), (20000, 3, 4, 2), (15000, 101, 12, 2), (1000, 30, 70, 2), (37, 5, 3, 2)]


@pytest.mark.parametrize("dtype", [np.float32, np.float64])
@pytest.mark.parametrize("n,d,k,sets", SHAPES)
def test_stacked_sets_equal_serial_restarts(hip, n, d, k, sets, dtype):
    X = blobs(n, d, k, dtype, seed=n + d)
    if hip.stack_width(n, d, k, dtype, sets) < sets:
        pytest.skip("shape does not hold %d sets" % sets)
    rng = np.random.default_rng(7)
    starts = [np.ascontiguousarray(X[rng.choice(n, size=k, replace=False)]) for _ in range(sets)]
    iters = 7
    with hip.Handle(n, d, k, dtype, sets=sets) as h:
        h.set_data(X)
        h.set_option("assign", "mfma_rowstat")  # (the final relabel runs ordinary kernels: these)
        for s in range(sets):
            h.select_set(s)
            h.set_centroids(starts[s])
        assert h.fit(iters, 0.0) == iters
        got = []
        for s in range(sets):
            h.select_set(s)
            got.append((h.centroids(), h.labels(), h.counts(), h.inertia()))
        assert h.set_iterations().tolist() == [iters] * sets
    for s in range(sets):
        C, L, cnt, inertia, _ = serial_fit(hip, X, k, starts[s], iters, 0.0)
        gC, gL, gcnt, ginertia = got[s]
        assert np.array_equal(gL, L), "set %d: %d labels differ" % (s, int((gL != L).sum()))
        assert np.array_equal(gcnt, cnt)
        if dtype == np.float32:
            # float32 rows add up exactly in the double-precision sums: bit for bit
            assert np.array_equal(gC, C)
            assert ginertia == inertia
        else:
            assert np.allclose(gC, C, rtol=1e-12, atol=1e-12)
            assert abs(ginertia - inertia) <= 1e-12 * inertia


def test_every_set_stops_at_its_own_iteration(hip):
    """With a threshold a set stops after the update whose squared shift is below it and keeps
    its centroids while the others go on (kmeans_impl.h:189-232, per set)."""
    n, d, k, sets = 40000, 32, 12, 3
    X = blobs(n, d, k, np.float32, seed=3)
    rng = np.random.default_rng(11)
    # one start at the true optimum's doorstep (converges at once), two poor ones
    good = serial_fit(hip, X, k, np.ascontiguousarray(X[rng.choice(n, size=k, replace=False)]), 40, 0.0)[0]
    starts = [good, np.ascontiguousarray(X[:k]), np.ascontiguousarray(X[rng.choice(n, size=k, replace=False)])]
    tol = 1e-3
    want = [serial_fit(hip, X, k, c0, 60, tol) for c0 in starts]
    with hip.Handle(n, d, k, np.float32, sets=sets) as h:
        h.set_data(X)
        h.set_option("assign", "mfma_rowstat")
        for s in range(sets):
            h.select_set(s)
            h.set_centroids(starts[s])
        h.fit(60, tol)
        its = h.set_iterations().tolist()
        assert its == [w[4] for w in want], (its, [w[4] for w in want])
        assert len(set(its)) > 1, "the starts were meant to converge at different iterations"
        for s in range(sets):
            h.select_set(s)
            assert np.array_equal(h.centroids(), want[s][0])
            assert np.array_equal(h.labels(), want[s][1])
            assert h.inertia() == want[s][3]


def test_per_set_seeding_and_limits(hip):
    n, d, k = 20000, 16, 10
    X = blobs(n, d, k, np.float32, seed=5)
    width = hip.stack_width(n, d, k, np.float32, 4096)  # as many as one CU's LDS holds
    assert 2 <= width < 4096
    assert hip.stack_width(500000, 784, 4096, np.float32, 4) == 1   # far beyond one CU's LDS
    with pytest.raises(hip.KMeansHipError):
        hip.Handle(n, d, k, np.float32, sets=width + 1)
    with hip.Handle(n, d, k, np.float32) as single, hip.Handle(n, d, k, np.float32, sets=2) as h:
        single.set_data(X)
        h.set_data(X)
        for s, (init, seed) in enumerate([("init_random_rows", 4), ("init_parallel", 9)]):
            getattr(single, init)(seed)
            h.select_set(s)
            getattr(h, init)(seed)
            assert np.array_equal(h.seed_rows(), single.seed_rows())
            assert np.array_equal(h.centroids(), single.centroids())
        h.select_set(0)
        h.init_plusplus(3)
        single.init_plusplus(3)
        assert np.array_equal(h.centroids(), single.centroids())
        with pytest.raises(hip.KMeansHipError):
            h.predict(X[:10])
        with pytest.raises(hip.KMeansHipError):
            h.select_set(2)


def test_estimator_restarts_keep_the_best(hip):
    import h2o4gpu_amd
    n, d, k = 30000, 32, 16
    X = blobs(n, d, k, np.float32, seed=8)
    data = X
    best = h2o4gpu_amd.KMeans(n_clusters=k, init="random", n_init=5, max_iter=15, tol=0, random_state=20).fit(data)
    singles = [h2o4gpu_amd.KMeans(n_clusters=k, init="random", n_init=1, max_iter=15, tol=0,
                                  random_state=20 + r).fit(data) for r in range(5)]
    inertias = [m.inertia_ for m in singles]
    assert abs(best.inertia_ - min(inertias)) <= 1e-6 * min(inertias)
    assert best.cluster_centers_.shape == (k, d) and best.labels_.shape == (n,)
    assert best.n_iter_ == 15


@pytest.mark.parametrize("dtype", [np.float32, np.float64])
@pytest.mark.parametrize("n,d,k,sets", [(60000, 16, 8, 4), (30000, 40, 12, 3), (20000, 5, 16, 5)])
def test_small_shapes_stacked_restarts_against_the_default_single_fit(hip, oracle, n, d, k, sets, dtype):
    """For k <= 16 and d <= 64 a single fit runs the scalar-order kernels (bit-identical to the
    oracle) while stacked restarts always run the matrix-core kernel with its own summation order
    (and 16-ulp keys in float32): restart r of an n_init fit is then the single fit from the same
    start only up to near-tie rows. Checked here by the usual bars, per iteration in lock-step
    (same centroids in: labels equal except near-ties, the update of the set's own labels equal
    to the oracle's) and end to end on the objective."""
    from parity import label_report
    X = blobs(n, d, k, dtype, seed=n + d + k)
    assert hip.stack_width(n, d, k, dtype, sets) >= sets
    rng = np.random.default_rng(17)
    starts = [np.ascontiguousarray(X[rng.choice(n, size=k, replace=False)]) for _ in range(sets)]
    tol = 1e-5 if dtype == np.float32 else 1e-12
    with hip.Handle(n, d, k, dtype, sets=sets) as h:
        h.set_data(X)
        for s in range(sets):
            h.select_set(s)
            h.set_centroids(starts[s])
        h.iterate(1)
        flips = 0
        for s in range(sets):
            h.select_set(s)
            L, C1 = h.labels(), h.centroids()
            wL = oracle.assign(X, starts[s], threads=4)
            flips += label_report(oracle, X, starts[s], L, wL)["mismatch"]
            wC, _ = oracle.update(X, L, starts[s], threads=4)
            assert np.allclose(C1, wC, rtol=tol, atol=tol * np.abs(wC).max())
        for s in range(sets):
            h.select_set(s)
            h.set_centroids(starts[s])
        assert h.fit(25, 0.0) == 25
        stacked = []
        for s in range(sets):
            h.select_set(s)
            stacked.append((h.centroids(), h.labels(), h.inertia()))
    for s in range(sets):
        with hip.Handle(n, d, k, dtype) as h1:
            h1.set_data(X)
            assert h1.assign_variant() == "valu"
            h1.set_centroids(starts[s])
            assert h1.fit(25, 0.0) == 25
            C, L, inertia = h1.centroids(), h1.labels(), h1.inertia()
        sC, sL, sinertia = stacked[s]
        # labels_ of a stacked set come from an ordinary relabel (the default family) against
        # the set's own centroids
        assert np.array_equal(sL, oracle.assign(X, sC, threads=4))
        assert abs(sinertia - inertia) <= 1e-5 * inertia
        if flips == 0 and np.array_equal(sL, L):
            assert np.allclose(sC, C, rtol=1e-4 if dtype == np.float32 else 1e-9,
                               atol=(1e-4 if dtype == np.float32 else 1e-9) * np.abs(C).max())
