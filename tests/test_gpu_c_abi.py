"""The reference's four entry points exercised through the SWIG-convention module and the
estimator on the GPU: argument handling, edge cases, layouts."""
import numpy as np
import pytest

from parity import label_report

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def shim(hip):
    from h2o4gpu_amd.libs import ch2o4gpu_gpu
    return ch2o4gpu_gpu


def blobs(n, d, k, dtype, seed):
    rng = np.random.default_rng(seed)
    centers = rng.uniform(-20, 20, size=(k, d))
    return np.ascontiguousarray((centers[rng.integers(0, k, size=n)] + rng.standard_normal((n, d))).astype(dtype)), centers


def fit(shim, X, k, iters, init, seed=1, tol=0.0, C0=None):
    n, d = X.shape
    fn = shim.make_ptr_float_kmeans if X.dtype == np.float32 else shim.make_ptr_double_kmeans
    pc = np.zeros(k * d, X.dtype)
    pl = np.zeros(n, np.int32)
    cen = np.empty([]) if C0 is None else C0.flatten()
    rc = fn(0, 0, seed, 0, 1, n, d, k, iters, init, tol, X.flatten(), cen, pc, pl)
    return rc, pc.reshape(k, d), pl


@pytest.mark.parametrize("dtype", [np.float32, np.float64])
def test_random_row_start_follows_the_reference_rule(shim, oracle, dtype):
    """init_from_data = 0: centroids start at rows v[0..k-1] of std::shuffle(iota(n),
    std::default_random_engine(seed)); with zero iterations' worth of movement excluded,
    the whole run must equal the oracle started from those rows."""
    X, _ = blobs(3000, 8, 5, dtype, 1)
    k, iters, seed = 5, 4, 1234
    rc, C, L = fit(shim, X, k, iters, 0, seed=seed)
    assert rc == 0
    rows = oracle.random_rows(seed, X.shape[0], k)
    wC, wL, _, _ = oracle.lloyd(X, X[rows], iters, 0.0)
    tol = 1e-4 if dtype == np.float32 else 1e-9
    assert np.allclose(C, wC, rtol=tol, atol=tol)
    assert np.array_equal(L, wL)
    rc, C2, L2 = fit(shim, X, k, iters, 0, seed=seed)
    # deterministic per seed: bit-identical for float32 (the double-precision LDS sums of
    # float32 data are exact); float64 sums depend on wavefront arrival order in the last bit
    assert np.array_equal(L, L2)
    assert np.array_equal(C, C2) if dtype == np.float32 else np.allclose(C, C2, rtol=1e-13, atol=1e-13)
    rc, C3, _ = fit(shim, X, k, iters, 0, seed=seed + 1)
    assert not np.array_equal(C, C3)


def test_k_larger_than_rows_is_clamped(shim, capfd):
    X = np.array([[0.0, 0.0], [10.0, 0.0], [0.0, 10.0]], np.float32)
    rc, C, L = fit(shim, X, 5, 3, 0, seed=3)
    assert rc == 0
    assert "Number of clusters adjusted" in capfd.readouterr().err
    # three clusters, each point its own centroid; the two extra centroid rows stay zero
    assert sorted(L.tolist()) == [0, 1, 2]
    assert np.array_equal(np.sort(C[:3], axis=0), np.sort(X, axis=0))
    assert not C[3:].any()


@pytest.mark.parametrize("dtype", [np.float32, np.float64])
def test_tiny_and_degenerate_shapes(shim, oracle, dtype):
    # one row, one feature, one cluster
    X = np.array([[3.5]], dtype)
    rc, C, L = fit(shim, X, 1, 2, 2, C0=np.array([[0.0]], dtype))
    assert rc == 0 and C[0, 0] == 3.5 and L.tolist() == [0]
    # all rows identical: one cluster takes everything, the others keep their start
    X = np.full((100, 3), 2.0, dtype)
    C0 = np.array([[2, 2, 2], [5, 5, 5], [-1, 0, 1]], dtype)
    rc, C, L = fit(shim, X, 3, 3, 2, C0=C0)
    assert rc == 0 and (L == 0).all()
    assert np.array_equal(C, C0)
    # duplicate centroids: ties go to the lowest index
    C0 = np.array([[0, 0, 0], [2, 2, 2], [2, 2, 2]], dtype)
    rc, C, L = fit(shim, X, 3, 1, 2, C0=C0)
    assert (L == 1).all()
    # d = 1, many clusters
    rng = np.random.default_rng(0)
    X = rng.normal(size=(500, 1)).astype(dtype)
    C0 = np.linspace(-2, 2, 9).reshape(9, 1).astype(dtype)
    rc, C, L = fit(shim, X, 9, 5, 2, C0=C0)
    wC, wL, _, _ = oracle.lloyd(X, C0, 5, 0.0)
    assert np.array_equal(L, wL) and np.allclose(C, wC, rtol=1e-5, atol=1e-6)


def test_rows_whose_distances_overflow_get_minus_one(shim, hip):
    """The reference starts the running minimum at FLT_MAX and leaves -1 when nothing is
    below it; such rows must not contribute to any centroid."""
    X = np.zeros((200, 2), np.float32)
    X[:, 0] = np.linspace(-1, 1, 200)
    X[7] = [3e19, 3e19]              # squared norm overflows float32 -> distances inf
    C0 = np.array([[-0.5, 0.0], [0.5, 0.0]], np.float32)
    with hip.Handle(200, 2, 2, np.float32) as h:
        h.set_data(X)
        h.set_centroids(C0)
        h.iterate(1)
        L, C, counts = h.labels(), h.centroids(), h.counts()
    assert L[7] == -1 and (np.delete(L, 7) >= 0).all()
    assert counts.sum() == 199 and np.isfinite(C).all()


@pytest.mark.parametrize("dtype", [np.float32, np.float64])
def test_predict_and_transform_entry_points(shim, oracle, dtype):
    X, centers = blobs(4000, 24, 33, dtype, 7)
    C = np.ascontiguousarray(centers.astype(dtype))
    n, d = X.shape
    k = C.shape[0]
    fn = shim.make_ptr_float_kmeans if dtype == np.float32 else shim.make_ptr_double_kmeans
    res = np.zeros(n, np.int32)
    rc = fn(1, 0, 0, 0, 1, n, d, k, 10, 0, 0.0, X.flatten(), C.flatten(), np.empty([], dtype), res)
    assert rc == 0
    label_report(oracle, X, C, res, oracle.assign(X, C))
    tf = shim.kmeans_transform_float if dtype == np.float32 else shim.kmeans_transform_double
    out = np.zeros(n * k, dtype)
    assert tf(0, 0, 1, n, d, k, X.flatten(), C.flatten(), out) == 0
    want = oracle.distances(X, C)                      # [k][n]
    eps = np.finfo(dtype).eps
    scale = 2 * (X.astype(np.float64) ** 2).sum(1).max()
    assert np.max(np.abs(out.reshape(k, n).astype(np.float64) - want)) <= 64 * eps * scale
    # inputs of another dtype / layout are converted like SWIG's IN_ARRAY1
    res2 = np.zeros(n, np.int32)
    Xf = np.asfortranarray(X).astype(np.float64 if dtype == np.float32 else np.float32)
    rc = fn(1, 0, 0, 0, 1, n, d, k, 10, 0, 0.0, np.ascontiguousarray(Xf).flatten(), C.flatten(),
            np.empty([], dtype), res2)
    assert rc == 0 and (res2 == res).mean() > 0.999


@pytest.mark.parametrize("dtype", [np.float32, np.float64])
def test_transform_in_several_batches(hip, dtype):
    """transform_host fills its [k][rows] host result batch by batch (strided copies, a
    ragged last batch that is not a multiple of the row tile) when the output exceeds its
    device buffer: the result must be the single-batch one and the float64 brute force."""
    n, d, k = 33333, 40, 300
    rng = np.random.default_rng(12)
    X = rng.standard_normal((n, d)).astype(dtype)
    C = rng.standard_normal((k, d)).astype(dtype)
    with hip.Handle(k, d, k, dtype) as h:
        h.set_centroids(C)
        whole = h.transform(X)
        # 1 MB per batch: 33333 rows x 300 distances go out in 38 (float32) / 77 batches
        h.set_option("transform_batch_mb", 1)
        parts = h.transform(X)
        assert parts.shape == (k, n) and np.array_equal(parts, whole)
        h.set_option("transform_batch_mb", 16)  # three batches, the last one ragged
        assert np.array_equal(h.transform(X), whole)
    rows = rng.choice(n, size=200, replace=False)
    want = ((X[rows][:, None, :].astype(np.float64) - C[None].astype(np.float64)) ** 2).sum(-1).T
    scale = 2 * (X.astype(np.float64) ** 2).sum(1).max()
    assert np.max(np.abs(whole[:, rows].astype(np.float64) - want)) <= 64 * np.finfo(dtype).eps * scale


@pytest.mark.parametrize("dtype", [np.float32, np.float64])
def test_transform_batches_through_the_staging_buffers(hip, dtype):
    """Batches of 24 MB and more come back through the pinned staging buffers, each batch's
    [k][its rows] block scattered into its columns of the [k][rows] result while the next
    batch is computed: the result must be the single-batch one, bit for bit (ragged last batch,
    batch widths that do not divide the 16 MB staging chunk)."""
    n, d, k = 200003, 16, 130
    rng = np.random.default_rng(5)
    X = rng.standard_normal((n, d)).astype(dtype)
    C = rng.standard_normal((k, d)).astype(dtype)
    with hip.Handle(k, d, k, dtype) as h:
        h.set_centroids(C)
        whole = h.transform(X)
        for mb in (32, 40):
            h.set_option("transform_batch_mb", mb)
            assert n * k * np.dtype(dtype).itemsize > 2 * (mb << 20)  # three batches or more
            assert np.array_equal(h.transform(X), whole)
        # one set of device buffers (what a failed allocation of the second set falls back to)
        h.set_option("transform_buffers", 1)
        assert np.array_equal(h.transform(X), whole)
    rows = rng.choice(n, size=100, replace=False)
    want = ((X[rows][:, None, :].astype(np.float64) - C[None].astype(np.float64)) ** 2).sum(-1).T
    scale = 2 * (X.astype(np.float64) ** 2).sum(1).max()
    assert np.max(np.abs(whole[:, rows].astype(np.float64) - want)) <= 64 * np.finfo(dtype).eps * scale


@pytest.mark.parametrize("dtype,n,d,k", [(np.float32, 301234, 128, 200), (np.float64, 150001, 120, 20),
                                         (np.float32, 2100000, 16, 8)])
def test_predict_of_a_large_input_goes_up_in_pieces(hip, dtype, n, d, k):
    """predict_host sends inputs of 128 MB and more to the device in pieces and assigns a piece
    while the next one is in transfer (ragged last piece): the labels must be those of one
    assignment pass over the same rows resident on the device."""
    rng = np.random.default_rng(n)
    X = rng.standard_normal((n, d)).astype(dtype)
    assert X.nbytes >= 128 << 20
    C = np.ascontiguousarray(X[rng.choice(n, size=k, replace=False)] + dtype(0.25))
    with hip.Handle(n, d, k, dtype) as h:
        h.set_data(X)
        h.set_centroids(C)
        h.assign()
        want = h.labels()
        got = h.predict(X)
    assert np.array_equal(got, want)


def test_bad_arguments_return_codes(shim):
    X = np.zeros((10, 2), np.float32)
    pc, pl = np.zeros(4, np.float32), np.zeros(10, np.int32)
    assert shim.make_ptr_float_kmeans(0, 0, 1, 0, 1, 10, 2, 0, 3, 0, 0.0, X.flatten(), np.empty([]), pc, pl) == -2
    assert shim.make_ptr_float_kmeans(0, 0, 1, 0, 1, 10, 2, 2, 3, 2, 0.0, X.flatten(), None, pc, pl) == -2
    with pytest.raises(TypeError):
        shim.make_ptr_float_kmeans(0, 0, 1, 0, 1, 10, 2, 2, 3, 0, 0.0, X.flatten(), np.empty([]),
                                   np.zeros(4, np.float64), pl)
    # max_iterations = 0: no update, labels stay zero-initialised as in the reference
    rc = shim.make_ptr_float_kmeans(0, 0, 1, 0, 1, 10, 2, 2, 0, 0, 0.0, X.flatten(), np.empty([]), pc, pl)
    assert rc == 0 and not pl.any()


@pytest.mark.parametrize("dtype", [np.float32, np.float64])
def test_estimator_round_trip(oracle, dtype):
    """h2o4gpu-style estimator on the GPU: shapes, dtypes and values of every public
    result (README example and test_model.R shapes included)."""
    from h2o4gpu_amd import KMeans
    X = np.array([[1, 1], [1, 4], [1, 0]], dtype)
    m = KMeans(n_clusters=2, random_state=1234, init="random", max_iter=5, tol=0)
    m.fit(X)
    assert m.backend == "h2o4gpu"
    assert m.cluster_centers_.shape == (2, 2) and m.labels_.shape == (3,) and m.labels_.dtype == np.int32
    assert m.predict(X).shape == (3,) and m.transform(X).shape == (3, 2)

    Xb, centers = blobs(5000, 10, 6, dtype, 3)
    C0 = (centers + 0.3).astype(dtype)
    m = KMeans(n_clusters=6, init=C0, max_iter=8, tol=0.0, random_state=5)
    m.fit(Xb)
    wC, wL, _, _ = oracle.lloyd(Xb, C0, 8, 0.0)
    tol = 1e-4 if dtype == np.float32 else 1e-9
    assert np.allclose(m.cluster_centers_, wC, rtol=tol, atol=tol)
    assert np.array_equal(m.labels_, wL) and np.array_equal(m.predict(Xb), wL)
    D = m.transform(Xb)                               # (rows, k), squared distances
    assert D.shape == (5000, 6) and D.flags.f_contiguous
    want = ((Xb[:, None, :].astype(np.float64) - wC[None].astype(np.float64)) ** 2).sum(-1)
    assert np.allclose(D, want, rtol=1e-3, atol=1e-2)
    assert np.array_equal(np.argmin(D, axis=1), m.labels_)
    assert abs(m.inertia_ - want.min(1).sum()) <= 1e-4 * m.inertia_
    assert abs(m.score(Xb) + m.inertia_) <= 1e-3 * m.inertia_
    # k-means++ start through the estimator: valid clustering of well separated blobs
    # (D^2 sampling can still seed one blob twice, so the best of a few seeds is compared)
    best = np.inf
    for seed in range(5):
        m2 = KMeans(n_clusters=6, init="k-means++", max_iter=20, tol=1e-6, random_state=seed)
        m2.fit(Xb)
        best = min(best, m2.inertia_)
    assert best <= 1.05 * m.inertia_
    assert np.array_equal(m2.fit_predict(Xb), m2.labels_)
    # integer input is cast to float32 as in the reference
    m3 = KMeans(n_clusters=2, init="random", max_iter=3, tol=0, random_state=1)
    m3.fit(np.array([[0, 0], [0, 1], [9, 9], [9, 8]]))
    assert m3.cluster_centers_.dtype == np.float32 and sorted(m3.labels_.tolist()) == [0, 0, 1, 1]


@pytest.mark.parametrize("dtype", [np.float32, np.float64])
def test_last_fit_info_reports_inertia_and_iterations(shim, oracle, dtype):
    """The side channel of the fit entry point: inertia equals the exact (float64, brute
    force) objective of the returned labels and centroids, the iteration count follows the
    reference's stop rule, and a thread that never fitted has nothing to report."""
    import threading
    X, centers = blobs(4000, 7, 5, dtype, 11)
    C0 = (centers + 0.2).astype(dtype)
    rc, C, L = fit(shim, X, 5, 6, 2, C0=C0)          # tol = 0: all 6 iterations run
    assert rc == 0
    inertia, iters = shim.last_fit_info()
    assert iters == 6
    want = ((X.astype(np.float64) - C.astype(np.float64)[L]) ** 2).sum()
    assert abs(inertia - want) <= (1e-5 if dtype == np.float32 else 1e-11) * want
    wC, wL, w_it, _ = oracle.lloyd(X, C0, 50, 1e-3)   # stops early on the shift threshold
    rc, C, L = fit(shim, X, 5, 50, 2, tol=1e-3, C0=C0)
    # the oracle returns the loop index at the break as the reference does
    # (kmeans_impl.h:246); the entry point reports the number of updates made, one more
    assert rc == 0 and shim.last_fit_info()[1] == w_it + 1 < 50
    seen = []
    t = threading.Thread(target=lambda: seen.append(shim.last_fit_info()))
    t.start()
    t.join()
    assert seen == [None]


def test_estimator_restarts_and_score(oracle):
    """n_init restarts keep the best of the seeds seed, seed+1, ...; n_iter_ and inertia_
    come from the native fit; score is the negated objective on new rows."""
    from h2o4gpu_amd import KMeans
    Xb, _ = blobs(6000, 6, 8, np.float32, 21)
    singles = []
    for seed in (40, 41, 42, 43):
        m = KMeans(n_clusters=8, init="random", max_iter=30, tol=1e-6, random_state=seed)
        m.fit(Xb)
        assert 1 <= m.n_iter_ <= 30
        singles.append(m.inertia_)
    multi = KMeans(n_clusters=8, init="random", n_init=4, max_iter=30, tol=1e-6, random_state=40)
    multi.fit(Xb)
    # (the restarts run stacked through the matrix-core kernel, the single fits of this small
    # shape through the scalar-order one: same optimum, minimum distances equal to rounding)
    assert abs(multi.inertia_ - min(singles)) <= 1e-5 * min(singles)
    want = ((Xb.astype(np.float64) - multi.cluster_centers_.astype(np.float64)[multi.labels_]) ** 2).sum()
    assert abs(multi.inertia_ - want) <= 1e-5 * want
    Xn, _ = blobs(1500, 6, 8, np.float32, 22)
    d2 = ((Xn[:, None, :].astype(np.float64) - multi.cluster_centers_[None].astype(np.float64)) ** 2).sum(-1)
    assert abs(multi.score(Xn) + d2.min(1).sum()) <= 1e-5 * d2.min(1).sum()


def test_concurrent_fits_from_two_threads(shim):
    """The entry points are re-entrant (the reference keeps per-device globals and is not,
    kmeans_labels.cu:11-49): two threads fitting different data at the same time get the
    results, and the last-fit record, of their own call."""
    import threading
    jobs = []
    for seed, (n, d, k) in enumerate([(40000, 24, 9), (25000, 40, 14)]):
        X, centers = blobs(n, d, k, np.float32, 50 + seed)
        C0 = (centers + 0.3).astype(np.float32)
        rc, C, L = fit(shim, X, k, 6, 2, C0=C0)
        assert rc == 0
        jobs.append((X, C0, k, C, L, shim.last_fit_info()))
    out = [None, None]

    def work(i):
        X, C0, k = jobs[i][:3]
        res = []
        for _ in range(5):
            rc, C, L = fit(shim, X, k, 6, 2, C0=C0)
            res.append((rc, C, L, shim.last_fit_info()))
        out[i] = res

    threads = [threading.Thread(target=work, args=(i,)) for i in range(2)]
    for t in threads:
        t.start()
    for t in threads:
        t.join()
    for i in range(2):
        _, _, _, wantC, wantL, want_info = jobs[i]
        for rc, C, L, info in out[i]:
            assert rc == 0 and np.array_equal(C, wantC) and np.array_equal(L, wantL)
            assert info == want_info


def test_sigint_stops_the_loop_when_handlers_are_enabled(hip):
    """Runs in a child process: the handler is process-wide and must not replace pytest's."""
    import json
    import os
    import subprocess
    import sys
    here = os.path.dirname(os.path.abspath(__file__))
    proc = subprocess.run([sys.executable, os.path.join(here, "signal_stop_check.py")],
                          capture_output=True, text=True, timeout=600)
    assert proc.returncode == 0, proc.stdout + proc.stderr
    r = json.loads(proc.stdout.strip().splitlines()[-1])
    assert r["rc"] == 0 and r["labels_in_range"]
    assert 1 <= r["iterations"] < 2_000_000       # stopped early ...
    assert "Signal caught" in proc.stderr         # ... for the stated reason


def test_fit_after_device_reset(hip):
    """cudaresetdevice / cudaresetdevice_bare between fits: the library's pinned staging
    buffers die with the device context and must be re-created, results unchanged."""
    import json
    import os
    import subprocess
    import sys
    here = os.path.dirname(os.path.abspath(__file__))
    proc = subprocess.run([sys.executable, os.path.join(here, "device_reset_check.py")],
                          capture_output=True, text=True, timeout=600)
    assert proc.returncode == 0, proc.stdout + proc.stderr
    r = json.loads(proc.stdout.strip().splitlines()[-1])
    assert r["rc"] == [0, 0, 0] and r["reset_rc"] == [0, 0]
    assert r["same_centroids"] and r["same_labels"]
