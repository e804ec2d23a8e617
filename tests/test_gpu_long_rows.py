"""Long rows with a handful of centroids (k <= 16, more than 64 features): the one-pass kernel
(`wave_row`: a wavefront along the features of four rows, sums fused) against the CPU oracle,
by the bars of the matrix-core kernels (its dot products are not summed in a scalar loop's
order), and against the tiled kernel it replaces on these shapes."""
import numpy as np
import pytest

from parity import label_report

pytestmark = pytest.mark.gpu


def blobs(n, d, k, dtype, seed, spread=4.0):
    rng = np.random.default_rng(seed)
    nb = max(k, 2)
    centres = rng.uniform(-spread, spread, size=(nb, d))
    X = centres[rng.integers(0, nb, size=n)] + rng.standard_normal((n, d))
    C = X[rng.choice(n, size=k, replace=False)] + 0.1 * rng.standard_normal((k, d))
    return np.ascontiguousarray(X.astype(dtype)), np.ascontiguousarray(C.astype(dtype))


# n, d, k: every count of 16-byte vectors per lane (1 to 4), partial last vectors, ragged last
# group of rows, k from 1 to 16, the largest model whose sums fit one CU's LDS
SHAPES = [
    (5001, 68, 3),
    (4099, 256, 16),
    (3000, 300, 10),
    (2050, 784, 10),
    (1027, 784, 16),
    (1500, 1024, 12),
    (777, 132, 1),
    (3, 200, 2),
    (1, 96, 1),
]


@pytest.mark.parametrize("dtype", [np.float32, np.float64])
@pytest.mark.parametrize("n,d,k", SHAPES)
def test_assign_and_fused_step_against_the_oracle(hip, oracle, n, d, k, dtype):
    if dtype == np.float64 and d > 512:
        pytest.skip("float64 rows beyond 512 features are the tiled kernel's")
    X, C = blobs(n, d, k, dtype, seed=n + d + k)
    with hip.Handle(n, d, k, dtype) as h:
        h.set_data(X)
        h.set_centroids(C)
        h.set_option("assign", "wave_row")   # (the default for up to 4 centroids, and beyond 128 float32 / from 256 float64 features)
        assert h.assign_variant() == "wave_row"
        h.assign()
        L, m = h.labels(), h.min_distances()
        h.set_centroids(C)
        h.iterate(1)                                   # the fused form: same labels, plus the update
        L1, counts, C1 = h.labels(), h.counts(), h.centroids()
        P = h.predict(X)
        h.set_option("assign", "mfma_tiled")
        h.set_centroids(C)
        h.assign()
        Lt = h.labels()
    want, wmin = oracle.assign(X, C, threads=4, return_mindist=True)
    nm = max(8.0, 0.7 * np.sqrt(d))
    label_report(oracle, X, C, L, want, noise_mult=nm)
    assert np.array_equal(L, L1)
    eps = float(np.finfo(dtype).eps)
    xx = (X.astype(np.float64) ** 2).sum(1)
    cc = (C.astype(np.float64) ** 2).sum(1)
    same = L == want
    assert np.all(np.abs(m[same].astype(np.float64) - wmin[same]) <= (4 * np.sqrt(d) + 40) * eps * (xx[same] + cc[want[same]]))
    # the update of the engine's own labels, as the oracle computes it
    wC, wcounts = oracle.update(X, L, C)
    assert np.array_equal(counts, wcounts)
    tol = 1e-5 if dtype == np.float32 else 1e-12
    assert np.allclose(C1, wC, rtol=tol, atol=tol * max(np.abs(wC).max(), 1e-30))
    # predict against the new centroids agrees with the oracle's pass over them
    label_report(oracle, X, C1, P, oracle.assign(X, C1, threads=4), noise_mult=nm)
    # the tiled kernel differs from it on near-tie rows at most
    if (Lt != L).any():
        label_report(oracle, X, C, Lt, L, noise_mult=nm)


@pytest.mark.parametrize("dtype", [np.float32, np.float64])
def test_whole_fit_against_the_oracle(hip, oracle, dtype):
    n, d, k = 20000, 320, 9
    X, C = blobs(n, d, k, dtype, seed=7, spread=6.0)
    with hip.Handle(n, d, k, dtype) as h:
        h.set_data(X)
        h.set_centroids(C)
        assert h.fit(6, 0.0) == 6
        assert h.assign_variant() == "wave_row"
        Cf, L, inertia = h.centroids(), h.labels(), h.inertia()
        assert np.array_equal(h.predict(X), L)
    wC, wL, _, _ = oracle.lloyd(X, C, 6, 0.0, threads=4)
    # well-separated blobs: no near-tie rows, the trajectories coincide
    assert np.array_equal(L, wL)
    tol = 1e-4 if dtype == np.float32 else 1e-9
    assert np.allclose(Cf, wC, rtol=tol, atol=tol * np.abs(wC).max())
    X64 = X.astype(np.float64)
    want = ((X64 - Cf.astype(np.float64)[L]) ** 2).sum()
    assert abs(inertia - want) <= 1e-4 * want


def test_rows_with_nan_get_no_label_and_join_no_sum(hip, oracle):
    n, d, k = 1000, 200, 5
    X, C = blobs(n, d, k, np.float32, seed=3)
    X[17, 5] = np.nan
    X[400, 199] = np.inf
    with hip.Handle(n, d, k, np.float32) as h:
        h.set_data(X)
        h.set_centroids(C)
        h.iterate(1)
        L, counts, C1 = h.labels(), h.counts(), h.centroids()
    assert L[17] == -1 and L[400] == -1
    assert counts.sum() == n - 2
    assert np.isfinite(C1).all()
    keep = np.ones(n, bool)
    keep[[17, 400]] = False
    want = oracle.assign(np.ascontiguousarray(X[keep]), C, threads=2)
    label_report(oracle, np.ascontiguousarray(X[keep]), C, L[keep], want, noise_mult=max(8.0, 0.7 * np.sqrt(d)))


def test_duplicate_centroids_lowest_index_wins(hip):
    n, d, k = 512, 128 + 64, 6
    X, C = blobs(n, d, k, np.float32, seed=11)
    C[4] = C[1]
    C[5] = C[0]
    with hip.Handle(n, d, k, np.float32) as h:
        h.set_data(X)
        h.set_centroids(C)
        h.assign()
        L = h.labels()
    assert not np.isin(L, [4, 5]).any()


def test_which_shapes_take_it_by_default(hip):
    for n, d, k, dtype, want in [(2000, 64, 8, np.float32, "valu"), (2000, 784, 17, np.float32, "mfma_tiled"),
                                 (2000, 1028, 8, np.float32, "mfma_tiled"), (2000, 786, 8, np.float32, "mfma_tiled"),
                                 (2000, 96, 8, np.float32, "mfma_rowstat"), (2000, 96, 8, np.float64, "wave_row"), (2000, 92, 8, np.float64, "mfma_tiled"),
                                 (2000, 200, 12, np.float64, "mfma_tiled"), (2000, 256, 12, np.float64, "wave_row"),
                                 (2000, 784, 10, np.float32, "wave_row"), (2000, 256, 16, np.float32, "wave_row"),
                                 (2000, 516, 4, np.float64, "mfma_tiled"), (2000, 96, 4, np.float32, "wave_row"),
                                 (2000, 96, 5, np.float32, "mfma_rowstat"), (2000, 72, 2, np.float64, "wave_row")]:
        with hip.Handle(n, d, k, dtype) as h:
            assert h.assign_variant() == want, (n, d, k, h.assign_variant())
