"""The float32 matrix-core kernels with their dot products on the bfloat16 matrix pipe
(option "fp32_split": 9 products of bfloat16 parts per feature pair, every one exact, or 6,
the three smallest left out) against the CPU oracle and against float64 brute force, through
the C ABI. The bar is the float32 matrix-core path's own: labels equal the oracle's except
rows whose two nearest centroids lie within rounding of each other, minimum distances within
the rounding of (xx + cc)."""
import numpy as np
import pytest

from parity import assert_centroids_close, label_report

pytestmark = pytest.mark.gpu


def blobs(n, d, k, spread=5.0, sigma=1.0, seed=0, scale=1.0):
    rng = np.random.default_rng(seed)
    centers = rng.uniform(-spread, spread, size=(k, d))
    X = centers[rng.integers(0, k, size=n)] + sigma * rng.standard_normal((n, d))
    return np.ascontiguousarray((scale * X).astype(np.float32))


# rows of exactly 16 / 32 / 64 features (16-byte loads of the slice as it lies in memory),
# rows padded up to those widths (9..63 features, whole vectors or not), models of one tile,
# of several, with a partly filled last tile, and one swept in LDS-sized chunks
SHAPES = [(4096, 32, 256), (5000, 32, 100), (3001, 64, 64), (2000, 24, 33), (1000, 16, 8),
          (900, 30, 70), (700, 9, 40), (513, 63, 20), (2500, 50, 130), (1, 16, 1), (130, 20, 2),
          (3000, 40, 600), (2000, 16, 3000)]
# the tiled kernel (more than 64 centroids): whole 16-feature stages, a last stage with 1 to
# 15 features, rows that are not whole vectors, 128- and 256-centroid blocks with partly
# filled last blocks, integer keys (below 128 features) and the float compare chain
TILED_SHAPES = [(4096, 32, 256), (1500, 128, 200), (2500, 100, 70), (1200, 256, 130), (900, 300, 257),
                (1800, 255, 140), (1300, 101, 300), (1100, 127, 1030), (1500, 120, 9000),
                (1200, 520, 2304), (700, 9, 100), (513, 63, 200), (600, 6, 80), (3, 17, 65)]


@pytest.mark.parametrize("split", [9, 6])
@pytest.mark.parametrize("variant,n,d,k", [("mfma_rowstat",) + c for c in SHAPES] +
                         [("mfma_tiled",) + c for c in TILED_SHAPES])
def test_assign_matches_oracle(hip, oracle, variant, n, d, k, split):
    X = blobs(n, d, max(k, 2), seed=n + d + k)
    rng = np.random.default_rng(k)
    if k <= n:
        C = np.ascontiguousarray(X[rng.choice(n, size=k, replace=False)])
    else:
        C = np.ascontiguousarray((X[rng.choice(n, size=k)] + 0.5 * rng.standard_normal((k, d))).astype(np.float32))
    with hip.Handle(n, d, k, np.float32) as h:
        h.set_data(X)
        h.set_centroids(C)
        h.set_option("assign", variant)
        h.set_option("fp32_split", split)
        name = h.assign_variant()
        h.assign()
        got, mind = h.labels(), h.min_distances()
        h.set_option("fp32_split", 0)
        assert h.assign_variant() == variant
        h.assign()
        plain, pmind = h.labels(), h.min_distances()
    want, wmind = oracle.assign(X, C, return_mindist=True)
    rep = label_report(oracle, X, C, got, want)
    scale = (X.astype(np.float64) ** 2).sum(1).max() + (C.astype(np.float64) ** 2).sum(1).max()
    eps = np.finfo(np.float32).eps
    assert np.max(np.abs(mind.astype(np.float64) - wmind)) <= (4 * np.sqrt(d) + 40) * eps * scale
    assert name == "%s_bf16x%d" % (variant, split)
    print("%s split %d n=%d d=%d k=%d: %s; %d labels differ from the float32 instructions'" %
          (variant, split, n, d, k, rep, int((got != plain).sum())))


def test_shapes_the_option_leaves_alone(hip):
    """Rows of fewer than 4 features, 64 centroids or fewer in the tiled kernel, rows padded to
    128 features in the row-stationary kernel, the small-model kernels: the float32
    instructions (or the vector ALU) run, and the results are the option-free ones bit for bit."""
    for n, d, k, variant, name in [(3000, 3, 100, "mfma_tiled", "mfma_tiled"), (3000, 40, 50, "mfma_tiled", "mfma_tiled"),
                                   (3000, 100, 90, "mfma_rowstat", "mfma_rowstat"), (3000, 20, 10, "auto", "valu")]:
        X = blobs(n, d, k, seed=n + d)
        C = np.ascontiguousarray(X[:k])
        out = []
        for split in (0, 6):
            with hip.Handle(n, d, k, np.float32) as h:
                h.set_data(X)
                h.set_centroids(C)
                h.set_option("assign", variant)
                h.set_option("fp32_split", split)
                assert h.assign_variant() == name
                h.assign()
                out.append((h.labels(), h.min_distances()))
        assert np.array_equal(out[0][0], out[1][0]) and np.array_equal(out[0][1], out[1][1])


@pytest.mark.parametrize("split", [9, 6])
@pytest.mark.parametrize("n,d,k", [(3000, 100, 300), (1000, 784, 4096), (2500, 37, 130), (129, 16, 65)])
def test_transform_matches_oracle(hip, oracle, n, d, k, split):
    X = blobs(n, d, 20, seed=k)
    rng = np.random.default_rng(d)
    C = np.ascontiguousarray((X[rng.choice(n, size=k)] + 0.5 * rng.standard_normal((k, d))).astype(np.float32))
    with hip.Handle(n, d, k, np.float32) as h:
        h.set_data(X)
        h.set_centroids(C)
        h.set_option("fp32_split", split)
        D = h.transform(X)
        h.set_option("fp32_split", 0)
        D0 = h.transform(X)
    want = oracle.distances(X, C)
    scale = (X.astype(np.float64) ** 2).sum(1).max() + (C.astype(np.float64) ** 2).sum(1).max()
    eps = np.finfo(np.float32).eps
    bound = (4 * np.sqrt(d) + 40) * eps * scale
    assert np.max(np.abs(D.astype(np.float64) - want)) <= bound
    assert np.max(np.abs(D0.astype(np.float64) - want)) <= bound
    assert not np.array_equal(D, D0)  # (the parts did run: same values to rounding, not bit for bit)


@pytest.mark.parametrize("variant", ["mfma_rowstat", "mfma_tiled"])
@pytest.mark.parametrize("split", [9, 6])
def test_distances_are_as_close_to_float64_as_the_float32_instructions(hip, split, variant):
    """Minimum distances of both paths against float64 brute force, in units of the rounding
    of (xx + cc). The keys the argmin compares drop four mantissa bits on both paths, so the
    exact-compare option is used for the float32 side and the split side is given twice its
    worst error plus those four bits."""
    n, d, k = 20000, 32, 96
    X = blobs(n, d, k, spread=40.0, sigma=3.0, seed=5)
    C = np.ascontiguousarray(X[np.random.default_rng(1).choice(n, size=k, replace=False)])
    X64, C64 = X.astype(np.float64), C.astype(np.float64)
    D = (X64 * X64).sum(1)[:, None] + (C64 * C64).sum(1)[None, :] - 2.0 * X64 @ C64.T
    truth, tl = D.min(1), D.argmin(1)
    unit = np.finfo(np.float32).eps * ((X64 * X64).sum(1) + (C64[tl] ** 2).sum(1))
    out = {}
    for name, opts in (("f32", {"exact_argmin": 1}), ("split", {"fp32_split": split})):
        with hip.Handle(n, d, k, np.float32) as h:
            h.set_data(X)
            h.set_centroids(C)
            h.set_option("assign", variant)
            for o, v in opts.items():
                h.set_option(o, v)
            h.assign()
            out[name] = (h.labels(), np.abs(h.min_distances().astype(np.float64) - truth) / unit)
    f32_err, split_err = out["f32"][1], out["split"][1]
    print("max error in units of eps*(xx+cc): float32 instructions %.2f, %d bfloat16 products %.2f" %
          (f32_err.max(), split, split_err.max()))
    assert split_err.max() <= 2 * f32_err.max() + 16
    assert int((out["split"][0] != tl).sum()) <= int((out["f32"][0] != tl).sum()) + 2


@pytest.mark.parametrize("split", [9, 6])
@pytest.mark.parametrize("n,d,k", [(60000, 32, 256), (30000, 64, 64), (20000, 20, 40), (15000, 48, 100)])
def test_fit_matches_oracle(hip, oracle, n, d, k, split):
    """The fused step (labels and sums in one kernel): lock-step beside the oracle (every
    iteration starts from the oracle's centroids; labels to the near-tie rule, the update of
    the engine's own labels to 1e-5), then a whole fit, whose objective must agree and which
    must repeat bit for bit."""
    X = blobs(n, d, k, spread=20.0, sigma=1.0, seed=n)
    rng = np.random.default_rng(3)
    centres = np.stack([X[rng.choice(n, 40)].mean(0) for _ in range(k)])  # rough, distinct starts
    C0 = np.ascontiguousarray(centres.astype(np.float32))
    iters = 6
    with hip.Handle(n, d, k, np.float32) as h:
        h.set_data(X)
        h.set_option("fp32_split", split)
        assert h.assign_variant() == "mfma_rowstat_bf16x%d" % split
        C = C0.copy()
        excused = 0
        for _ in range(iters):
            h.set_centroids(C)
            h.iterate(1)
            L = h.labels()
            rep = label_report(oracle, X, C, L, oracle.assign(X, C, threads=4))
            excused += rep["excused"]
            wC, wcounts = oracle.update(X, L, C)
            assert np.array_equal(h.counts(), wcounts)
            assert np.allclose(h.centroids(), wC, rtol=1e-5, atol=1e-5 * np.abs(wC).max())
            C = wC
        h.set_centroids(C0)
        assert h.fit(iters, 0.0) == iters
        Cg, Lg, inertia = h.centroids(), h.labels(), h.inertia()
        h.set_centroids(C0)
        h.fit(iters, 0.0)
        assert np.array_equal(h.centroids(), Cg) and np.array_equal(h.labels(), Lg), "fit does not repeat"
    print("fit split %d n=%d d=%d k=%d: %d near-tie rows excused in lock-step" % (split, n, d, k, excused))
    wC, wL, _, _ = oracle.lloyd(X, C0, iters, 0.0, threads=4)
    X64 = X.astype(np.float64)
    want_inertia = ((X64 - wC.astype(np.float64)[wL]) ** 2).sum()
    assert abs(inertia - want_inertia) <= 1e-4 * want_inertia


def test_stacked_sets_take_the_option(hip):
    n, d, k, sets = 30000, 32, 20, 3
    X = blobs(n, d, k, seed=9)
    rng = np.random.default_rng(7)
    starts = [np.ascontiguousarray(X[rng.choice(n, size=k, replace=False)]) for _ in range(sets)]
    with hip.Handle(n, d, k, np.float32, sets=sets) as h:
        h.set_data(X)
        h.set_option("fp32_split", 9)
        for s in range(sets):
            h.select_set(s)
            h.set_centroids(starts[s])
        h.fit(5, 0.0)
        got = []
        for s in range(sets):
            h.select_set(s)
            got.append((h.centroids(), h.labels(), h.inertia()))
    for s in range(sets):
        with hip.Handle(n, d, k, np.float32) as h:
            h.set_data(X)
            h.set_option("assign", "mfma_rowstat")
            h.set_option("fp32_split", 9)
            h.set_centroids(starts[s])
            h.fit(5, 0.0)
            assert np.array_equal(h.labels(), got[s][1])
            assert np.array_equal(h.centroids(), got[s][0])
            assert h.inertia() == got[s][2]


def test_option_values(hip):
    with hip.Handle(100, 32, 4, np.float32) as h:
        for bad in (1, 3, 12, -9):
            with pytest.raises(hip.KMeansHipError):
                h.set_option("fp32_split", bad)
    X = blobs(2000, 32, 40, seed=2).astype(np.float64)
    with hip.Handle(2000, 32, 40, np.float64) as h:  # float64: accepted, without effect
        h.set_data(X)
        h.set_centroids(X[:40])
        h.set_option("assign", "mfma_rowstat")
        h.set_option("fp32_split", 9)
        assert h.assign_variant() == "mfma_rowstat"
        h.assign()


@pytest.mark.timeout(900)
@pytest.mark.parametrize("name,e2e_iters,fit_iters,split", [("C3", 6, 20, 9), ("C3", 6, 20, 6), ("C2", 20, 20, 9),
                                                            ("C2", 20, 20, 6), ("C4", 2, 4, 6), ("C5", 1, 2, 6)])
def test_full_benchmark_shape(hip, oracle, name, e2e_iters, fit_iters, split):
    """The float32 benchmark shapes that run on the matrix cores, at full size with the option
    on: one Lloyd step on all rows beside the oracle at the start and at the fitted centroids,
    and a fixed number of iterations end to end, to the same bars as the float32 instructions'
    full-size test. 500k x 784, k = 4096 also transforms its 100,000 held-out rows."""
    from h2o4gpu_amd import datasets
    from test_gpu_configs import _end_to_end_all_rows, _lockstep_all_rows, _start, _transform_check
    X, k, _ = datasets.make(name, 1.0, np.float32)
    n, d = X.shape
    tag = "%s float32 bf16x%d" % (name, split)
    with hip.Handle(n, d, k, np.float32) as h:
        h.set_data(X)
        C0 = _start(name, X, k, h)
        h.set_option("fp32_split", split)
        assert h.assign_variant() == ("mfma_rowstat_bf16x%d" if name in ("C2", "C3") else "mfma_tiled_bf16x%d") % split
        start = _lockstep_all_rows(hip, oracle, h, X, C0, np.float32, tag + " start")
        h.set_centroids(C0)
        h.fit(fit_iters, 0.0)
        C, L = h.centroids(), h.labels()
        h.set_centroids(C0)
        h.fit(fit_iters, 0.0)
        assert np.array_equal(h.centroids(), C) and np.array_equal(h.labels(), L), "fit does not repeat"
        fitted = _lockstep_all_rows(hip, oracle, h, X, C, np.float32, tag + " fitted")
        e2e = _end_to_end_all_rows(hip, oracle, h, X, C0, np.float32, e2e_iters, tag)
        if name == "C5":
            h.set_centroids(C)
            _transform_check(h, C)
    print("full shape %s: start %s\nfitted %s\nend to end %s" % (tag, start, fitted, e2e))


def test_environment_variable_reaches_the_reference_entry_points(hip, oracle, monkeypatch):
    """make_ptr_float_kmeans has no argument for the option: H2O4GPU_KMEANS_FP32_SPLIT sets it
    for every handle created afterwards."""
    from h2o4gpu_amd.libs import ch2o4gpu_gpu
    n, d, k = 40000, 32, 64
    X = blobs(n, d, k, spread=20.0, seed=4)
    C0 = np.ascontiguousarray(X[np.random.default_rng(2).choice(n, size=k, replace=False)])

    def fit():
        centres = np.zeros(k * d, np.float32)
        labels = np.zeros(n, np.int32)
        rc = ch2o4gpu_gpu.make_ptr_float_kmeans(0, 0, 1, 0, 1, n, d, k, 5, 2, 0.0, X.flatten(), C0.flatten(),
                                                centres, labels)
        assert rc == 0
        return centres.reshape(k, d), labels

    plain = fit()
    monkeypatch.setenv("H2O4GPU_KMEANS_FP32_SPLIT", "6")
    with hip.Handle(n, d, k, np.float32) as h:
        assert h.assign_variant() == "mfma_rowstat_bf16x6"
    split = fit()
    monkeypatch.setenv("H2O4GPU_KMEANS_FP32_SPLIT", "7")  # not a value of the option: ignored
    with hip.Handle(n, d, k, np.float32) as h:
        assert h.assign_variant() == "mfma_rowstat"
    monkeypatch.delenv("H2O4GPU_KMEANS_FP32_SPLIT")
    assert not np.array_equal(plain[0], split[0])  # another summation order: not bit for bit
    wC, wL, _, _ = oracle.lloyd(X, C0, 5, 0.0, threads=4)
    X64 = X.astype(np.float64)
    want = ((X64 - wC.astype(np.float64)[wL]) ** 2).sum()
    for C, L in (plain, split):
        if np.array_equal(L, wL):
            assert_centroids_close(C, wC, np.float32)
        # (a start on random rows splits blobs: near-tie rows that flip move the trajectory,
        # the objective stays)
        got = ((X64 - C.astype(np.float64)[L]) ** 2).sum()
        assert abs(got - want) <= 1e-4 * want


@pytest.mark.parametrize("variant", ["mfma_rowstat", "mfma_tiled"])
def test_non_finite_rows_and_centroids(hip, oracle, variant):
    """The parts of an infinity or a NaN are not finite either: such rows get label -1, such
    centroids are never chosen (kmeans_labels.h:360-377), their neighbours are unaffected."""
    n, d, k = 2048, 32, 80
    X = blobs(n, d, k, seed=99)
    C = np.ascontiguousarray(X[np.random.default_rng(1).choice(n, size=k, replace=False)])
    X[5, 3] = np.nan
    X[70, :] = np.nan
    X[130, 0] = np.inf
    X[131, 7] = -np.inf
    X[1999, d - 1] = np.nan
    C[4, 2] = np.nan
    C[17, :] = np.inf
    bad_rows = [5, 70, 130, 131, 1999]
    with hip.Handle(n, d, k, np.float32) as h:
        h.set_data(X)
        h.set_centroids(C)
        h.set_option("assign", variant)
        h.set_option("fp32_split", 6)
        assert h.assign_variant() == variant + "_bf16x6"
        h.assign()
        got = h.labels()
        h.update()
        counts = h.counts()
    want = oracle.assign(X, C)
    assert np.all(want[bad_rows] == -1) and np.all(got[bad_rows] == -1)
    assert not np.any(np.isin(got, [4, 17]))
    good = np.ones(n, bool)
    good[bad_rows] = False
    remap = np.delete(np.arange(k), [4, 17])
    inv = {int(c): i for i, c in enumerate(remap)}
    g2 = np.array([inv[int(c)] for c in got[good]], np.int32)
    w2 = np.array([inv[int(c)] for c in want[good]], np.int32)
    label_report(oracle, np.ascontiguousarray(X[good]), np.ascontiguousarray(np.delete(C, [4, 17], axis=0)), g2, w2)
    assert counts.sum() == n - len(bad_rows)


@pytest.mark.parametrize("variant", ["mfma_rowstat", "mfma_tiled"])
@pytest.mark.parametrize("scale", [1e15, 1e-15])
def test_large_and_small_magnitudes(hip, oracle, variant, scale):
    """bfloat16 has float32's exponent range: data scaled by 1e15 (squares near 1e32) and by
    1e-15 (squares near 1e-28) split exactly and label as unscaled data does."""
    n, d, k = 6000, 32, 70
    X = blobs(n, d, k, seed=8, scale=scale)
    C = np.ascontiguousarray(X[np.random.default_rng(5).choice(n, size=k, replace=False)])
    with hip.Handle(n, d, k, np.float32) as h:
        h.set_data(X)
        h.set_centroids(C)
        h.set_option("assign", variant)
        h.set_option("fp32_split", 6)
        h.assign()
        got, mind = h.labels(), h.min_distances()
    want, wmind = oracle.assign(X, C, return_mindist=True)
    label_report(oracle, X, C, got, want)
    s2 = (X.astype(np.float64) ** 2).sum(1).max() + (C.astype(np.float64) ** 2).sum(1).max()
    assert np.max(np.abs(mind.astype(np.float64) - wmind)) <= (4 * np.sqrt(d) + 40) * np.finfo(np.float32).eps * s2


@pytest.mark.parametrize("variant,k,pairs", [("mfma_rowstat", 192, [(7, 36), (3, 160)]),
                                             ("mfma_tiled", 192, [(7, 36), (3, 160)]),
                                             ("mfma_tiled", 1024, [(7, 36), (3, 800), (100, 901)])])
def test_duplicate_centroids_lowest_index_wins(hip, oracle, variant, k, pairs):
    """Identical centroids give bit-identical distances on the bfloat16 pipe too; the strict
    '<' of the reference (kmeans_labels.h:360-377) sends every tied row to the lower index,
    across 32-centroid tiles and across centroid blocks."""
    n, d = 24000, 32
    rng = np.random.default_rng(k + 11)
    centers = rng.uniform(-10, 10, size=(k, d))
    X = np.ascontiguousarray((centers[rng.integers(0, k, size=n)] + 0.3 * rng.standard_normal((n, d))).astype(np.float32))
    C0 = np.ascontiguousarray((centers + 0.05).astype(np.float32))
    for lo, hi in pairs:
        C0[hi] = C0[lo]
    want = oracle.assign(X, C0, threads=4)
    assert not np.isin(want, [hi for _, hi in pairs]).any()
    for fuse in (1, 0):
        with hip.Handle(n, d, k, np.float32) as h:
            h.set_data(X)
            h.set_centroids(C0)
            h.set_option("assign", variant)
            h.set_option("fp32_split", 6)
            h.set_option("fuse", fuse)
            h.assign()
            assert np.array_equal(h.labels(), want), "assignment-only pass"
            h.iterate(1)
            assert np.array_equal(h.labels(), want), "Lloyd step, fuse=%d" % fuse
            C1 = h.centroids()
        for lo, hi in pairs:
            assert np.array_equal(C1[hi], C0[hi]) and not np.array_equal(C1[lo], C0[lo])
