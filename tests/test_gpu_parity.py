"""GPU parity: every kernel of the engine against the CPU oracle, through the C ABI."""
import numpy as np
import pytest

from parity import assert_centroids_close, label_report

pytestmark = pytest.mark.gpu

RNG = np.random.default_rng(20240607)


def blobs(n, d, k, dtype, spread=5.0, sigma=1.0, seed=0):
    rng = np.random.default_rng(seed)
    centers = rng.uniform(-spread, spread, size=(k, d))
    lab = rng.integers(0, k, size=n)
    X = centers[lab] + sigma * rng.standard_normal((n, d))
    return np.ascontiguousarray(X.astype(dtype))


ASSIGN_CASES = [
    # (n, d, k) covering padding of rows, features and centroids in every variant
    (1000, 16, 8), (777, 5, 3), (4096, 32, 256), (5000, 32, 100), (3001, 64, 64),
    (2000, 24, 33), (1500, 128, 40), (2500, 100, 70), (1200, 256, 130), (900, 300, 257),
    (64, 8, 64), (1, 4, 1), (130, 2, 2), (3000, 40, 600), (2100, 66, 1030),
    # rows that are not a whole number of 16-byte vectors
    (1800, 255, 140), (1300, 101, 300), (900, 30, 70), (1100, 127, 1030), (700, 9, 40), (513, 63, 20),
    # float32 models beyond 4 MB: the tiled kernel's 256-centroid block (integer keys below 128
    # features, float compare from there on; 520 features leave a quarter-filled last stage)
    (1500, 120, 9000), (1200, 520, 2304),
]


@pytest.mark.parametrize("dtype", [np.float32, np.float64])
@pytest.mark.parametrize("variant", ["valu", "mfma_rowstat", "mfma_tiled"])
@pytest.mark.parametrize("n,d,k", ASSIGN_CASES)
def test_assign_matches_oracle(hip, oracle, n, d, k, variant, dtype):
    X = blobs(n, d, max(k, 2), dtype, seed=n + d + k)
    if k <= n:
        C = np.ascontiguousarray(X[RNG.choice(n, size=k, replace=False)])
    else:  # more centroids than rows: rows drawn with repeats, nudged apart
        C = np.ascontiguousarray((X[RNG.choice(n, size=k)] + 0.5 * RNG.standard_normal((k, d))).astype(dtype))
    with hip.Handle(n, d, k, dtype) as h:
        h.set_data(X)
        h.set_centroids(C)
        try:
            h.set_option("assign", variant)
        except hip.KMeansHipError:
            pytest.skip("variant not available")
        if h.assign_variant() == "unsupported":
            pytest.skip("shape outside %s" % variant)
        h.assign()
        got = h.labels()
        mind = h.min_distances()
    want, wmind = oracle.assign(X, C, return_mindist=True)
    if variant == "valu":
        # same association as the scalar loop: bit-exact
        assert np.array_equal(got, want)
        assert np.array_equal(mind, wmind)
    else:
        rep = label_report(oracle, X, C, got, want)
        scale = (X.astype(np.float64) ** 2).sum(1).max() + (C.astype(np.float64) ** 2).sum(1).max()
        eps = np.finfo(dtype).eps
        # MFMA summation order differs from the scalar loop (rounding of order
        # sqrt(d)*eps*(xx+cc)); the float32 epilogue compares distances at 16 ulp
        assert np.max(np.abs(mind.astype(np.float64) - wmind)) <= (4 * np.sqrt(d) + 40) * eps * scale
        print("assign %s %s n=%d d=%d k=%d: %s" % (variant, np.dtype(dtype).name, n, d, k, rep))


@pytest.mark.parametrize("dtype", [np.float32, np.float64])
@pytest.mark.parametrize("buckets", [1, 0])
@pytest.mark.parametrize("n,d,k", [(5000, 32, 256), (3000, 16, 8), (2000, 7, 5), (4000, 256, 300),
                                   (1000, 784, 130), (70000, 64, 64), (300, 3, 300), (9000, 1100, 70),
                                   (5000, 130, 90), (6000, 51, 700), (3000, 256, 700), (9000, 40, 5000),
                                   (4000, 301, 50), (3000, 101, 2000), (2000, 1101, 60), (2500, 5, 40)])
def test_update_matches_oracle(hip, oracle, n, d, k, buckets, dtype):
    X = blobs(n, d, k, dtype, seed=7 * n + k)
    C = np.ascontiguousarray(X[RNG.choice(n, size=k, replace=False)])
    labels = RNG.integers(0, k, size=n).astype(np.int32)
    labels[labels == 1] = 0  # cluster 1 empty: must keep its old centroid
    labels[::97] = -1        # rows without a label (all distances overflowed) are skipped
    with hip.Handle(n, d, k, dtype) as h:
        h.set_data(X)
        h.set_centroids(C)
        h.set_labels(labels)
        h.set_option("buckets", buckets)
        shift2 = h.update()
        got = h.centroids()
        counts = h.counts()
    want, wcounts = oracle.update(X, labels, C)
    assert np.array_equal(counts, wcounts)
    if k > 1:
        assert np.array_equal(got[1], C[1])
    tol = 1e-5 if dtype == np.float32 else 1e-12
    assert np.allclose(got, want, rtol=tol, atol=tol * np.abs(want).max())
    ws2 = ((C.astype(np.float64) - want.astype(np.float64)) ** 2).sum()
    assert abs(shift2 - ws2) <= 1e-4 * ws2 + 1e-30


@pytest.mark.parametrize("dtype", [np.float32, np.float64])
@pytest.mark.parametrize("exact", [0, 1])
@pytest.mark.parametrize("variant,k,pairs", [
    # (lower, higher) index of two identical centroids. 7 / 36: same lane group, the later
    # 32-centroid tile on a LOWER accumulator number; 3 / 160: the same across two
    # 128-centroid blocks of the tiled kernel; 3 / 800: across two LDS chunks of a
    # row-stationary sweep (k = 1024 at d = 32 is swept in two launches)
    ("mfma_rowstat", 192, [(7, 36), (3, 160)]),
    ("mfma_tiled", 192, [(7, 36), (3, 160)]),
    ("mfma_rowstat", 1024, [(7, 36), (3, 800)]),
    ("mfma_tiled", 1024, [(7, 36), (3, 800), (100, 901)]),
])
def test_duplicate_centroids_lowest_index_wins(hip, oracle, variant, k, pairs, exact, dtype):
    """Identical centroids give bit-identical distances; the reference's strict '<'
    (kmeans_labels.h:360-377) sends every tied row to the LOWER index, so the update moves
    that centroid and leaves the higher one where it was. Well-separated blobs: no other
    near-tie exists, labels must equal the oracle's exactly and one update must match."""
    n, d = 24000, 32
    rng = np.random.default_rng(k + 11)
    centers = rng.uniform(-10, 10, size=(k, d))
    X = np.ascontiguousarray((centers[rng.integers(0, k, size=n)]
                              + 0.3 * rng.standard_normal((n, d))).astype(dtype))
    C0 = np.ascontiguousarray((centers + 0.05).astype(dtype))
    for lo, hi in pairs:
        C0[hi] = C0[lo]
    want = oracle.assign(X, C0, threads=4)
    wC, wcounts = oracle.update(X, want, C0, threads=4)
    his = [hi for _, hi in pairs]
    assert not np.isin(want, his).any() and all((want == lo).sum() > 0 for lo, _ in pairs)
    tol = 1e-5 if dtype == np.float32 else 1e-12
    for fuse in (1, 0):
        with hip.Handle(n, d, k, dtype) as h:
            h.set_data(X)
            h.set_centroids(C0)
            h.set_option("assign", variant)
            h.set_option("exact_argmin", exact)
            h.set_option("fuse", fuse)
            h.assign()
            assert np.array_equal(h.labels(), want), "assignment-only pass"
            h.iterate(1)
            got, counts, C1 = h.labels(), h.counts(), h.centroids()
        assert np.array_equal(got, want), "Lloyd step, fuse=%d" % fuse
        assert np.array_equal(counts, wcounts)
        assert np.allclose(C1, wC, rtol=tol, atol=tol * np.abs(wC).max())
        for lo, hi in pairs:
            assert np.array_equal(C1[hi], C0[hi]) and not np.array_equal(C1[lo], C0[lo])


@pytest.mark.parametrize("d,k,pairs", [
    # 7 / 36: two tiles of one wavefront; 3 / 160: the two wavefronts of a 256-centroid block;
    # 3 / 300 and 100 / 8000: different blocks
    (120, 9000, [(7, 36), (3, 160), (40, 300), (100, 8000)]),
    (520, 2304, [(7, 36), (3, 160), (40, 300), (100, 2100)]),
])
def test_duplicate_centroids_in_the_wide_block(hip, oracle, d, k, pairs):
    """The tie rule in the tiled kernel's 256-centroid form (float32 models beyond 4 MB)."""
    n = 6000
    rng = np.random.default_rng(k)
    centers = rng.uniform(-10, 10, size=(k, d))
    lab = rng.integers(0, k, size=n)
    lab[:40] = np.repeat([lo for lo, _ in pairs], 10)  # every duplicated centroid has rows
    X = np.ascontiguousarray((centers[lab] + 0.3 * rng.standard_normal((n, d))).astype(np.float32))
    C0 = np.ascontiguousarray((centers + 0.05).astype(np.float32))
    for lo, hi in pairs:
        C0[hi] = C0[lo]
    want = oracle.assign(X, C0, threads=4)
    assert not np.isin(want, [hi for _, hi in pairs]).any()
    with hip.Handle(n, d, k, np.float32) as h:
        h.set_data(X)
        h.set_centroids(C0)
        h.set_option("assign", "mfma_tiled")
        h.assign()
        assert np.array_equal(h.labels(), want)
        h.iterate(1)
        C1 = h.centroids()
    for lo, hi in pairs:
        assert np.array_equal(C1[hi], C0[hi]) and not np.array_equal(C1[lo], C0[lo])


@pytest.mark.parametrize("n,d,k,dtype,exact", [
    # float32 rows are summed in double, which is exact whatever the order: every path repeats
    (200000, 16, 8, np.float32, True), (150000, 32, 256, np.float32, True),
    (100000, 64, 64, np.float32, True), (80000, 40, 600, np.float32, True),
    # sums that do not fit LDS: rows ordered by label with a stable sort, fixed windows and
    # a fixed tree, so float64 repeats bit for bit as well
    (60000, 256, 700, np.float64, True), (60000, 256, 700, np.float32, True),
    (30000, 784, 1100, np.float32, True), (50000, 130, 1500, np.float64, True),
    # float64 rows through the LDS-privatised sums are added in arrival order inside a
    # workgroup: repeatable to rounding only
    (100000, 32, 64, np.float64, False),
])
def test_two_identical_fits_repeat(hip, n, d, k, dtype, exact):
    """The same fit twice in one process and once more on a fresh handle: labels always
    identical; centroids bit-identical wherever the sums are order-independent (float32
    rows) or taken in a fixed order (the bucketed update of large models)."""
    X = blobs(n, d, min(k, 64), dtype, spread=6.0, sigma=2.0, seed=n + d)
    C0 = np.ascontiguousarray(X[np.random.default_rng(k).choice(n, size=k, replace=False)])
    runs = []
    for fresh in range(2):
        with hip.Handle(n, d, k, dtype) as h:
            h.set_data(X)
            for _ in range(2 - fresh):
                h.set_centroids(C0)
                assert h.fit(4, 0.0) == 4
                runs.append((h.centroids(), h.labels(), h.inertia()))
    C, L, inertia = runs[0]
    for Cr, Lr, ir in runs[1:]:
        if exact:
            assert np.array_equal(Cr, C) and np.array_equal(Lr, L) and ir == inertia
        else:
            assert np.allclose(Cr, C, rtol=1e-12, atol=1e-12 * np.abs(C).max())


def separated_problem(n, d, k, dtype, seed, spread=10.0, offset=0.5):
    """Blobs plus one start per blob (true centre + offset). No blob is split by the
    start, so no row sits on a decision boundary and a last-bit difference in a
    distance cannot flip a label: end-to-end runs are then comparable to 1e-4 even
    when clusters are small. (With a split blob one flipped near-tie moves a centroid
    by |x - c| / cluster size, which for small clusters exceeds 1e-4 although both
    answers are valid.)"""
    rng = np.random.default_rng(seed)
    centers = rng.uniform(-spread, spread, size=(k, d))
    X = np.ascontiguousarray((centers[rng.integers(0, k, size=n)] + rng.standard_normal((n, d))).astype(dtype))
    C0 = np.ascontiguousarray((centers + offset).astype(dtype))
    return X, C0


@pytest.mark.parametrize("dtype", [np.float32, np.float64])
@pytest.mark.parametrize("fuse", [1, 0])
@pytest.mark.parametrize("variant", ["auto", "mfma_rowstat", "mfma_tiled"])
def test_lloyd_end_to_end(hip, oracle, variant, fuse, dtype):
    n, d, k, iters = 20000, 32, 40, 12
    X, C0 = separated_problem(n, d, k, dtype, seed=5)
    with hip.Handle(n, d, k, dtype) as h:
        h.set_data(X)
        h.set_centroids(C0)
        h.set_option("assign", variant)
        h.set_option("fuse", fuse)
        done = h.fit(iters, 0.0)
        C = h.centroids()
        labels = h.labels()
    assert done == iters
    wC, wlabels, it, _ = oracle.lloyd(X, C0, iters, 0.0, threads=4)
    assert it == iters - 1
    assert_centroids_close(C, wC, dtype)
    rep = label_report(oracle, X, wC, labels, wlabels)
    print("lloyd %s fuse=%d %s: %s" % (variant, fuse, np.dtype(dtype).name, rep))


@pytest.mark.parametrize("dtype", [np.float32, np.float64])
@pytest.mark.parametrize("variant", ["auto", "mfma_tiled"])
def test_lloyd_lockstep_random_row_start(hip, oracle, variant, dtype):
    """Random-row start (blobs get split, near-ties exist): every iteration the engine
    and the oracle start from the SAME centroids; labels must agree up to excused
    near-ties and the engine's new centroids must equal the oracle update of the
    engine's own labels."""
    n, d, k, iters = 30000, 32, 48, 8
    X = blobs(n, d, k, dtype, spread=8.0, seed=21)
    C = np.ascontiguousarray(X[np.random.default_rng(3).choice(n, size=k, replace=False)])
    tol = 1e-5 if dtype == np.float32 else 1e-12
    excused = 0
    with hip.Handle(n, d, k, dtype) as h:
        h.set_data(X)
        h.set_option("assign", variant)
        for _ in range(iters):
            h.set_centroids(C)
            h.iterate(1)
            labels = h.labels()
            Cn = h.centroids()
            rep = label_report(oracle, X, C, labels, oracle.assign(X, C, threads=4))
            excused += rep["excused"]
            wC, _ = oracle.update(X, labels, C)
            assert np.allclose(Cn, wC, rtol=tol, atol=tol * np.abs(wC).max())
            C = wC
    print("lockstep %s %s: excused near-tie rows over %d iterations: %d" %
          (variant, np.dtype(dtype).name, iters, excused))


@pytest.mark.parametrize("dtype", [np.float32, np.float64])
@pytest.mark.parametrize("n,d,k", [(30000, 32, 256), (9999, 16, 20), (5000, 64, 64), (4097, 24, 50)])
def test_fused_step_equals_separate_kernels(hip, oracle, n, d, k, dtype):
    """fit/iterate may run assign+accumulate as one kernel: same labels, same counts,
    centroids equal up to summation order, and both match the oracle step."""
    X = blobs(n, d, k, dtype, seed=3 * n + k)
    C0 = np.ascontiguousarray(X[RNG.choice(n, size=k, replace=False)])
    out = {}
    for fuse in (1, 0):
        with hip.Handle(n, d, k, dtype) as h:
            h.set_data(X)
            h.set_centroids(C0)
            h.set_option("assign", "mfma_rowstat")
            h.set_option("fuse", fuse)
            h.iterate(1)
            out[fuse] = (h.labels(), h.counts(), h.centroids())
    assert np.array_equal(out[1][0], out[0][0])
    assert np.array_equal(out[1][1], out[0][1])
    tol = 1e-5 if dtype == np.float32 else 1e-12
    assert np.allclose(out[1][2], out[0][2], rtol=tol, atol=tol * np.abs(out[0][2]).max())
    wl = oracle.assign(X, C0)
    rep = label_report(oracle, X, C0, out[1][0], wl)
    wC, wcounts = oracle.update(X, out[1][0], C0)
    assert np.array_equal(out[1][1], wcounts)
    assert np.allclose(out[1][2], wC, rtol=tol, atol=tol * np.abs(wC).max())
    print("fused step %s n=%d d=%d k=%d: %s" % (np.dtype(dtype).name, n, d, k, rep))


@pytest.mark.parametrize("dtype", [np.float32, np.float64])
@pytest.mark.parametrize("n,d,k", [(100000, 16, 8), (5001, 3, 2), (777, 64, 16), (3000, 33, 11), (256, 8, 1),
                                   (40000, 4, 16), (30001, 8, 7), (9000, 2, 4), (5000, 6, 3), (4000, 1, 2),
                                   # feature counts between the register sizes: rows that straddle the
                                   # 16-byte vectors of a block, padded and unpadded LDS rows, a last
                                   # block whose values do not fill a vector
                                   (5003, 30, 8), (777, 31, 5), (20001, 50, 16), (9001, 46, 3), (6000, 12, 9),
                                   (4099, 63, 13), (2051, 62, 4), (12345, 20, 8), (1025, 5, 2), (300, 7, 16),
                                   (255, 13, 6), (257, 15, 1), (100001, 24, 12),
                                   # large enough for the staged row-norm kernel (4M values and more)
                                   (300001, 16, 8), (140003, 30, 5), (70001, 63, 9), (1050000, 4, 3)])
def test_small_shape_fused_step_is_bit_exact(hip, oracle, n, d, k, dtype):
    """k <= 16 and d <= 64: the one-pass VALU step. Labels and minimum distances are
    bit-identical to the scalar CPU loop; float32 centroids are bit-identical to the
    oracle update (exact double sums, rounded once)."""
    X = blobs(n, d, max(k, 2), dtype, seed=n + k)
    C0 = np.ascontiguousarray(X[RNG.choice(n, size=k, replace=False)])
    res = {}
    for fuse in (1, 0):
        with hip.Handle(n, d, k, dtype) as h:
            h.set_data(X)
            h.set_centroids(C0)
            h.set_option("fuse", fuse)
            assert h.assign_variant() == "valu"
            h.iterate(1)
            res[fuse] = (h.labels(), h.min_distances(), h.counts(), h.centroids())
    wl, wm = oracle.assign(X, C0, return_mindist=True)
    wC, wcounts = oracle.update(X, wl, C0)
    for fuse in (1, 0):
        L, M, counts, C = res[fuse]
        assert np.array_equal(L, wl) and np.array_equal(M, wm) and np.array_equal(counts, wcounts)
        if dtype == np.float32:
            assert np.array_equal(C, wC)
        else:
            assert np.allclose(C, wC, rtol=1e-13, atol=1e-13)


@pytest.mark.parametrize("dtype", [np.float32, np.float64])
def test_threshold_stop(hip, oracle, dtype):
    n, d, k = 6000, 8, 5
    # one start per blob (true centre + offset): no blob is split, so no row sits
    # on a boundary and a last-bit difference cannot flip a label
    rng = np.random.default_rng(11)
    centers = rng.uniform(-20.0, 20.0, size=(k, d))
    X = np.ascontiguousarray((centers[rng.integers(0, k, size=n)] + rng.standard_normal((n, d))).astype(dtype))
    C0 = np.ascontiguousarray((centers + 0.5).astype(dtype))
    thr = 1e-3
    with hip.Handle(n, d, k, dtype) as h:
        h.set_data(X)
        h.set_centroids(C0)
        done = h.fit(200, thr)
        C = h.centroids()
        L = h.labels()
        inertia = h.inertia()
        # The convergence scalar is read one iteration behind the queue: at the stop the
        # queued iteration's update is dropped. The handle must be left exactly at the
        # stopping point: same centroids and labels from a fresh assignment pass, and
        # the next step continues from them.
        h.assign()
        assert np.array_equal(h.labels(), L) and h.inertia() == inertia
        h.iterate(1)
        C_next = h.centroids()
        # max_iterations reached while the threshold never triggers: no queued iteration
        h.set_centroids(C0)
        assert h.fit(2, 1e-30) == 2
        C2, L2 = h.centroids(), h.labels()
    wC, wL, it, hist = oracle.lloyd(X, C0, 200, thr, threads=2)
    assert done == it + 1 and done < 200
    assert_centroids_close(C, wC, dtype)
    assert np.array_equal(L, wL)
    wnext, _ = oracle.update(X, L, C)
    assert_centroids_close(C_next, wnext, dtype)
    w2C, w2L, _, _ = oracle.lloyd(X, C0, 2, 0.0, threads=2)
    assert_centroids_close(C2, w2C, dtype)
    assert np.array_equal(L2, w2L)


@pytest.mark.parametrize("dtype", [np.float32, np.float64])
@pytest.mark.parametrize("n,d,k", [(1000, 16, 8), (3000, 64, 70), (700, 300, 130), (129, 5, 17)])
def test_transform_matches_oracle(hip, oracle, n, d, k, dtype):
    X = blobs(n, d, k, dtype, seed=n)
    C = np.ascontiguousarray(X[RNG.choice(n, size=k, replace=False)])
    with hip.Handle(k, d, k, dtype) as h:
        h.set_centroids(C)
        got = h.transform(X)
    want = oracle.distances(X, C, threads=2)
    scale = (X.astype(np.float64) ** 2).sum(1).max() * 2
    eps = np.finfo(dtype).eps
    assert got.shape == (k, n)
    assert np.max(np.abs(got.astype(np.float64) - want)) <= 4 * np.sqrt(d) * eps * scale


@pytest.mark.parametrize("dtype", [np.float32, np.float64])
@pytest.mark.parametrize("n,d,k,seed", [(5000, 6, 12, 3), (20000, 32, 40, 11), (3000, 100, 25, 5), (1500, 3, 7, 0),
                                        (4000, 101, 20, 2), (2500, 7, 9, 4),
                                        (6000, 300, 12, 7), (4100, 257, 6, 8)])  # long rows: 256-row workgroups
def test_kmeanspp_seeding(hip, oracle, n, d, k, seed, dtype):
    """k-means++ on the device: same draw rule as the CPU restatement (same generator
    calls, same fixed-tree block sums), so the chosen rows agree; the minimum distances
    differ only by summation order."""
    X = blobs(n, d, k, dtype, spread=30.0, seed=n + k)
    with hip.Handle(n, d, k, dtype) as h:
        h.set_data(X)
        h.init_plusplus(seed)
        rows = h.seed_rows()
        C = h.centroids()
        mind = h.min_distances()
        h.init_plusplus(seed)
        assert np.array_equal(rows, h.seed_rows())          # deterministic per seed
    want_rows, want_mind = oracle.kmeanspp(X, k, seed)
    assert np.array_equal(C, X[rows])
    assert len(set(rows.tolist())) == k
    scale = (X.astype(np.float64) ** 2).sum(1).max() * 2
    eps = np.finfo(dtype).eps
    if np.array_equal(rows, want_rows):
        assert np.max(np.abs(mind.astype(np.float64) - want_mind)) <= 8 * np.sqrt(d) * eps * scale
    else:
        # a draw landed within rounding of a boundary between two rows: allowed, but the
        # first differing pick must be such a boundary case and quality must be the same
        i = int(np.nonzero(rows != want_rows)[0][0])
        assert i > 0
        pot_g = mind.astype(np.float64).sum()
        pot_o = want_mind.astype(np.float64).sum()
        assert abs(pot_g - pot_o) <= 0.2 * pot_o
        print("k-means++ picks diverged at pick %d of %d" % (i, k))


@pytest.mark.parametrize("dtype", [np.float32, np.float64])
@pytest.mark.parametrize("variant", ["valu", "mfma_rowstat", "mfma_tiled"])
def test_non_finite_rows_and_centroids(hip, oracle, variant, dtype):
    """NaN / infinity follow the reference's relabel rule (kmeans_labels.h:360-377): a
    distance that is not below FLT_MAX never wins, a row with no such distance gets
    label -1 and is left out of the sums; a centroid holding a NaN is never chosen;
    rows and centroids next to them are unaffected."""
    n, d, k = 2048, 32, 40
    X = blobs(n, d, k, dtype, seed=99)
    C = np.ascontiguousarray(X[RNG.choice(n, size=k, replace=False)])
    X[5, 3] = np.nan
    X[70, :] = np.nan
    X[130, 0] = np.inf
    X[131, 7] = -np.inf
    X[1999, d - 1] = np.nan
    C[4, 2] = np.nan
    C[17, :] = np.inf
    bad_rows = [5, 70, 130, 131, 1999]
    with hip.Handle(n, d, k, dtype) as h:
        h.set_data(X)
        h.set_centroids(C)
        h.set_option("assign", variant)
        if h.assign_variant() == "unsupported":
            pytest.skip("shape outside %s" % variant)
        h.assign()
        got = h.labels()
        h.update()
        counts = h.counts()
        newC = h.centroids()
    want = oracle.assign(X, C)
    assert np.all(want[bad_rows] == -1) and np.all(got[bad_rows] == -1)
    assert not np.any(np.isin(got, [4, 17])) and not np.any(np.isin(want, [4, 17]))
    good = np.ones(n, bool)
    good[bad_rows] = False
    Cf = np.delete(C, [4, 17], axis=0)   # near-tie analysis on the finite part only
    remap = np.delete(np.arange(k), [4, 17])
    inv = {int(c): i for i, c in enumerate(remap)}
    g2 = np.array([inv[int(c)] for c in got[good]], np.int32)
    w2 = np.array([inv[int(c)] for c in want[good]], np.int32)
    if variant == "valu":
        assert np.array_equal(g2, w2)
    else:
        label_report(oracle, np.ascontiguousarray(X[good]), np.ascontiguousarray(Cf), g2, w2)
    wC, wcounts = oracle.update(X, got, C)
    assert np.array_equal(counts, wcounts) and counts.sum() == n - len(bad_rows)
    keep = counts > 0
    tol = 1e-5 if dtype == np.float32 else 1e-12
    assert np.allclose(newC[keep], wC[keep], rtol=tol, atol=tol * np.abs(wC[keep]).max())
    # empty clusters (the two poisoned ones among them) keep their old coordinates, NaN included
    assert np.array_equal(newC[~keep], C[~keep], equal_nan=True)


def test_more_than_two_to_the_31_elements(hip, oracle):
    """Row offsets are 64-bit: 70,000,000 x 32 float32 (2.24e9 elements, 8.96 GB) through
    the fused step, checked on the first, middle and last rows against the oracle and by
    mass conservation."""
    n, d, k = 70_000_000, 32, 64
    rng = np.random.default_rng(31)
    centers = rng.uniform(-40, 40, size=(k, d)).astype(np.float32)
    block = 1_000_000
    base = (centers[rng.integers(0, k, size=block)] + rng.standard_normal((block, d), dtype=np.float32))
    X = np.empty((n, d), np.float32)
    for b in range(n // block):
        np.add(base, np.float32(1e-3 * b), out=X[b * block:(b + 1) * block])
    C0 = np.ascontiguousarray(centers + np.float32(0.3))
    with hip.Handle(n, d, k, np.float32) as h:
        h.set_data(X)
        h.set_centroids(C0)
        h.iterate(1)             # fused assign + sums, finalize
        C1 = h.centroids()
        counts = h.counts()
        labels = h.labels()
    assert counts.sum() == n
    for lo in (0, 34_999_000, n - 3000):
        rows = slice(lo, lo + 3000)
        want = oracle.assign(np.ascontiguousarray(X[rows]), C0)
        label_report(oracle, np.ascontiguousarray(X[rows]), C0, labels[rows], want)
    assert np.array_equal(np.bincount(labels, minlength=k), counts)
    # centroid of cluster c = mean of its rows: check two clusters in float64 on the host
    for c in (0, k - 1):
        m = X[labels == c].astype(np.float64).mean(0)
        assert np.allclose(C1[c], m, rtol=1e-5, atol=1e-4)


@pytest.mark.parametrize("dtype", [np.float32, np.float64])
@pytest.mark.parametrize("k", [130, 9000])
def test_tiled_every_feature_count(hip, k, dtype):
    """The tiled kernel deals the features of a row that is not a whole number of stages evenly
    over its stages: every feature count from 4 to 140 (and a few long ones), with the 128-centroid
    block (k = 130) and the 256-centroid one (float32 models beyond 4 MB: k = 9000 from 117
    features on), against float64 brute force. A feature left out or taken twice moves a distance
    by far more than the tolerance."""
    n = 257
    rng = np.random.default_rng(k)
    eps = np.finfo(dtype).eps
    ds = list(range(4, 141)) + [250, 271, 519, 777]
    if k > 1000:
        ds = [d for d in ds if d >= 117 and (d < 141 and d % 3 == 0 or d > 141)] + [118, 121, 125]
    bad = []
    for d in ds:
        X = np.ascontiguousarray((3.0 * rng.standard_normal((n, d))).astype(dtype))
        C = np.ascontiguousarray((3.0 * rng.standard_normal((k, d))).astype(dtype))
        with hip.Handle(n, d, k, dtype) as h:
            h.set_data(X)
            h.set_centroids(C)
            h.set_option("assign", "mfma_tiled")
            assert h.assign_variant() == "mfma_tiled"
            h.assign()
            got, mind = h.labels(), h.min_distances()
        X64, C64 = X.astype(np.float64), C.astype(np.float64)
        D = (X64 ** 2).sum(1)[:, None] + (C64 ** 2).sum(1)[None, :] - 2.0 * X64 @ C64.T
        best = D.min(1)
        scale = (X64 ** 2).sum(1).max() + (C64 ** 2).sum(1).max()
        tol = (4 * np.sqrt(d) + 40) * eps * scale
        if np.abs(mind - best).max() > tol or (D[np.arange(n), got] - best).max() > tol:
            bad.append((d, float(np.abs(mind - best).max()), float((D[np.arange(n), got] - best).max()), tol))
    assert not bad, bad


def _random_shapes(count, seed):
    """Seeded shapes spread over every dispatch rule: feature counts around the vector
    and MFMA-slice boundaries, models from one centroid to several LDS chunks."""
    rng = np.random.default_rng(seed)
    d_pool = [1, 2, 3, 4, 5, 7, 8, 9, 12, 15, 16, 17, 20, 24, 31, 32, 33, 40, 48, 63, 64, 65, 72, 96,
              100, 127, 128, 129, 160, 200, 256, 257, 300, 384, 520]
    shapes = []
    for _ in range(count):
        d = int(rng.choice(d_pool))
        k = int(rng.choice([1, 2, 3, 8, 16, 17, 31, 32, 33, 50, 64, 65, 100, 128, 129, 200, 256, 300,
                            500, 700, 1000, 1500, 2500]))
        n = int(rng.integers(max(k, 2), 12000))
        shapes.append((n, d, k))
    return shapes


@pytest.mark.parametrize("dtype", [np.float32, np.float64])
def test_one_step_on_random_shapes(hip, oracle, dtype):
    """One Lloyd step (the kernels the dispatcher picks by itself) on 60 seeded shapes and a
    dozen extreme ones (thousands of features, more centroids than fit any LDS chunking, one
    feature, one centroid):
    labels against the oracle up to excused near-ties, counts and new centroids against
    the oracle update of the engine's own labels."""
    tol = 1e-5 if dtype == np.float32 else 1e-12
    seen = {}
    extremes = [(3000, 5000, 3), (2000, 2049, 17), (30000, 3, 20000), (25000, 16, 12000), (6000, 1, 300),
                (4000, 700, 600), (5000, 1023, 129), (70000, 2, 2), (12000, 130, 4097), (9000, 64, 9000),
                (300, 4000, 300), (100000, 7, 1)]
    for (n, d, k) in _random_shapes(60, 2024) + extremes:
        X = blobs(n, d, max(k, 2), dtype, seed=n + 3 * d + 7 * k)
        C0 = np.ascontiguousarray(X[np.random.default_rng(n).choice(n, size=k, replace=False)])
        with hip.Handle(n, d, k, dtype) as h:
            h.set_data(X)
            h.set_centroids(C0)
            variant = h.assign_variant()
            h.iterate(1)
            labels, counts, C1 = h.labels(), h.counts(), h.centroids()
        where = "n=%d d=%d k=%d %s %s" % (n, d, k, variant, np.dtype(dtype).name)
        rep = label_report(oracle, X, C0, labels, oracle.assign(X, C0, threads=4))
        wC, wcounts = oracle.update(X, labels, C0)
        assert np.array_equal(counts, wcounts), where
        assert np.allclose(C1, wC, rtol=tol, atol=tol * np.abs(wC).max()), where
        seen[variant] = seen.get(variant, 0) + 1
        if rep["mismatch"]:
            print("random shape %s: %s" % (where, rep))
    assert {"valu", "mfma_rowstat", "mfma_tiled"} <= set(seen) <= {"valu", "mfma_rowstat", "mfma_tiled", "wave_row"}, seen
    if dtype == np.float32:
        assert "wave_row" in seen, seen
