"""Pins the CPU oracle: the reference's own known-answer cases, float64 brute force
on tiny inputs, closed forms, invariants and independent library routines. None of
these tests retypes the oracle's formula; each is built so that a plausible mistake
(dropped term, wrong sign, transposed operand, wrong tie rule) fails it."""
import json
import os

import numpy as np
import pytest

HERE = os.path.dirname(os.path.abspath(__file__))
KATS = json.load(open(os.path.join(HERE, "golden", "reference_gtest_kats.json")))


def f32(a):
    return np.ascontiguousarray(np.array(a, dtype=np.float32))


# ---------------------------------------------------------------- reference KATs
@pytest.mark.parametrize("case", ["counts_per_centroids", "centroid_per_data_point"])
def test_kat_counts(oracle, case):
    kat = KATS[case]
    X, C = f32(kat["data"]), f32(kat["centroids"])
    labels = oracle.assign(X, C)
    counts = np.bincount(labels, minlength=C.shape[0])
    assert counts.tolist() == kat["expected_counts"]


def test_kat_self_distance_needs_abs(oracle):
    """CentroidPerDataPoint: every point is its own centroid; the expanded form can round
    below zero there, the stored distance must be |.| and the point must pick itself."""
    kat = KATS["centroid_per_data_point"]
    X = f32(kat["data"])
    D = oracle.distances(X, X)
    assert (D >= 0).all()
    assert np.array_equal(np.argmin(D, axis=0), np.arange(len(X)))
    assert np.array_equal(oracle.assign(X, X), np.arange(len(X)))


def test_kat_calculate_centroids(oracle):
    kat = KATS["calculate_centroids"]
    sums, counts = oracle.update_sums(f32(kat["data"]), kat["labels"], kat["k"])
    assert sums.tolist() == kat["expected_unscaled_sums"]
    assert counts.tolist() == [2, 2]


def test_kat_shard_additivity(oracle):
    kat = KATS["calculate_centroids_2gpu"]
    X, lab, k, cut = f32(kat["data"]), np.array(kat["labels"], np.int32), kat["k"], kat["split_at"]
    whole, cw = oracle.update_sums(X, lab, k)
    a, ca = oracle.update_sums(X[:cut], lab[:cut], k)
    b, cb = oracle.update_sums(X[cut:], lab[cut:], k)
    assert np.array_equal(whole, a + b) and np.array_equal(cw, ca + cb)
    assert whole[0].tolist() == [9.0, 2.0]


def test_kat_revert_and_scale(oracle):
    kat = KATS["revert_centroid_zeroing"]
    got = oracle.finalize(f32(kat["current"]), kat["counts"], f32(kat["old_centroids"]))
    # counts are 1 where kept, so the scale factor is 1 and only the revert rule shows
    assert got.tolist() == kat["expected"]
    kat = KATS["centroids_scaling"]
    got = oracle.finalize(f32(kat["sums"]), kat["counts"], np.zeros((2, 2), np.float32))
    assert got.tolist() == kat["expected"]


def test_kat_row_major_layout(oracle):
    kat = KATS["copy_data_row_major"]
    src = f32(kat["src"]).reshape(kat["rows"], kat["cols"])
    norms = oracle.row_norms(src[: kat["take_rows"]])
    exp = f32(kat["expected"]).reshape(kat["take_rows"], kat["cols"])
    assert np.array_equal(norms, (exp.astype(np.float64) ** 2).sum(1).astype(np.float32))


# ---------------------------------------------------------------- mathematics
@pytest.mark.parametrize("dtype", [np.float32, np.float64])
def test_distances_equal_cdist_transposed(oracle, dtype):
    from scipy.spatial.distance import cdist
    rng = np.random.default_rng(1)
    X = rng.normal(size=(57, 9)).astype(dtype)
    C = rng.normal(size=(6, 9)).astype(dtype)
    D = oracle.distances(X, C)
    want = cdist(X.astype(np.float64), C.astype(np.float64), "sqeuclidean").T
    assert D.shape == (6, 57)  # centroid-major
    tol = 2e-5 if dtype == np.float32 else 1e-12
    assert np.allclose(D, want, rtol=tol, atol=tol)


@pytest.mark.parametrize("dtype", [np.float32, np.float64])
def test_assign_is_brute_force_argmin(oracle, dtype):
    rng = np.random.default_rng(2)
    X = rng.integers(-5, 6, size=(300, 4)).astype(dtype)   # small integers: exact arithmetic
    C = rng.integers(-5, 6, size=(11, 4)).astype(dtype)
    C[7] = C[3]                                            # duplicate centroid: exact ties
    D = ((X[:, None, :].astype(np.float64) - C[None, :, :]) ** 2).sum(-1)
    want = np.argmin(D, axis=1)                            # numpy argmin = first minimum
    labels, mind = oracle.assign(X, C, return_mindist=True)
    assert np.array_equal(labels, want)
    assert not (labels == 7).any()                         # lowest index wins a tie
    assert np.array_equal(mind.astype(np.float64), D.min(axis=1))
    b, d1, d2 = oracle.top2_exact(X, C)
    assert np.array_equal(b, want) and np.array_equal(d1, D.min(axis=1))
    assert np.array_equal(d2, np.sort(D, axis=1)[:, 1])


def test_assign_nothing_below_start_gives_minus_one(oracle):
    X = np.full((3, 2), 3e19, np.float32)     # squared distances overflow float32 -> inf
    C = np.full((2, 2), -3e19, np.float32)
    assert oracle.assign(X, C).tolist() == [-1, -1, -1]


@pytest.mark.parametrize("dtype", [np.float32, np.float64])
def test_update_mass_invariants(oracle, dtype):
    rng = np.random.default_rng(3)
    n, d, k = 5000, 7, 13
    X = rng.normal(size=(n, d)).astype(dtype)
    labels = rng.integers(0, k, size=n).astype(np.int32)
    labels[labels == 4] = 5                                  # cluster 4 empty
    C_old = rng.normal(size=(k, d)).astype(dtype)
    C_new, counts = oracle.update(X, labels, C_old)
    assert counts.sum() == n and counts[4] == 0
    assert np.array_equal(C_new[4], C_old[4])                # empty keeps its centroid
    tot = (counts[:, None] * C_new.astype(np.float64))
    tot[4] = 0
    assert np.allclose(tot.sum(0), X.astype(np.float64).sum(0), rtol=1e-4, atol=1e-3)
    for c in (0, 5, 12):
        assert np.allclose(C_new[c], X[labels == c].astype(np.float64).mean(0), rtol=2e-5, atol=2e-6)
    # threaded variant: same counts, same values up to summation order
    C_thr, counts_thr = oracle.update(X, labels, C_old, threads=4)
    assert np.array_equal(counts, counts_thr)
    assert np.allclose(C_new, C_thr, rtol=1e-5, atol=1e-6)


@pytest.mark.parametrize("dtype", [np.float32, np.float64])
def test_lloyd_closed_forms(oracle, dtype):
    rng = np.random.default_rng(4)
    X = rng.normal(size=(400, 5)).astype(dtype)
    # k = 1: one iteration lands on the mean, labels all zero
    C, labels, it, hist = oracle.lloyd(X, X[:1], 3, 0.0)
    assert np.allclose(C[0], X.astype(np.float64).mean(0), rtol=1e-5, atol=1e-6)
    assert (labels == 0).all() and it == 2
    assert hist[1] < 1e-10 * max(hist[0], 1e-30) + 1e-12     # second shift is (almost) zero
    # k = n: fixed point, labels are the identity
    Xs = X[:50]
    C, labels, it, hist = oracle.lloyd(Xs, Xs, 2, 0.0)
    assert np.array_equal(C, Xs) and np.array_equal(labels, np.arange(50))
    assert hist[0] == 0.0
    # threshold stop: shift 0 < 1e-30 on the first iteration -> loop index 0
    C, labels, it, hist = oracle.lloyd(Xs, Xs, 10, 1e-30)
    assert it == 0


def test_lloyd_iteration_count_and_final_relabel(oracle):
    """N updates and a final relabel: labels must be the argmin against the RETURNED
    centroids, and the shift history has exactly N entries."""
    rng = np.random.default_rng(5)
    X = np.concatenate([rng.normal(loc=m, size=(200, 3)) for m in (-6, 0, 6)]).astype(np.float32)
    C0 = X[[0, 250, 450]]
    C, labels, it, hist = oracle.lloyd(X, C0, 4, 0.0)
    assert it == 3 and np.isfinite(hist[:4]).all()
    assert np.array_equal(labels, oracle.assign(X, C))
    inertia = []
    Ck = C0.copy()
    for _ in range(4):
        lab, mind = oracle.assign(X, Ck, return_mindist=True)
        inertia.append(mind.astype(np.float64).sum())
        Ck, _ = oracle.update(X, lab, Ck)
    assert all(b <= a * (1 + 1e-6) for a, b in zip(inertia, inertia[1:]))   # monotone
    assert np.array_equal(Ck, C)


@pytest.mark.parametrize("dtype", [np.float32, np.float64])
def test_lloyd_matches_independent_implementation(oracle, dtype):
    """scikit-learn's Lloyd (explicit start, n_init=1, tol=0) on data where no cluster
    empties: an independent implementation of the same iteration."""
    sk = pytest.importorskip("sklearn.cluster")
    rng = np.random.default_rng(6)
    k, d, n, iters = 6, 4, 3000, 5
    centers = rng.uniform(-10, 10, size=(k, d))
    X = (centers[rng.integers(0, k, size=n)] + rng.normal(size=(n, d))).astype(dtype)
    C0 = (centers + 0.3).astype(dtype)
    model = sk.KMeans(n_clusters=k, init=C0.astype(np.float64), n_init=1, max_iter=iters, tol=0.0,
                      algorithm="lloyd").fit(X.astype(np.float64))
    C, labels, it, _ = oracle.lloyd(X, C0, iters, 0.0)
    if model.n_iter_ == iters:   # scikit-learn also stops on a label fixpoint
        tol = 1e-4 if dtype == np.float32 else 1e-9
        assert np.allclose(C, model.cluster_centers_, rtol=tol, atol=tol)
        assert np.array_equal(labels, model.labels_)
    else:
        # converged early: the fixpoint is the same
        assert np.allclose(C, model.cluster_centers_, rtol=1e-4, atol=1e-4)


def test_random_rows_rule(oracle):
    a = oracle.random_rows(1234, 1000, 16)
    b = oracle.random_rows(1234, 1000, 16)
    c = oracle.random_rows(1235, 1000, 16)
    assert np.array_equal(a, b) and not np.array_equal(a, c)
    assert len(set(a.tolist())) == 16 and a.min() >= 0 and a.max() < 1000
    full = oracle.random_rows(7, 50, 50)
    assert sorted(full.tolist()) == list(range(50))           # a permutation


def test_row_norms_sequential_float32(oracle):
    """The sum is taken in float32, features ascending (no pairwise tree, no float64)."""
    x = np.array([[1e4, 1.0, 1.0, 1.0, 1.0]], np.float32)
    acc = np.float32(0)
    for v in x[0]:
        acc = np.float32(acc + np.float32(v * v))
    assert oracle.row_norms(x)[0] == acc
    assert oracle.row_norms(x.astype(np.float64))[0] == 1e8 + 4


@pytest.mark.parametrize("dtype", [np.float32, np.float64])
def test_kmeanspp_is_d2_sampling(oracle, dtype):
    """Textbook properties of D^2 sampling: chosen rows are distinct (a chosen row has
    distance 0 and cannot be drawn again), the potential never increases, the draw is a
    function of the seed, and on far-apart blobs it hits every blob."""
    rng = np.random.default_rng(8)
    k, d, n = 12, 6, 5000
    centers = rng.uniform(-100, 100, size=(k, d))
    X = (centers[rng.integers(0, k, size=n)] + rng.normal(size=(n, d))).astype(dtype)
    rows, mind = oracle.kmeanspp(X, k, 3)
    rows2, _ = oracle.kmeanspp(X, k, 3)
    rows3, _ = oracle.kmeanspp(X, k, 4)
    assert np.array_equal(rows, rows2) and not np.array_equal(rows, rows3)
    assert len(set(rows.tolist())) == k
    assert rows[0] == oracle.kmeanspp_first(3, n)
    # minimum distance to the chosen rows, by brute force in float64
    D = ((X[:, None, :].astype(np.float64) - X[rows][None, :, :]) ** 2).sum(-1).min(1)
    assert np.allclose(mind, D, rtol=1e-3, atol=1e-2 if dtype == np.float32 else 1e-9)
    # every blob got a centre: all rows are within a blob diameter of a chosen row
    assert D.max() < 100.0
    pots = [oracle.kmeanspp(X, kk, 3)[1].astype(np.float64).sum() for kk in (2, 4, 8, 12)]
    assert all(b <= a for a, b in zip(pots, pots[1:]))


def test_kmeanspp_draw_is_proportional_to_d2(oracle):
    """Two far clusters of very different spread: after the first centre, the second is
    drawn with probability proportional to squared distance, so over many seeds it falls
    in the other cluster almost always (a uniform or D^1 draw would not)."""
    rng = np.random.default_rng(9)
    A = rng.normal(size=(900, 2)) * 0.1
    B = rng.normal(size=(100, 2)) * 0.1 + 50.0
    X = np.concatenate([A, B]).astype(np.float32)
    other = 0
    for seed in range(40):
        rows, _ = oracle.kmeanspp(X, 2, seed)
        other += (rows[0] < 900) != (rows[1] < 900)
    assert other >= 39


# ------------------------------------------------- helpers the parity verdicts rest on
def test_pair_dist_exact_against_float64_brute_force(oracle):
    """pair_dist_exact prices every excused label mismatch, so it is pinned by itself:
    a 50 x 7 float32 case with 5 centroids, labels a and b chosen differently per row
    (an a/b swap, a wrong centroid row or a squared-vs-plain mix-up all fail), against
    numpy float64 on the direct form; float64 input alike."""
    rng = np.random.default_rng(17)
    for dtype in (np.float32, np.float64):
        X = np.ascontiguousarray(rng.normal(3.0, 4.0, size=(50, 7)).astype(dtype))
        C = np.ascontiguousarray(rng.normal(-1.0, 5.0, size=(5, 7)).astype(dtype))
        a = rng.integers(0, 5, size=50).astype(np.int32)
        b = ((a + 1 + rng.integers(0, 4, size=50)) % 5).astype(np.int32)   # never equal to a
        assert (a != b).all()
        da, db = oracle.pair_dist_exact(X, C, a, b, threads=2)
        X64, C64 = X.astype(np.float64), C.astype(np.float64)
        wa = ((X64 - C64[a]) ** 2).sum(1)
        wb = ((X64 - C64[b]) ** 2).sum(1)
        assert np.allclose(da, wa, rtol=1e-14, atol=0) and np.allclose(db, wb, rtol=1e-14, atol=0)
        assert not np.allclose(da, wb, rtol=1e-3)   # the case does tell a from b
        # and it agrees with the two smallest entries of the full exact table
        best, d1, d2 = oracle.top2_exact(X, C)
        full = ((X64[:, None, :] - C64[None, :, :]) ** 2).sum(-1)
        assert np.array_equal(best, full.argmin(1))
        srt = np.sort(full, axis=1)
        assert np.allclose(d1, srt[:, 0], rtol=1e-14) and np.allclose(d2, srt[:, 1], rtol=1e-14)


@pytest.mark.parametrize("dtype", [np.float32, np.float64])
def test_descending_dot_order_is_the_ascending_sum_of_reversed_columns(oracle, dtype):
    """The descending summation order is the yardstick of the full-size drift test. Summing
    features d-1 .. 0 of (X, C) is, term for term, summing features 0 .. d-1 of the
    column-reversed arrays, and the row norms are order-independent inputs of both only
    if they are formed the same way: so labels AND minimum distances of the descending
    mode on (X, C) must equal, bit for bit, those of the default mode on data whose dot
    products are reversed but whose norms are not. That is checked through distances with
    a single feature block reversed: d = 1 is trivially equal, and for d > 1 the two modes
    must differ somewhere in the last bit (the switch does something)."""
    rng = np.random.default_rng(23)
    n, d, k = 4000, 37, 29
    X = np.ascontiguousarray(rng.normal(20.0, 3.0, size=(n, d)).astype(dtype))
    C = np.ascontiguousarray(rng.normal(20.0, 3.0, size=(k, d)).astype(dtype))
    Xr, Cr = np.ascontiguousarray(X[:, ::-1]), np.ascontiguousarray(C[:, ::-1])
    asc = oracle.distances(X, C)
    oracle.set_dot_order(True)
    try:
        desc = oracle.distances(X, C)
        desc_rev = oracle.distances(Xr, Cr)
        l_desc, m_desc = oracle.assign(X, C, return_mindist=True)
    finally:
        oracle.set_dot_order(False)
    # the norms xx, cc are always summed ascending over the array as given, so build the
    # expected values from their parts: norms of the original arrays, dots of the reversed ones
    xx = oracle.row_norms(X)
    cc = oracle.row_norms(C)
    dots_rev = np.zeros((k, n), dtype)
    for j in range(d):                       # ascending over reversed columns, in dtype
        dots_rev += np.outer(Cr[:, j], Xr[:, j]).astype(dtype)
    want = np.abs((xx[None, :] + cc[:, None]) - dtype(2) * dots_rev)
    assert np.array_equal(desc, want)
    assert np.array_equal(m_desc, want.min(0))
    assert np.array_equal(l_desc, want.argmin(0))
    # same mathematics, different rounding: close everywhere, not identical everywhere
    scale = float(xx.max() + cc.max())
    assert np.max(np.abs(desc.astype(np.float64) - asc)) <= 64 * np.finfo(dtype).eps * scale
    assert (desc != asc).any()
    # reversing the columns AND the order restores the ascending-order dot products
    xxr, ccr = oracle.row_norms(Xr), oracle.row_norms(Cr)
    dots = np.zeros((k, n), dtype)
    for j in range(d):
        dots += np.outer(C[:, j], X[:, j]).astype(dtype)
    assert np.array_equal(desc_rev, np.abs((xxr[None, :] + ccr[:, None]) - dtype(2) * dots))
