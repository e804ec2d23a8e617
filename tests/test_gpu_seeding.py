"""k-means|| on the device (the reference's init_from_data == 1) against the CPU
restatement of kmeans_parallel (src/gpu/kmeans/kmeans_h2o4gpu.cu:331-563) and of its
host k-means++ over the candidates (:154-279), through the C ABI."""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu


def blobs(n, d, k, dtype, seed, spread=20.0):
    rng = np.random.default_rng(seed)
    centres = rng.uniform(-spread, spread, size=(k, d))
    return np.ascontiguousarray((centres[rng.integers(0, k, size=n)] +
                                 rng.standard_normal((n, d))).astype(dtype))


def run_device(hip, X, k, seed, variant=None, split=0):
    n, d = X.shape
    with hip.Handle(n, d, k, X.dtype) as h:
        h.set_data(X)
        if variant:
            h.set_option("assign", variant)
        h.set_option("fp32_split", split)
        h.init_parallel(seed)
        info = h.parallel_seed_info()
        info["centroids"] = h.centroids()
        info["seed_rows"] = h.seed_rows()
        h.init_parallel(seed)
        again = h.parallel_seed_info()
        assert np.array_equal(info["cand_rows"], again["cand_rows"])  # deterministic per seed
        assert np.array_equal(info["chosen"], again["chosen"])
        assert np.array_equal(info["centroids"], h.centroids())
    return info


@pytest.mark.parametrize("dtype", [np.float32, np.float64])
@pytest.mark.parametrize("n,d,k,seed", [(20000, 8, 12, 5), (9000, 16, 20, 9), (30000, 3, 40, 123),
                                        (5000, 33, 7, 1), (2500, 64, 64, 77), (294, 189, 67, 3),
                                        (3000, 300, 90, 11)])
def test_candidates_weights_and_centres_equal_the_oracle(hip, oracle, n, d, k, seed, dtype):
    """With the scalar-order distance kernel every distance is the oracle's bit for bit, the
    sum of the costs uses the same fixed tree, and the acceptance test is integer and IEEE
    arithmetic: candidates, potentials, weights and the k chosen centres must be equal."""
    X = blobs(n, d, k, dtype, seed=n + d)
    got = run_device(hip, X, k, seed, "valu")
    want = oracle.kmeans_parallel(X, k, seed, threads=4)
    assert np.array_equal(got["round_count"], want["round_count"])
    assert np.array_equal(got["cand_rows"], want["cand_rows"])
    assert np.array_equal(got["phi"], want["phi"])
    M = len(want["cand_rows"])
    assert M > k
    if k == 7:
        # three rounds, and the last one still adds candidates: no round has measured the rows
        # against those, so the engine's weights need its extra pass over them
        assert want["round_count"][2] > 0
    # (the engine takes the weights from the nearest candidate noted round by round, the
    # oracle from one pass over all candidates)
    assert np.array_equal(got["weights"], want["weights"].astype(np.float64))
    assert np.array_equal(got["chosen"], want["chosen"])
    assert np.array_equal(got["centroids"], want["centroids"])
    assert np.array_equal(got["seed_rows"], want["cand_rows"][want["chosen"]])


@pytest.mark.parametrize("dtype,split", [(np.float32, 0), (np.float64, 0), (np.float32, 6)])
@pytest.mark.parametrize("n,d,k,seed", [(20000, 32, 64, 3), (6000, 200, 300, 4), (12000, 128, 40, 8)])
def test_matrix_core_rounds_differ_only_at_the_threshold(hip, oracle, n, d, k, seed, dtype, split):
    """The matrix-core kernels sum the dot products in another order (with the bfloat16-parts
    option as well), so a cost can differ from the oracle's in its last bits: a row may then
    fall on the other side of its threshold only when 2k * cost / potential is within rounding
    of it."""
    X = blobs(n, d, k, dtype, seed=n + d)
    got = run_device(hip, X, k, seed, split=split)
    want = oracle.kmeans_parallel(X, k, seed, threads=4)
    thr = np.array([oracle.row_threshold(seed, int(r)) for r in range(n)], np.float64)
    C = got["centroids"]
    assert np.array_equal(C, X[got["cand_rows"][got["chosen"]]])
    assert len(set(got["chosen"].tolist())) == k
    if np.array_equal(got["cand_rows"], want["cand_rows"]):
        # (a row that is a candidate itself costs exactly 0 in the oracle, where both norms and
        # the dot product are the same sum, and a rounding residue of a few eps * 2|x|^2 on the
        # matrix cores: with a third of the rows among the candidates the potentials of the
        # late rounds differ by about 1e-5)
        assert np.allclose(got["phi"], want["phi"], rtol=3e-5 if dtype == np.float32 else 1e-12)
        # cells: a row between two candidates may be counted for either
        assert np.abs(got["weights"] - want["weights"]).sum() <= max(4, n // 1000)
        if np.array_equal(got["weights"], want["weights"].astype(np.float64)):
            assert np.array_equal(got["chosen"], want["chosen"])
        return
    # first round whose lists differ: every differing row must sit on its threshold
    pos = 1
    X64 = X.astype(np.float64)
    running = np.full(n, np.inf)
    known = [int(want["cand_rows"][0])]
    tol = 1e-4 if dtype == np.float32 else 1e-10
    for r in range(8):
        a = got["cand_rows"][pos:pos + got["round_count"][r]]
        b = want["cand_rows"][pos:pos + want["round_count"][r]]
        running = np.minimum(running, ((X64[:, None, :] - X64[known][None, :, :]) ** 2).sum(-1).min(1))
        if not np.array_equal(a, b):
            odd = np.setxor1d(a, b)
            prob = 2.0 * k * running[odd] / running.sum()
            assert (np.abs(prob - thr[odd]) <= tol * (1 + thr[odd])).all()
            return
        known = [int(v) for v in b] if len(b) else known
        pos += len(b)


@pytest.mark.parametrize("dtype", [np.float32, np.float64])
@pytest.mark.parametrize("n,d,k,seed", [(20000, 32, 64, 3), (6000, 200, 300, 4), (3000, 7, 5, 2)])
def test_picks_from_the_distance_matrix_and_from_a_kernel_per_pick_agree(hip, n, d, k, seed, dtype):
    """The centres are picked either from one matrix of all distances between candidates
    (the default) or with one kernel per pick (models whose matrix exceeds 1 GiB; option
    seed_matrix = 0): the two sum the dot products in different orders, so the picks are the same
    until two candidates' weighted distances tie within rounding (every later pick then depends
    on which of the two was taken)."""
    X = blobs(n, d, k, dtype, seed=n + d)
    res = []
    for matrix in (1, 0):
        with hip.Handle(n, d, k, dtype) as h:
            h.set_data(X)
            h.set_option("seed_matrix", matrix)
            h.init_parallel(seed)
            info = h.parallel_seed_info()
            res.append((info["cand_rows"], info["weights"], info["chosen"], h.centroids()))
    assert len(res[0][0]) > k  # more candidates than centres: the picks do run
    assert np.array_equal(res[0][0], res[1][0]) and np.array_equal(res[0][1], res[1][1])
    ca, cb = res[0][2], res[1][2]
    assert len(set(ca.tolist())) == k and len(set(cb.tolist())) == k
    if np.array_equal(ca, cb):
        assert np.array_equal(res[0][3], res[1][3])
        return
    p = int(np.argmax(ca != cb))  # first pick that differs: a tie within rounding
    assert p > 0
    cand = X[res[0][0]].astype(np.float64)
    w = res[0][1].astype(np.float64).copy()
    w[ca[:p]] = 0
    best = ((cand[:, None, :] - cand[ca[:p]][None, :, :]) ** 2).sum(-1).min(1)
    val = w * best
    tol = 1e-4 if dtype == np.float32 else 1e-10
    assert abs(val[ca[p]] - val[cb[p]]) <= tol * val.max(), (p, val[ca[p]], val[cb[p]], val.max())


@pytest.mark.parametrize("dtype", [np.float32, np.float64])
@pytest.mark.parametrize("n,d,k,seed", [(40000, 32, 64, 3), (9000, 200, 300, 4), (25000, 16, 24, 6),
                                        (15000, 100, 600, 2)])
def test_default_path_weights_equal_one_pass_over_all_candidates(hip, oracle, n, d, k, seed, dtype):
    """The weights come from the nearest candidate noted round by round, and with the default
    (matrix-core) kernels every round's model has another size and may run another kernel family,
    so a row's distances to candidates of different rounds need not be summed alike. The
    reference counts the rows per nearest candidate in ONE pass over all candidates
    (count_pts_per_centroid, kmeans_h2o4gpu.h:90-126): the engine's weights may differ from that
    pass only by rows whose two nearest candidates are a near-tie (1e-5 relative gap, or the
    rounding floor 8 eps (|x|^2 + |c|^2) of the expanded form), each of which moves one unit
    of weight from one candidate to another."""
    X = blobs(n, d, k, dtype, seed=n + d + 1, spread=6.0)
    with hip.Handle(n, d, k, dtype) as h:
        h.set_data(X)
        h.init_parallel(seed)
        info = h.parallel_seed_info()
    cand = np.ascontiguousarray(X[info["cand_rows"]])
    M = cand.shape[0]
    assert M > k and info["weights"] is not None
    assert info["weights"].sum() == n
    one_pass = oracle.assign(X, cand, threads=8)
    want = np.bincount(one_pass, minlength=M).astype(np.float64)
    moved = np.abs(info["weights"] - want).sum()
    best, d1, d2 = oracle.top2_exact(X, cand, threads=8)
    xx = (X.astype(np.float64) ** 2).sum(1)
    floor = 8 * float(np.finfo(dtype).eps) * 2 * xx            # (candidates are rows: |c|^2 ~ |x|^2)
    near_tie = ((d2 - d1) <= 1e-5 * d2) | ((d2 - d1) <= floor)
    assert moved <= 2 * int(near_tie.sum()), (moved, int(near_tie.sum()))


def test_fit_entry_point_seeds_with_kmeans_parallel(hip, oracle):
    """init_from_data == 1 through make_ptr_float_kmeans; zero iterations return the seeds."""
    from h2o4gpu_amd.libs import ch2o4gpu_gpu
    n, d, k, seed = 8000, 12, 10, 21
    X = blobs(n, d, k, np.float32, seed=5)
    centres = np.zeros(k * d, np.float32)
    labels = np.zeros(n, np.int32)
    rc = ch2o4gpu_gpu.make_ptr_float_kmeans(0, 0, seed, 0, 1, n, d, k, 0, 1, 0.0, X.flatten(),
                                            np.empty([], np.float32), centres, labels)
    assert rc == 0
    # no iteration, no relabel: the labels are the zeros the reference's vector starts with
    # (kmeans_h2o4gpu.cu:747), not what the seeding left in its scratch
    assert not labels.any()
    with hip.Handle(n, d, k, np.float32) as h:
        h.set_data(X)
        h.init_parallel(seed)
        assert np.array_equal(centres.reshape(k, d), h.centroids())
        assert not h.labels().any()
        with pytest.raises(hip.KMeansHipError):
            h.inertia()
    want = oracle.kmeans_parallel(X, k, seed, threads=4)
    assert np.array_equal(centres.reshape(k, d), want["centroids"])
    # and a real fit from that start lowers the objective below the seeds' own
    rc = ch2o4gpu_gpu.make_ptr_float_kmeans(0, 0, seed, 0, 1, n, d, k, 10, 1, 0.0, X.flatten(),
                                            np.empty([], np.float32), centres, labels)
    assert rc == 0
    _, mind0 = oracle.assign(X, want["centroids"], return_mindist=True)
    _, mind1 = oracle.assign(X, centres.reshape(k, d), return_mindist=True)
    assert mind1.sum(dtype=np.float64) < mind0.sum(dtype=np.float64)


def test_fewer_candidates_than_centres(hip, oracle):
    """kmeans_h2o4gpu.cu:536-540: the candidates become the first centres, zero rows follow."""
    X = blobs(6, 4, 3, np.float32, seed=1)
    k, seed = 6, 7
    got = run_device(hip, X, k, seed)
    want = oracle.kmeans_parallel(X, k, seed)
    M = len(want["cand_rows"])
    assert M <= k and got["weights"] is None
    assert np.array_equal(got["cand_rows"], want["cand_rows"])
    assert np.array_equal(got["centroids"], want["centroids"])
    assert got["seed_rows"].tolist() == want["cand_rows"].tolist() + [-1] * (k - M)


def test_estimator_names_for_the_seeding(hip):
    import h2o4gpu_amd
    X = blobs(4000, 10, 6, np.float32, seed=3)
    a = h2o4gpu_amd.KMeans(n_clusters=6, init="k-means++", max_iter=5, tol=0, random_state=4).fit(X)
    b = h2o4gpu_amd.KMeans(n_clusters=6, init="k-means||", max_iter=5, tol=0, random_state=4).fit(X)
    c = h2o4gpu_amd.KMeans(n_clusters=6, init="d2-sampling", max_iter=5, tol=0, random_state=4).fit(X)
    assert np.array_equal(a.cluster_centers_, b.cluster_centers_)
    assert c.cluster_centers_.shape == a.cluster_centers_.shape
    with pytest.raises(ValueError):
        h2o4gpu_amd.KMeans(n_clusters=6, init="farthest")
