"""Pins the oracle's restatement of the reference's k-means|| seeding
(kmeans_parallel, src/gpu/kmeans/kmeans_h2o4gpu.cu:331-563, and the host k-means++ over the
candidates, :154-279) by what can be fixed without a CUDA build:

* the random streams: published known answers of the two generators, the row thresholds
  against rocThrust's own host code (the same header text CUDA thrust ships), the host
  sampler's thresholds against an independent MT19937 (numpy's);
* pick_point_idx_weighted: small cases worked out from the thresholds alone;
* the rounds: every candidate recomputed from float64 brute-force distances and the row
  thresholds; candidates are rows of the data, found in row order, the potential never grows;
* the reduction to k centres: weights are the sizes of the nearest-candidate cells.

Parity against a run of the reference itself stays unpinned: the distances come out of
cuBLAS there and the sum of the minima out of thrust::reduce, both in an unspecified order."""
import os
import shutil
import subprocess
import tempfile

import numpy as np
import pytest


# ---------------------------------------------------------------- generators
def test_minstd_known_answer(oracle):
    """[rand.predef]: the 10000th call of a default-constructed minstd_rand (seed 1) is
    399268537; thrust documents the same value for its minstd_rand."""
    assert oracle.minstd_nth(1, 10000) == 399268537
    # seed 0 is replaced by 1 (a zero state would stay zero)
    assert oracle.minstd_nth(0, 10000) == 399268537
    # one step by hand: 48271 * 7 mod (2^31 - 1)
    assert oracle.minstd_nth(7, 1) == 48271 * 7
    assert oracle.minstd_nth(123456789, 2) == (123456789 * 48271 % 2147483647) * 48271 % 2147483647
    # a negative seed converts to uint32 first
    assert oracle.minstd_nth(-5, 1) == ((2 ** 32 - 5) % 2147483647) * 48271 % 2147483647


ROCTHRUST_PROBE = r"""
#include <thrust/random.h>
#include <cstdio>
#include <cstdlib>
// the three calls of the reference's acceptance test for one row
int main(int argc, char **argv) {
  for (int a = 1; a + 1 < argc; a += 2) {
    const int seed = atoi(argv[a]);
    const long long row = atoll(argv[a + 1]);
    thrust::default_random_engine rng(seed);
    thrust::uniform_real_distribution<> dist(0.0, 1.0);
    rng.discard(row);
    const float u = dist(rng);
    printf("%.9g\n", u);
  }
  return 0;
}
"""


def test_row_thresholds_equal_rocthrust_host_code(oracle):
    hipcc = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    if not os.path.exists(hipcc):
        pytest.skip("no hipcc: rocThrust's host code cannot be compiled")
    cases = [(1, 0), (1, 1), (77, 0), (77, 5), (12345, 99999), (2147483647, 3), (0, 17), (-3, 1000),
             (987654321, 1234567)]
    with tempfile.TemporaryDirectory() as tmp:
        src = os.path.join(tmp, "probe.cpp")
        exe = os.path.join(tmp, "probe")
        open(src, "w").write(ROCTHRUST_PROBE)
        r = subprocess.run([hipcc, "-O1", "-std=c++17", "--offload-arch=gfx950", "-w", src, "-o", exe],
                           capture_output=True, text=True)
        if r.returncode != 0:
            pytest.skip("rocThrust probe does not compile here: " + r.stderr[-300:])
        args = [str(v) for c in cases for v in c]
        out = subprocess.run([exe] + args, capture_output=True, text=True, check=True).stdout.split()
    want = np.array([float(v) for v in out], np.float32)
    got = np.array([oracle.row_threshold(s, r) for s, r in cases], np.float32)
    assert np.array_equal(got, want), (got, want)
    assert ((got >= 0) & (got <= 1)).all()


def mt19937_raw(seed, count):
    """Raw 32-bit outputs of std::mt19937(seed), from numpy's independent implementation
    (the legacy RandomState seeds with the same init_genrand)."""
    rs = np.random.RandomState(seed)
    return [int(v) for v in rs.randint(0, 2 ** 32, size=count, dtype=np.uint64)]


def std_uniform01(seed, count):
    """std::uniform_real_distribution<double>(0,1) over mt19937(seed): libstdc++ forms
    (x0 + x1 * 2^32) / 2^64 from two calls, rounded to double once."""
    raw = mt19937_raw(seed, 2 * count)
    out = []
    for i in range(count):
        v = float(raw[2 * i] + raw[2 * i + 1] * 2 ** 32) / 2.0 ** 64
        out.append(np.nextafter(1.0, 0.0) if v >= 1.0 else v)
    return np.array(out)


def test_mt19937_emulation_known_answer():
    """[rand.predef]: the 10000th call of a default-constructed mt19937 (seed 5489)."""
    assert mt19937_raw(5489, 10000)[-1] == 4123659995


# ---------------------------------------------------------------- pick_point_idx_weighted
@pytest.mark.parametrize("dtype", [np.float32, np.float64])
def test_pick_point_first_share_above_its_threshold(oracle, dtype):
    seed = 42
    u = std_uniform01(seed, 8).astype(dtype)
    # shares w_i / sum(w); entry i is taken when its share exceeds the i-th draw
    for trial in range(20):
        rng = np.random.default_rng(trial)
        w = rng.integers(1, 50, size=8).astype(dtype)
        share = w / w.sum(dtype=dtype)
        hits = np.nonzero(share > u)[0]
        if len(hits):
            want = int(hits[0])
        else:  # last entry that reached the running maximum
            best, want = dtype(0), 0
            for i, s in enumerate(share):
                if s >= best:
                    best, want = s, i
        assert oracle.pick_point_idx_weighted(seed, w) == want
    # an entry holding the whole weight is taken at once when it comes first ...
    assert oracle.pick_point_idx_weighted(seed, np.array([5, 0, 0], dtype)) == 0
    # ... and whatever the draws are when it comes later (share 1 > u in [0, 1))
    assert oracle.pick_point_idx_weighted(seed, np.array([0, 0, 9, 0], dtype)) == 2
    # equal small shares that never exceed a draw: the LAST of the maxima (>=, not >)
    small = np.full(8, 1, dtype)
    if not (small / small.sum() > u).any():
        assert oracle.pick_point_idx_weighted(seed, small) == 7


def test_pick_point_weights_times_distances(oracle):
    seed = 3
    u = std_uniform01(seed, 4)
    w = np.array([2.0, 1.0, 4.0, 3.0])
    dist = np.array([0.0, 10.0, 0.5, 2.0])
    share = w * dist / float((w * dist).sum())
    hits = np.nonzero(share > u)[0]
    want = int(hits[0]) if len(hits) else int(np.nonzero(share == share.max())[0][-1])
    assert oracle.pick_point_idx_weighted(seed, w, dist) == want
    # swapping the two arrays' roles gives the same product: same answer
    assert oracle.pick_point_idx_weighted(seed, dist, w) == want
    # every draw is taken afresh for every call: same arguments, same answer
    assert oracle.pick_point_idx_weighted(seed, w, dist) == want


def test_weighted_kmeanspp_on_a_line(oracle):
    """Four candidates on a line, worked by hand from the thresholds: the first centre comes
    from the weights alone, a chosen candidate has weight 0 afterwards, and the running
    minimum uses the expanded form without an absolute value."""
    seed = 11
    u = std_uniform01(seed, 4)
    data = np.array([[0.0], [1.0], [10.0], [11.0]])
    w = np.array([3.0, 1.0, 2.0, 4.0])

    def pick(values):
        share = values / values.sum()
        hits = np.nonzero(share > u[:len(values)])[0]
        if len(hits):
            return int(hits[0])
        best, idx = 0.0, 0
        for i, s in enumerate(share):
            if s >= best:
                best, idx = s, i
        return idx

    chosen = []
    wt = w.copy()
    first = pick(wt)
    chosen.append(first)
    wt[first] = 0
    best = (data[:, 0] - data[first, 0]) ** 2
    for _ in range(2):
        nxt = pick(wt * best)
        chosen.append(nxt)
        wt[nxt] = 0
        best[nxt] = 0
        best = np.minimum(best, (data[:, 0] - data[nxt, 0]) ** 2)
    got = oracle.weighted_kmeanspp(seed, data, w, 3)
    assert got.tolist() == chosen
    assert len(set(chosen)) == 3


# ---------------------------------------------------------------- the rounds
def blobs(n, d, k, seed, dtype):
    rng = np.random.default_rng(seed)
    centres = rng.uniform(-10, 10, size=(k, d))
    return (centres[rng.integers(0, k, size=n)] + rng.standard_normal((n, d))).astype(dtype)


@pytest.mark.parametrize("dtype,n,d,k,seed", [(np.float32, 6000, 7, 12, 5), (np.float64, 4000, 16, 20, 9),
                                               (np.float32, 3000, 3, 40, 123)])
def test_rounds_against_brute_force(oracle, dtype, n, d, k, seed):
    X = blobs(n, d, k, seed, dtype)
    res = oracle.kmeans_parallel(X, k, seed, threads=2)
    cand, rc, phi = res["cand_rows"], res["round_count"], res["phi"]
    rounds = min(8, int(2 + np.log(k)))
    assert (rc[rounds:] == 0).all() and (phi[rounds:] == 0).all()
    assert len(cand) == 1 + rc.sum()
    assert cand[0] == oracle.kmeanspp_first(seed, n)
    assert ((cand >= 0) & (cand < n)).all()
    # the potential never grows, and the candidate count stays near 2k per round once the
    # first centre is in place (each row is taken with probability 2k * cost / potential)
    assert (np.diff(phi[:rounds]) <= 0).all()
    assert rc[:rounds].max() <= 2 * k + 8 * np.sqrt(2 * k) + 8
    thr = np.array([oracle.row_threshold(seed, int(r)) for r in range(n)], np.float64)
    X64 = X.astype(np.float64)
    known = [int(cand[0])]
    pos = 1
    running = np.full(n, np.inf)
    margin = 1e-4 if dtype == np.float32 else 1e-10
    for r in range(rounds):
        new = cand[pos:pos + rc[r]]
        assert (np.diff(new) > 0).all(), "a round lists its rows in ascending order"
        cost = ((X64[:, None, :] - X64[known][None, :, :]) ** 2).sum(-1).min(1)
        running = np.minimum(running, cost)
        total = running.sum()
        assert abs(total - phi[r]) <= 1e-4 * total
        prob = 2.0 * k * running / total
        sure_in = np.nonzero(prob > thr * (1 + margin) + margin)[0]
        sure_out = np.nonzero(prob < thr * (1 - margin) - margin)[0]
        assert np.isin(sure_in, new).all(), "round %d misses rows the rule takes" % r
        assert not np.isin(sure_out, new).any(), "round %d takes rows the rule rejects" % r
        known = [int(v) for v in new] if len(new) else known
        pos += rc[r]
    # reduction to k centres
    M = len(cand)
    C = res["centroids"]
    chosen = res["chosen"]
    if M <= k:
        assert res["weights"] is None
        assert np.array_equal(C[:M], X[cand]) and not C[M:].any()
        return
    w = res["weights"]
    assert w.sum() == n
    cells = ((X64[:, None, :] - X64[cand][None, :, :]) ** 2).sum(-1).argmin(1)
    want_w = np.bincount(cells, minlength=M)
    assert np.abs(w - want_w).sum() <= max(2, n // 500)  # near-ties may fall either way
    assert ((chosen >= 0) & (chosen < M)).all() and len(set(chosen.tolist())) == k
    assert np.array_equal(C, X[cand[chosen]])
    assert chosen.tolist() == oracle.weighted_kmeanspp(seed, X[cand], w, k).tolist()


def test_fewer_candidates_than_centres_are_padded_with_zero_rows(oracle):
    """kmeans_h2o4gpu.cu:536-540: with at most k candidates they become the first centres
    and the remaining rows stay zero."""
    X = blobs(6, 4, 3, 1, np.float32)  # a chosen row costs nothing afterwards: at most 6 candidates
    res = oracle.kmeans_parallel(X, 10, 7)
    M = len(res["cand_rows"])
    assert 1 < M <= 10
    assert res["weights"] is None
    assert res["chosen"].tolist() == list(range(M)) + [-1] * (10 - M)
    assert np.array_equal(res["centroids"][:M], X[res["cand_rows"]])
    assert not res["centroids"][M:].any()


def test_identical_rows_stop_after_the_first_round(oracle):
    """A potential of zero skips the selection (kmeans_h2o4gpu.cu:430-432)."""
    X = np.ones((50, 3), np.float32)
    res = oracle.kmeans_parallel(X, 4, 2)
    assert len(res["cand_rows"]) == 1 and not res["phi"].any()
