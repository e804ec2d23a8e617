"""Seeded random shapes and call sequences through the C ABI against the CPU oracle: the
fixed cases of the other files cover what was thought of, these cover what was not. Every
case prints its parameters before it runs, so a failure names its shape."""
import numpy as np
import pytest

from parity import label_report

pytestmark = pytest.mark.gpu


def _data(rng, n, d, k, dtype):
    nb = max(min(k, 40), 2)
    centers = rng.uniform(-6, 6, size=(nb, d))
    return np.ascontiguousarray((centers[rng.integers(0, nb, size=n)] + rng.standard_normal((n, d))).astype(dtype))


def _shape(rng, dmax=1200, kmax=3000, nmax=60000):
    d = int(rng.choice([rng.integers(1, 9), rng.integers(9, 70), rng.integers(70, 300), rng.integers(300, dmax)],
                       p=[0.2, 0.45, 0.25, 0.1]))
    k = int(rng.choice([rng.integers(1, 17), rng.integers(17, 300), rng.integers(300, kmax)], p=[0.25, 0.5, 0.25]))
    n = int(rng.choice([rng.integers(1, 200), rng.integers(200, 20000), rng.integers(20000, nmax)], p=[0.15, 0.6, 0.25]))
    return n, d, k


def _noise_mult(d):
    # the rounding floor of a float dot product grows with the square root of its length
    return max(8.0, 0.7 * np.sqrt(d))


@pytest.mark.parametrize("seed", [11, 12])
def test_one_step_predict_and_transform(hip, oracle, seed):
    """One Lloyd step, predict and transform of random shapes with a random kernel family and
    random options (fused or not, sort-based update or not, float compare or keys, bfloat16
    parts or not): labels to the near-tie rule, the update of the engine's own labels and the
    distances to rounding."""
    rng = np.random.default_rng(seed)
    done = 0
    while done < 150:
        dtype = np.float32 if rng.random() < 0.6 else np.float64
        n, d, k = _shape(rng)
        if n * d > 2e7 or n * k > 4e7:
            continue
        k = min(k, n) if rng.random() < 0.8 else k
        variant = str(rng.choice(["auto", "auto", "valu", "mfma_rowstat", "mfma_tiled"]))
        opts = {"fuse": int(rng.integers(0, 2)), "buckets": int(rng.integers(0, 2)),
                "exact_argmin": int(rng.integers(0, 2)), "fp32_split": int(rng.choice([0, 6, 9]))}
        print("seed %d case %d: %s n=%d d=%d k=%d %s %s" % (seed, done, np.dtype(dtype).name, n, d, k, variant, opts),
              flush=True)
        tol = 1e-5 if dtype == np.float32 else 1e-12
        X = _data(rng, n, d, k, dtype)
        if k <= n:
            C0 = np.ascontiguousarray(X[rng.choice(n, size=k, replace=False)])
        else:
            C0 = np.ascontiguousarray((X[rng.choice(n, size=k)] + 0.5 * rng.standard_normal((k, d))).astype(dtype))
        m = min(n, 150)
        with hip.Handle(n, d, k, dtype) as h:
            h.set_data(X)
            h.set_centroids(C0)
            try:
                h.set_option("assign", variant)
            except hip.KMeansHipError:
                pass
            if h.assign_variant() == "unsupported":
                h.set_option("assign", "auto")
            for o, v in opts.items():
                h.set_option(o, v)
            h.iterate(1)
            labels, counts, C1 = h.labels(), h.counts(), h.centroids()
            D = h.transform(X[:m])
            P = h.predict(X[:m])
            h.set_option("transform_batch_mb", 1)
            assert np.array_equal(h.transform(X[:m]), D)
        label_report(oracle, X, C0, labels, oracle.assign(X, C0, threads=8), noise_mult=_noise_mult(d))
        wC, wcounts = oracle.update(X, labels, C0)
        assert np.array_equal(counts, wcounts)
        assert np.allclose(C1, wC, rtol=tol, atol=tol * np.abs(wC).max())
        Xm = np.ascontiguousarray(X[:m])
        wantD = oracle.distances(Xm, C1)
        scale = max(np.abs(wantD).max(), float((Xm.astype(np.float64) ** 2).sum(1).max()))
        assert np.allclose(D, wantD, rtol=1e-3 if dtype == np.float32 else 1e-9,
                           atol=(1e-4 if dtype == np.float32 else 1e-10) * scale)
        label_report(oracle, Xm, C1, P, oracle.assign(Xm, C1), noise_mult=_noise_mult(d))
        done += 1


@pytest.mark.parametrize("seed", [31])
def test_fits_entry_points_and_restarts(hip, oracle, seed):
    """Whole fits with and without a threshold (predicting the training rows gives back the
    labels, the objective agrees with the oracle's fit), the reference's entry points with
    every start and 0 to 5 iterations, stacked restarts against serial ones, and k-means||
    with the scalar-order kernels against the oracle."""
    from h2o4gpu_amd.libs import ch2o4gpu_gpu
    rng = np.random.default_rng(seed)
    done = 0
    while done < 100:
        op = str(rng.choice(["fit", "stacked", "parallel", "entry"]))
        dtype = np.float32 if rng.random() < 0.6 else np.float64
        n, d, k = _shape(rng, dmax=400, kmax=900, nmax=30000)
        n, k = max(n, 2), max(min(k, n), 1)
        if d >= 200 or n * k > 2e7:
            continue
        split = int(rng.choice([0, 6])) if dtype == np.float32 else 0
        print("seed %d case %d: %s %s n=%d d=%d k=%d split=%d" % (seed, done, op, np.dtype(dtype).name, n, d, k, split),
              flush=True)
        X = _data(rng, n, d, k, dtype)
        C0 = np.ascontiguousarray(X[rng.choice(n, size=k, replace=False)])
        X64 = X.astype(np.float64)
        nm = _noise_mult(d)
        if op == "fit":
            tol = float(rng.choice([0.0, 1e-3, 1e-1]))
            iters = int(rng.integers(1, 12))
            with hip.Handle(n, d, k, dtype) as h:
                h.set_data(X)
                h.set_option("fp32_split", split)
                h.set_centroids(C0)
                it = h.fit(iters, tol)
                C, L, inertia = h.centroids(), h.labels(), h.inertia()
                assert np.array_equal(h.predict(X), L)
            assert it == iters if tol == 0.0 else 1 <= it <= iters
            label_report(oracle, X, C, L, oracle.assign(X, C, threads=8), noise_mult=nm)
            got = ((X64 - C.astype(np.float64)[L]) ** 2).sum()
            assert abs(inertia - got) <= 1e-4 * got + 1e-6 * (X64 ** 2).sum()
            if d > 1 and k <= n // 20:  # (tiny clusters in one dimension: near-ties move the trajectory)
                wC, wL, _, _ = oracle.lloyd(X, C0, iters, tol, threads=8)
                want = ((X64 - wC.astype(np.float64)[wL]) ** 2).sum()
                assert abs(got - want) <= 1e-2 * want + 1e-9
        elif op == "stacked":
            sets = int(rng.integers(2, 5))
            if hip.stack_width(n, d, k, dtype, sets) < sets:
                continue
            starts = [np.ascontiguousarray(X[rng.choice(n, size=k, replace=False)]) for _ in range(sets)]
            iters = int(rng.integers(1, 6))
            with hip.Handle(n, d, k, dtype, sets=sets) as h:
                h.set_data(X)
                h.set_option("assign", "mfma_rowstat")
                for s in range(sets):
                    h.select_set(s)
                    h.set_centroids(starts[s])
                h.fit(iters, 0.0)
                got = []
                for s in range(sets):
                    h.select_set(s)
                    got.append((h.centroids(), h.labels(), h.inertia()))
            for s in range(sets):
                with hip.Handle(n, d, k, dtype) as h:
                    h.set_data(X)
                    h.set_option("assign", "mfma_rowstat")
                    h.set_centroids(starts[s])
                    h.fit(iters, 0.0)
                    assert np.array_equal(h.labels(), got[s][1])
                    if dtype == np.float32:
                        assert np.array_equal(h.centroids(), got[s][0])
                    else:
                        assert np.allclose(h.centroids(), got[s][0], rtol=1e-12, atol=1e-12)
        elif op == "parallel":
            sd = int(rng.integers(0, 1000))
            with hip.Handle(n, d, k, dtype) as h:
                h.set_data(X)
                h.set_option("assign", "valu")
                h.init_parallel(sd)
                info, C = h.parallel_seed_info(), h.centroids()
                assert not h.labels().any()
            want = oracle.kmeans_parallel(X, k, sd, threads=4)
            assert np.array_equal(info["cand_rows"], want["cand_rows"])
            assert np.array_equal(info["chosen"], want["chosen"]) and np.array_equal(C, want["centroids"])
        else:
            iters = int(rng.integers(0, 6))
            init = int(rng.choice([0, 1, 2, 3]))
            fit = ch2o4gpu_gpu.make_ptr_float_kmeans if dtype == np.float32 else ch2o4gpu_gpu.make_ptr_double_kmeans
            centres, labels = np.zeros(k * d, dtype), np.zeros(n, np.int32)
            assert fit(0, 0, 5, 0, 1, n, d, k, iters, init, 0.0, X.flatten(), C0.flatten(), centres, labels) == 0
            C = centres.reshape(k, d)
            assert np.isfinite(C).all()
            if iters == 0:  # no relabel: the zeros the reference's label vector starts with
                assert not labels.any()
                labels = oracle.assign(X, C, threads=8)
            else:
                label_report(oracle, X, C, labels, oracle.assign(X, C, threads=8), noise_mult=nm)
            m = min(n, 100)
            Xm = np.ascontiguousarray(X[:m])
            res = np.zeros(m, np.int32)
            assert fit(1, 0, 5, 0, 1, m, d, k, 0, 0, 0.0, Xm.flatten(), C.flatten(), np.empty([], dtype), res) == 0
            label_report(oracle, Xm, C, res, labels[:m], noise_mult=nm)
            tf = ch2o4gpu_gpu.kmeans_transform_float if dtype == np.float32 else ch2o4gpu_gpu.kmeans_transform_double
            dist = np.zeros(m * k, dtype)
            assert tf(0, 0, 1, m, d, k, Xm.flatten(), C.flatten(), dist) == 0
            wantD = oracle.distances(Xm, C)
            scale = max(np.abs(wantD).max(), float((Xm.astype(np.float64) ** 2).sum(1).max()))
            assert np.allclose(dist.reshape(k, m), wantD, rtol=1e-3 if dtype == np.float32 else 1e-9,
                               atol=(1e-4 if dtype == np.float32 else 1e-10) * scale)
        done += 1
