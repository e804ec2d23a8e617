"""Child process of test_gpu_torch_input.py: rows handed over as PyTorch-ROCm tensors
(device memory, adopted without a copy) must give the results of the same rows handed
over as host arrays. Prints one JSON object. Not collected by pytest."""
import json
import os
import sys

import numpy as np
import torch  # imported before the engine: both then share one HIP runtime

sys.path.insert(0, os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
from h2o4gpu_amd import KMeans  # noqa: E402


def main():
    out = {}
    rng = np.random.default_rng(7)
    for dtype in (np.float32, np.float64):
        tag = np.dtype(dtype).name
        k, d, n = 12, 24, 50_000
        centers = rng.uniform(-30, 30, size=(k, d))
        X = np.ascontiguousarray((centers[rng.integers(0, k, size=n)] +
                                  rng.standard_normal((n, d))).astype(dtype))
        C0 = (centers + 0.25).astype(dtype)
        Xd = torch.from_numpy(X).to("cuda:0")
        host = KMeans(n_clusters=k, init=C0, max_iter=7, tol=0.0, random_state=3).fit(X)
        dev = KMeans(n_clusters=k, init=C0, max_iter=7, tol=0.0, random_state=3).fit(Xd)
        scale = float(np.abs(host.cluster_centers_).max())
        out[tag + "_centroids_maxdiff"] = float(np.abs(host.cluster_centers_.astype(np.float64) -
                                                       dev.cluster_centers_).max()) / scale
        out[tag + "_labels_equal"] = bool(np.array_equal(host.labels_, dev.labels_))
        out[tag + "_inertia"] = [host.inertia_, dev.inertia_]
        out[tag + "_n_iter"] = [host.n_iter_, dev.n_iter_]
        out[tag + "_predict_equal"] = bool(np.array_equal(host.predict(X), dev.predict(Xd)))
        out[tag + "_score"] = [host.score(X), dev.score(Xd)]
        Dh = host.transform(X[:4096])
        Dd = dev.transform(Xd[:4096])
        out[tag + "_transform_is_tensor"] = bool(isinstance(Dd, torch.Tensor) and Dd.is_cuda)
        out[tag + "_transform_shape"] = list(Dd.shape)
        out[tag + "_transform_equal"] = bool(np.array_equal(Dh, Dd.cpu().numpy()))
        # seeded starts take the same rows whether the data came from host or device
        for init in ("random", "k-means++"):
            a = KMeans(n_clusters=k, init=init, max_iter=3, tol=0.0, random_state=11).fit(X)
            b = KMeans(n_clusters=k, init=init, max_iter=3, tol=0.0, random_state=11).fit(Xd)
            out["%s_%s_close" % (tag, init)] = bool(np.allclose(a.cluster_centers_, b.cluster_centers_,
                                                                rtol=1e-12, atol=1e-12))
        # restarts (stacked where the shape allows) on device rows and on host rows agree
        a = KMeans(n_clusters=k, init="random", n_init=3, max_iter=3, tol=0.0, random_state=5).fit(X)
        b = KMeans(n_clusters=k, init="random", n_init=3, max_iter=3, tol=0.0, random_state=5).fit(Xd)
        out[tag + "_restarts_close"] = bool(np.allclose(a.cluster_centers_, b.cluster_centers_, rtol=1e-12,
                                                       atol=1e-12) and
                                           abs(a.inertia_ - b.inertia_) <= 1e-12 * a.inertia_)
    # device rows that start 4 or 8 bytes into an allocation (not 16-byte aligned): every
    # kernel family must take its unaligned path and give the aligned result
    unaligned = {}
    for dtype in (np.float32, np.float64):
        for (k, d, n) in ((8, 16, 20_011), (8, 30, 20_011), (5, 3, 9_001), (40, 32, 20_011),
                          (200, 24, 20_011), (70, 100, 8_003), (3000, 8, 20_011)):
            centers = rng.uniform(-30, 30, size=(k, d))
            X = np.ascontiguousarray((centers[rng.integers(0, k, size=n)] +
                                      rng.standard_normal((n, d))).astype(dtype))
            C0 = (centers + 0.25).astype(dtype)
            base = torch.empty(n * d + 1, dtype=torch.from_numpy(X).dtype, device="cuda:0")
            Xd = base[1:].view(n, d)
            Xd.copy_(torch.from_numpy(X))
            assert Xd.data_ptr() % 16 != 0
            host = KMeans(n_clusters=k, init=C0, max_iter=3, tol=0.0, random_state=3).fit(X)
            dev = KMeans(n_clusters=k, init=C0, max_iter=3, tol=0.0, random_state=3).fit(Xd)
            scale = float(np.abs(host.cluster_centers_).max())
            diff = float(np.abs(host.cluster_centers_.astype(np.float64) - dev.cluster_centers_).max()) / scale
            unaligned["%s k=%d d=%d" % (np.dtype(dtype).name, k, d)] = [
                bool(np.array_equal(host.labels_, dev.labels_)), diff,
                bool(np.array_equal(host.predict(X), dev.predict(Xd)))]
    out["unaligned"] = unaligned
    # a non-contiguous view is refused, a CPU tensor goes the host way
    try:
        KMeans(n_clusters=2, init="random", max_iter=1).fit(Xd[:, ::2])
        out["strided_refused"] = False
    except ValueError:
        out["strided_refused"] = True
    m = KMeans(n_clusters=3, init="random", max_iter=2, random_state=1).fit(torch.from_numpy(X[:100]))
    out["cpu_tensor_ok"] = m.cluster_centers_.shape == (3, X.shape[1])
    print(json.dumps(out), flush=True)


if __name__ == "__main__":
    main()
