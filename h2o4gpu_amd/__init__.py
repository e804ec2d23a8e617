"""MI355X (gfx950) k-means engine with the interface of h2o4gpu's KMeans.

    from h2o4gpu_amd import KMeans
    model = KMeans(n_clusters=8, init='random', max_iter=20, tol=0).fit(X)

The compute path is libh2o4gpu_kmeans_hip.so (hand-written HIP kernels behind the C ABI
declared in include/h2o4gpu_kmeans.h); build it with `python -m h2o4gpu_amd.build`.
"""
from .solvers.kmeans import KMeans, KMeansH2O  # noqa: F401

__all__ = ["KMeans", "KMeansH2O"]
