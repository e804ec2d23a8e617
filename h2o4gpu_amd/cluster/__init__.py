"""`h2o4gpu_amd.cluster`: the clustering namespace of the scikit-learn-shaped surface.

The reference builds `h2o4gpu.cluster` from a renamed copy of scikit-learn's `cluster`
package and injects its own estimator into it (scripts/prepare_sklearn.sh:65-66), so that
`from h2o4gpu.cluster import KMeans` gives the GPU-backed selector while scikit-learn's own
class stays reachable as `KMeansSklearn`. Same names here, on the installed scikit-learn:

    from h2o4gpu_amd.cluster import KMeans          # backend selector (GPU engine by default)
    from h2o4gpu_amd.cluster import KMeansH2O       # the GPU estimator itself
    from h2o4gpu_amd.cluster import KMeansSklearn   # scikit-learn's KMeans, untouched

Both estimators follow scikit-learn's estimator protocol (`get_params` / `set_params`
round-trip through the constructor), so `sklearn.base.clone`, `Pipeline` and the
model-selection tools accept them.
"""
from ..solvers.kmeans import KMeans, KMeansH2O  # noqa: F401

__all__ = ["KMeans", "KMeansH2O", "KMeansSklearn"]


def __getattr__(name):
    # scikit-learn is imported only when its class is asked for
    if name == "KMeansSklearn":
        from sklearn.cluster import KMeans as _SkKMeans
        return _SkKMeans
    raise AttributeError("module %r has no attribute %r" % (__name__, name))
