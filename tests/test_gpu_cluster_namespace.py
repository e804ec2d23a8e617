"""`h2o4gpu_amd.cluster` on the GPU: the estimator taken from the scikit-learn-shaped namespace
(reference: scripts/prepare_sklearn.sh:65-66 injects the GPU estimator into `h2o4gpu.cluster`),
cloned and run as a step of a scikit-learn Pipeline, against the CPU oracle."""
import numpy as np
import pytest

from parity import assert_centroids_close, label_report

pytestmark = pytest.mark.gpu


def _blobs(n, d, k, dtype, seed):
    rng = np.random.default_rng(seed)
    centers = rng.uniform(-20, 20, size=(k, d))
    X = centers[rng.integers(0, k, size=n)] + rng.standard_normal((n, d)) * rng.uniform(0.5, 3.0, size=d)
    return np.ascontiguousarray(X.astype(dtype)), centers


@pytest.mark.parametrize("dtype", [np.float32, np.float64])
def test_cloned_estimator_in_a_pipeline_equals_the_oracle(oracle, dtype):
    from sklearn.base import clone
    from sklearn.pipeline import Pipeline
    from sklearn.preprocessing import StandardScaler
    from h2o4gpu_amd.cluster import KMeans, KMeansH2O

    n, d, k, iters = 20000, 16, 6, 8
    X, centers = _blobs(n, d, k, dtype, 31)
    scaler = StandardScaler().fit(X)
    Xs = np.ascontiguousarray(scaler.transform(X).astype(dtype))
    C0 = np.ascontiguousarray((scaler.transform(centers) + 0.1).astype(dtype))

    proto = KMeans(n_clusters=k, init=C0, max_iter=iters, tol=0, backend="h2o4gpu")
    est = clone(proto)
    assert est is not proto and est.get_params()["n_clusters"] == k
    pipe = Pipeline([("scale", StandardScaler()), ("km", est)]).fit(X)
    model = pipe.named_steps["km"]
    assert model.backend == "h2o4gpu" and isinstance(model.model, KMeansH2O)
    # the scaler hands the estimator float64 or float32 rows as it received them
    wC, wL, _, _ = oracle.lloyd(Xs, C0, iters, 0.0, threads=4)
    assert model.cluster_centers_.shape == (k, d) and model.cluster_centers_.dtype == np.dtype(dtype)
    assert_centroids_close(model.cluster_centers_, wC, dtype)
    rep = label_report(oracle, Xs, wC, model.labels_, wL)
    assert rep["mismatch"] == 0, rep
    assert np.array_equal(pipe.predict(X), wL)
    assert model.n_iter_ == iters

    # as the first step: fit_transform gives (rows, k) squared distances to the fitted centres
    first = Pipeline([("km", clone(proto)), ("scale", StandardScaler(with_mean=False, with_std=False))])
    D = first.fit_transform(Xs)
    assert D.shape == (n, k)
    Cf = first.named_steps["km"].cluster_centers_
    assert_centroids_close(Cf, wC, dtype)
    want = oracle.distances(Xs, np.ascontiguousarray(Cf), threads=4).T          # (rows, k)
    eps = float(np.finfo(dtype).eps)
    xx = (Xs.astype(np.float64) ** 2).sum(1)[:, None]
    cc = (Cf.astype(np.float64) ** 2).sum(1)[None, :]
    err = np.abs(D.astype(np.float64) - want.astype(np.float64)) / (eps * (xx + cc))
    assert err.max() <= 4 * np.sqrt(d) + 40, err.max()
    assert np.array_equal(np.argmin(D, axis=1), wL)

    # score through the namespace's class: negated objective of the oracle's result
    obj = float(oracle.assign(Xs, wC, threads=4, return_mindist=True)[1].astype(np.float64).sum())
    assert abs(model.score(Xs) + obj) <= 1e-4 * obj


def test_grid_search_accepts_the_estimator():
    """Model selection over the namespace's estimator: every candidate is a clone fitted on the
    GPU; the winner is the candidate with the true number of blobs."""
    from sklearn.model_selection import GridSearchCV
    from h2o4gpu_amd.cluster import KMeans

    X, _ = _blobs(6000, 8, 5, np.float32, 4)
    gs = GridSearchCV(KMeans(init="random", max_iter=30, tol=1e-6, random_state=3, n_init=3,
                             backend="h2o4gpu"),
                      {"n_clusters": [2, 5]}, cv=2, refit=True)
    gs.fit(X)
    assert gs.best_params_["n_clusters"] == 5
    assert gs.best_estimator_.cluster_centers_.shape == (5, 8)
    assert gs.best_estimator_.predict(X).shape == (6000,)
