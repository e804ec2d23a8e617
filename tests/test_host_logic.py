"""Host-side logic above the C ABI: the estimator's argument mapping (checked against
the call sites of the reference's kmeans.py), the SWIG-convention shim, the data
generators. A recording stand-in replaces the native module; nothing is computed."""
import numpy as np
import pytest

from h2o4gpu_amd.solvers import kmeans as km


class RecordingLib:
    def __init__(self):
        self.calls = []

    def _fill(self, name, args):
        self.calls.append((name, args))
        return 0

    def make_ptr_float_kmeans(self, *a):
        if a[0] == 0:
            a[13][:] = np.arange(a[13].size)
            a[14][:] = 1
        else:
            a[14][:] = 2
        return self._fill("make_ptr_float_kmeans", a)

    def make_ptr_double_kmeans(self, *a):
        if a[0] == 0:
            a[13][:] = 0.5
            a[14][:] = 0
        return self._fill("make_ptr_double_kmeans", a)

    def kmeans_transform_float(self, *a):
        a[8][:] = np.arange(a[8].size)
        return self._fill("kmeans_transform_float", a)

    def kmeans_transform_double(self, *a):
        return self._fill("kmeans_transform_double", a)


@pytest.fixture
def model(monkeypatch):
    monkeypatch.setattr("h2o4gpu_amd.util.gpu.device_count", lambda n_gpus=0: (1, 1))
    lib = RecordingLib()
    m = km.KMeansH2O(n_clusters=3, init="random", max_iter=7, tol=0.25, random_state=42, gpu_id=0)
    monkeypatch.setattr(m, "_load_lib", lambda: lib)
    return m, lib


def test_fit_call_matches_reference_call_site(model):
    """Reference kmeans.py:485-497: (0, verbose, seed, gpu_id, n_gpus, rows, cols, k,
    max_iter, c_init, tol, c_data, centroids, pred_centers, pred_labels)."""
    m, lib = model
    X = np.arange(20, dtype=np.int64).reshape(10, 2)           # not float: cast to float32
    m.fit(X)
    name, a = lib.calls[0]
    assert name == "make_ptr_float_kmeans"
    assert a[:11] == (0, 0, 42, 0, 1, 10, 2, 3, 7, 0, 0.25)
    assert a[11].dtype == np.float32 and a[11].shape == (20,)  # flattened C order
    assert np.array_equal(a[11], X.astype(np.float32).flatten())
    assert a[12].ndim == 0                                     # np.empty([]) as in the reference
    assert a[13].shape == (6,) and a[13].dtype == np.float32
    assert a[14].shape == (10,) and a[14].dtype == np.int32
    assert m.cluster_centers_.shape == (3, 2) and m.labels_.shape == (10,)
    assert m.cluster_centers_[1, 0] == 2.0                     # row-major reshape (k, cols)


def test_init_mapping_and_double_path(model):
    m, lib = model
    m.init = "k-means++"
    m.fit(np.zeros((5, 2), np.float64))
    name, a = lib.calls[0]
    assert name == "make_ptr_double_kmeans" and a[9] == 1 and a[11].dtype == np.float64
    m.init = np.ones((3, 2))
    m.fit(np.zeros((5, 2), np.float32))
    name, a = lib.calls[1]
    assert a[9] == 2 and a[12].shape == (6,) and a[12].dtype == np.float32


def test_predict_and_transform_call_sites(model):
    """Reference kmeans.py:369-372 and :410-422."""
    m, lib = model
    m.cluster_centers_ = np.zeros((3, 2), np.float32)
    X = np.ones((4, 2), np.float32)
    res = m.predict(X)
    name, a = lib.calls[0]
    assert a[:11] == (1, 0, 42, 0, 1, 4, 2, 3, 7, 0, 0.25)
    assert a[12].shape == (6,) and a[13].ndim == 0 and res.dtype == np.int32 and (res == 2).all()
    D = m.transform(X)
    name, a = lib.calls[1]
    assert name == "kmeans_transform_float" and a[:6] == (0, 0, 1, 4, 2, 3)
    # library layout is [k][rows]; the estimator returns (rows, k) with D[i, c] = buf[c*rows + i]
    assert D.shape == (4, 3) and D[1, 2] == 2 * 4 + 1
    with pytest.raises(AssertionError):
        m.predict(np.ones((4, 5), np.float32))


def test_setters_validate(model):
    m, _ = model
    with pytest.raises(ValueError):
        m.n_clusters = 0
    with pytest.raises(ValueError):
        m.max_iter = 0
    with pytest.raises(ValueError):
        m.gpu_id = -1
    with pytest.raises(ValueError):
        km.KMeansH2O(init="nonsense")
    assert m.get_params()["n_clusters"] == 3
    m.set_params(tol=0.5)
    assert m.tol == 0.5
    with pytest.raises(ValueError):
        m.set_params(bogus=1)


def test_nonfinite_data_is_refused(model):
    m, _ = model
    with pytest.raises(AssertionError):
        m.fit(np.array([[0.0, np.nan], [1.0, 2.0]]))


def test_without_a_device_the_estimator_raises_and_the_selector_uses_sklearn(monkeypatch):
    """No device: the GPU estimator refuses to compute (no CPU stand-in for the engine);
    the backend selector takes scikit-learn only when asked to (n_gpus=0 / backend)."""
    monkeypatch.setattr("h2o4gpu_amd.util.gpu.device_count", lambda n_gpus=0: (0, 0))
    X = np.random.default_rng(0).standard_normal((50, 3)).astype(np.float32)
    m = km.KMeansH2O(n_clusters=2, init="random", random_state=1)
    with pytest.raises(RuntimeError, match="usable GPU"):
        m.fit(X)
    m.cluster_centers_ = X[:2]
    for call in (m.predict, m.transform, m.score):
        with pytest.raises(RuntimeError, match="usable GPU"):
            call(X)
    with pytest.raises(RuntimeError, match="no usable GPU"):
        km.KMeans(n_clusters=2)
    sk = km.KMeans(n_clusters=2, n_gpus=0, random_state=1, n_init=1).fit(X)
    assert sk.cluster_centers_.shape == (2, 3)


def test_native_status_is_not_ignored(model):
    """The reference drops the entry points' return value (kmeans.py:485-497); here a
    non-zero status raises."""
    m, lib = model
    lib._fill = lambda name, args: -3
    with pytest.raises(RuntimeError, match="status -3"):
        m.fit(np.zeros((4, 2), np.float32))
    m.cluster_centers_ = np.zeros((3, 2), np.float32)
    with pytest.raises(RuntimeError, match="status -3"):
        m.predict(np.zeros((4, 2), np.float32))
    with pytest.raises(RuntimeError, match="status -3"):
        m.transform(np.zeros((4, 2), np.float32))


def test_swig_shim_conversions():
    from h2o4gpu_amd.libs import ch2o4gpu_gpu as shim
    p, keep = shim._in_array(np.empty([]), np.float32)          # 0-d array: converted, not NULL
    assert p is not None and keep.dtype == np.float32
    assert shim._in_array(None, np.float32) == (None, None)     # non-array -> NULL
    with pytest.raises(TypeError):
        shim._inplace_array(np.zeros(3, np.float64), np.float32, "x")
    with pytest.raises(TypeError):
        shim._inplace_array(np.zeros((4, 2), np.float32)[:, 0], np.float32, "x")


def test_datasets_are_deterministic_and_shaped():
    from h2o4gpu_amd import datasets
    X1, k, iters = datasets.make("C1", scale=0.02)
    X2, _, _ = datasets.make("C1", scale=0.02)
    assert X1.shape == (2000, 16) and k == 8 and iters == 20 and np.array_equal(X1, X2)
    X3, k3, _ = datasets.make("C3", scale=0.001)
    assert X3.shape == (10000, 32) and k3 == 256 and X3.dtype == np.float32
    X4, _, _ = datasets.make("C4", scale=0.002, dtype=np.float64)
    assert X4.dtype == np.float64 and X4.shape[1] == 256 and np.abs(X4).max() <= 25
    X5, _, _ = datasets.make("C5", scale=0.02)
    frac0 = (X5 == 0).mean()
    assert 0.68 < frac0 < 0.72 and X5.max() <= 255 and (X5 == np.round(X5)).all()
    H = datasets.make_holdout("C5", 100)
    assert H.shape == (100, 784) and not np.array_equal(H, X5[:100])
    C0 = datasets.seeded_row_init(X3, k3, 5)
    assert C0.shape == (256, 32) and len({r.tobytes() for r in C0}) == 256


def test_more_clusters_than_rows_keeps_one_shape(model):
    """n_clusters > rows: the library fits with k = rows (kmeans_h2o4gpu.cu:630-635) and the
    estimator's centre array keeps n_clusters rows; predict and transform then hand the
    library exactly as many centroids as that array holds."""
    m, lib = model
    m.n_clusters = 5
    X = np.arange(6, dtype=np.float32).reshape(3, 2)            # 3 rows, 5 clusters asked for
    m.fit(X)
    assert m.cluster_centers_.shape == (5, 2)
    m.predict(X)
    name, a = lib.calls[-1]
    assert a[7] == 5 and a[12].size == 5 * 2
    D = m.transform(X)
    name, a = lib.calls[-1]
    assert a[5] == 5 and a[7].size == 5 * 2 and D.shape == (3, 5)
    # a centre array shorter than n_clusters (set by hand, or left by an older fit) is
    # never over-read: k follows the array
    m.cluster_centers_ = np.zeros((3, 2), np.float32)
    m.predict(X)
    assert lib.calls[-1][1][7] == 3 and lib.calls[-1][1][12].size == 6
    assert m.transform(X).shape == (3, 3)


def test_cluster_namespace_clone_and_pipeline(monkeypatch):
    """The scikit-learn-shaped surface (reference: scripts/prepare_sklearn.sh:65-66 puts the
    estimator into the `cluster` namespace): importable from h2o4gpu_amd.cluster, accepted by
    sklearn.base.clone and by a two-step Pipeline in both positions."""
    from sklearn.base import clone
    from sklearn.pipeline import Pipeline
    from sklearn.preprocessing import StandardScaler
    import sklearn.cluster
    from h2o4gpu_amd import cluster
    assert cluster.KMeans is km.KMeans and cluster.KMeansH2O is km.KMeansH2O
    assert cluster.KMeansSklearn is sklearn.cluster.KMeans
    monkeypatch.setattr("h2o4gpu_amd.util.gpu.device_count", lambda n_gpus=0: (1, 1))
    lib = RecordingLib()
    monkeypatch.setattr(km.KMeansH2O, "_load_lib", lambda self: lib)
    est = cluster.KMeans(n_clusters=3, init="random", max_iter=7, tol=0.25, random_state=42,
                         backend="h2o4gpu")
    twin = clone(est)
    assert twin is not est and twin.backend == "h2o4gpu"
    assert twin.get_params() == est.get_params() and twin.get_params()["n_clusters"] == 3
    inner = clone(est.model)
    assert isinstance(inner, km.KMeansH2O) and inner.get_params() == est.model.get_params()
    assert est.set_params(max_iter=9) is est and est.get_params()["max_iter"] == 9
    with pytest.raises(ValueError):
        est.set_params(backend="sklearn")
    X = np.random.default_rng(0).standard_normal((20, 2)).astype(np.float32)
    last = Pipeline([("scale", StandardScaler()), ("km", clone(est))]).fit(X)
    assert last.predict(X).shape == (20,) and lib.calls[-1][0] == "make_ptr_float_kmeans"
    first = Pipeline([("km", clone(est)), ("scale", StandardScaler())])
    assert first.fit_transform(X).shape == (20, 3)
    # the CPU backend clones into the CPU backend
    cpu = clone(cluster.KMeans(n_clusters=2, n_gpus=0, random_state=1, n_init=1))
    assert cpu.backend == "sklearn"


class FakeHandle:
    """Stands in for kmeans_hip.Handle: records which set got which seed and lets each
    restart end with an inertia that depends on its seed only."""

    def __init__(self, log, sets):
        self.log, self.sets, self.cur = log, sets, 0
        self.seed = [None] * sets
        log.append(("create", sets))

    def __enter__(self):
        return self

    def __exit__(self, *exc):
        self.log.append(("close",))

    def select_set(self, s):
        assert 0 <= s < self.sets
        self.cur = s

    def init_random_rows(self, seed):
        self.seed[self.cur] = seed
        self.log.append(("seed", self.cur, seed))

    def fit(self, max_iter, tol):
        assert all(s is not None for s in self.seed)
        self.log.append(("fit", tuple(self.seed)))
        return max_iter

    def set_iterations(self):
        return np.array([3 + s for s in self.seed], np.int32)

    def inertia(self):
        return float((self.seed[self.cur] * 7) % 11)

    def centroids(self):
        return np.full((3, 2), self.seed[self.cur], np.float32)

    def labels(self):
        return np.full(10, self.seed[self.cur], np.int32)


@pytest.mark.parametrize("restarts,width,want_sets,want_groups", [(4, 3, 2, 2), (5, 8, 5, 1), (7, 3, 3, 3),
                                                                  (3, 1, 1, 3)])
def test_restarts_are_grouped_into_balanced_stacks(model, monkeypatch, restarts, width, want_sets, want_groups):
    """n_init restarts use seeds random_state, random_state + 1, ...; as many as the shape
    allows run stacked, in balanced groups on one handle (one upload); a spare set of the last
    group repeats a seed and is ignored; the restart with the lowest inertia is kept."""
    m, _ = model
    m.n_init = restarts
    log = []
    monkeypatch.setattr("h2o4gpu_amd.libs.kmeans_hip.stack_width", lambda rows, cols, k, dtype, r: min(width, r))
    m._fit_on_handle(lambda sets: FakeHandle(log, sets), 10, 2, np.float32, 3, None)
    assert log[0] == ("create", want_sets) and log[-1] == ("close",)
    assert sum(1 for e in log if e[0] == "create") == 1          # the rows are set up once
    fits = [e for e in log if e[0] == "fit"]
    assert len(fits) == want_groups
    seeds = sorted({s for f in fits for s in f[1]})
    assert seeds == list(range(42, 42 + restarts))                # every restart ran, none beyond
    best = min(range(42, 42 + restarts), key=lambda s: ((s * 7) % 11, s))
    assert m.inertia_ == float((best * 7) % 11)
    assert (m.cluster_centers_ == best).all() and (m.labels_ == best).all()
    assert m.n_iter_ == (3 + best if want_sets > 1 else 7)
