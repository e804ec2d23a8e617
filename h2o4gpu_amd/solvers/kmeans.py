"""K-Means estimator with the interface of h2o4gpu.KMeans.

Mirrors src/interface_py/h2o4gpu/solvers/kmeans.py of the reference: the same
constructor arguments and defaults (:131-148, :685-702), attributes, dtype rule,
argument order of the native calls (:369-372, :410-418, :485-497) and result shapes,
on top of the gfx950 engine. Differences, all additive:
  * `init` may be an ndarray of shape (n_clusters, n_features): it is passed to the
    engine as starting centroids (init_from_data=2) instead of forcing the
    scikit-learn backend;
  * `inertia_` is filled after fit (the reference leaves it None, :187);
  * when scikit-learn is chosen as backend it is the installed scikit-learn (the
    reference uses its own renamed copy);
  * `init='k-means++'` runs k-means|| as in the reference (whose native side does so for
    that name); `'k-means||'` is accepted as a second name for it and `'d2-sampling'`
    selects textbook k-means++ (one centre per pass, drawn proportionally to the squared
    distance to the nearest chosen centre);
  * `n_init` restarts, `n_iter_` and a native `score`. Restarts run stacked through the
    matrix-core kernel wherever the shape allows; a single fit of a small model (k <= 16,
    d <= 64) runs the scalar-order kernels instead, so restart r of an `n_init` fit equals
    the `n_init=1` fit with `random_state + r` up to rows whose two nearest centroids are a
    near-tie (1e-5 relative), not bit for bit; `labels_` always come from an ordinary relabel
    against the returned centroids, so they equal `predict` on the same rows;
  * fit / predict / score / transform accept rows that already live on the GPU (any
    object with `__cuda_array_interface__`, e.g. a PyTorch-ROCm tensor): the engine adopts
    the pointer, nothing crosses PCIe (the reference re-uploads the rows on every call,
    kmeans_h2o4gpu.cu:679,857,930).
"""
import sys

import numpy as np


def _to_np(data):
    """Reference solvers/utils.py:_get_data/_to_np for the dense-matrix case: numpy
    array, 2-D, float32 unless the data already is float64/float32."""
    if not isinstance(data, np.ndarray) and not callable(getattr(data, "values", data.__class__)):
        data = data.values  # pandas (a tensor's `values` is a method and stays as it is)
    arr = np.asarray(data)
    if arr.ndim == 1:
        arr = arr.reshape(-1, 1)
    if arr.dtype not in (np.float32, np.float64):
        arr = arr.astype(np.float32)
    return arr


class _DeviceRows:
    """A C-contiguous (rows, cols) float32/float64 array in device memory."""

    def __init__(self, owner, ptr, rows, cols, dtype):
        self.owner, self.ptr, self.rows, self.cols, self.dtype = owner, ptr, rows, cols, dtype


def _device_rows(X):
    """_DeviceRows for an object exposing `__cuda_array_interface__`, else None. Work
    queued on the array by its owner must have finished; for PyTorch tensors the current
    stream is synchronised here."""
    try:
        cai = getattr(X, "__cuda_array_interface__", None)
    except Exception:  # PyTorch raises for CPU tensors and tensors that require grad
        return None
    if not isinstance(cai, dict):
        return None
    shape = tuple(cai["shape"])
    dtype = np.dtype(cai["typestr"])
    if dtype not in (np.dtype(np.float32), np.dtype(np.float64)):
        raise TypeError("device input must be float32 or float64, got %s" % dtype)
    if len(shape) != 2:
        raise ValueError("device input must be 2-D (rows, cols), got shape %s" % (shape,))
    strides = cai.get("strides")
    if strides is not None and tuple(strides) != (shape[1] * dtype.itemsize, dtype.itemsize):
        raise ValueError("device input must be C-contiguous")
    torch = sys.modules.get("torch")
    if torch is not None and isinstance(X, torch.Tensor):
        torch.cuda.current_stream(X.device).synchronize()
    return _DeviceRows(X, int(cai["data"][0]), int(shape[0]), int(shape[1]), dtype)


def _check_data_content(do_check, name, data):
    """Reference solvers/utils.py:144-158."""
    if do_check == 1 and np.size(data):
        # the library's parallel pass over the raw values where it can be used ...
        if isinstance(data, np.ndarray) and data.dtype in (np.float32, np.float64) \
                and data.flags.c_contiguous:
            try:
                from ..libs import kmeans_hip
                finite = kmeans_hip.host_all_finite(data)
            except Exception:  # no native library here: numpy below  # pylint: disable=broad-except
                finite = None
            if finite is not None:
                # (the reference's first assertion fires for NaN as well as for infinities)
                assert finite, "%s contains Inf" % name
                return
        # ... else the same two assertions as the reference, from the extremes (a NaN
        # propagates into both, an infinity into one of them): two passes and no boolean
        # temporary the size of the data
        lo, hi = np.min(data), np.max(data)
        assert np.isfinite(lo) and np.isfinite(hi), "%s contains Inf" % name
        assert not (np.isnan(lo) or np.isnan(hi)), "%s contains NA" % name


def assert_satisfies(value, cond, message):
    """Reference typecheck.typechecks.assert_satisfies, reduced to what the setters use."""
    if not cond:
        raise ValueError("%s (got %r)" % (message, value))


def _clusterer_tags():
    """scikit-learn's estimator tags (1.6 and later ask every estimator for them; the two
    classes here do not inherit BaseEstimator, as in the reference)."""
    from sklearn.utils import Tags, TargetTags, TransformerTags
    return Tags(estimator_type="clusterer", target_tags=TargetTags(required=False),
                transformer_tags=TransformerTags())


class KMeansH2O:
    """K-Means on the GPU (reference class KMeansH2O, kmeans.py:18-588)."""

    def __init__(self, n_clusters=8, init='k-means++', n_init=1, max_iter=300, tol=1e-4,
                 precompute_distances='auto', verbose=0, random_state=None, copy_x=True, n_jobs=1,
                 algorithm='auto', gpu_id=0, n_gpus=-1, do_checks=1):
        if isinstance(tol, np.floating):
            tol = tol.item()
        if isinstance(init, str) and init not in ['random', 'k-means++', 'k-means||', 'd2-sampling']:
            raise ValueError("Invalid initialization method. Should be 'k-means++' or 'random' "
                             "but got '%s'." % init)
        self.init = init
        self._n_clusters = n_clusters
        self._gpu_id = gpu_id
        from ..util.gpu import device_count
        (self.n_gpus, self.devices) = device_count(n_gpus)
        self._max_iter = max_iter
        self.tol = tol
        self._did_sklearn_fit = 0
        self.verbose = verbose
        self.do_checks = do_checks
        self.n_init = n_init
        self.precompute_distances = precompute_distances
        self.copy_x = copy_x
        self.n_jobs = n_jobs
        self.algorithm = algorithm
        if random_state is None:
            import random
            self.random_state = random.randint(0, 32000)
        else:
            self.random_state = random_state
        self.cluster_centers_ = None
        self.labels_ = None
        self.inertia_ = None
        self.n_iter_ = None
        self.sklearn_model = None
        self.double_precision = 0

    def __sklearn_tags__(self):
        return _clusterer_tags()

    _PARAMS = ["algorithm", "copy_x", "do_checks", "gpu_id", "init", "max_iter", "n_clusters", "n_gpus",
               "n_init", "n_jobs", "precompute_distances", "random_state", "tol", "verbose"]

    @classmethod
    def _get_param_names(cls):
        return list(cls._PARAMS)

    def get_params(self, deep=True):
        return {key: getattr(self, key, None) for key in self._get_param_names()}

    def set_params(self, **params):
        valid = self.get_params(deep=True)
        for key, value in params.items():
            if key not in valid:
                raise ValueError('Invalid parameter %s for estimator %s. Check the list of available '
                                 'parameters with `estimator.get_params().keys()`.'
                                 % (key, self.__class__.__name__))
            setattr(self, key, value)
        return self

    def fit(self, X, y=None):
        dev = _device_rows(X)
        if dev is not None:
            self._fit_device(dev)
        else:
            X_np = _to_np(X)
            _check_data_content(self.do_checks, "X", X_np)
            self._fit(X_np)
        self._did_sklearn_fit = 0
        return self

    def _device_handle(self, dev, k, sets=1):
        """A handle that adopts the device rows (no copy)."""
        if self._load_lib() is None:
            raise RuntimeError("device input needs a usable GPU")
        from ..libs import kmeans_hip
        h = kmeans_hip.Handle(dev.rows, dev.cols, k, dev.dtype, gpu_id=self._gpu_id, verbose=self.verbose,
                              sets=sets)
        h.set_data_device(dev.ptr, keepalive=dev.owner)
        return h

    def _seed_handle(self, h, start, seed):
        """Initial centroids of the handle's selected set."""
        if start is not None:
            h.set_centroids(start)
        elif self.init in ("k-means++", "k-means||"):
            h.init_parallel(seed)
        elif self.init == "d2-sampling":
            h.init_plusplus(seed)
        else:
            h.init_random_rows(seed)

    def _fit_on_handle(self, make_handle, rows, cols, dtype, k, start):
        """Runs the restarts (seeds random_state, random_state + 1, ...) on rows that stay on
        the device, keeps the one with the lowest inertia, and sets the fitted attributes.
        As many restarts as the shape allows run stacked: their centroid sets form one model,
        one kernel labels every row against all of them and sums the rows per set, so every
        iteration reads the rows once for the whole group (the reference documents n_init > 1
        as unsupported, kmeans.py:722-725). make_handle(sets) returns a handle that holds
        the rows."""
        from ..libs import kmeans_hip
        restarts = 1 if start is not None else max(1, int(self.n_init or 1))
        width = kmeans_hip.stack_width(rows, cols, k, dtype, restarts) if restarts > 1 else 1
        groups = -(-restarts // width)
        sets = -(-restarts // groups)  # balanced groups; a spare set repeats the group's first start
        best = None
        with make_handle(sets) as h:
            for g in range(groups):
                members = [g * sets + s for s in range(sets)]
                for s, r in enumerate(members):
                    if sets > 1:
                        h.select_set(s)
                    self._seed_handle(h, start, self.random_state + (r if r < restarts else members[0]))
                n_iter = h.fit(self._max_iter, self.tol)
                iters = h.set_iterations() if sets > 1 else [n_iter]
                for s, r in enumerate(members):
                    if r >= restarts:
                        continue
                    if sets > 1:
                        h.select_set(s)
                    inertia = h.inertia() if self._max_iter > 0 else None
                    if best is None or (inertia is not None and inertia < best[2]):
                        best = (h.centroids(), h.labels(), inertia, int(iters[s]))
        centers, self.labels_, self.inertia_, self.n_iter_ = best
        if k < self._n_clusters:
            # more clusters asked for than rows: the fit ran with k = rows (kmeans_h2o4gpu.cu:630-635);
            # the result keeps n_clusters rows, the rest zero, exactly as the host-pointer entry point
            # leaves its preallocated array, so predict / transform see one shape whichever path fitted
            centers = np.concatenate([centers, np.zeros((self._n_clusters - k, cols), centers.dtype)])
        self.cluster_centers_ = centers
        return self.cluster_centers_, self.labels_

    def _fit_device(self, dev):
        """fit on rows resident in device memory, through the handle entry points: same
        start rules, loop and outputs as the host-pointer entry point."""
        self.double_precision = 1 if dev.dtype == np.float64 else 0
        k = min(self._n_clusters, dev.rows)  # clamp as kmeans_h2o4gpu.cu:630-635
        start = None
        if isinstance(self.init, np.ndarray):
            assert self.init.shape == (self._n_clusters, dev.cols), \
                "init must have shape (n_clusters, n_features)"
            start = np.ascontiguousarray(self.init[:k], dtype=dev.dtype)
        return self._fit_on_handle(lambda sets: self._device_handle(dev, k, sets), dev.rows, dev.cols,
                                   dev.dtype, k, start)

    def sklearn_fit(self, X, y=None):
        assert self.cluster_centers_ is not None, "Centroids are None. Run fit() first."
        if self._did_sklearn_fit == 0:
            X_np = _to_np(X)
            _check_data_content(self.do_checks, "X", X_np)
            self._did_sklearn_fit = 1
            import sklearn.cluster as sk_cluster
            self.sklearn_model = sk_cluster.KMeans(self._n_clusters, max_iter=1,
                                                   init=self.cluster_centers_, n_init=1)
            self.sklearn_model.fit(X_np)
            self.sklearn_model.cluster_centers_ = self.cluster_centers_

    def predict(self, X):
        lib = self._require_lib("predict")
        cols, rows = self._validate_centroids(X)
        dev = _device_rows(X)
        if dev is not None:
            with self._device_handle(dev, self.cluster_centers_.shape[0]) as h:
                h.set_centroids(self.cluster_centers_)
                h.assign()
                return h.labels()
        X_np = _to_np(X)
        _check_data_content(self.do_checks, "X", X_np)
        c_X_np = self._toc(X_np)
        cluster_centers_ = self._toc(self.cluster_centers_, convert=False)
        c_res = np.zeros(rows, np.int32)
        c_kmeans = lib.make_ptr_float_kmeans if self.double_precision == 0 else lib.make_ptr_double_kmeans
        k = int(self.cluster_centers_.shape[0])  # (== n_clusters after fit; the array decides)
        status = c_kmeans(1, self.verbose, self.random_state, self._gpu_id, self.n_gpus, rows, cols,
                          k, self._max_iter, 0, self.tol, c_X_np, cluster_centers_,
                          np.empty([], X_np.dtype), c_res)
        if status:
            raise RuntimeError("KMeans predict failed in the native library (status %d)" % status)
        return c_res

    def sklearn_predict(self, X, y=None):
        _check_data_content(self.do_checks, "X", X)
        self.sklearn_fit(X)
        return self.sklearn_model.predict(X)

    def transform(self, X, y=None):
        """Squared distances to every centre, shape (rows, n_clusters) (the reference returns
        the squared values, kmeans.py:389-422 with kmeans_h2o4gpu.cu:937-950)."""
        lib = self._require_lib("transform")
        cols, rows = self._validate_centroids(X)
        dev = _device_rows(X)
        if dev is not None:
            return self._transform_device(X, dev)
        X_np = _to_np(X)
        c_X_np = self._toc(X_np)
        cluster_centers_ = self._toc(self.cluster_centers_, convert=False)
        k = int(self.cluster_centers_.shape[0])  # (== n_clusters after fit; the array decides)
        owned = getattr(lib, "kmeans_transform_owned", None)
        if owned is not None:  # adopt the library's buffer instead of zero-filling and copying
            status, c_res = owned(self.verbose, self._gpu_id, self.n_gpus, rows, cols, k,
                                  c_X_np, cluster_centers_, X_np.dtype)
            if status != 0:
                raise RuntimeError("KMeans transform failed in the native library (status %d)" % status)
            return np.reshape(c_res, (rows, k), order='F')
        c_res = np.zeros(rows * k, X_np.dtype)
        fn = lib.kmeans_transform_float if self.double_precision == 0 else lib.kmeans_transform_double
        status = fn(self.verbose, self._gpu_id, self.n_gpus, rows, cols, k, c_X_np,
                    cluster_centers_, c_res)
        if status:
            raise RuntimeError("KMeans transform failed in the native library (status %d)" % status)
        return np.reshape(c_res, (rows, k), order='F')

    def _transform_device(self, X, dev):
        """Distances of device rows, left on the device: a (rows, k) view of the engine's
        centroid-major [k][rows] result, i.e. the same Fortran-ordered layout the host path
        returns. The output buffer comes from the array's own library."""
        torch = sys.modules.get("torch")
        if torch is None or not isinstance(X, torch.Tensor):
            raise TypeError("transform of device rows returns a device array and is available "
                            "for PyTorch tensors; pass host rows otherwise")
        k = self.cluster_centers_.shape[0]
        out = torch.empty((k, dev.rows), dtype=X.dtype, device=X.device)
        torch.cuda.current_stream(X.device).synchronize()
        with self._device_handle(dev, k) as h:
            h.set_centroids(self.cluster_centers_)
            h.transform_resident(out.data_ptr())
        return out.t()

    def sklearn_transform(self, X, y=None):
        _check_data_content(self.do_checks, "X", X)
        self.sklearn_fit(X)
        return self.sklearn_model.transform(X)

    def fit_transform(self, X, y=None):
        return self.fit(X, y).transform(X)

    def fit_predict(self, X, y=None):
        return self.fit(X, y).labels_

    def _fit(self, data):
        lib = self._require_lib("fit")
        c_data = self._toc(data)
        rows = np.shape(data)[0]
        cols = np.shape(data)[1]
        centroids = np.empty([])
        if isinstance(self.init, np.ndarray):
            init_arr = np.asarray(self.init)
            assert init_arr.shape == (self._n_clusters, cols), \
                "init must have shape (n_clusters, n_features)"
            c_init = 2
            centroids = np.ascontiguousarray(init_arr, dtype=data.dtype).flatten()
        elif self.init in ("k-means++", "k-means||"):
            c_init = 1  # kmeans.py:472-475; the native side runs k-means|| for it, as the reference
        elif self.init == "d2-sampling":
            c_init = 3
        else:
            c_init = 0
        fn = lib.make_ptr_float_kmeans if self.double_precision == 0 else lib.make_ptr_double_kmeans
        # n_init restarts (seed, seed+1, ...) keep the lowest inertia; the reference runs one
        # (kmeans.py:722-725). Restarts are pointless when the start is given.
        restarts = 1 if c_init == 2 else max(1, int(self.n_init or 1))
        if restarts > 1:
            # the rows go to the device once and stay there for all restarts
            from ..libs import kmeans_hip
            k = min(self._n_clusters, rows)
            dtype = np.float64 if self.double_precision else np.float32
            host = np.ascontiguousarray(np.reshape(c_data, (rows, cols)), dtype=dtype)

            def make_handle(sets):
                h = kmeans_hip.Handle(rows, cols, k, dtype, gpu_id=self._gpu_id, verbose=self.verbose,
                                      sets=sets)
                h.set_data(host)
                return h
            return self._fit_on_handle(make_handle, rows, cols, dtype, k, None)
        best = None
        owned = getattr(lib, "kmeans_fit_owned", None)
        for r in range(restarts):
            if owned is not None:  # adopt the library's buffers: no zero-fill, no copy
                status, pred_centers, pred_labels = owned(
                    self.verbose, self.random_state + r, self._gpu_id, self.n_gpus, rows, cols,
                    self._n_clusters, self._max_iter, c_init, self.tol, c_data, centroids, data.dtype)
                if status == 0 and pred_centers.size < cols * self._n_clusters:
                    # more clusters asked for than rows: the library clamps k (kmeans_h2o4gpu.cu:630-635)
                    pred_centers = np.concatenate([pred_centers, np.zeros(
                        cols * self._n_clusters - pred_centers.size, data.dtype)])
            else:
                pred_centers = np.zeros(cols * self._n_clusters, data.dtype)
                pred_labels = np.zeros(rows, dtype=np.int32)
                status = fn(0, self.verbose, self.random_state + r, self._gpu_id, self.n_gpus, rows,
                            cols, self._n_clusters, self._max_iter, c_init, self.tol, c_data, centroids,
                            pred_centers, pred_labels)
            if status != 0:
                raise RuntimeError("KMeans fit failed in the native library (status %d)" % status)
            # a module that offers only the reference's entry points has no such getter
            getter = getattr(lib, "last_fit_info", None)
            info = getter() if getter is not None else None
            inertia, n_iter = info if info is not None else (None, None)
            if best is None or (inertia is not None and inertia < best[2]):
                best = (pred_centers, pred_labels, inertia, n_iter)
        pred_centers, pred_labels, self.inertia_, self.n_iter_ = best
        self.cluster_centers_ = np.reshape(pred_centers, (self._n_clusters, cols))
        self.labels_ = np.reshape(pred_labels, rows)
        return self.cluster_centers_, self.labels_

    def score(self, X, y=None):
        """Opposite of the k-means objective of X under the fitted centres: the rows go to
        the device once, one assignment pass, and the minimum distances are summed there."""
        self._validate_centroids(X)
        if self._load_lib() is None:
            raise RuntimeError("score needs a usable GPU")
        from ..libs import kmeans_hip
        dev = _device_rows(X)
        if dev is not None:
            with self._device_handle(dev, self.cluster_centers_.shape[0]) as h:
                h.set_centroids(self.cluster_centers_)
                h.assign()
                return -h.inertia()
        X_np = _to_np(X)
        dtype = np.float64 if X_np.dtype == np.float64 else np.float32
        X_np = np.ascontiguousarray(X_np, dtype=dtype)
        with kmeans_hip.Handle(X_np.shape[0], X_np.shape[1], int(self.cluster_centers_.shape[0]), dtype,
                               gpu_id=self._gpu_id, verbose=self.verbose) as h:
            h.set_data(X_np)
            h.set_centroids(np.ascontiguousarray(self.cluster_centers_, dtype=dtype))
            h.assign()
            return -h.inertia()

    def _toc(self, data, convert=True):
        if convert and data.dtype != np.float64 and data.dtype != np.float32:
            self._print_verbose(1, "Detected numeric data format which is not supported. "
                                   "Casting to np.float32.")
            data = np.asarray(data, dtype=np.float32)
        if data.dtype == np.float64:
            self._print_verbose(1, "Detected np.float64 data")
            self.double_precision = 1
        elif data.dtype == np.float32:
            self._print_verbose(1, "Detected np.float32 data")
            self.double_precision = 0
        # row-major and contiguous, without the copy flatten() always makes
        return np.ascontiguousarray(data).reshape(-1)

    def _print_verbose(self, level, msg):
        if self.verbose > level:
            print(msg)
            sys.stdout.flush()

    def _load_lib(self):
        """The native module, or None when no GPU can be used (the caller then falls back
        to scikit-learn, as in the reference kmeans.py:532-546)."""
        if (self.n_gpus == 0) or (self.devices == 0):
            self._print_verbose(0, "H2O KMeans for CPU not yet supported.")
            return None
        from ..libs import ch2o4gpu_gpu
        self._print_verbose(0, "\nUsing GPU KMeans solver with %d GPUs.\n" % self.n_gpus)
        return ch2o4gpu_gpu

    def _require_lib(self, what):
        lib = self._load_lib()
        if lib is None:
            raise RuntimeError("KMeansH2O.%s needs a usable GPU (n_gpus=%r, visible devices %r); "
                               "use KMeans(backend='sklearn') to run on the CPU"
                               % (what, self.n_gpus, self.devices))
        return lib

    def _validate_centroids(self, X):
        assert self.cluster_centers_ is not None, "Centroids are None. Run fit() first."
        rows = np.shape(X)[0]
        cols = np.shape(X)[1]
        centroids_dim = np.shape(self.cluster_centers_)[1]
        assert cols == centroids_dim, \
            "The dimension of X [%d] and centroids [%d] is not equal." % (cols, centroids_dim)
        return cols, rows

    @property
    def n_clusters(self):
        return self._n_clusters

    @n_clusters.setter
    def n_clusters(self, value):
        assert_satisfies(value, value > 0, "Number of clusters must be positive.")
        self._n_clusters = value

    @property
    def gpu_id(self):
        return self._gpu_id

    @gpu_id.setter
    def gpu_id(self, value):
        assert_satisfies(value, value >= 0, "GPU ID must be non-negative.")
        self._gpu_id = value

    @property
    def max_iter(self):
        return self._max_iter

    @max_iter.setter
    def max_iter(self, value):
        assert_satisfies(value, value > 0, "Number of maximum iterations must be non-negative.")
        self._max_iter = value


class KMeans:
    """Backend selector (reference class KMeans, kmeans.py:591-829): 'auto' uses the GPU
    engine when a device is usable, 'sklearn' forces scikit-learn, 'h2o4gpu' forces the
    engine. The environment variable H2O4GPU_BACKEND overrides the argument."""

    def __init__(self, n_clusters=8, init='k-means++', n_init=1, max_iter=300, tol=1e-4,
                 precompute_distances='auto', verbose=0, random_state=None, copy_x=True, n_jobs=1,
                 algorithm='auto', gpu_id=0, n_gpus=-1, do_checks=1, backend='auto'):
        import os
        _backend = os.environ.get('H2O4GPU_BACKEND', None)
        if _backend is not None:
            backend = _backend
        self._backend_arg = backend
        # constructor arguments as given: what get_params reports, so that
        # KMeans(**est.get_params()) rebuilds the same selection (sklearn.base.clone)
        self._ctor_args = dict(n_clusters=n_clusters, init=init, n_init=n_init, max_iter=max_iter, tol=tol,
                               precompute_distances=precompute_distances, verbose=verbose,
                               random_state=random_state, copy_x=copy_x, n_jobs=n_jobs,
                               algorithm=algorithm, gpu_id=gpu_id, n_gpus=n_gpus, do_checks=do_checks,
                               backend=backend)
        self.do_sklearn = backend == 'sklearn'
        self.model_h2o4gpu = KMeansH2O(n_clusters=n_clusters, init=init, n_init=n_init, max_iter=max_iter,
                                       tol=tol, precompute_distances=precompute_distances,
                                       verbose=verbose, random_state=random_state, copy_x=copy_x,
                                       n_jobs=n_jobs, algorithm=algorithm, gpu_id=gpu_id, n_gpus=n_gpus,
                                       do_checks=do_checks)
        # (scikit-learn knows the engine's two extra seeding names only as 'k-means++')
        sk_init = 'k-means++' if isinstance(init, str) and init in ('k-means||', 'd2-sampling') else init
        self._sk_args = dict(n_clusters=n_clusters, init=sk_init, n_init=n_init, max_iter=max_iter, tol=tol,
                             verbose=verbose, random_state=random_state, copy_x=copy_x)
        self.model_sklearn = None
        # scikit-learn is used only when asked for (backend='sklearn' or n_gpus=0). The
        # reference also drops to scikit-learn silently when no GPU library or device is
        # found (kmeans.py:766-773); here that case raises instead, so a missing build or
        # device is never mistaken for a GPU run.
        # pylint: disable=protected-access
        if not self.do_sklearn and n_gpus != 0 and self.model_h2o4gpu._load_lib() is None:
            raise RuntimeError("KMeans(backend=%r): no usable GPU (visible devices: %d). Pass "
                               "backend='sklearn' or n_gpus=0 to run scikit-learn on the CPU."
                               % (backend, self.model_h2o4gpu.devices))
        if self.do_sklearn or n_gpus == 0:
            if backend == 'h2o4gpu':
                raise RuntimeError("backend='h2o4gpu' was requested with n_gpus=0")
            self.backend = 'sklearn'
            self.model = self._sklearn()
            KMeans._print_verbose(verbose, 0, "Using ScikitLearn backend.")
        else:
            self.backend = 'h2o4gpu'
            self.model = self.model_h2o4gpu
            KMeans._print_verbose(verbose, 0, "Using h2o4gpu backend.")
        self.cluster_centers_ = None
        self.labels_ = None
        self.inertia_ = None

    def _sklearn(self):
        if self.model_sklearn is None:
            import sklearn.cluster as sk_cluster
            self.model_sklearn = sk_cluster.KMeans(**self._sk_args)
        return self.model_sklearn

    def fit(self, X, y=None):
        res = self.model.fit(X, y)
        self.set_attributes()
        return res

    def fit_predict(self, X, y=None):
        res = self.model.fit_predict(X, y)
        self.set_attributes()
        return res

    def fit_transform(self, X, y=None):
        res = self.model.fit_transform(X, y)
        self.set_attributes()
        return res

    def get_params(self, deep=True):
        # the selector's own constructor arguments, refreshed from the selected model for
        # the ones it knows (set_params or attribute assignment may have changed them)
        params = dict(self._ctor_args)
        for key, value in self.model.get_params(deep).items():
            if key in params and key not in ("n_gpus", "random_state", "tol"):
                params[key] = value
        return params

    def predict(self, X):
        res = self.model.predict(X)
        self.set_attributes()
        return res

    def score(self, X, y=None):
        """Opposite of the k-means objective on X (scikit-learn's definition)."""
        return self.model.score(X, y)

    def set_params(self, **params):
        params = dict(params)
        if "backend" in params:
            # the backend is chosen at construction; the same value is accepted silently
            backend = params.pop("backend")
            if backend != self._backend_arg:
                raise ValueError("backend is fixed at construction (%r); build a new KMeans for %r"
                                 % (self._backend_arg, backend))
        known = self.model.get_params(deep=False)
        unknown = [key for key in params if key not in self._ctor_args]
        if unknown:
            raise ValueError("Invalid parameter %s for estimator KMeans." % unknown[0])
        self.model.set_params(**{key: value for key, value in params.items() if key in known})
        self._ctor_args.update(params)
        self.set_attributes()
        return self

    def __sklearn_tags__(self):
        return _clusterer_tags()

    def transform(self, X):
        res = self.model.transform(X)
        self.set_attributes()
        return res

    def set_attributes(self):
        for name in ("cluster_centers_", "labels_", "inertia_", "n_iter_"):
            setattr(self, name, getattr(self.model, name, None))

    @staticmethod
    def _print_verbose(verbose, level, msg):
        if verbose > level:
            print(msg)
            sys.stdout.flush()
