"""ctypes binding of libh2o4gpu_kmeans_hip.so (the C ABI in include/h2o4gpu_kmeans.h).

The library is the only compute path: if it is missing or cannot be loaded the
import of this module's `lib()` raises, nothing falls back to the CPU.
"""
import ctypes
import os

import numpy as np

_PKG = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
# H2O4GPU_KMEANS_LIB may point at another build of the same library
LIB_PATH = os.environ.get("H2O4GPU_KMEANS_LIB") or os.path.join(_PKG, "libh2o4gpu_kmeans_hip.so")

c_int = ctypes.c_int
c_size_t = ctypes.c_size_t
c_double = ctypes.c_double
c_float = ctypes.c_float
c_void_p = ctypes.c_void_p
c_char_p = ctypes.c_char_p
P = ctypes.POINTER

# every symbol include/h2o4gpu_kmeans.h declares: name -> (restype, argtypes)
PROTOTYPES = {
    "make_ptr_float_kmeans": (c_int, [c_int, c_int, c_int, c_int, c_int, c_size_t, c_size_t, c_int,
                                      c_int, c_int, c_float, c_void_p, c_void_p,
                                      P(c_void_p), P(c_void_p)]),
    "make_ptr_double_kmeans": (c_int, [c_int, c_int, c_int, c_int, c_int, c_size_t, c_size_t, c_int,
                                       c_int, c_int, c_double, c_void_p, c_void_p,
                                       P(c_void_p), P(c_void_p)]),
    "kmeans_transform_float": (c_int, [c_int, c_int, c_int, c_size_t, c_size_t, c_int, c_void_p,
                                       c_void_p, P(c_void_p)]),
    "kmeans_transform_double": (c_int, [c_int, c_int, c_int, c_size_t, c_size_t, c_int, c_void_p,
                                        c_void_p, P(c_void_p)]),
    "get_gpu_info_c": (c_int, [c_int] * 9 + [P(ctypes.c_uint), c_void_p, c_void_p, c_void_p,
                                             P(c_char_p), c_void_p, c_void_p, c_void_p, c_void_p,
                                             c_void_p, c_void_p, c_void_p, c_void_p]),
    "get_compute_capability": (c_int, [c_int, P(c_int), P(c_int), P(c_int)]),
    "cudaresetdevice": (c_int, [c_int, c_int]),
    "cudaresetdevice_bare": (c_int, []),
    "h2o4gpu_kmeans_device_count": (c_int, []),
    "h2o4gpu_kmeans_last_fit_info": (c_int, [P(c_double), P(c_int)]),
    "h2o4gpu_kmeans_host_all_finite": (c_int, [c_void_p, c_size_t, c_int]),
    "h2o4gpu_kmeans_random_start_rows": (c_int, [c_int, c_size_t, c_int, c_void_p]),
    "h2o4gpu_kmeans_create": (c_int, [P(c_void_p), c_int, c_size_t, c_size_t, c_int, c_int, c_int]),
    "h2o4gpu_kmeans_destroy": (c_int, [c_void_p]),
    "h2o4gpu_kmeans_stack_width": (c_int, [c_int, c_size_t, c_size_t, c_int, c_int]),
    "h2o4gpu_kmeans_create_stacked": (c_int, [P(c_void_p), c_int, c_size_t, c_size_t, c_int, c_int, c_int,
                                              c_int]),
    "h2o4gpu_kmeans_select_set": (c_int, [c_void_p, c_int]),
    "h2o4gpu_kmeans_set_iterations": (c_int, [c_void_p, c_void_p]),
    "h2o4gpu_kmeans_set_data_host": (c_int, [c_void_p, c_void_p]),
    "h2o4gpu_kmeans_set_data_device": (c_int, [c_void_p, c_void_p]),
    "h2o4gpu_kmeans_set_centroids_host": (c_int, [c_void_p, c_void_p]),
    "h2o4gpu_kmeans_init_random_rows": (c_int, [c_void_p, c_int]),
    "h2o4gpu_kmeans_init_plusplus": (c_int, [c_void_p, c_int]),
    "h2o4gpu_kmeans_init_parallel": (c_int, [c_void_p, c_int]),
    "h2o4gpu_kmeans_parallel_seed_info": (c_int, [c_void_p, c_int, c_void_p, P(c_int), c_void_p, c_void_p,
                                                  c_void_p, c_void_p]),
    "h2o4gpu_kmeans_get_seed_rows": (c_int, [c_void_p, c_void_p]),
    "h2o4gpu_kmeans_fit": (c_int, [c_void_p, c_int, c_double, P(c_int)]),
    "h2o4gpu_kmeans_assign": (c_int, [c_void_p]),
    "h2o4gpu_kmeans_update": (c_int, [c_void_p, P(c_double)]),
    "h2o4gpu_kmeans_set_labels_host": (c_int, [c_void_p, c_void_p]),
    "h2o4gpu_kmeans_iterate": (c_int, [c_void_p, c_int]),
    "h2o4gpu_kmeans_get_centroids": (c_int, [c_void_p, c_void_p]),
    "h2o4gpu_kmeans_get_labels": (c_int, [c_void_p, c_void_p]),
    "h2o4gpu_kmeans_get_counts": (c_int, [c_void_p, c_void_p]),
    "h2o4gpu_kmeans_get_min_distances": (c_int, [c_void_p, c_void_p]),
    "h2o4gpu_kmeans_inertia": (c_int, [c_void_p, P(c_double)]),
    "h2o4gpu_kmeans_predict_host": (c_int, [c_void_p, c_size_t, c_void_p, c_void_p]),
    "h2o4gpu_kmeans_transform_host": (c_int, [c_void_p, c_size_t, c_void_p, c_void_p]),
    "h2o4gpu_kmeans_transform_resident": (c_int, [c_void_p, c_void_p]),
    "h2o4gpu_kmeans_set_option": (c_int, [c_void_p, c_char_p, c_int]),
    "h2o4gpu_kmeans_timer_start": (c_int, [c_void_p]),
    "h2o4gpu_kmeans_timer_stop": (c_int, [c_void_p, P(c_float)]),
    "h2o4gpu_kmeans_profile": (c_int, [c_void_p, c_int]),
    "h2o4gpu_kmeans_kernel_time": (c_int, [c_void_p, c_char_p, P(c_int), P(c_double)]),
    "h2o4gpu_kmeans_assign_variant": (c_char_p, [c_void_p]),
    "h2o4gpu_kmeans_copy_probe": (c_int, [c_int, c_size_t, c_int, P(c_float)]),
    "h2o4gpu_kmeans_bandwidth_probe": (c_int, [c_int, c_int, c_size_t, c_int, P(c_float)]),
    "h2o4gpu_kmeans_predict_device_noalloc": (c_int, [c_int, c_size_t, c_size_t, c_int, c_void_p,
                                                      c_void_p, c_void_p, c_void_p]),
}

NOALLOC_SCRATCH_BYTES = 16 << 20

_lib = None
_libc = None


class KMeansHipError(RuntimeError):
    """A C-ABI call returned a negative status."""

    def __init__(self, fn, code):
        names = {-1: "allocation failed", -2: "bad argument", -3: "HIP device error",
                 -4: "call order / missing state", -5: "beyond the fixed scratch buffer"}
        RuntimeError.__init__(self, "%s returned %d (%s)" % (fn, code, names.get(code, "?")))
        self.code = code


def lib():
    """Loads the shared library (once). Raises if it has not been built."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise ImportError(
                "%s is missing: build it with `python -m h2o4gpu_amd.build` "
                "(hipcc, gfx950). There is no CPU fallback." % LIB_PATH)
        handle = ctypes.CDLL(LIB_PATH)
        for name, (res, args) in PROTOTYPES.items():
            fn = getattr(handle, name)  # AttributeError if the symbol is not exported
            fn.restype = res
            fn.argtypes = args
        _lib = handle
    return _lib


def libc_free(ptr):
    global _libc
    if _libc is None:
        _libc = ctypes.CDLL(None)
        _libc.free.argtypes = [c_void_p]
        _libc.free.restype = None
    _libc.free(ptr)


def _check(fn, rc):
    if rc != 0:
        raise KMeansHipError(fn, rc)


def _vp(a):
    return a.ctypes.data_as(c_void_p)


def stack_width(rows, cols, k, dtype, max_sets):
    """How many restarts of a k-cluster fit one stacked handle can run at once for this shape."""
    return int(lib().h2o4gpu_kmeans_stack_width(np.dtype(dtype).itemsize, int(rows), int(cols), int(k),
                                                int(max_sets)))


ASSIGN_VARIANTS = {"auto": 0, "valu": 1, "mfma_rowstat": 2, "mfma_tiled": 3, "wave_row": 4}


class Handle:
    """Resident data set + model working set on one GPU (part 3 of the C ABI)."""

    def __init__(self, rows, cols, k, dtype=np.float32, gpu_id=0, verbose=0, sets=1):
        """sets > 1: a stacked handle holding that many independent centroid sets (restarts)
        over the same rows; see stack_width() for how many a shape allows."""
        self.dtype = np.dtype(dtype)
        if self.dtype not in (np.dtype(np.float32), np.dtype(np.float64)):
            raise TypeError("float32 or float64 only")
        self.rows, self.cols, self.k = int(rows), int(cols), int(k)
        self.sets = int(sets)
        self._h = c_void_p()
        self._keep = None
        _check("create", lib().h2o4gpu_kmeans_create_stacked(ctypes.byref(self._h), self.dtype.itemsize,
                                                             self.rows, self.cols, self.k, self.sets,
                                                             gpu_id, verbose))

    def select_set(self, s):
        """Stacked handle: the set that set_centroids, init_*, centroids, labels, counts,
        min_distances, seed_rows and inertia address."""
        _check("select_set", lib().h2o4gpu_kmeans_select_set(self._h, int(s)))

    def set_iterations(self):
        """Stacked handle: centroid updates each set made in the last fit."""
        out = np.empty(self.sets, np.int32)
        _check("set_iterations", lib().h2o4gpu_kmeans_set_iterations(self._h, _vp(out)))
        return out

    def close(self):
        if self._h:
            lib().h2o4gpu_kmeans_destroy(self._h)
            self._h = c_void_p()

    def __del__(self):
        try:
            self.close()
        except Exception:  # interpreter shutdown
            pass

    def __enter__(self):
        return self

    def __exit__(self, *exc):
        self.close()

    def _arr(self, a, shape):
        a = np.ascontiguousarray(a, dtype=self.dtype)
        if a.shape != shape:
            raise ValueError("expected shape %s, got %s" % (shape, a.shape))
        return a

    def set_data(self, X):
        X = self._arr(X, (self.rows, self.cols))
        _check("set_data_host", lib().h2o4gpu_kmeans_set_data_host(self._h, _vp(X)))

    def set_data_device(self, ptr, keepalive=None):
        self._keep = keepalive
        _check("set_data_device", lib().h2o4gpu_kmeans_set_data_device(self._h, c_void_p(ptr)))

    def set_centroids(self, C):
        C = self._arr(C, (self.k, self.cols))
        _check("set_centroids_host", lib().h2o4gpu_kmeans_set_centroids_host(self._h, _vp(C)))

    def init_random_rows(self, seed):
        _check("init_random_rows", lib().h2o4gpu_kmeans_init_random_rows(self._h, seed))

    def init_plusplus(self, seed):
        _check("init_plusplus", lib().h2o4gpu_kmeans_init_plusplus(self._h, seed))

    def init_parallel(self, seed):
        """k-means|| as the reference runs it (its init_from_data == 1)."""
        _check("init_parallel", lib().h2o4gpu_kmeans_init_parallel(self._h, seed))

    def parallel_seed_info(self):
        """What the last init_parallel found: dict with cand_rows, round_count [8], phi [8],
        weights (None when there were at most k candidates) and chosen [k]."""
        m = c_int(0)
        rc = np.zeros(8, np.int32)
        phi = np.zeros(8, np.float64)
        chosen = np.empty(self.k, np.int32)
        _check("parallel_seed_info", lib().h2o4gpu_kmeans_parallel_seed_info(
            self._h, 0, None, ctypes.byref(m), _vp(rc), _vp(phi), None, _vp(chosen)))
        cand = np.empty(m.value, np.int32)
        w = np.empty(m.value, np.float64)
        _check("parallel_seed_info", lib().h2o4gpu_kmeans_parallel_seed_info(
            self._h, m.value, _vp(cand), None, None, None, _vp(w), None))
        return {"cand_rows": cand, "round_count": rc, "phi": phi,
                "weights": w if m.value > self.k else None, "chosen": chosen}

    def seed_rows(self):
        out = np.empty(self.k, np.int32)
        _check("get_seed_rows", lib().h2o4gpu_kmeans_get_seed_rows(self._h, _vp(out)))
        return out

    def fit(self, max_iter, threshold=0.0):
        it = c_int(0)
        _check("fit", lib().h2o4gpu_kmeans_fit(self._h, max_iter, threshold, ctypes.byref(it)))
        return it.value

    def assign(self):
        _check("assign", lib().h2o4gpu_kmeans_assign(self._h))

    def update(self, want_shift=True):
        s = c_double(0.0)
        _check("update", lib().h2o4gpu_kmeans_update(self._h, ctypes.byref(s) if want_shift else None))
        return s.value

    def iterate(self, steps):
        """Enqueue `steps` x (assign + update); returns without waiting."""
        _check("iterate", lib().h2o4gpu_kmeans_iterate(self._h, int(steps)))

    def set_labels(self, labels):
        labels = np.ascontiguousarray(labels, np.int32)
        assert labels.shape == (self.rows,)
        _check("set_labels_host", lib().h2o4gpu_kmeans_set_labels_host(self._h, _vp(labels)))

    def centroids(self):
        C = np.empty((self.k, self.cols), self.dtype)
        _check("get_centroids", lib().h2o4gpu_kmeans_get_centroids(self._h, _vp(C)))
        return C

    def labels(self):
        out = np.empty(self.rows, np.int32)
        _check("get_labels", lib().h2o4gpu_kmeans_get_labels(self._h, _vp(out)))
        return out

    def counts(self):
        out = np.empty(self.k, np.int32)
        _check("get_counts", lib().h2o4gpu_kmeans_get_counts(self._h, _vp(out)))
        return out

    def min_distances(self):
        out = np.empty(self.rows, self.dtype)
        _check("get_min_distances", lib().h2o4gpu_kmeans_get_min_distances(self._h, _vp(out)))
        return out

    def inertia(self):
        v = c_double(0.0)
        _check("inertia", lib().h2o4gpu_kmeans_inertia(self._h, ctypes.byref(v)))
        return v.value

    def predict(self, X):
        X = np.ascontiguousarray(X, dtype=self.dtype)
        assert X.ndim == 2 and X.shape[1] == self.cols
        out = np.empty(X.shape[0], np.int32)
        _check("predict_host", lib().h2o4gpu_kmeans_predict_host(self._h, X.shape[0], _vp(X), _vp(out)))
        return out

    def transform(self, X):
        """Squared distances, centroid-major: result[c, i]."""
        X = np.ascontiguousarray(X, dtype=self.dtype)
        assert X.ndim == 2 and X.shape[1] == self.cols
        out = np.empty((self.k, X.shape[0]), self.dtype)
        _check("transform_host", lib().h2o4gpu_kmeans_transform_host(self._h, X.shape[0], _vp(X), _vp(out)))
        return out

    def transform_resident(self, d_ptr):
        _check("transform_resident", lib().h2o4gpu_kmeans_transform_resident(self._h, c_void_p(d_ptr)))

    def set_option(self, name, value):
        if name == "assign" and isinstance(value, str):
            value = ASSIGN_VARIANTS[value]
        _check("set_option", lib().h2o4gpu_kmeans_set_option(self._h, name.encode(), int(value)))

    def assign_variant(self):
        return lib().h2o4gpu_kmeans_assign_variant(self._h).decode()

    def timer_start(self):
        _check("timer_start", lib().h2o4gpu_kmeans_timer_start(self._h))

    def timer_stop(self):
        ms = c_float(0.0)
        _check("timer_stop", lib().h2o4gpu_kmeans_timer_stop(self._h, ctypes.byref(ms)))
        return ms.value

    def profile(self, on):
        _check("profile", lib().h2o4gpu_kmeans_profile(self._h, 1 if on else 0))

    def kernel_time(self, name):
        n = c_int(0)
        ms = c_double(0.0)
        _check("kernel_time", lib().h2o4gpu_kmeans_kernel_time(self._h, name.encode(), ctypes.byref(n),
                                                               ctypes.byref(ms)))
        return n.value, ms.value


def copy_probe(nbytes, reps=10, gpu_id=0):
    """Average milliseconds of one device-to-device copy of nbytes."""
    ms = c_float(0.0)
    _check("copy_probe", lib().h2o4gpu_kmeans_copy_probe(gpu_id, nbytes, reps, ctypes.byref(ms)))
    return ms.value


PROBE_KINDS = {"copy": 0, "read": 1, "write": 2, "memcpy": 3}


def bandwidth_probe(kind, nbytes, reps=10, gpu_id=0):
    """Average milliseconds of one streaming pass over nbytes: kind "read" (read only), "write"
    (write only), "copy" (a kernel that reads and writes nbytes) or "memcpy" (hipMemcpy device
    to device)."""
    ms = c_float(0.0)
    _check("bandwidth_probe", lib().h2o4gpu_kmeans_bandwidth_probe(gpu_id, PROBE_KINDS[kind], nbytes, reps,
                                                                    ctypes.byref(ms)))
    return ms.value


def random_start_rows(seed, rows, k):
    """Rows a fit with init_from_data = 0 starts from (host-only computation)."""
    out = np.empty(k, np.int32)
    _check("random_start_rows", lib().h2o4gpu_kmeans_random_start_rows(int(seed), int(rows), int(k), _vp(out)))
    return out


def host_all_finite(arr):
    """True when every value of a C-contiguous float32/float64 host array is finite (one
    parallel pass on host threads; no device is touched)."""
    if arr.dtype not in (np.float32, np.float64) or not arr.flags.c_contiguous:
        raise TypeError("host_all_finite wants a C-contiguous float32 or float64 array")
    rc = lib().h2o4gpu_kmeans_host_all_finite(_vp(arr), int(arr.size), int(arr.itemsize))
    _check("host_all_finite", min(rc, 0))
    return rc == 1


def last_fit_info():
    """(inertia, iterations) of this thread's last successful fit through the
    make_ptr_*_kmeans entry points, or None when there is none."""
    inertia, iters = c_double(0.0), c_int(0)
    if lib().h2o4gpu_kmeans_last_fit_info(ctypes.byref(inertia), ctypes.byref(iters)) != 0:
        return None
    return float(inertia.value), int(iters.value)


def device_count():
    return int(lib().h2o4gpu_kmeans_device_count())


def predict_device_noalloc(dtype, rows, cols, k, d_X, d_centroids, d_labels, stream=None):
    """Queues the assignment of device-resident rows (raw device addresses) on `stream`
    without allocating anything; see part 4 of the C header."""
    rc = lib().h2o4gpu_kmeans_predict_device_noalloc(np.dtype(dtype).itemsize, int(rows), int(cols),
                                                     int(k), c_void_p(d_X), c_void_p(d_centroids),
                                                     c_void_p(d_labels), c_void_p(stream))
    _check("predict_device_noalloc", rc)
