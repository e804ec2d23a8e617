"""ctypes binding of oracle/liboracle_kmeans.so (test infrastructure only)."""
import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB = os.path.join(_HERE, "liboracle_kmeans.so")

_i64 = ctypes.c_int64
_int = ctypes.c_int
_dbl = ctypes.c_double
_vp = ctypes.c_void_p


def build_oracle(force=False):
    """Compile the oracle with g++ (make -C oracle)."""
    if force and os.path.exists(_LIB):
        os.remove(_LIB)
    subprocess.check_call(["make", "-C", _HERE, "liboracle_kmeans.so"],
                          stdout=subprocess.DEVNULL)
    return _LIB


def _ptr(a):
    return None if a is None else a.ctypes.data_as(_vp)


class Oracle:
    """Thin numpy front for the C++ restatement. dtype picks the f32/f64 symbols."""

    def __init__(self, lib):
        self.lib = lib
        self.max_threads = int(lib.oracle_max_threads())

    @staticmethod
    def _suf(dtype):
        dtype = np.dtype(dtype)
        if dtype == np.float32:
            return "f32"
        if dtype == np.float64:
            return "f64"
        raise TypeError("oracle handles float32/float64 only, got %s" % dtype)

    def _fn(self, name, dtype):
        return getattr(self.lib, "oracle_%s_%s" % (name, self._suf(dtype)))

    @staticmethod
    def _prep(X, C=None):
        X = np.ascontiguousarray(X)
        assert X.ndim == 2
        if C is not None:
            C = np.ascontiguousarray(C, dtype=X.dtype)
            assert C.ndim == 2 and C.shape[1] == X.shape[1]
        return X, C

    def row_norms(self, X, threads=1):
        X, _ = self._prep(X)
        out = np.empty(X.shape[0], X.dtype)
        f = self._fn("row_norms", X.dtype)
        f(_i64(X.shape[0]), _int(X.shape[1]), _ptr(X), _ptr(out), _int(threads))
        return out

    def assign(self, X, C, threads=1, return_mindist=False):
        X, C = self._prep(X, C)
        n, d = X.shape
        labels = np.empty(n, np.int32)
        mind = np.empty(n, X.dtype) if return_mindist else None
        self._fn("assign", X.dtype)(_i64(n), _int(d), _int(C.shape[0]), _ptr(X),
                                    _ptr(C), _ptr(labels), _ptr(mind), _int(threads))
        return (labels, mind) if return_mindist else labels

    def distances(self, X, C, threads=1):
        """Squared distances, centroid-major: result[c, i]."""
        X, C = self._prep(X, C)
        n, d = X.shape
        k = C.shape[0]
        D = np.empty((k, n), X.dtype)
        self._fn("distances", X.dtype)(_i64(n), _int(d), _int(k), _ptr(X), _ptr(C),
                                       _ptr(D), _int(threads))
        return D

    def update_sums(self, X, labels, k, threads=1):
        X, _ = self._prep(X)
        n, d = X.shape
        labels = np.ascontiguousarray(labels, np.int32)
        sums = np.empty((k, d), X.dtype)
        counts = np.empty(k, np.int32)
        self._fn("update_sums", X.dtype)(_i64(n), _int(d), _int(k), _ptr(X),
                                         _ptr(labels), _ptr(sums), _ptr(counts),
                                         _int(threads))
        return sums, counts

    def finalize(self, sums, counts, old_c):
        sums = np.ascontiguousarray(sums)
        old_c = np.ascontiguousarray(old_c, sums.dtype)
        counts = np.ascontiguousarray(counts, np.int32)
        k, d = sums.shape
        new_c = np.empty_like(sums)
        self._fn("finalize", sums.dtype)(_int(d), _int(k), _ptr(sums), _ptr(counts),
                                         _ptr(old_c), _ptr(new_c))
        return new_c

    def update(self, X, labels, C, threads=1):
        """Returns (new centroids, counts); C is not modified."""
        X, C = self._prep(X, C)
        n, d = X.shape
        k = C.shape[0]
        labels = np.ascontiguousarray(labels, np.int32)
        Cn = C.copy()
        counts = np.empty(k, np.int32)
        self._fn("update", X.dtype)(_i64(n), _int(d), _int(k), _ptr(X), _ptr(labels),
                                    _ptr(Cn), _ptr(counts), _int(threads))
        return Cn, counts

    def lloyd(self, X, C0, max_iter, threshold=0.0, threads=1):
        """Returns (centroids, labels, iteration index at exit, shift^2 history)."""
        X, C0 = self._prep(X, C0)
        n, d = X.shape
        k = C0.shape[0]
        C = C0.copy()
        labels = np.full(n, -1, np.int32)
        hist = np.full(max(max_iter, 1), np.nan, np.float64)
        fn = self._fn("lloyd", X.dtype)
        fn.restype = _int
        it = fn(_i64(n), _int(d), _int(k), _ptr(X), _ptr(C), _ptr(labels),
                _int(max_iter), _dbl(threshold), _int(threads), _ptr(hist))
        return C, labels, int(it), hist

    def top2_exact(self, X, C, threads=1):
        X, C = self._prep(X, C)
        n, d = X.shape
        best = np.empty(n, np.int32)
        d1 = np.empty(n, np.float64)
        d2 = np.empty(n, np.float64)
        self._fn("top2_exact", X.dtype)(_i64(n), _int(d), _int(C.shape[0]), _ptr(X),
                                        _ptr(C), _ptr(best), _ptr(d1), _ptr(d2),
                                        _int(threads))
        return best, d1, d2

    def pair_dist_exact(self, X, C, a, b, threads=1):
        X, C = self._prep(X, C)
        n, d = X.shape
        a = np.ascontiguousarray(a, np.int32)
        b = np.ascontiguousarray(b, np.int32)
        da = np.empty(n, np.float64)
        db = np.empty(n, np.float64)
        self._fn("pair_dist_exact", X.dtype)(_i64(n), _int(d), _ptr(X), _ptr(C),
                                             _ptr(a), _ptr(b), _ptr(da), _ptr(db),
                                             _int(threads))
        return da, db

    def set_dot_order(self, descending):
        """Summation order of the distance dot product: features ascending (False,
        default) or descending (True)."""
        self.lib.oracle_set_dot_order(_int(1 if descending else 0))

    def random_rows(self, seed, n, k):
        idx = np.empty(k, np.int32)
        self.lib.oracle_random_rows(_int(seed), _i64(n), _int(k), _ptr(idx))
        return idx

    def kmeanspp(self, X, k, seed):
        """Rows chosen by k-means++ (D^2 sampling) and the final minimum distances."""
        X, _ = self._prep(X)
        n, d = X.shape
        rows = np.empty(k, np.int32)
        mind = np.empty(n, X.dtype)
        self._fn("kmeanspp", X.dtype)(_i64(n), _int(d), _int(k), _ptr(X), _int(seed), _ptr(rows),
                                      _ptr(mind))
        return rows, mind

    def minstd_nth(self, seed, nth):
        """Value of the nth call (nth >= 1) of thrust's default_random_engine seeded with seed."""
        self.lib.oracle_minstd_nth.restype = ctypes.c_uint
        return int(self.lib.oracle_minstd_nth(_int(seed), _i64(nth)))

    def row_threshold(self, seed, row):
        """The k-means|| acceptance threshold of a data row (float)."""
        self.lib.oracle_kmeans_parallel_row_threshold.restype = ctypes.c_float
        return float(self.lib.oracle_kmeans_parallel_row_threshold(_int(seed), _i64(row)))

    def pick_point_idx_weighted(self, seed, weights, data=None):
        weights = np.ascontiguousarray(weights)
        if data is not None:
            data = np.ascontiguousarray(data, weights.dtype)
        fn = self._fn("pick_point_idx_weighted", weights.dtype)
        fn.restype = _int
        return int(fn(_int(seed), _int(weights.shape[0]), _ptr(data), _ptr(weights)))

    def weighted_kmeanspp(self, seed, data, weights, k):
        """Candidate indices chosen by the reference's host k-means++ over weighted candidates."""
        data = np.ascontiguousarray(data)
        weights = np.ascontiguousarray(weights, data.dtype)
        m, d = data.shape
        chosen = np.empty(k, np.int32)
        self._fn("weighted_kmeanspp", data.dtype)(_int(seed), _int(m), _int(d), _int(k), _ptr(data),
                                                  _ptr(weights), _ptr(chosen))
        return chosen

    def kmeans_parallel(self, X, k, seed, threads=1, cap=None):
        """k-means|| as the reference runs it. Returns a dict: cand_rows (data row of every
        candidate, in the order found), round_count [8], phi [8], weights (None when there
        were at most k candidates), chosen [k] (candidate index, -1 = zero row), centroids."""
        X, _ = self._prep(X)
        n, d = X.shape
        cap = int(cap if cap is not None else min(n * 8 + 1, max(64 * k + 64, 4096)))
        cand = np.empty(cap, np.int32)
        rc = np.zeros(8, np.int32)
        phi = np.zeros(8, np.float64)
        weights = np.zeros(cap, X.dtype)
        chosen = np.empty(k, np.int32)
        C = np.empty((k, d), X.dtype)
        fn = self._fn("kmeans_parallel", X.dtype)
        fn.restype = _int
        m = int(fn(_i64(n), _int(d), _int(k), _ptr(X), _int(seed), _int(cap), _ptr(cand), _ptr(rc),
                   _ptr(phi), _ptr(weights), _ptr(chosen), _ptr(C), _int(threads)))
        if m < 0:
            raise RuntimeError("k-means||: more than %d candidates" % cap)
        return {"cand_rows": cand[:m].copy(), "round_count": rc, "phi": phi,
                "weights": weights[:m].copy() if m > k else None, "chosen": chosen, "centroids": C}

    def kmeanspp_first(self, seed, n):
        self.lib.oracle_kmeanspp_first.restype = _int
        return int(self.lib.oracle_kmeanspp_first(_int(seed), _i64(n)))


_cached = None


def load_oracle(build_if_missing=True):
    global _cached
    if _cached is None:
        if not os.path.exists(_LIB):
            if not build_if_missing:
                raise FileNotFoundError(_LIB)
            build_oracle()
        _cached = Oracle(ctypes.CDLL(_LIB))
    return _cached
