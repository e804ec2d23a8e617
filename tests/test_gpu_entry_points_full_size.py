"""The five benchmark configurations, at their full size, through the four C symbols a binding
of the reference calls (make_ptr_float_kmeans / make_ptr_double_kmeans with dopredict 0 and 1,
kmeans_transform_float; reference: src/gpu/kmeans/kmeans_h2o4gpu.cu:1060-1097, :817-975).

tests/test_gpu_configs.py checks the handle-level fit of the same shapes against the CPU oracle
on all rows. This file ties the entry points to that: from pageable host arrays and the same
start they must return the handle-level centroids and labels bit for bit, predict on ALL rows
must return the fit's labels, and the transform entry point must return the handle-level
matrix, which is compared with the oracle's distances over the whole [k][rows] result.
"""
import ctypes

import numpy as np
import pytest

from h2o4gpu_amd import datasets
from parity import record

pytestmark = pytest.mark.gpu

THREADS = 16

# name, dtype: Lloyd iterations are the benchmark's own (datasets.SHAPES)
CONFIGS = [
    ("C1", np.float32),
    ("C2", np.float32),
    ("C3", np.float32),
    ("C4", np.float32),
    ("C4", np.float64),
    ("C5", np.float32),
]


def _void(a):
    return a.ctypes.data_as(ctypes.c_void_p)


def _predict_entry(hip, X, C):
    """make_ptr_*_kmeans(dopredict = 1, ...) called as a C client would: raw pointers in,
    the library's malloc()ed label buffer out."""
    n, d = X.shape
    k = C.shape[0]
    lib = hip.lib()
    fn = lib.make_ptr_float_kmeans if X.dtype == np.float32 else lib.make_ptr_double_kmeans
    pc, pl = ctypes.c_void_p(), ctypes.c_void_p()
    rc = fn(1, 0, 0, 0, 1, n, d, k, 0, 0, 0.0, _void(X), _void(C), ctypes.byref(pc), ctypes.byref(pl))
    assert rc == 0, rc
    assert not pc.value, "predict must not set pred_centroids"
    assert pl.value
    try:
        return np.ctypeslib.as_array(ctypes.cast(pl.value, ctypes.POINTER(ctypes.c_int32)), shape=(n,)).copy()
    finally:
        hip.libc_free(pl)


@pytest.mark.timeout(900)
@pytest.mark.parametrize("name,dtype", CONFIGS)
def test_entry_points_reproduce_the_handle_fit(hip, oracle, full_data, name, dtype):
    from h2o4gpu_amd.libs import ch2o4gpu_gpu as shim
    X, k, iters = full_data(name, dtype)
    n, d = X.shape
    seed = datasets.SHAPES[name][3]
    with hip.Handle(n, d, k, dtype) as h:
        h.set_data(X)
        if name == "C4":
            h.init_plusplus(seed)          # the benchmark's k-means++ start, computed once
            C0 = h.centroids()
        else:
            C0 = datasets.seeded_row_init(X, k, seed)
        h.set_centroids(C0)
        assert h.fit(iters, 0.0) == iters
        Ch, Lh, inertia_h = h.centroids(), h.labels(), h.inertia()
        variant = h.assign_variant()
        Dh = H = None
        if name == "C5":
            H = datasets.make_holdout("C5", 100_000)
            Dh = h.transform(H)
    # fit: dopredict = 0, init_from_data = 2 (start from the centroids argument), threshold 0
    rc, Ce, Le = shim.kmeans_fit_owned(0, seed, 0, 1, n, d, k, iters, 2, 0.0, X.reshape(-1), C0.reshape(-1), dtype)
    assert rc == 0
    Ce = Ce.reshape(k, d)
    assert Ce.dtype == np.dtype(dtype) and Le.dtype == np.int32 and Le.shape == (n,)
    assert np.array_equal(Ce, Ch), "%s: entry-point centroids differ from the handle fit" % name
    assert np.array_equal(Le, Lh), "%s: %d labels differ from the handle fit" % (name, int((Le != Lh).sum()))
    info = shim.last_fit_info()
    assert info is not None and info[1] == iters
    assert abs(info[0] - inertia_h) <= 1e-12 * inertia_h
    # predict: dopredict = 1 on ALL rows returns the fit's labels (they come from the final
    # relabel against the returned centroids)
    Lp = _predict_entry(hip, X, np.ascontiguousarray(Ce))
    assert np.array_equal(Lp, Le), "%s: predict differs from labels_ on %d rows" % (name, int((Lp != Le).sum()))
    entry = {"kind": "entry_points", "config": name, "dtype": np.dtype(dtype).name, "n": n, "d": d, "k": k,
             "variant": variant, "iterations": iters, "fit_bit_equal_to_handle": True,
             "predict_rows": n, "predict_equals_labels": True}
    if name == "C5":
        rc, De = shim.kmeans_transform_owned(0, 0, 1, H.shape[0], d, k, H.reshape(-1), Ce.reshape(-1), dtype)
        assert rc == 0
        De = De.reshape(k, H.shape[0])
        assert np.array_equal(De, Dh), "transform entry point differs from the handle transform"
        del Dh
        entry.update(_whole_transform_against_the_oracle(oracle, H, Ce, De))
    record(entry)
    print("entry points %s" % entry)


def _whole_transform_against_the_oracle(oracle, H, C, D):
    """Every element of the [k][rows] result against the oracle's distances (its float32
    restatement of |xx + cc - 2 x.c| with the features summed in ascending order). Two correct
    float32 evaluations of that form differ by rounding of a d-term sum whose terms are of the
    size of xx + cc: the bar is (4 sqrt(d) + 40) eps (xx + cc) per element."""
    k, d = C.shape
    m = H.shape[0]
    want = oracle.distances(H, C, threads=THREADS)        # [k][m], float32
    assert want.shape == D.shape == (k, m)
    eps = float(np.finfo(H.dtype).eps)
    xx = (H.astype(np.float64) ** 2).sum(1)
    cc = (C.astype(np.float64) ** 2).sum(1)
    mult = 4.0 * np.sqrt(d) + 40.0
    worst = 0.0
    for lo in range(0, k, 256):                          # 256 x 100,000 doubles at a time
        hi = min(k, lo + 256)
        err = np.abs(D[lo:hi].astype(np.float64) - want[lo:hi].astype(np.float64))
        err /= eps * (xx[None, :] + cc[lo:hi, None])
        worst = max(worst, float(err.max()))
    assert worst <= mult, "transform differs from the oracle by %.1f eps (xx + cc), bar %.1f" % (worst, mult)
    return {"transform_elements": int(k) * int(m), "transform_worst_err_in_eps_xx_cc": worst,
            "transform_bar_in_eps_xx_cc": mult}
