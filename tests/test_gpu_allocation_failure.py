"""The reference's one documented failure code on the device: -1 when the working set cannot be
allocated (reference: src/gpu/kmeans/kmeans_impl.h:67-105 returns -1 after log_error,
kmeans_h2o4gpu.cu:758-761 passes it on). Nothing here goes beyond hipMalloc refusing a size:
no kernel runs on the oversized shape."""
import ctypes

import numpy as np
import pytest

pytestmark = pytest.mark.gpu

COLS = 4096


def _free_bytes(shim):
    free = np.zeros(16, np.uint64)
    status, n = shim.get_gpu_info_c(0, 0, 0, 0, 1, 0, 0, 0, 0, None, None, free, None, None, None,
                                    None, None, None, None, None, None)
    assert status == 0 and n >= 1 and free[0] > 0
    return int(free[0])


def _small_fit_works(hip, oracle):
    rng = np.random.default_rng(3)
    X = rng.standard_normal((5000, 12)).astype(np.float32)
    C0 = np.ascontiguousarray(X[:7] + np.float32(0.5))
    with hip.Handle(5000, 12, 7, np.float32) as h:
        h.set_data(X)
        h.set_centroids(C0)
        assert h.fit(4, 0.0) == 4
        C, L = h.centroids(), h.labels()
    wC, wL, _, _ = oracle.lloyd(X, C0, 4, 0.0)
    assert np.array_equal(L, wL) and np.allclose(C, wC, rtol=1e-5, atol=1e-6)


def test_rows_beyond_free_memory_return_minus_one(hip, oracle, capfd):
    from h2o4gpu_amd.libs import ch2o4gpu_gpu as shim
    free = _free_bytes(shim)
    rows = int(free * 1.25) // (COLS * 4)
    assert rows < 2 ** 31
    small = np.zeros((8, COLS), np.float32)           # never read: the allocation fails first

    # handle level: the per-row working set of create() (labels, norms, minimum distances,
    # 12 bytes per row) fits, the rows themselves do not
    h = ctypes.c_void_p()
    lib = hip.lib()
    assert lib.h2o4gpu_kmeans_create(ctypes.byref(h), 4, rows, COLS, 8, 0, 0) == 0
    try:
        capfd.readouterr()
        rc = lib.h2o4gpu_kmeans_set_data_host(h, small.ctypes.data_as(ctypes.c_void_p))
        assert rc == -1
        assert capfd.readouterr().err == "", "verbose = 0 must stay silent"
    finally:
        assert lib.h2o4gpu_kmeans_destroy(h) == 0
    _small_fit_works(hip, oracle)

    # the reference's entry point: same shape, pageable host pointers, verbose at the error
    # level (200) prints the reference's message; the out-parameters stay untouched
    C0 = np.zeros((8, COLS), np.float32)
    pc, pl = ctypes.c_void_p(), ctypes.c_void_p()
    for verbose, want_message in ((0, False), (200, True)):
        rc = lib.make_ptr_float_kmeans(0, verbose, 1, 0, 1, rows, COLS, 8, 3, 2, 0.0,
                                       small.ctypes.data_as(ctypes.c_void_p),
                                       C0.ctypes.data_as(ctypes.c_void_p),
                                       ctypes.byref(pc), ctypes.byref(pl))
        err = capfd.readouterr().err
        assert rc == -1 and not pc.value and not pl.value
        assert ("Unable to allocate memory" in err and "KMeans algorithm failed" in err) == want_message, err
        if not want_message:
            assert err == ""
    # a working set that cannot be allocated at create() (k * cols beyond free memory)
    h = ctypes.c_void_p()
    kbig = int(free * 1.25) // (COLS * 8 * 2) + 256
    assert lib.h2o4gpu_kmeans_create(ctypes.byref(h), 8, kbig, COLS, kbig, 0, 0) == -1 and not h.value
    # the device is as usable as before
    assert _free_bytes(shim) >= 0.98 * free
    _small_fit_works(hip, oracle)
