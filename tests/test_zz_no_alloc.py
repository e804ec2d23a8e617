"""The entry point that allocates nothing (part 4 of the C header) against the existing
predict entry point, through the C ABI.

Device buffers come straight from the HIP runtime the engine itself is linked against
(its functions are looked up through the engine's library handle, so a second copy of the
runtime that another package may have brought into the process is never picked). Two calls in a row share the library's fixed scratch array, the second one
with a smaller input: stale contents of the first call must not show."""
import ctypes

import numpy as np
import pytest

pytestmark = pytest.mark.gpu

_hip = None


def hiprt():
    global _hip
    if _hip is None:
        from h2o4gpu_amd.libs import kmeans_hip
        rt = kmeans_hip.lib()   # dlsym on the engine's handle also searches its dependencies
        rt.hipMalloc.argtypes = [ctypes.POINTER(ctypes.c_void_p), ctypes.c_size_t]
        rt.hipFree.argtypes = [ctypes.c_void_p]
        rt.hipMemcpy.argtypes = [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_size_t, ctypes.c_int]
        rt.hipMemset.argtypes = [ctypes.c_void_p, ctypes.c_int, ctypes.c_size_t]
        rt.hipStreamCreateWithFlags.argtypes = [ctypes.POINTER(ctypes.c_void_p), ctypes.c_uint]
        rt.hipStreamSynchronize.argtypes = [ctypes.c_void_p]
        rt.hipStreamDestroy.argtypes = [ctypes.c_void_p]
        rt.hipMemGetInfo.argtypes = [ctypes.POINTER(ctypes.c_size_t), ctypes.POINTER(ctypes.c_size_t)]
        _hip = rt
    return _hip


def free_device_bytes():
    fr, tot = ctypes.c_size_t(0), ctypes.c_size_t(0)
    assert hiprt().hipMemGetInfo(ctypes.byref(fr), ctypes.byref(tot)) == 0
    return fr.value


class DeviceBuffer:
    def __init__(self, nbytes):
        self.ptr = ctypes.c_void_p()
        self.nbytes = nbytes
        assert hiprt().hipMalloc(ctypes.byref(self.ptr), max(nbytes, 16)) == 0

    def upload(self, a):
        a = np.ascontiguousarray(a)
        assert a.nbytes <= self.nbytes
        assert hiprt().hipMemcpy(self.ptr, a.ctypes.data_as(ctypes.c_void_p), a.nbytes, 1) == 0

    def download(self, shape, dtype):
        out = np.empty(shape, dtype)
        assert hiprt().hipMemcpy(out.ctypes.data_as(ctypes.c_void_p), self.ptr, out.nbytes, 2) == 0
        return out

    def free(self):
        hiprt().hipFree(self.ptr)


def problem(n, d, k, dtype, seed):
    rng = np.random.default_rng(seed)
    centers = rng.uniform(-8, 8, size=(k, d))
    X = np.ascontiguousarray((centers[rng.integers(0, k, size=n)] + rng.standard_normal((n, d))).astype(dtype))
    C = np.ascontiguousarray(X[rng.choice(n, size=k, replace=False)])
    return X, C


# (first call, second smaller call): every kernel family of the assignment, models that
# need centroid padding, rows that are not whole 16-byte vectors
CASES = [
    ((200_000, 32, 256), (50_001, 32, 100)),    # row-stationary, then fewer rows and centroids
    ((60_000, 16, 8), (777, 5, 3)),             # small-model kernels
    ((20_000, 256, 300), (3_000, 100, 70)),     # tiled
    ((90_000, 24, 1500), (10_000, 24, 33)),     # row-stationary sweep in chunks, then one chunk
]


@pytest.mark.parametrize("dtype", [np.float32, np.float64])
@pytest.mark.parametrize("first,second", CASES)
def test_noalloc_predict_equals_predict_host(hip, oracle, first, second, dtype):
    stream = ctypes.c_void_p()
    assert hiprt().hipStreamCreateWithFlags(ctypes.byref(stream), 1) == 0   # non-blocking
    try:
        for call, (n, d, k) in enumerate((first, second)):
            X, C = problem(n, d, k, dtype, seed=n + k)
            with hip.Handle(k, d, k, dtype) as h:
                h.set_centroids(C)
                want = h.predict(X)                      # the existing entry point
            dX, dC, dL = DeviceBuffer(X.nbytes), DeviceBuffer(C.nbytes), DeviceBuffer(4 * n)
            try:
                dX.upload(X)
                dC.upload(C)
                assert hiprt().hipMemset(dL.ptr, 0xFF, 4 * n) == 0
                hip.predict_device_noalloc(dtype, n, d, k, dX.ptr.value, dC.ptr.value, dL.ptr.value,
                                           stream.value)
                assert hiprt().hipStreamSynchronize(stream) == 0
                got = dL.download(n, np.int32)
                # the same call again (the shape's one-time set-up is behind it): the device's
                # free memory is the same before, while the work is queued, and after
                before = free_device_bytes()
                hip.predict_device_noalloc(dtype, n, d, k, dX.ptr.value, dC.ptr.value, dL.ptr.value,
                                           stream.value)
                queued = free_device_bytes()
                assert hiprt().hipStreamSynchronize(stream) == 0
                assert before == queued == free_device_bytes(), "the call changed the device's free memory"
                assert np.array_equal(dL.download(n, np.int32), got)
            finally:
                dX.free(); dC.free(); dL.free()
            where = "call %d: n=%d d=%d k=%d %s" % (call, n, d, k, np.dtype(dtype).name)
            # same kernels on the same values: identical labels, not just near-tie equal
            assert np.array_equal(got, want), where
            # and both agree with the CPU oracle up to near-ties
            from parity import label_report
            label_report(oracle, X, C, got, oracle.assign(X, C, threads=4))
    finally:
        hiprt().hipStreamDestroy(stream)


def test_noalloc_rejects_inputs_beyond_its_scratch(hip):
    """Nothing is queued and a distinct error comes back when the fixed array is too small;
    bad arguments are told apart from that."""
    dX, dC, dL = DeviceBuffer(1024), DeviceBuffer(1024), DeviceBuffer(1024)
    try:
        rows = hip.NOALLOC_SCRATCH_BYTES // 8 + 1     # 2 * rows * 4 bytes alone exceed it
        with pytest.raises(hip.KMeansHipError) as e:
            hip.predict_device_noalloc(np.float32, rows, 4, 2, dX.ptr.value, dC.ptr.value, dL.ptr.value)
        assert e.value.code == -5
        with pytest.raises(hip.KMeansHipError) as e:   # model too large: 4096 x 2048 doubles
            hip.predict_device_noalloc(np.float64, 10, 2048, 4096, dX.ptr.value, dC.ptr.value, dL.ptr.value)
        assert e.value.code == -5
        with pytest.raises(hip.KMeansHipError) as e:
            hip.predict_device_noalloc(np.float32, 10, 4, 2, 0, dC.ptr.value, dL.ptr.value)
        assert e.value.code == -2
    finally:
        dX.free(); dC.free(); dL.free()
