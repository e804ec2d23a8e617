"""Python module with the call surface of h2o4gpu's SWIG module `ch2o4gpu_gpu`
(reference: src/swig/ch2o4gpu_gpu.i, src/swig/solver/kmeans.i, src/swig/util/gpu.i),
restricted to what the k-means estimator uses, bound to the gfx950 engine with ctypes.

Calling convention reproduced from the reference's numpy typemaps
(src/swig/numpy.i:3136-3204):
  * `srcdata`, `centroids` (T* IN_ARRAY1): any numpy array is converted to a contiguous
    array of T; anything that is not an array becomes NULL.
  * `pred_centroids`, `pred_labels`, `preds` (T** INPLACE_ARRAY1): must be a contiguous
    numpy array of exactly T. SWIG passes the address of the array's data pointer, so the
    library's malloc()ed result buffer replaces the array storage. Here the result is
    copied into the caller's array and the library buffer is freed: same visible effect
    (the array the caller preallocated holds the result on return), no leaked storage.
"""
import ctypes

import numpy as np

from . import kmeans_hip as _k


def _in_array(obj, dtype):
    """IN_ARRAY1: (pointer or None, keepalive)."""
    if isinstance(obj, np.ndarray):
        arr = np.ascontiguousarray(obj, dtype=dtype)
        return arr.ctypes.data_as(ctypes.c_void_p), arr
    return None, None


def _inplace_array(obj, dtype, name):
    if not isinstance(obj, np.ndarray) or obj.dtype != np.dtype(dtype):
        raise TypeError("%s must be a numpy array of %s" % (name, np.dtype(dtype).name))
    if not obj.flags.c_contiguous:
        raise TypeError("%s must be contiguous" % name)
    return obj


def _take(slot, dest, count):
    """Copy `count` elements from the library buffer in `slot` into dest, free the buffer."""
    if not slot.value:
        return
    try:
        flat = dest.reshape(-1) if dest.ndim else dest.reshape(1)
        ncopy = min(int(count), flat.size)
        if ncopy > 0:
            ctypes.memmove(flat.ctypes.data, slot.value, ncopy * flat.itemsize)
    finally:
        _k.libc_free(slot)


def _adopt(slot, count, dtype):
    """A numpy array over the library's malloc()ed buffer (no copy); the buffer is freed
    when the last view of it goes away. This is what SWIG's INPLACE_ARRAY1(T**) typemap
    does by re-pointing the caller's array, minus the stranded original storage."""
    import weakref
    if not slot.value or count <= 0:
        _k.libc_free(slot)
        return np.empty(0, dtype)
    ctype = {np.dtype(np.float32): ctypes.c_float, np.dtype(np.float64): ctypes.c_double,
             np.dtype(np.int32): ctypes.c_int32}[np.dtype(dtype)]
    buf = (ctype * int(count)).from_address(slot.value)
    weakref.finalize(buf, _k.libc_free, ctypes.c_void_p(slot.value))
    return np.frombuffer(buf, dtype=dtype)


def kmeans_transform_owned(verbose, gpu_id, n_gpu, m, n, k, srcdata, centroids, dtype):
    """kmeans_transform_float/double without the preallocated output array: returns
    (status, preds) where preds ([k*m], centroid-major) owns the library's buffer. Not part
    of the reference's module; the estimator uses it to skip zero-filling and copying an
    m x k array."""
    dtype = np.dtype(dtype)
    fn_name = "kmeans_transform_float" if dtype == np.float32 else "kmeans_transform_double"
    lib = _k.lib()
    src_p, _src_keep = _in_array(srcdata, dtype)
    cen_p, _cen_keep = _in_array(centroids, dtype)
    slot = ctypes.c_void_p()
    rc = getattr(lib, fn_name)(int(verbose), int(gpu_id), int(n_gpu), int(m), int(n), int(k), src_p, cen_p,
                               ctypes.byref(slot))
    return rc, _adopt(slot, int(m) * int(k) if rc == 0 else 0, dtype)


def kmeans_fit_owned(verbose, seed, gpu_id, n_gpu, mTrain, n, k, max_iterations, init_from_data,
                     threshold, srcdata, centroids, dtype):
    """make_ptr_float/double_kmeans(dopredict=0, ...) without preallocated outputs: returns
    (status, centroids [min(k, mTrain) * n], labels [mTrain]), both owning the library's
    buffers. Not part of the reference's module; the estimator uses it to skip zero-filling
    and copying the result arrays."""
    dtype = np.dtype(dtype)
    fn_name = "make_ptr_float_kmeans" if dtype == np.float32 else "make_ptr_double_kmeans"
    lib = _k.lib()
    src_p, _src_keep = _in_array(srcdata, dtype)
    cen_p, _cen_keep = _in_array(centroids, dtype)
    pc_slot, pl_slot = ctypes.c_void_p(), ctypes.c_void_p()
    rc = getattr(lib, fn_name)(0, int(verbose), int(seed), int(gpu_id), int(n_gpu), int(mTrain), int(n),
                               int(k), int(max_iterations), int(init_from_data), float(threshold), src_p,
                               cen_p, ctypes.byref(pc_slot), ctypes.byref(pl_slot))
    ok = rc == 0
    k_eff = min(int(k), int(mTrain))
    return rc, _adopt(pc_slot, k_eff * int(n) if ok else 0, dtype), \
        _adopt(pl_slot, int(mTrain) if ok else 0, np.int32)


def _make_ptr(fn_name, dtype, dopredict, verbose, seed, gpu_id, n_gpu, mTrain, n, k, max_iterations,
              init_from_data, threshold, srcdata, centroids, pred_centroids, pred_labels):
    lib = _k.lib()
    src_p, _src_keep = _in_array(srcdata, dtype)
    cen_p, _cen_keep = _in_array(centroids, dtype)
    pred_labels = _inplace_array(pred_labels, np.int32, "pred_labels")
    pc_slot = ctypes.c_void_p()
    pl_slot = ctypes.c_void_p()
    if dopredict == 0:
        pred_centroids = _inplace_array(pred_centroids, dtype, "pred_centroids")
    rc = getattr(lib, fn_name)(int(dopredict), int(verbose), int(seed), int(gpu_id), int(n_gpu),
                               int(mTrain), int(n), int(k), int(max_iterations), int(init_from_data),
                               float(threshold), src_p, cen_p, ctypes.byref(pc_slot),
                               ctypes.byref(pl_slot))
    k_eff = min(int(k), int(mTrain))
    if dopredict == 0:
        _take(pc_slot, pred_centroids, k_eff * int(n))
    _take(pl_slot, pred_labels, int(mTrain))
    return rc


def make_ptr_float_kmeans(dopredict, verbose, seed, gpu_id, n_gpu, mTrain, n, k, max_iterations,
                          init_from_data, threshold, srcdata, centroids, pred_centroids, pred_labels):
    return _make_ptr("make_ptr_float_kmeans", np.float32, dopredict, verbose, seed, gpu_id, n_gpu, mTrain,
                     n, k, max_iterations, init_from_data, threshold, srcdata, centroids, pred_centroids,
                     pred_labels)


def make_ptr_double_kmeans(dopredict, verbose, seed, gpu_id, n_gpu, mTrain, n, k, max_iterations,
                           init_from_data, threshold, srcdata, centroids, pred_centroids, pred_labels):
    return _make_ptr("make_ptr_double_kmeans", np.float64, dopredict, verbose, seed, gpu_id, n_gpu, mTrain,
                     n, k, max_iterations, init_from_data, threshold, srcdata, centroids, pred_centroids,
                     pred_labels)


def _transform(fn_name, dtype, verbose, gpu_id, n_gpu, m, n, k, srcdata, centroids, preds):
    lib = _k.lib()
    src_p, _src_keep = _in_array(srcdata, dtype)
    cen_p, _cen_keep = _in_array(centroids, dtype)
    preds = _inplace_array(preds, dtype, "preds")
    slot = ctypes.c_void_p()
    rc = getattr(lib, fn_name)(int(verbose), int(gpu_id), int(n_gpu), int(m), int(n), int(k), src_p, cen_p,
                               ctypes.byref(slot))
    _take(slot, preds, int(m) * int(k))
    return rc


def kmeans_transform_float(verbose, gpu_id, n_gpu, m, n, k, srcdata, centroids, preds):
    return _transform("kmeans_transform_float", np.float32, verbose, gpu_id, n_gpu, m, n, k, srcdata,
                      centroids, preds)


def kmeans_transform_double(verbose, gpu_id, n_gpu, m, n, k, srcdata, centroids, preds):
    return _transform("kmeans_transform_double", np.float64, verbose, gpu_id, n_gpu, m, n, k, srcdata,
                      centroids, preds)


def get_gpu_info_c(verbose, return_memory, return_name, return_usage, return_free_memory,
                   return_capability, return_memory_by_pid, return_usage_by_pid, return_all,
                   gpu_percent_usage, gpu_total_memory, gpu_free_memory, gpu_name, majors, minors,
                   num_pids, pids, usedGpuMemorys, num_pids_usage, pids_usage, usedGpuUsage):
    """Returns (status, n_gpus) and fills the in-place arrays, as the SWIG wrapper does
    (int *OUTPUT n_gpus; src/swig/util/gpu.i:55-93). gpu_name is a list of strings that
    is updated in place."""
    lib = _k.lib()
    n = ctypes.c_uint(0)
    nslots = len(gpu_name) if gpu_name is not None else 0
    bufs = [ctypes.create_string_buffer(100) for _ in range(nslots)]
    names = (ctypes.c_char_p * max(nslots, 1))(*[ctypes.cast(b, ctypes.c_char_p) for b in bufs])

    def vp(a):
        return a.ctypes.data_as(ctypes.c_void_p) if isinstance(a, np.ndarray) else None

    status = lib.get_gpu_info_c(int(verbose), int(return_memory), int(return_name), int(return_usage),
                                int(return_free_memory), int(return_capability),
                                int(return_memory_by_pid), int(return_usage_by_pid), int(return_all),
                                ctypes.byref(n), vp(gpu_percent_usage), vp(gpu_total_memory),
                                vp(gpu_free_memory), names if nslots else None, vp(majors), vp(minors),
                                vp(num_pids), vp(pids), vp(usedGpuMemorys), vp(num_pids_usage),
                                vp(pids_usage), vp(usedGpuUsage))
    for i in range(min(nslots, n.value)):
        gpu_name[i] = bufs[i].value.decode(errors="replace")
    return status, int(n.value)


def get_compute_capability(d_idx):
    """Returns (status, major, minor, ratioperf) like the SWIG int *OUTPUT mapping."""
    major, minor, ratio = ctypes.c_int(0), ctypes.c_int(0), ctypes.c_int(0)
    status = _k.lib().get_compute_capability(int(d_idx), ctypes.byref(major), ctypes.byref(minor),
                                             ctypes.byref(ratio))
    return status, major.value, minor.value, ratio.value


def cudaresetdevice(wDev, nDev):
    return _k.lib().cudaresetdevice(int(wDev), int(nDev))


def cudaresetdevice_bare():
    return _k.lib().cudaresetdevice_bare()


def last_fit_info():
    """(inertia, iterations) of this thread's last successful make_ptr_*_kmeans fit, or
    None. Not part of the reference's module: its entry points cannot return either."""
    return _k.last_fit_info()
