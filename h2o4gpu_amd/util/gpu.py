"""Device count helper (reference: src/interface_py/h2o4gpu/util/gpu.py:14-36,152-212)."""
import numpy as np


def get_gpu_info_c(verbose=0):
    """Returns (number of visible devices, total memory per device); 0 devices when the
    runtime sees none. A missing or unloadable library raises ImportError: there is no
    silent CPU path."""
    max_gpus = 16
    total_mems = np.zeros(max_gpus, dtype=np.uint64)
    try:
        from ..libs import ch2o4gpu_gpu as lib
        dummy_i = np.zeros(max_gpus, dtype=np.int32)
        dummy_u = np.zeros(max_gpus, dtype=np.uint32)
        dummy_l = np.zeros(max_gpus, dtype=np.uint64)
        status, n = lib.get_gpu_info_c(verbose, 1, 0, 0, 0, 0, 0, 0, 0, dummy_i, total_mems, dummy_l, None,
                                       dummy_i.copy(), dummy_i.copy(), dummy_u, dummy_u.copy(), dummy_l.copy(),
                                       dummy_u.copy(), dummy_u.copy(), dummy_l.copy())
        if status != 0:
            return 0, total_mems[:0]
        return n, total_mems[:n]
    except OSError as e:  # the library exists but the loader rejected it
        raise ImportError("cannot load the k-means engine: %s" % e)


def device_count(n_gpus=0):
    """Adjusted n_gpus and all available devices (reference util/gpu.py:14-36)."""
    available_device_count = get_gpu_info_c()[0]
    if n_gpus < 0:
        if available_device_count >= 0:
            n_gpus = available_device_count
        else:
            n_gpus = 1
    if n_gpus > available_device_count:
        n_gpus = available_device_count
    return n_gpus, available_device_count
