"""The C-ABI library loads and exports every symbol include/h2o4gpu_kmeans.h declares.
No compute calls here (no GPU in this container)."""
import ctypes
import os
import re

import numpy as np
import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "h2o4gpu_kmeans.h")


def declared_functions():
    text = open(HEADER).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    names = re.findall(r"^\s*(?:const\s+)?(?:int|char)\s*\*?\s*(\w+)\s*\(", text, flags=re.M)
    return sorted(set(names))


def test_header_parses_as_c():
    import subprocess
    subprocess.check_call(["gcc", "-std=c99", "-fsyntax-only", "-x", "c", HEADER])


def test_library_exports_every_declared_symbol(hip):
    lib = ctypes.CDLL(hip.LIB_PATH)
    names = declared_functions()
    assert len(names) >= 30
    for name in names:
        assert hasattr(lib, name), "symbol %s is declared in the header but not exported" % name
    assert set(names) == set(hip.PROTOTYPES), (
        "binding and header disagree: %s" % sorted(set(names) ^ set(hip.PROTOTYPES)))


def test_reference_entry_points_are_present(hip):
    lib = hip.lib()
    for name in ("make_ptr_float_kmeans", "make_ptr_double_kmeans", "kmeans_transform_float",
                 "kmeans_transform_double", "get_gpu_info_c"):
        assert getattr(lib, name) is not None


def test_bad_arguments_are_rejected_without_a_device(hip):
    lib = hip.lib()
    h = ctypes.c_void_p()
    assert lib.h2o4gpu_kmeans_create(ctypes.byref(h), 3, 10, 2, 2, 0, 0) == -2     # elem size
    assert lib.h2o4gpu_kmeans_create(ctypes.byref(h), 4, 0, 2, 2, 0, 0) == -2      # no rows
    assert lib.h2o4gpu_kmeans_create(ctypes.byref(h), 4, 10, 2, 0, 0, 0) == -2     # no centroids
    assert lib.h2o4gpu_kmeans_create(None, 4, 10, 2, 2, 0, 0) == -2
    assert lib.h2o4gpu_kmeans_assign(None) == -2
    slot_c, slot_l = ctypes.c_void_p(), ctypes.c_void_p()
    rc = lib.make_ptr_float_kmeans(0, 0, 1, 0, 1, 10, 2, 2, 5, 0, 0.0, None, None,
                                   ctypes.byref(slot_c), ctypes.byref(slot_l))
    assert rc == -2 and not slot_c.value and not slot_l.value


@pytest.mark.skipif(os.path.exists("/dev/kfd"), reason="a GPU is present")
def test_no_device_is_an_error_not_a_fallback(hip):
    assert hip.device_count() == 0
    with pytest.raises(hip.KMeansHipError):
        hip.Handle(100, 4, 3)
    from h2o4gpu_amd import KMeans
    with pytest.raises(RuntimeError):
        KMeans(n_clusters=2)
    X = np.zeros((4, 2), np.float32)
    from h2o4gpu_amd.libs import ch2o4gpu_gpu
    out_c, out_l = np.zeros(4, np.float32), np.zeros(4, np.int32)
    assert ch2o4gpu_gpu.make_ptr_float_kmeans(0, 0, 1, 0, 1, 4, 2, 2, 3, 0, 0.0, X.flatten(),
                                              np.empty([]), out_c, out_l) != 0


def test_random_start_rows_equal_the_standard_library_shuffle(hip, oracle):
    """The engine computes the first k entries of std::shuffle(iota(n),
    default_random_engine(seed)) without shuffling n entries; the oracle makes the two
    standard-library calls as the reference writes them (kmeans_h2o4gpu.cu:662-669).
    Both sides of libstdc++'s 46340-row switch, generator edge seeds, k from 1 to n."""
    for n in (1, 2, 3, 10, 257, 1000, 46339, 46340, 46341, 46342, 50000, 100003, 1_000_000):
        for k in (1, 2, 7, 64, 256, 1000, n):
            if k > n:
                continue
            for seed in (0, 1, 7, 1234, 2147483646, 2147483647):
                want = oracle.random_rows(seed, n, k)
                got = hip.random_start_rows(seed, n, k)
                assert np.array_equal(got, want), (n, k, seed)
    assert hip.lib().h2o4gpu_kmeans_random_start_rows(1, 5, 6, None) == -2


def test_host_all_finite_matches_numpy():
    """The estimator's input check as one parallel pass over the raw values: same verdict
    as np.isfinite(...).all() (reference solvers/utils.py:144-158), no device involved."""
    from h2o4gpu_amd.libs import kmeans_hip
    rng = np.random.default_rng(3)
    for dt in (np.float32, np.float64):
        a = rng.standard_normal(2_500_003).astype(dt)          # large enough for several threads
        assert kmeans_hip.host_all_finite(a) is True
        for pos in (0, 1, a.size // 3, a.size - 1):
            for bad in (np.inf, -np.inf, np.nan):
                b = a.copy()
                b[pos] = bad
                assert kmeans_hip.host_all_finite(b) is False
        info = np.finfo(dt)
        edge = np.array([info.max, -info.max, info.tiny, info.smallest_subnormal, 0.0, -0.0], dt)
        assert kmeans_hip.host_all_finite(edge) is True
        assert kmeans_hip.host_all_finite(np.zeros(0, dt)) is True
    with pytest.raises(TypeError):
        kmeans_hip.host_all_finite(np.zeros(4, np.int32))
    with pytest.raises(TypeError):
        kmeans_hip.host_all_finite(np.zeros((4, 4), np.float32)[:, ::2])
