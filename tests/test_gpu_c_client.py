"""The shared library called from compiled C (tests/c_abi_client.c), no Python between
the caller and the entry points."""
import os
import subprocess

import numpy as np
import pytest

HERE = os.path.dirname(os.path.abspath(__file__))
CLIENT = os.path.join(HERE, "c_abi_client")
ROWS, COLS, K, ITERS = 6000, 12, 7, 5


def client_data():
    i = np.arange(ROWS)[:, None]
    j = np.arange(COLS)[None, :]
    X = (np.float32(3.0) * (i % K).astype(np.float32) +
         np.float32(0.01) * ((i * 7 + j * 13) % 100).astype(np.float32)).astype(np.float32)
    C0 = (np.float32(3.0) * np.arange(K, dtype=np.float32)[:, None] + np.float32(0.25)) * np.ones((1, COLS), np.float32)
    return np.ascontiguousarray(X), np.ascontiguousarray(C0.astype(np.float32))


CXX_CLIENT = os.path.join(HERE, "cxx_abi_client")


def test_cxx_client_builds_from_the_template_header():
    """include/h2o4gpu_kmeans.hpp mirrors the reference's C++ templates
    (src/include/solver/kmeans.h:16-54); a caller written against them compiles with g++
    and resolves the library (no GPU needed to check that)."""
    if not os.path.exists(CXX_CLIENT):
        subprocess.check_call(["g++", "-O1", "-Wall", "-Wextra", "-std=c++17", "-o", CXX_CLIENT,
                               CXX_CLIENT + ".cpp", "-L" + os.path.join(HERE, "..", "h2o4gpu_amd"),
                               "-lh2o4gpu_kmeans_hip", "-Wl,-rpath,$ORIGIN/../h2o4gpu_amd"])
    out = subprocess.run(["ldd", CXX_CLIENT], capture_output=True, text=True).stdout
    line = [l for l in out.splitlines() if "libh2o4gpu_kmeans_hip.so" in l]
    assert line and "not found" not in line[0], out


@pytest.mark.gpu
def test_cxx_client_runs():
    proc = subprocess.run([CXX_CLIENT], capture_output=True, text=True, timeout=300)
    assert proc.returncode == 0, proc.stdout + proc.stderr
    assert proc.stdout.split() == ["float", "ok", "double", "ok"]


def test_client_is_built_against_the_public_header():
    """build() compiles the client with gcc from the header alone; it must resolve the
    library next to the package (no GPU needed to check the link)."""
    if not os.path.exists(CLIENT):  # a tree where build() has not run yet: gcc only, no GPU
        subprocess.check_call(["gcc", "-O1", "-Wall", "-Wextra", "-std=c99", "-o", CLIENT, CLIENT + ".c",
                               "-L" + os.path.join(HERE, "..", "h2o4gpu_amd"), "-lh2o4gpu_kmeans_hip",
                               "-Wl,-rpath,$ORIGIN/../h2o4gpu_amd"])
    out = subprocess.run(["ldd", CLIENT], capture_output=True, text=True).stdout
    line = [l for l in out.splitlines() if "libh2o4gpu_kmeans_hip.so" in l]
    assert line and "not found" not in line[0], out


@pytest.mark.gpu
def test_c_client_results_match_the_oracle(oracle):
    proc = subprocess.run([CLIENT], capture_output=True, text=True, timeout=300)
    assert proc.returncode == 0, proc.stdout + proc.stderr
    rows = [l.split() for l in proc.stdout.splitlines()]
    kv = {r[0]: r[1:] for r in rows if r[0] not in ("centroid", "dist")}
    assert kv["fit_rc"] == ["0"] and kv["predict_rc"] == ["0", "same_as_fit", "1"]
    assert kv["transform_rc"] == ["0"]
    X, C0 = client_data()
    wC, wL, _, _ = oracle.lloyd(X, C0, ITERS, 0.0)
    C = np.array([[float(v) for v in r[2:]] for r in rows if r[0] == "centroid"], np.float32)
    assert C.shape == (K, COLS)
    assert np.allclose(C, wC, rtol=1e-4, atol=1e-4)
    want_sum = int((wL.astype(np.int64) * (np.arange(ROWS) % 97 + 1)).sum())
    assert int(kv["label_checksum"][0]) == want_sum
    assert kv["info_rc"][0] == "0" and int(kv["info_rc"][2]) == ITERS
    inertia = float(kv["info_rc"][4])
    want_inertia = ((X.astype(np.float64) - wC.astype(np.float64)[wL]) ** 2).sum()
    assert abs(inertia - want_inertia) <= 1e-4 * want_inertia
    D = np.array([[float(v) for v in r[2:]] for r in rows if r[0] == "dist"], np.float64)
    want = ((X[:16, None, :].astype(np.float64) - C[None].astype(np.float64)) ** 2).sum(-1).T
    assert D.shape == (K, 16) and np.allclose(D, want, rtol=1e-3, atol=1e-3)
