"""The tiled matrix-core kernel in its two forms, operands fetched by direct-to-LDS loads
(rows and centroids whole stages, 16-byte aligned) and staged through registers (every other
shape; option tiled_direct = 0): both against the CPU oracle by the usual bars, and against
each other, on shapes that exercise what differs between them (one stage only, the ring
wrapping inside a centroid block and across blocks, partial last row tiles and centroid blocks,
models on both sides of the 128- / 256-centroid block rule, both precisions, transform)."""
import numpy as np
import pytest

from parity import label_report

pytestmark = pytest.mark.gpu


def data(n, d, k, dtype, seed):
    rng = np.random.default_rng(seed)
    centres = rng.uniform(-6, 6, size=(k, d))
    X = centres[rng.integers(0, k, size=n)] + rng.standard_normal((n, d))
    C = centres + 0.3 * rng.standard_normal((k, d))
    return np.ascontiguousarray(X.astype(dtype)), np.ascontiguousarray(C.astype(dtype))


# n, d, k: d a multiple of 32 (float32 stages of 16 or 32 features) or 16 (float64)
SHAPES = [
    (5000, 32, 130),      # one stage of 32 features, two centroid blocks, the second mostly padding
    (4099, 64, 256),      # 256-centroid block, ragged last row tile
    (3000, 96, 500),      # stages do not divide the ring evenly across blocks
    (2048, 256, 1024),    # the benchmark's row length
    (1500, 160, 129),     # 128-centroid block chosen (padding rule), last block one centroid
    (700, 16, 200),       # float64 only: one 16-feature stage (float32 goes through registers)
    (1027, 784, 300),     # 49 stages of 16 in the wide block
]


@pytest.mark.parametrize("dtype", [np.float32, np.float64])
@pytest.mark.parametrize("n,d,k", SHAPES)
def test_both_forms_against_the_oracle_and_each_other(hip, oracle, n, d, k, dtype):
    X, C = data(n, d, k, dtype, seed=n + d + k)
    got = {}
    m_rows = min(n, 777)
    with hip.Handle(n, d, k, dtype) as h:
        h.set_data(X)
        h.set_option("assign", "mfma_tiled")
        for direct in (1, 0):
            h.set_option("tiled_direct", direct)
            h.set_centroids(C)
            h.assign()
            got[direct] = (h.labels(), h.min_distances(), h.transform(X[:m_rows]))
    want, wmin = oracle.assign(X, C, threads=4, return_mindist=True)
    eps = float(np.finfo(dtype).eps)
    xx = (X.astype(np.float64) ** 2).sum(1)
    cc = (C.astype(np.float64) ** 2).sum(1)
    bar = (4 * np.sqrt(d) + 40) * eps
    wD = oracle.distances(np.ascontiguousarray(X[:m_rows]), C, threads=4)
    for direct in (1, 0):
        L, m, D = got[direct]
        label_report(oracle, X, C, L, want)
        same = L == want
        assert np.all(np.abs(m[same].astype(np.float64) - wmin[same]) <= bar * (xx[same] + cc[want[same]]))
        assert D.shape == (k, m_rows)
        err = np.abs(D.astype(np.float64) - wD.astype(np.float64)) / (eps * (xx[None, :m_rows] + cc[:, None]))
        assert err.max() <= 4 * np.sqrt(d) + 40, (direct, err.max())
    # The two forms add the same products in the same order and close a block of centroids with the
    # same expression: the same bits, whichever block width either of them chose.
    assert np.array_equal(got[1][0], got[0][0])
    assert np.array_equal(got[1][1], got[0][1])
    assert np.array_equal(got[1][2], got[0][2])


def test_unaligned_rows_fall_back_to_registers(hip, oracle):
    """Rows that are whole stages but start at an address that is only element-aligned (a device
    pointer 4 bytes into an allocation) cannot use the direct loads; the result must not change
    by a bit."""
    import ctypes
    rt = hip.lib()   # the HIP runtime the engine is linked against (dlsym searches its dependencies)
    rt.hipMalloc.argtypes = [ctypes.POINTER(ctypes.c_void_p), ctypes.c_size_t]
    rt.hipFree.argtypes = [ctypes.c_void_p]
    rt.hipMemcpy.argtypes = [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_size_t, ctypes.c_int]
    n, d, k = 3000, 64, 200
    X, C = data(n, d, k, np.float32, seed=5)
    buf = ctypes.c_void_p()
    assert rt.hipMalloc(ctypes.byref(buf), X.nbytes + 16) == 0
    try:
        rows = ctypes.c_void_p(buf.value + 4)
        assert rt.hipMemcpy(rows, X.ctypes.data_as(ctypes.c_void_p), X.nbytes, 1) == 0
        with hip.Handle(n, d, k, np.float32) as h:
            h.set_option("assign", "mfma_tiled")
            h.set_data_device(rows.value)
            h.set_centroids(C)
            h.assign()
            L, m = h.labels(), h.min_distances()
    finally:
        rt.hipFree(buf)
    label_report(oracle, X, C, L, oracle.assign(X, C, threads=4))
    with hip.Handle(n, d, k, np.float32) as h:
        h.set_option("assign", "mfma_tiled")
        h.set_data(X)
        h.set_centroids(C)
        h.assign()
        assert np.array_equal(h.labels(), L) and np.array_equal(h.min_distances(), m)


@pytest.mark.parametrize("n,d,k,direct", [
    (20000, 256, 1024, 1),    # direct loads
    (20000, 256, 1024, 0),    # the same shape staged through registers
    (20000, 298, 1000, 1),    # rows that are not whole stages: through registers whatever the option says
    (20000, 142, 40, 1),      # the 64-centroid block
])
def test_float32_distances_carry_the_rounding_noise_of_a_scalar_loop(hip, oracle, n, d, k, direct):
    """Both forms of the tiled kernel sum the dot product from zero and add -(xx + cc)/2 when a
    block of centroids is complete, which is the order of the reference's GEMM with beta = 1
    (kmeans_labels.cu:158-165) and of the oracle's scalar loop. Accumulators that start at
    -(xx + cc)/2 round every partial sum at the size of xx + cc and carry 1.5 times the noise
    (rms 3.0 against 2.0 eps (xx + cc) at 256 features), which flips near-tie rows that a scalar
    loop decides the other way. Measured here: the error of every returned distance against
    float64, in units of eps (xx + cc), for the engine's transform and for the oracle's."""
    rng = np.random.default_rng(d + k)
    X = (rng.standard_normal((n, d)) * 3 + rng.integers(0, 20, (n, 1))).astype(np.float32)
    C = np.ascontiguousarray(X[rng.choice(n, size=k, replace=False)] + rng.standard_normal((k, d)).astype(np.float32))
    m = 4000
    with hip.Handle(n, d, k, np.float32) as h:
        h.set_data(X)
        h.set_option("assign", "mfma_tiled")
        h.set_option("tiled_direct", direct)
        h.set_centroids(C)
        D = h.transform(X[:m]).T.astype(np.float64)           # [m][k]
        h.set_option("exact_argmin", 1)
        h.assign()
        L, md = h.labels()[:m], h.min_distances()[:m].astype(np.float64)
    wD = oracle.distances(np.ascontiguousarray(X[:m]), C, threads=4).T.astype(np.float64)
    X64, C64 = X[:m].astype(np.float64), C.astype(np.float64)
    xx, cc = (X64 * X64).sum(1)[:, None], (C64 * C64).sum(1)[None, :]
    truth = np.abs(xx + cc - 2.0 * X64 @ C64.T)
    unit = float(np.finfo(np.float32).eps) * (xx + cc)
    e_engine, e_oracle = (D - truth) / unit, (wD - truth) / unit
    rms_e, rms_o = np.sqrt((e_engine ** 2).mean()), np.sqrt((e_oracle ** 2).mean())
    print("d=%d k=%d direct=%d: engine rms %.2f max %.1f, oracle rms %.2f max %.1f" % (
        d, k, direct, rms_e, np.abs(e_engine).max(), rms_o, np.abs(e_oracle).max()))
    assert abs(e_engine.mean()) <= 0.2
    assert rms_e <= 1.25 * rms_o + 0.1, (rms_e, rms_o)
    # the assignment pass returns the same numbers as the transform for the rows' own minima
    e_min = (md - truth[np.arange(m), L]) / unit[np.arange(m), L]
    assert np.sqrt((e_min ** 2).mean()) <= 1.25 * rms_o + 0.1
