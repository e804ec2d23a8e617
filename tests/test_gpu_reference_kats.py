"""The reference's own known-answer cases (tests/cpp/gpu/kmeans/*.cu, transcribed in
tests/golden/reference_gtest_kats.json) run through the engine on the GPU, on every
kernel variant that can take the shape, in both precisions."""
import json
import os

import numpy as np
import pytest

pytestmark = pytest.mark.gpu
HERE = os.path.dirname(os.path.abspath(__file__))
KATS = json.load(open(os.path.join(HERE, "golden", "reference_gtest_kats.json")))
VARIANTS = ["valu", "mfma_rowstat", "mfma_tiled"]


def labels_counts(hip, X, C, variant, dtype):
    X = np.ascontiguousarray(X, dtype)
    C = np.ascontiguousarray(C, dtype)
    with hip.Handle(X.shape[0], X.shape[1], C.shape[0], dtype) as h:
        h.set_data(X)
        h.set_centroids(C)
        h.set_option("assign", variant)
        h.assign()
        labels = h.labels()
    return labels, np.bincount(labels, minlength=C.shape[0])


@pytest.mark.parametrize("dtype", [np.float32, np.float64])
@pytest.mark.parametrize("variant", VARIANTS)
def test_counts_per_centroids(hip, variant, dtype):
    kat = KATS["counts_per_centroids"]
    _, counts = labels_counts(hip, kat["data"], kat["centroids"], variant, dtype)
    assert counts.tolist() == kat["expected_counts"]


@pytest.mark.parametrize("dtype", [np.float32, np.float64])
@pytest.mark.parametrize("variant", VARIANTS)
def test_centroid_per_data_point(hip, variant, dtype):
    """Every point coincides with one centroid: the rounded self-distance |xx + cc - 2 x.c|
    must win (the reference keeps the fabs for this case, kmeans_labels.cu:183-244)."""
    kat = KATS["centroid_per_data_point"]
    labels, counts = labels_counts(hip, kat["data"], kat["centroids"], variant, dtype)
    assert counts.tolist() == kat["expected_counts"]
    assert labels.tolist() == list(range(len(kat["data"])))


def one_update(hip, X, labels, C_old, dtype, buckets=1):
    X = np.ascontiguousarray(X, dtype)
    C_old = np.ascontiguousarray(C_old, dtype)
    with hip.Handle(X.shape[0], X.shape[1], C_old.shape[0], dtype) as h:
        h.set_data(X)
        h.set_centroids(C_old)
        h.set_labels(np.asarray(labels, np.int32))
        h.set_option("buckets", buckets)
        h.update()
        return h.centroids(), h.counts()


@pytest.mark.parametrize("dtype", [np.float32, np.float64])
def test_calculate_centroids_and_scaling(hip, dtype):
    """calculate_centroids gives the unscaled sums; the engine returns sum * (1/count)."""
    kat = KATS["calculate_centroids"]
    C, counts = one_update(hip, kat["data"], kat["labels"], np.zeros((kat["k"], 2)), dtype)
    sums = np.asarray(kat["expected_unscaled_sums"], np.float64)
    assert counts.tolist() == [2, 2]
    assert np.array_equal(C, (sums * (1.0 / counts[:, None])).astype(dtype))
    kat = KATS["centroids_scaling"]
    counts = kat["counts"]
    sums = np.asarray(kat["sums"], dtype)
    # rows that reproduce the given sums and counts: sum/count repeated count times
    X = np.concatenate([np.repeat((sums[c] / counts[c])[None], counts[c], axis=0) for c in range(2)])
    labels = np.repeat(np.arange(2), counts)
    C, got_counts = one_update(hip, X, labels, np.zeros((2, 2)), dtype)
    assert got_counts.tolist() == counts
    assert np.allclose(C, np.asarray(kat["expected"]), rtol=1e-6)


@pytest.mark.parametrize("dtype", [np.float32, np.float64])
def test_sums_of_two_halves_add_up(hip, dtype):
    """CalculateCentroids2GPU: the sums over two shards equal the sums over the whole set."""
    kat = KATS["calculate_centroids_2gpu"]
    X = np.asarray(kat["data"], dtype)
    labels = np.asarray(kat["labels"])
    s = kat["split_at"]
    k = kat["k"]
    whole, wc = one_update(hip, X, labels, np.zeros((k, 2)), dtype)
    a, ac = one_update(hip, X[:s], labels[:s], np.zeros((k, 2)), dtype)
    b, bc = one_update(hip, X[s:], labels[s:], np.zeros((k, 2)), dtype)
    assert (ac + bc).tolist() == wc.tolist()
    got = a.astype(np.float64) * ac[:, None] + b.astype(np.float64) * bc[:, None]
    assert np.allclose(got, whole.astype(np.float64) * wc[:, None], rtol=1e-6)


@pytest.mark.parametrize("dtype", [np.float32, np.float64])
def test_empty_cluster_keeps_its_centroid(hip, dtype):
    """RevertCentroidZeroing: counts {1,0,1} -> the middle centroid is the old one."""
    kat = KATS["revert_centroid_zeroing"]
    cur = np.asarray(kat["current"], dtype)
    X = cur[[0, 2]]                      # one row each for clusters 0 and 2
    C, counts = one_update(hip, X, [0, 2], kat["old_centroids"], dtype)
    assert counts.tolist() == kat["counts"]
    assert np.array_equal(C, np.asarray(kat["expected"], dtype))


def test_readme_example_shapes(hip):
    from h2o4gpu_amd import KMeans
    kat = KATS["readme_example_shapes"]
    X = np.asarray(kat["data"], np.float32)
    m = KMeans(n_clusters=kat["k"], random_state=1234).fit(X)
    assert m.cluster_centers_.shape == (2, 2)
    assert m.predict(X).shape == (3,) and m.transform(X).shape == (3, 2)
