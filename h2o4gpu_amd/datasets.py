"""Seeded synthetic inputs for the five k-means benchmark shapes.

Every shape is produced by numpy.random.Generator(PCG64(seed)) in row chunks, so
the same (name, scale) always yields the same bytes, whatever machine runs it.
`scale` shrinks the row count (never d or k) so the CPU checker finishes in
seconds; scale=1.0 is the full benchmark shape.
"""
import numpy as np

# name -> (rows, cols, k, seed, Lloyd iterations)
SHAPES = {
    "C1": (100_000, 16, 8, 1001, 20),
    "C2": (1_000_000, 64, 64, 1002, 50),
    "C3": (10_000_000, 32, 256, 1003, 30),
    "C4": (2_000_000, 256, 1024, 1004, 20),
    "C5": (500_000, 784, 4096, 1005, 15),
}

_CHUNK = 1 << 18


def _rows(name, scale):
    n = SHAPES[name][0]
    k = SHAPES[name][2]
    return max(int(round(n * scale)), 2 * k)


def _blob_rows(rng, centers, sizes_or_n, sigma, dtype, shuffle_assign):
    """Rows = centre[label] + sigma*N(0,1); labels drawn or laid out by sizes."""
    k, d = centers.shape
    if np.isscalar(sizes_or_n):
        n = int(sizes_or_n)
        labels = None
    else:
        sizes = np.asarray(sizes_or_n, np.int64)
        n = int(sizes.sum())
        labels = np.repeat(np.arange(k, dtype=np.int32), sizes)
        if shuffle_assign:
            rng.shuffle(labels)
    X = np.empty((n, d), dtype)
    for lo in range(0, n, _CHUNK):
        hi = min(n, lo + _CHUNK)
        if labels is None:
            lab = rng.integers(0, k, size=hi - lo)
        else:
            lab = labels[lo:hi]
        noise = rng.standard_normal((hi - lo, d), dtype=np.float32)
        X[lo:hi] = (centers[lab] + sigma * noise).astype(dtype, copy=False)
    return X


def make(name, scale=1.0, dtype=np.float32):
    """Returns (X, k, iterations) for benchmark shape `name`."""
    n_full, d, k, seed, iters = SHAPES[name]
    n = _rows(name, scale)
    rng = np.random.Generator(np.random.PCG64(seed))
    dtype = np.dtype(dtype)
    if name == "C1":
        centers = rng.uniform(-10.0, 10.0, size=(k, d)).astype(np.float32)
        X = _blob_rows(rng, centers, n, 1.0, dtype, False)
    elif name == "C2":
        centers = (5.0 * rng.standard_normal((k, d))).astype(np.float32)
        w = rng.dirichlet(np.ones(k))
        sizes = np.floor(w * n).astype(np.int64)
        sizes[np.argmax(sizes)] += n - sizes.sum()
        X = _blob_rows(rng, centers, sizes, 2.0, dtype, True)
    elif name == "C3":
        centers = rng.uniform(-50.0, 50.0, size=(k, d)).astype(np.float32)
        sizes = np.full(k, n // k, np.int64)
        sizes[: n - sizes.sum()] += 1
        X = _blob_rows(rng, centers, sizes, 3.0, dtype, True)
    elif name == "C4":
        centers = (4.0 * rng.standard_normal((k, d))).astype(np.float32)
        X = _blob_rows(rng, centers, n, 1.0, dtype, False)
        n_out = n // 10
        rows = rng.choice(n, size=n_out, replace=False)
        for lo in range(0, n_out, _CHUNK):
            hi = min(n_out, lo + _CHUNK)
            X[rows[lo:hi]] = rng.uniform(-20.0, 20.0, size=(hi - lo, d)).astype(dtype)
    elif name == "C5":
        X = _image_like(rng, n, d, dtype)
    else:
        raise KeyError(name)
    return X, k, iters


def _image_like(rng, n, d, dtype):
    X = np.empty((n, d), dtype)
    for lo in range(0, n, _CHUNK // 4):
        hi = min(n, lo + _CHUNK // 4)
        vals = rng.integers(1, 256, size=(hi - lo, d), dtype=np.int16)
        keep = rng.random((hi - lo, d), dtype=np.float32) >= 0.7
        X[lo:hi] = np.where(keep, vals, 0).astype(dtype)
    return X


def make_holdout(name, rows, dtype=np.float32):
    """Held-out rows from the generator of `name` (a later stream of the same seed)."""
    n_full, d, k, seed, iters = SHAPES[name]
    rng = np.random.Generator(np.random.PCG64(seed).jumped(1))
    if name != "C5":
        raise KeyError("held-out rows are defined for C5 only")
    return _image_like(rng, rows, d, np.dtype(dtype))


def seeded_row_init(X, k, seed):
    """k distinct seeded-random rows of X (numpy stream; used where the benchmark
    text asks for 'seeded-random row init' and both sides are fed the same rows)."""
    rng = np.random.Generator(np.random.PCG64(seed))
    idx = rng.choice(X.shape[0], size=k, replace=False)
    return np.ascontiguousarray(X[np.sort(idx)])
