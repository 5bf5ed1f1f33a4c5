"""Frozen synthetic data generators for the five benchmark configurations (used by the
throughput benchmark, the benchmark CLI and the parity tests; no computation of the KMeans
path lives here).

Each generator draws, in the stated order, from `rng = np.random.default_rng(seed)`:
centres, (per-blob std), (blob sizes), the Gaussian noise, a row permutation, the initial
rows, (the weights).  Data are generated in fp64 blob by blob and cast at the end; arrays are
C-contiguous (n_samples, n_features).  `n` can be overridden to get a smaller problem with
the same structure (used by the parity tests).
"""

import numpy as np


def _blobs(rng, centers, sizes, stds, dtype, chunk=1 << 20):
    n = int(np.sum(sizes))
    d = centers.shape[1]
    y = np.repeat(np.arange(len(sizes)), sizes)
    X = np.empty((n, d), dtype=dtype)
    std_per_row = np.asarray(stds, dtype=np.float64)[y] if np.ndim(stds) else None
    for lo in range(0, n, chunk):
        hi = min(lo + chunk, n)
        noise = rng.standard_normal((hi - lo, d))
        if std_per_row is not None:
            noise *= std_per_row[lo:hi, None]
        else:
            noise *= float(stds)
        X[lo:hi] = (centers[y[lo:hi]] + noise).astype(dtype)
    perm = rng.permutation(n)
    return X[perm], y[perm]


def _equal_sizes(n, k):
    sizes = np.full(k, n // k, dtype=np.int64)
    sizes[: n % k] += 1
    return sizes


def config1(n=100_000):
    """fp32, 14 features, 127 equal isotropic blobs (std 1), unit weights, tol 0."""
    rng = np.random.default_rng(0)
    d, k = 14, 127
    centers = rng.uniform(-10, 10, (k, d))
    X, _ = _blobs(rng, centers, _equal_sizes(n, k), 1.0, np.float32)
    init = X[rng.choice(n, k, replace=False)].copy()
    w = np.ones(n, dtype=np.float32)
    return dict(X=X, init=init, sample_weight=w, k=k, max_iter=100, tol=0.0, name="C1")


def config2(n=5_000_000):
    """fp32, 14 features, 127 blobs with std in [0.5, 2], Dirichlet sizes, weights in [0.5, 1.5]."""
    rng = np.random.default_rng(1)
    d, k = 14, 127
    centers = rng.uniform(-10, 10, (k, d))
    stds = rng.uniform(0.5, 2.0, k)
    sizes = rng.multinomial(n, rng.dirichlet(np.ones(k)))
    X, _ = _blobs(rng, centers, sizes, stds, np.float32)
    init = X[rng.choice(n, k, replace=False)].copy()
    w = rng.uniform(0.5, 1.5, n).astype(np.float32)
    return dict(X=X, init=init, sample_weight=w, k=k, max_iter=100, tol=0.0, name="C2")


def config3(n=1_000_000, d=256, k=1024):
    """fp32, 256 features, 1024 equal blobs, centres N(0, 4 I), std 1, unit weights."""
    rng = np.random.default_rng(2)
    centers = rng.normal(0.0, 2.0, (k, d))
    X, _ = _blobs(rng, centers, _equal_sizes(n, k), 1.0, np.float32)
    init = X[rng.choice(n, k, replace=False)].copy()
    w = np.ones(n, dtype=np.float32)
    return dict(X=X, init=init, sample_weight=w, k=k, max_iter=50, tol=0.0, name="C3")


def config4(n=1_000_000, d=64, k=256):
    """kmeans++ only: fp32, 64 features, 256 equal blobs in [-5, 5]^64, std 1, RNG seed 3."""
    rng = np.random.default_rng(3)
    centers = rng.uniform(-5, 5, (k, d))
    X, _ = _blobs(rng, centers, _equal_sizes(n, k), 1.0, np.float32)
    w = np.ones(n, dtype=np.float32)
    return dict(X=X, sample_weight=w, k=k, seed=3, n_local_trials=2 + int(np.log(k)), name="C4")


def config5(n=2_000_000, d=32, n_blobs=48, k=64):
    """fp64 with forced empty clusters: 48 blobs (std 0.5), k = 64 = 48 random rows + 16 far
    centroids at +1e3 * (1 + j * 1e-3) in every coordinate; tol 1e-4 (relative)."""
    rng = np.random.default_rng(4)
    centers = rng.uniform(-10, 10, (n_blobs, d))
    X, _ = _blobs(rng, centers, _equal_sizes(n, n_blobs), 0.5, np.float64)
    init = np.empty((k, d), dtype=np.float64)
    init[:n_blobs] = X[rng.choice(n, n_blobs, replace=False)]
    for j in range(k - n_blobs):
        init[n_blobs + j] = 1e3 * (1 + j * 1e-3)
    w = np.ones(n, dtype=np.float64)
    return dict(X=X, init=init, sample_weight=w, k=k, max_iter=100, tol=1e-4, name="C5")
