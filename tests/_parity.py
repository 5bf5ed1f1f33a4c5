"""Shared parity checks: GPU results against the CPU oracle."""

import numpy as np

# north-star tolerances
RTOL = {np.dtype(np.float32): 1e-5, np.dtype(np.float64): 1e-12}
NEAR_TIE = 1e-6


def sq_distances_f64(X, centers, rows):
    """Exact (fp64) squared distances of the given sample rows to every centroid."""
    Xr = np.asarray(X[rows], dtype=np.float64)
    C = np.asarray(centers, dtype=np.float64)
    return ((Xr[:, None, :] - C[None, :, :]) ** 2).sum(axis=2)


def assert_labels_match(labels_gpu, labels_ref, X, centers, max_fraction=1e-3):
    """Labels equal except at near-ties: d(x, c_gpu) - d(x, c_ref) <= 1e-6 * max_c d(x, c), distances in fp64."""
    labels_gpu = np.asarray(labels_gpu).astype(np.int64)
    labels_ref = np.asarray(labels_ref).astype(np.int64)
    assert labels_gpu.shape == labels_ref.shape
    bad = np.flatnonzero(labels_gpu != labels_ref)
    if bad.size == 0:
        return 0
    assert bad.size <= max(1, int(max_fraction * labels_ref.size)), (
        f"{bad.size} of {labels_ref.size} labels differ"
    )
    dist = sq_distances_f64(X, centers, bad)
    d_gpu = dist[np.arange(bad.size), labels_gpu[bad]]
    d_ref = dist[np.arange(bad.size), labels_ref[bad]]
    tol = NEAR_TIE * dist.max(axis=1)
    # one-sided: a label whose exact distance is SMALLER than that of the oracle's label is the
    # better arg-min (the oracle evaluates in the input precision and loses such near-ties itself)
    excess = d_gpu - d_ref
    worst = np.max(excess / dist.max(axis=1))
    assert np.all(excess <= tol), (
        f"{bad.size} label mismatches, worst relative gap {worst:.3e} exceeds the near-tie bound"
    )
    return bad.size


def assert_centers_close(c_gpu, c_ref, dtype, scale_rtol=None):
    """|gpu - ref| <= rtol * (|ref| + norm scale): rtol 1e-5 (fp32) / 1e-12 (fp64) relative to
    the coordinate, with the per-centroid max-norm as floor for coordinates near zero."""
    c_gpu = np.asarray(c_gpu, dtype=np.float64)
    c_ref = np.asarray(c_ref, dtype=np.float64)
    rtol = scale_rtol if scale_rtol is not None else RTOL[np.dtype(dtype)]
    scale = np.abs(c_ref).max(axis=1, keepdims=True)
    err = np.abs(c_gpu - c_ref)
    bound = rtol * np.maximum(np.abs(c_ref), scale)
    assert np.all(err <= bound), f"max centroid error / bound = {np.max(err / np.maximum(bound, 1e-300)):.3f}"
