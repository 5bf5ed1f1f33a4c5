"""numpy restatement of the reference KMeans path.  TEST INFRASTRUCTURE ONLY.

Arrays use the natural (n_samples, n_features) / (n_clusters, n_features) orientation;
the reference works on the transposes (X_t, centroids_t) but no arithmetic depends on it.
Everything marked "in T" is evaluated in the input floating dtype, one IEEE operation
at a time, in the reference's order.

Function                      follows (reference file:line)                    pinned by
----------------------------  -----------------------------------------------  ---------------------------------
half_sq_norms                 common/kernels.py:127-143                        closed form (tests/test_oracle_kmeans.py)
pseudo_distances/assign       kernels/_base_kmeans_kernel_funcs.py:266-301,    brute-force argmin of ||x-c||^2 in fp64;
                              :359-366; kernels/compute_labels.py:75-168       sklearn _labels_inertia; predict(centers)=arange
                                                                               (reference test_kmeans.py:113-122)
sq_dist_to_assigned /         kernels/compute_inertia.py:16-39                 closed form sum w||x-c||^2 with signed weights
per_sample_inertia                                                             (reference test_kmeans.py:182-205)
euclidean_distances           kernels/compute_euclidean_distances.py:136-152   closed form / scipy cdist (test_kmeans.py:161-179)
lloyd_step / lloyd            drivers.py:43-393, kernels/lloyd_single_step.py  sklearn _kmeans_single_lloyd (labels equal,
                              :338-414, kernels/utils.py:88-167,               centers/inertia allclose, same n_iter);
                              common/kernels.py:69-80                          4-point toy (test_kmeans.py:125-158)
relocate_empty_clusters       drivers.py:396-433, kernels/utils.py:23-74       sklearn _relocate_empty_clusters_dense;
                                                                               reference test_kmeans.py:208-248
prepare_data_for_lloyd /      drivers.py:436-589                               np.mean, sklearn _tolerance
restore_data_after_lloyd
kmeans_plusplus               drivers.py:735-910, kernels/kmeans_plusplus.py   known answer -865.257501
                                                                               (reference test_kmeans.py:251-325)
is_same_clustering /          kernels/utils.py:198-279                         sklearn _is_same_clustering; answer 7
count_distinct_clusters                                                        (reference test_kmeans.py:448-457)

Deliberate departures from the reference's literal behaviour (each one is a reference
defect with no stable output to reproduce):
  * the strict-convergence flag is armed before the second iteration
    (drivers.py:176,328-332 leaves it uninitialised on the first one);
  * `tol` is scaled by the true mean feature variance (the reference's fused-square
    reduction, common/reductions.py:440-449, squares partial sums again);
  * relocation distances: `relocation="sklearn"` (default) measures to the centroids the
    labels were computed from, `relocation="literal"` to the un-normalised sums
    (drivers.py:252-259).  PARITY UNPINNED for the `literal` branch: nothing outside this
    file fixes its output (the reference's own relocation test passes with either);
  * far samples are paired with empty clusters canonically: empty ids ascending, samples
    by descending distance then ascending index (the reference's order comes from atomics);
  * kmeans++ `sampler="exact"` searches an fp64 inclusive scan, `sampler="literal"`
    repeats the sequential running sum in T (kernels/kmeans_plusplus.py:92-100).
"""

import numpy as np

from . import rng as _rng


# --------------------------------------------------------------------------- distances


def half_sq_norms(centers):
    """(sum_f c_f^2) / 2 per centroid, accumulated feature by feature in T."""
    centers = np.asarray(centers)
    T = centers.dtype.type
    acc = np.zeros(centers.shape[0], dtype=T)
    for f in range(centers.shape[1]):
        acc = acc + centers[:, f] * centers[:, f]
    return acc / T(2)


def pseudo_distances(X, centers, half=None):
    """half||c||^2 - <x, c>, dot product accumulated feature 0, 1, ... in T."""
    X = np.asarray(X)
    centers = np.asarray(centers)
    if half is None:
        half = half_sq_norms(centers)
    n, d = X.shape
    dot = X[:, 0:1] * centers[None, :, 0]
    for f in range(1, d):
        dot += X[:, f : f + 1] * centers[None, :, f]
    return half[None, :] - dot


def assign_labels(X, centers, chunk=8192, return_margin=False):
    """Label = argmin of the pseudo distance; strict `<` so the lowest index wins ties.

    With `return_margin`, also returns per sample (second-best - best) of the pseudo
    distance and max_c |pseudo|, which the tests use to recognise near-ties.
    """
    X = np.asarray(X)
    centers = np.asarray(centers)
    half = half_sq_norms(centers)
    n = X.shape[0]
    labels = np.empty(n, dtype=np.uint32)
    margin = np.empty(n, dtype=np.float64) if return_margin else None
    for lo in range(0, n, chunk):
        pd = pseudo_distances(X[lo : lo + chunk], centers, half)
        lab = np.argmin(pd, axis=1)
        labels[lo : lo + chunk] = lab
        if return_margin:
            if pd.shape[1] > 1:
                part = np.partition(pd.astype(np.float64), 1, axis=1)
                margin[lo : lo + chunk] = part[:, 1] - part[:, 0]
            else:
                margin[lo : lo + chunk] = np.inf
    if return_margin:
        return labels, margin
    return labels


def sq_dist_to_assigned(X, centers, labels):
    """sum_f (x_f - c_f)^2 to the assigned centroid, accumulated in feature order in T."""
    X = np.asarray(X)
    centers = np.asarray(centers)
    T = X.dtype.type
    C = centers[np.asarray(labels).astype(np.int64)]
    acc = np.zeros(X.shape[0], dtype=T)
    for f in range(X.shape[1]):
        diff = X[:, f] - C[:, f]
        acc = acc + diff * diff
    return acc


def per_sample_inertia(X, sample_weight, centers, labels):
    return sq_dist_to_assigned(X, centers, labels) * np.asarray(sample_weight)


def inertia(X, sample_weight, centers, labels):
    return per_sample_inertia(X, sample_weight, centers, labels).sum(dtype=np.float64)


def euclidean_distances(X, centers, chunk=8192):
    """sqrt(sum_f (c_f - x_f)^2) for every (sample, centroid) pair, shape (n, k)."""
    X = np.asarray(X)
    centers = np.asarray(centers)
    T = X.dtype.type
    n, d = X.shape
    out = np.empty((n, centers.shape[0]), dtype=T)
    for lo in range(0, n, chunk):
        Xc = X[lo : lo + chunk]
        acc = np.zeros((Xc.shape[0], centers.shape[0]), dtype=T)
        for f in range(d):
            diff = centers[None, :, f] - Xc[:, f : f + 1]
            acc += diff * diff
        out[lo : lo + chunk] = np.sqrt(acc)
    return out


# --------------------------------------------------------------------------- Lloyd


def weighted_sums(X, sample_weight, labels, n_clusters):
    """Per-cluster sum of w*x (product in T, accumulation in fp64, result in T) and of w.

    The reference accumulates with unordered float atomics (lloyd_single_step.py:400-414),
    so only the exact sums, not a rounding order, can be restated.
    """
    X = np.asarray(X)
    T = X.dtype.type
    w = np.asarray(sample_weight, dtype=T)
    lab = np.asarray(labels).astype(np.int64)
    sums = np.empty((n_clusters, X.shape[1]), dtype=np.float64)
    for f in range(X.shape[1]):
        sums[:, f] = np.bincount(lab, weights=(X[:, f] * w).astype(np.float64), minlength=n_clusters)
    sizes = np.bincount(lab, weights=w.astype(np.float64), minlength=n_clusters)
    return sums.astype(T), sizes.astype(T)


def top_k_indices(values, k):
    """Indices of the k largest values: descending value, ties by ascending index."""
    values = np.asarray(values)
    if k > values.shape[0]:
        raise ValueError("k larger than the number of items")
    order = np.lexsort((np.arange(values.shape[0]), -values.astype(np.float64)))
    return order[:k].astype(np.int64)


def relocate_empty_clusters(X, sample_weight, sums, sizes, labels, sq_dist):
    """Move each empty cluster onto one of the samples farthest from its centroid.

    Works on the un-normalised sums, like kernels/utils.py:23-74.  Returns the far
    sample indices used (empty array if nothing was relocated).
    """
    T = X.dtype.type
    empty = np.flatnonzero(sizes == 0)
    if empty.size == 0:
        return np.empty(0, dtype=np.int64)
    if not (np.max(sq_dist) > 0):
        # more clusters than distinct samples: nothing sensible to move
        return np.empty(0, dtype=np.int64)
    far = top_k_indices(sq_dist, empty.size)
    for cluster, i in zip(empty, far):
        w = T(sample_weight[i])
        old = int(labels[i])
        addend = X[i] * w
        sums[old] = sums[old] - addend
        sums[cluster] = addend
        sizes[old] = sizes[old] - w
        sizes[cluster] = w
    return far


def lloyd_iterations(X, sample_weight, centers_init, max_iter=300, tol=0.0, relocation="sklearn"):
    """Generator over Lloyd iterations.

    Yields dict(labels, centers, sizes, shift, n_iter, strict, n_empty) after each one.
    """
    X = np.asarray(X)
    T = X.dtype.type
    w = np.asarray(sample_weight, dtype=T)
    centers = np.array(centers_init, dtype=T, copy=True)
    k = centers.shape[0]
    prev_labels = None
    n_iter = 0
    shift = np.inf
    while n_iter < max_iter and shift > tol:
        labels = assign_labels(X, centers)
        sums, sizes = weighted_sums(X, w, labels, k)
        n_empty = int(np.count_nonzero(sizes == 0))
        if n_empty:
            ref_centers = centers if relocation == "sklearn" else sums
            sq = sq_dist_to_assigned(X, ref_centers, labels)
            relocate_empty_clusters(X, w, sums, sizes, labels, sq)
        new_centers = np.empty_like(sums)
        heaviest = int(np.argmax(sizes))
        for c in range(k):
            if sizes[c] != 0:
                new_centers[c] = sums[c] / sizes[c]
        for c in range(k):
            if sizes[c] == 0:
                new_centers[c] = new_centers[heaviest]
        n_iter += 1
        strict = prev_labels is not None and np.array_equal(labels, prev_labels)
        diff = centers - new_centers
        shift = float(np.sum((diff * diff).astype(np.float64)))
        centers = new_centers
        prev_labels = labels
        yield dict(labels=labels, centers=centers, sizes=sizes, shift=shift, n_iter=n_iter,
                   strict=strict, n_empty=n_empty)
        if strict:
            return


def lloyd(X, sample_weight, centers_init, max_iter=300, tol=0.0, relocation="sklearn"):
    """Single Lloyd run: returns (labels u32, inertia, centers (k, d), n_iter)."""
    X = np.asarray(X)
    T = X.dtype.type
    centers = np.array(centers_init, dtype=T, copy=True)
    n_iter = 0
    for state in lloyd_iterations(X, sample_weight, centers_init, max_iter, tol, relocation):
        centers = state["centers"]
        n_iter = state["n_iter"]
    labels = assign_labels(X, centers)
    return labels, inertia(X, sample_weight, centers, labels), centers, n_iter


# --------------------------------------------------------------------------- centering


def prepare_data_for_lloyd(X, init, tol, sample_weight):
    """Returns (X_centered, X_mean or None, init_centered, tol_scaled, weights_are_uniform)."""
    X = np.asarray(X)
    T = X.dtype.type
    n, d = X.shape
    X_mean = (X.sum(axis=0, dtype=np.float64) / n).astype(T)
    if float(np.sum(X_mean.astype(np.float64) ** 2)) == 0.0:
        X_mean = None
        Xc = X
    else:
        Xc = X - X_mean
        if isinstance(init, np.ndarray):
            init = init - X_mean
    variance = float(np.sum(Xc.astype(np.float64) ** 2)) / (n * d)
    w = np.asarray(sample_weight, dtype=T)
    uniform = bool(T(w.sum(dtype=np.float64)) == T(w[0]) * T(n))
    return Xc, X_mean, init, variance * tol, uniform


def restore_data_after_lloyd(centers, X_mean):
    if X_mean is None:
        return centers
    return centers + X_mean


# --------------------------------------------------------------------------- kmeans++


def kpp_uniform_table(n_clusters, n_local_trials, seed, dtype):
    """start_raw and U[c-1, t] = the uniform trial t draws when centre c is picked.

    Trial t always advances state t; state 0 first serves the raw draw that picks the
    starting centre (common/random.py:29-38, drivers.py:830).
    """
    gen = _rng.Xoroshiro128pp(n_local_trials, seed)
    start_raw = gen.next_raw(0)
    table = np.empty((max(n_clusters - 1, 0), n_local_trials), dtype=dtype)
    for c in range(n_clusters - 1):
        for t in range(n_local_trials):
            table[c, t] = gen.uniform(t, dtype)
    return start_raw, table


def _sample_literal(closest, total, u):
    """kernels/kmeans_plusplus.py:92-100: sequential running sum in T (-1 when rv == 0)."""
    T = closest.dtype.type
    rv = T(u) * T(total)
    cum = np.cumsum(closest, dtype=T)  # numpy's cumsum is the same sequential recurrence
    idx = int(np.searchsorted(cum, rv, side="left"))
    if not rv > T(0):
        return -1
    return min(idx, closest.shape[0] - 1)


def _sample_exact(closest, u):
    """fp64 inclusive scan; rv = u * total in fp64; first j with cum_j >= rv, clipped."""
    cum = np.cumsum(closest.astype(np.float64))
    rv = np.float64(u) * cum[-1]
    idx = int(np.searchsorted(cum, rv, side="left"))
    return min(max(idx, 0), closest.shape[0] - 1)


def kmeans_plusplus(X, sample_weight, n_clusters, seed, sampler="exact", return_trace=False):
    """kmeans++ seeding; returns (centers (k, d), indices int32 (k,))."""
    X = np.asarray(X)
    T = X.dtype.type
    n, d = X.shape
    w = np.asarray(sample_weight, dtype=T)
    n_trials = 2 + int(np.log(n_clusters))
    start_raw, table = kpp_uniform_table(n_clusters, n_trials, seed, T)
    indices = np.full(n_clusters, -1, dtype=np.int32)
    indices[0] = start_raw % n

    def wdist(i):
        acc = np.zeros(n, dtype=T)
        for f in range(d):
            diff = X[:, f] - X[i, f]
            acc = acc + diff * diff
        return acc * w

    closest = wdist(indices[0])
    total = T(closest.sum(dtype=np.float64))
    trace = []
    for c in range(1, n_clusters):
        cands = np.empty(n_trials, dtype=np.int64)
        for t in range(n_trials):
            if sampler == "literal":
                # -1 (rv <= 0) is used by the reference's next kernel as an index from the end
                cands[t] = _sample_literal(closest, total, table[c - 1, t]) % n
            else:
                cands[t] = _sample_exact(closest, table[c - 1, t])
        rows = np.stack([np.minimum(wdist(int(i)), closest) for i in cands])
        potentials = rows.sum(axis=1, dtype=np.float64)
        best = int(np.argmin(potentials.astype(T) if sampler == "literal" else potentials))
        closest = rows[best]
        total = T(potentials[best])
        indices[c] = cands[best]
        trace.append((cands.copy(), potentials.copy(), best))
    centers = X[indices.astype(np.int64)].copy()
    if return_trace:
        return centers, indices, trace
    return centers, indices


# --------------------------------------------------------------------------- label helpers


def is_same_clustering(labels1, labels2, n_clusters):
    """Equal up to a permutation of the labels (the mapping labels1 -> labels2 is a function)."""
    mapping = np.full(n_clusters, -1, dtype=np.int64)
    for a, b in zip(np.asarray(labels1).tolist(), np.asarray(labels2).tolist()):
        if mapping[a] == -1:
            mapping[a] = b
        elif mapping[a] != b:
            return False
    return True


def count_distinct_clusters(labels):
    return int(np.unique(np.asarray(labels)).shape[0])
