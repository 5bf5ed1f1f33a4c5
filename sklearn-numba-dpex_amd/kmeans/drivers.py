"""Host drivers of the KMeans path: the operator interface of the reference's
sklearn_numba_dpex/kmeans/drivers.py (same function names, argument meaning and returns),
orchestrating the HIP kernels of libmi355x_kmeans.so through the C ABI.

Arrays are torch ROCm tensors used as device buffers, in the reference's transposed layout:
`X_t` (n_features, n_samples), `centroids_t` (n_features, n_clusters), both C-contiguous.
Labels are 32-bit (torch.int32 holding the uint32 values the kernels write).
"""

import numpy as np
import torch

from .. import _capi
from .._capi import LloydStatus, check, lib, ptr
from ..common._buffers import contiguous, dcode, require_cuda, workspace
from ..common.kernels import broadcast_rows, divide_by, transposed_copy
from ..common.random import create_xoroshiro128pp_states, get_random_raw, raw_to_uniform
from ..common.reductions import sum_reduction
from ..common.topk import topk_idx

# How many Lloyd iterations may be enqueued before the host next reads the status.
_MAX_LOOKAHEAD = 16



def lloyd(
    X_t,
    sample_weight,
    centroids_t,
    use_uniform_weights=False,
    max_iter=300,
    verbose=False,
    tol=1e-4,
    relocation="sklearn",
    flags=None,
):
    """Single Lloyd run (reference: kmeans/drivers.py:43-393).

    Returns (assignments_idx (n,), inertia numpy scalar, centroids_t (d, k), n_iteration).

    The loop state (iteration count, convergence, empty clusters) lives on the device, and
    every kernel of an iteration is a no-op once the state is terminal, so iterations are
    enqueued ahead and the host reads the status once per batch instead of three times per
    iteration.

    relocation: which centroids the distances that rank samples for empty-cluster relocation
    are measured to: "sklearn" = the centroids the labels were computed from (what
    scikit-learn does), "literal" = the un-normalised sums (kmeans/drivers.py:252-259).

    flags: kernel selection (KMX_FLAG_* of the C header); None = the defaults `_capi` took from
    the environment when it was imported.
    """
    require_cuda()
    X_t = contiguous(X_t)
    sample_weight = contiguous(sample_weight)
    d, n = X_t.shape
    k = centroids_t.shape[1]
    dev, dt, dc = X_t.device, X_t.dtype, dcode(X_t)
    stream = _capi.current_stream()

    plan = _capi.lloyd_plan(n, d, k, dc, flags)
    ws_bytes = plan.workspace_bytes
    ws = workspace(ws_bytes, dev)
    cent = [contiguous(centroids_t).clone(), torch.empty((d, k), dtype=dt, device=dev)]
    labels = [torch.empty(n, dtype=torch.int32, device=dev) for _ in range(2)]
    sizes = torch.empty(k, dtype=dt, device=dev)
    empty_list = torch.empty(k, dtype=torch.int32, device=dev)
    verbose = bool(verbose)

    # the wide fp32 path and the bucketed sums add up each cluster's rows from a row-major copy
    # of X (one transpose per run, n * d extra elements of HBM): whole cache lines per sample
    X_rm = None
    reads_rowmajor = lib.kmx_lloyd_plan_reads_rowmajor(plan)
    if reads_rowmajor < 0:
        check(reads_rowmajor, "kmx_lloyd_plan_reads_rowmajor")
    if reads_rowmajor == 1:
        try:
            X_rm = transposed_copy(X_t)
        except torch.cuda.OutOfMemoryError:
            X_rm = None  # the kernels then gather the feature-major array (slower, same results)

    check(lib.kmx_lloyd_init(plan, ptr(ws), ws_bytes, ptr(X_t), ptr(sample_weight), ptr(cent[0]), int(max_iter),
                             float(tol), stream),
          "kmx_lloyd_init")

    status = LloydStatus()
    enqueued = 0
    lookahead = 1
    while True:
        for _ in range(lookahead):
            a, b = enqueued % 2, (enqueued + 1) % 2
            check(lib.kmx_lloyd_iter(plan, ptr(X_t), ptr(X_rm), ptr(sample_weight), ptr(cent[a]), ptr(cent[b]),
                                     ptr(labels[a]), ptr(labels[b]), ptr(sizes), ptr(empty_list),
                                     ptr(ws), ws_bytes, stream), "kmx_lloyd_iter")
            enqueued += 1
        check(lib.kmx_lloyd_status_read(ptr(ws), status, stream), "kmx_lloyd_status_read")

        if status.state == _capi.KMX_NEED_RELOCATION:
            j = status.n_iter  # the iteration that stopped: reads cent[j % 2], wrote sums to the other
            a, b = j % 2, (j + 1) % 2
            _relocate_empty_clusters(
                status.n_empty, X_t, sample_weight, cent[b], sizes, labels[b], empty_list,
                cent[a] if relocation == "sklearn" else cent[b],
            )
            check(lib.kmx_lloyd_finalize(plan, ptr(cent[a]), ptr(cent[b]), ptr(sizes), ptr(ws), ws_bytes,
                                         stream), "kmx_lloyd_finalize")
            enqueued = j + 1
            lookahead = 1
            check(lib.kmx_lloyd_status_read(ptr(ws), status, stream), "kmx_lloyd_status_read")

        if verbose:
            j = status.n_iter
            # inertia of the labels just computed w.r.t. the centroids they were computed from
            inertia = _inertia(X_t, sample_weight, cent[(j - 1) % 2], labels[j % 2])
            print(f"Iteration {j - 1}, inertia {inertia:5.3e}")

        if status.state != _capi.KMX_RUNNING:
            break
        enqueued = status.n_iter
        lookahead = 1 if verbose else min(2 * lookahead, _MAX_LOOKAHEAD)

    n_iteration = status.n_iter
    if verbose:
        converged_at = n_iteration - 1
        if status.state == _capi.KMX_CONVERGED_STRICT or status.shift_sum == 0:
            print(f"Converged at iteration {converged_at}: strict convergence.")
        elif status.shift_sum <= tol:
            print(f"Converged at iteration {converged_at}: center shift "
                  f"{status.shift_sum} within tolerance {tol}.")

    # labels for the final centroids and the exact inertia (kmeans/drivers.py:356-391)
    best = cent[n_iteration % 2]
    assignments_idx = labels[0]
    inertia = _assign_with_inertia(X_t, sample_weight, best, assignments_idx, flags)[0]
    return assignments_idx, inertia, best, n_iteration


def _assign(X_t, centroids_t, labels_out, flags=None):
    d, n = X_t.shape
    k = centroids_t.shape[1]
    dc = dcode(X_t)
    flags = _capi.DEFAULT_FLAGS if flags is None else int(flags)
    ws_bytes = lib.kmx_assign_workspace_bytes_for(n, d, k, dc, flags)
    ws = workspace(ws_bytes, X_t.device, tag="assign")
    check(lib.kmx_assign_labels(ptr(X_t), ptr(centroids_t), ptr(labels_out), ptr(ws), ws_bytes, n, d, k,
                                dc, flags, _capi.current_stream()), "kmx_assign_labels")


def _assign_with_inertia(X_t, sample_weight, centroids_t, labels_out, flags=None):
    """Labels into `labels_out` and the weighted inertia of that labelling as a 1-element numpy
    array, in one library call (one pass over X where the screened label kernel applies)."""
    d, n = X_t.shape
    k = centroids_t.shape[1]
    dc = dcode(X_t)
    flags = _capi.DEFAULT_FLAGS if flags is None else int(flags)
    ws_bytes = lib.kmx_assign_inertia_workspace_bytes(n, d, k, dc, flags)
    ws = workspace(ws_bytes, X_t.device, tag="assign_inertia")
    out = torch.empty(1, dtype=X_t.dtype, device=X_t.device)
    check(lib.kmx_assign_labels_inertia(ptr(X_t), ptr(sample_weight), ptr(centroids_t), ptr(labels_out), ptr(out),
                                        ptr(ws), ws_bytes, n, d, k, dc, flags, _capi.current_stream()),
          "kmx_assign_labels_inertia")
    return out.cpu().numpy()


def _per_sample_inertia(X_t, sample_weight, centroids_t, labels, out=None):
    d, n = X_t.shape
    k = centroids_t.shape[1]
    if out is None:
        out = torch.empty(n, dtype=X_t.dtype, device=X_t.device)
    check(lib.kmx_per_sample_inertia(ptr(X_t), ptr(sample_weight), ptr(centroids_t), ptr(labels), ptr(out),
                                     n, d, k, dcode(X_t), _capi.current_stream()), "kmx_per_sample_inertia")
    return out


def _inertia_array(X_t, sample_weight, centroids_t, labels):
    """1-element numpy array: the weighted sum of squared distances to the assigned centroids
    (the per-sample values are summed inside the kernel, not written out)."""
    d, n = X_t.shape
    k = centroids_t.shape[1]
    ws_bytes = lib.kmx_inertia_workspace_bytes(n)
    ws = workspace(ws_bytes, X_t.device, tag="inertia")
    out = torch.empty(1, dtype=X_t.dtype, device=X_t.device)
    check(lib.kmx_inertia(ptr(X_t), ptr(sample_weight), ptr(centroids_t), ptr(labels), ptr(out), ptr(ws), ws_bytes,
                          n, d, k, dcode(X_t), _capi.current_stream()), "kmx_inertia")
    return out.cpu().numpy()


def _inertia(X_t, sample_weight, centroids_t, labels):
    return _inertia_array(X_t, sample_weight, centroids_t, labels)[0]


def _relocate_empty_clusters(
    n_empty_clusters,
    X_t,
    sample_weight,
    centroids_t,
    cluster_sizes,
    assignments_idx,
    empty_clusters_list,
    distance_centroids_t,
):
    """Moves every empty cluster onto one of the samples farthest from its centroid
    (reference: kmeans/drivers.py:396-433 and the distance pass at :239-259).

    `centroids_t` holds the un-normalised sums and is updated in place together with
    `cluster_sizes`.  Pairing is canonical: empty cluster ids ascending (the order the
    reduction kernel lists them in) with samples by descending distance, ties by ascending
    index.
    """
    d, n = X_t.shape
    k = centroids_t.shape[1]
    # unit weights: the unweighted squared distance to the assigned centroid
    sq_dist = _per_sample_inertia(X_t, None, distance_centroids_t, assignments_idx)
    far = topk_idx(sq_dist, int(n_empty_clusters))
    if not float(sq_dist[far[0]]) > 0.0:
        # more clusters than distinct samples: nothing to relocate; the finalisation parks
        # the empty clusters on the heaviest one
        return
    check(lib.kmx_relocate_empty_clusters(ptr(X_t), ptr(sample_weight), ptr(assignments_idx), ptr(far),
                                          ptr(empty_clusters_list), int(n_empty_clusters), None,
                                          ptr(centroids_t), ptr(cluster_sizes), n, d, k, dcode(X_t),
                                          _capi.current_stream()), "kmx_relocate_empty_clusters")


def prepare_data_for_lloyd(X_t, init, tol, sample_weight, copy_x):
    """Centres X (and an array `init`) on the feature means, scales `tol` by the mean feature
    variance and tests whether the weights are uniform (reference: kmeans/drivers.py:436-545).

    Returns (X_t, X_mean or None, init, tol, sample_weight_is_uniform).  The variance is the
    true sum of squares / (n * d): the reference's fused-square reduction squares its partial
    sums again on every pass (common/reductions.py:440-449), which is not reproduced.
    """
    require_cuda()
    d, n = X_t.shape
    X_t = contiguous(X_t)
    X_mean = sum_reduction(X_t, axis=1)
    divide_by(X_mean, n)
    X_sum_squared = sum_reduction(X_mean, square=True)
    if float(X_sum_squared[0]) == 0.0:
        X_mean = None
    else:
        if copy_x:
            X_t = X_t.clone()
        broadcast_rows(X_t, X_mean, "minus")
        if isinstance(init, torch.Tensor):
            broadcast_rows(init, X_mean, "minus")

    variance = sum_reduction(X_t.reshape(-1), square=True)
    tol = (float(variance.cpu().numpy()[0]) / (d * n)) * tol

    sample_weight_sum = sum_reduction(sample_weight).cpu().numpy()[0]
    first = sample_weight[:1].cpu().numpy()[0]
    sample_weight_is_uniform = bool(sample_weight_sum == first * first.dtype.type(n))
    return X_t, X_mean, init, tol, sample_weight_is_uniform


def restore_data_after_lloyd(X_t, best_centers_t, X_mean, copy_x):
    """Adds the feature means back to the centres, and to X when it was centred in place
    (reference: kmeans/drivers.py:548-589)."""
    if X_mean is None:
        return
    if best_centers_t is not None:
        if not best_centers_t.is_contiguous():
            raise ValueError("best_centers_t must be the C-contiguous (d, k) centroid buffer")
        broadcast_rows(best_centers_t, X_mean, "plus")
    if not copy_x:
        broadcast_rows(X_t, X_mean, "plus")


def is_same_clustering(labels1, labels2, n_clusters):
    """True if the labelings are equal up to a permutation (reference: kmeans/drivers.py:592-602)."""
    n = labels1.shape[0]
    mapping = torch.empty(n_clusters, dtype=torch.int32, device=labels1.device)
    result = torch.empty(1, dtype=torch.int32, device=labels1.device)
    check(lib.kmx_is_same_clustering(ptr(contiguous(labels1)), ptr(contiguous(labels2)), ptr(mapping),
                                     ptr(result), n, int(n_clusters), _capi.current_stream()),
          "kmx_is_same_clustering")
    return bool(result.cpu().numpy()[0])


def get_nb_distinct_clusters(labels, n_clusters):
    """Number of distinct labels (reference: kmeans/drivers.py:605-627)."""
    seen = torch.empty(n_clusters, dtype=torch.int32, device=labels.device)
    result = torch.empty(1, dtype=torch.int32, device=labels.device)
    check(lib.kmx_count_distinct_clusters(ptr(contiguous(labels)), ptr(seen), ptr(result), labels.shape[0],
                                          int(n_clusters), _capi.current_stream()),
          "kmx_count_distinct_clusters")
    return result.cpu().numpy()[0]


def get_labels_inertia(X_t, centroids_t, sample_weight, with_inertia):
    """Labels for given centroids and, optionally, the inertia as a 1-element numpy array
    (reference: kmeans/drivers.py:630-699)."""
    require_cuda()
    X_t = contiguous(X_t)
    centroids_t = contiguous(centroids_t)
    n = X_t.shape[1]
    assignments_idx = torch.empty(n, dtype=torch.int32, device=X_t.device)
    if not with_inertia:
        _assign(X_t, centroids_t, assignments_idx)
        return assignments_idx, None
    return assignments_idx, _assign_with_inertia(X_t, contiguous(sample_weight), centroids_t, assignments_idx)


def get_euclidean_distances(X_t, Y_t):
    """(n_samples, n_clusters) view of the (n_clusters, n_samples) distance buffer
    (reference: kmeans/drivers.py:702-732)."""
    require_cuda()
    X_t = contiguous(X_t)
    Y_t = contiguous(Y_t)
    d, n = X_t.shape
    k = Y_t.shape[1]
    distances_t = torch.empty((k, n), dtype=X_t.dtype, device=X_t.device)
    check(lib.kmx_euclidean_distances(ptr(X_t), ptr(Y_t), ptr(distances_t), n, d, k, dcode(X_t),
                                      _capi.current_stream()), "kmx_euclidean_distances")
    return distances_t.T


def kpp_uniforms(n_clusters, n_local_trials, random_state, dtype):
    """Starting raw draw and the table U[c - 1, t] of the uniform that trial t draws when
    centre c is picked (state t serves trial t; state 0 first serves the raw draw that picks
    the starting centre: common/random.py:29-38, kmeans/drivers.py:799-803, 830)."""
    states = create_xoroshiro128pp_states(n_local_trials, seed=random_state)
    start_raw = get_random_raw(states)
    raw = states.next_raw_all(n_steps=max(n_clusters - 1, 0))
    return start_raw, raw_to_uniform(raw, dtype).astype(np.float64)


def kmeans_plusplus(X_t, sample_weight, n_clusters, random_state, sampler="scan"):
    """kmeans++ seeding (reference: kmeans/drivers.py:735-910).

    Returns (centers_t (d, k), center_indices int32 (k,)).  The uniform draws are generated
    on the host (integer RNG, a few values per centre) and uploaded once; the whole seeding
    then runs on the device without a host round trip.

    sampler: "scan" (default) finds the candidates by searching the fp64 inclusive scan of the
    closest-distance array; "literal" repeats the reference's serial running sum in the compute
    dtype (kmeans/kernels/kmeans_plusplus.py:79-100) and so picks the reference's candidates for
    the same draws, at about 8 ns per sample and centre.
    """
    if sampler not in ("scan", "literal"):
        raise ValueError(f"sampler must be 'scan' or 'literal', got {sampler!r}")
    require_cuda()
    X_t = contiguous(X_t)
    sample_weight = contiguous(sample_weight)
    d, n = X_t.shape
    dev, dc = X_t.device, dcode(X_t)
    n_local_trials = 2 + int(np.log(n_clusters))
    np_dtype = np.float32 if X_t.dtype == torch.float32 else np.float64

    start_raw, table = kpp_uniforms(n_clusters, n_local_trials, random_state, np_dtype)
    starting_center_id = int(start_raw % n)
    uniforms = torch.from_numpy(table).to(dev) if table.size else torch.zeros(1, dtype=torch.float64, device=dev)

    centers_t = torch.empty((d, n_clusters), dtype=X_t.dtype, device=dev)
    center_indices = torch.full((n_clusters,), -1, dtype=torch.int32, device=dev)
    ws_bytes = lib.kmx_kpp_workspace_bytes(n, d, n_clusters, n_local_trials, dc)
    if ws_bytes == 0:
        raise ValueError(f"kmeans++ does not support n_local_trials={n_local_trials}")
    ws = workspace(ws_bytes, dev)
    check(lib.kmx_kpp_run(ptr(X_t), ptr(sample_weight), ptr(uniforms), starting_center_id, ptr(centers_t),
                          ptr(center_indices), ptr(ws), ws_bytes, n, d, n_clusters, n_local_trials, dc,
                          _capi.KMX_KPP_SAMPLER_LITERAL if sampler == "literal" else _capi.KMX_KPP_SAMPLER_SCAN,
                          _capi.current_stream()), "kmx_kpp_run")
    return centers_t, center_indices
