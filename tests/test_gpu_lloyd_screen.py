"""GPU tests of the fp32 Lloyd step whose labels are screened on the fp16 matrix cores
(kernel variant 61): inputs chosen so that the certification fails for many, all or none of
the samples, exact ties, features of very different scale, offsets far from the origin.
Everything is compared with the CPU oracle (labels: exact except fp64 near-ties; exact ties
must go to the lowest index, as in the reference's running arg-min,
sklearn_numba_dpex/kmeans/kernels/_base_kmeans_kernel_funcs.py:228-267)."""

import ctypes

import numpy as np
import pytest

from oracle import kmeans as ok
from tests._parity import assert_centers_close, assert_labels_match

pytestmark = pytest.mark.gpu


# The library screens the labels only where that is the faster kernel (from about ten features
# on); the tests here want the screened kernel on every shape it can run.
SCREEN = 0x20   # KMX_FLAG_LABELS_SCREEN
ALL_F32 = 0x10  # KMX_FLAG_LABELS_F32
WIDE = 0x3      # KMX_FLAG_PATH_MFMA: the wide path also for the few clusters that are left to the tiled product


def _one_iteration(X, w, init, cuda, flags=SCREEN):
    """kmx_lloyd_init + one kmx_lloyd_iter through the C ABI; returns labels, new centroids
    (or the sums when a cluster is empty), sizes, status, variant, samples evaluated in fp32."""
    import torch

    from sklearn_numba_dpex_amd import _capi
    from sklearn_numba_dpex_amd._capi import lib, ptr

    n, d = X.shape
    k = init.shape[0]
    dev = lambda a: torch.as_tensor(np.ascontiguousarray(a), device=cuda)
    X_t, w_d, c_in = dev(X.T), dev(w), dev(init.T)
    c_out = torch.empty_like(c_in)
    labels_prev = torch.zeros(n, dtype=torch.int32, device=cuda)
    labels = torch.full((n,), -1, dtype=torch.int32, device=cuda)
    sizes = torch.empty(k, dtype=X_t.dtype, device=cuda)
    empty = torch.empty(k, dtype=torch.int32, device=cuda)
    plan = _capi.lloyd_plan(n, d, k, _capi.dtype_code(X.dtype), flags)
    ws_bytes = plan.workspace_bytes
    ws = torch.empty(ws_bytes, dtype=torch.uint8, device=cuda)
    stream = _capi.current_stream()
    variant = plan.variant
    _capi.check(lib.kmx_lloyd_init(plan, ptr(ws), ws_bytes, ptr(X_t), ptr(w_d), ptr(c_in), 10, 0.0, stream), "init")
    X_rm = dev(X) if variant in (42, 63) else None  # the wide path sums (and screens) with a row-major copy
    _capi.check(lib.kmx_lloyd_iter(plan, ptr(X_t), ptr(X_rm), ptr(w_d), ptr(c_in), ptr(c_out), ptr(labels_prev),
                                   ptr(labels), ptr(sizes), ptr(empty), ptr(ws), ws_bytes, stream), "iter")
    status = _capi.LloydStatus()
    _capi.check(lib.kmx_lloyd_status_read(ptr(ws), status, stream), "status")
    rechecked = ctypes.c_uint32(0)
    _capi.check(lib.kmx_lloyd_recheck_count(plan, ptr(ws), ctypes.byref(rechecked), stream), "recheck")
    return (labels.cpu().numpy().astype(np.int64), c_out.cpu().numpy().T, sizes.cpu().numpy(), status, variant,
            int(rechecked.value))


def _check_against_oracle(X, w, init, labels, c_out, sizes, status):
    k = init.shape[0]
    assert labels.min() >= 0 and labels.max() < k
    assert_labels_match(labels, ok.assign_labels(X, init), X, init)
    sums, ref_sizes = ok.weighted_sums(X, w, labels, k)
    np.testing.assert_allclose(sizes, ref_sizes, rtol=1e-5 if X.dtype == np.float32 else 1e-12)
    assert status.n_empty == int(np.count_nonzero(ref_sizes == 0))
    if status.n_empty == 0:
        assert_centers_close(c_out, sums / ref_sizes[:, None], X.dtype)
    else:
        assert_centers_close(c_out, sums, X.dtype)


def _blobs(n, d, k, seed, offset=0.0, scale=1.0):
    rng = np.random.default_rng(seed)
    centers = rng.uniform(-10, 10, (k, d))
    X = ((centers[rng.integers(0, k, n)] + rng.standard_normal((n, d))) * scale + offset).astype(np.float32)
    init = X[rng.choice(n, k, replace=False)].copy()
    w = rng.uniform(0.5, 1.5, n).astype(np.float32)
    return X, w, init


@pytest.mark.parametrize("shape", [(20_000, 14, 127), (10_003, 9, 45), (4_096, 16, 16), (3_001, 17, 40),
                                   (5_000, 32, 64), (777, 1, 20), (2_000, 2, 33), (64, 31, 16),
                                   # more than 64 KB of LDS per workgroup
                                   (20_000, 16, 512), (9_000, 14, 600), (6_000, 8, 512), (5_000, 32, 128),
                                   # three and four K steps (eight waves, the whole LDS of a compute unit)
                                   (6_000, 33, 16), (6_000, 48, 64), (5_003, 64, 64), (6_000, 40, 127),
                                   (6_000, 64, 120), (7_001, 63, 20), (6_000, 33, 200),
                                   # 17 to 32 features that need more than half the LDS of a compute unit: the
                                   # three-step kernel (one workgroup, all of the LDS) with an empty third step
                                   (9_000, 20, 300), (8_000, 32, 256), (6_001, 17, 280)])
def test_screened_step_matches_oracle(cuda, shape):
    n, d, k = shape
    X, w, init = _blobs(n, d, k, seed=n + d)
    labels, c_out, sizes, status, variant, rechecked = _one_iteration(X, w, init, cuda)
    assert variant == 61
    _check_against_oracle(X, w, init, labels, c_out, sizes, status)
    # on blob data only a small fraction of the labels needs the fp32 evaluation
    assert rechecked <= 8 + n // 20


def _labels_only(X, C, cuda, roomy=True, flags=SCREEN):
    """kmx_assign_labels through the C ABI (the screened label kernels; with roomy=False the
    minimal workspace, with which wide shapes take the all-fp32 kernel)."""
    import torch

    from sklearn_numba_dpex_amd import _capi
    from sklearn_numba_dpex_amd._capi import lib, ptr

    n, d = X.shape
    k = C.shape[0]
    X_t = torch.as_tensor(np.ascontiguousarray(X.T), device=cuda)
    c_t = torch.as_tensor(np.ascontiguousarray(C.T), device=cuda)
    labels = torch.full((n,), -1, dtype=torch.int32, device=cuda)
    ws_bytes = (lib.kmx_assign_workspace_bytes_for(n, d, k, 0, flags) if roomy
                else lib.kmx_assign_workspace_bytes(d, k, 0))
    ws = torch.empty(max(ws_bytes, 16), dtype=torch.uint8, device=cuda)
    _capi.check(lib.kmx_assign_labels(ptr(X_t), ptr(c_t), ptr(labels), ptr(ws), ws_bytes, n, d, k, 0, flags,
                                      _capi.current_stream()), "assign")
    return labels.cpu().numpy().astype(np.int64)


@pytest.mark.parametrize("shape", [(20_000, 14, 127), (10_003, 9, 45), (4_096, 16, 16), (3_001, 17, 40),
                                   (5_000, 32, 64), (777, 1, 20), (2_000, 2, 33), (64, 31, 16),
                                   (20_000, 16, 512), (9_000, 14, 600), (5_000, 32, 128),
                                   (6_000, 33, 16), (6_000, 48, 64), (5_003, 64, 64), (6_000, 40, 127),
                                   (6_000, 64, 120), (7_001, 63, 20),
                                   (9_000, 20, 300), (8_000, 32, 256), (9_000, 24, 440)])
def test_screened_labels_only_match_oracle(cuda, shape):
    n, d, k = shape
    X, _, init = _blobs(n, d, k, seed=n + d + 1)
    labels = _labels_only(X, init, cuda)
    assert labels.min() >= 0 and labels.max() < k
    assert_labels_match(labels, ok.assign_labels(X, init), X, init)


@pytest.mark.parametrize("factor", [1e-6, 0.3, 7.0, 300.0, 1e6])
def test_labels_only_with_samples_of_another_magnitude_than_the_centroids(cuda, factor):
    """The labels-only kernel takes its scale from the centroids: samples far larger overflow
    fp16 (and must then be evaluated in fp32), samples far smaller lose all their bits; the
    labels must be the oracle's either way."""
    rng = np.random.default_rng(31)
    n, d, k = 6_000, 14, 40
    C = rng.uniform(-4, 4, (k, d)).astype(np.float32)
    X = (rng.uniform(-4, 4, (n, d)) * factor).astype(np.float32)
    labels = _labels_only(X, C, cuda)
    assert_labels_match(labels, ok.assign_labels(X, C), X, C)


def test_labels_only_ties_and_zero_centroids(cuda):
    rng = np.random.default_rng(37)
    n, d, k = 5_000, 8, 24
    X = rng.standard_normal((n, d)).astype(np.float32)
    C = rng.standard_normal((k, d)).astype(np.float32)
    C[5] = C[2]                                    # duplicates: the lower index wins
    C[9] = C[2]
    labels = _labels_only(X, C, cuda)
    ref = ok.assign_labels(X, C)
    assert not np.any(labels == 5) and not np.any(labels == 9)
    assert_labels_match(labels, ref, X, C)
    zeros = _labels_only(X, np.zeros((k, d), dtype=np.float32), cuda)
    assert np.all(zeros == 0)


def test_default_choice_between_screened_and_fp32_step(cuda):
    """With flags = 0 the screen is used where it is the faster kernel."""
    from sklearn_numba_dpex_amd._capi import lib

    for (d, k), variant in {(14, 127): 61, (2, 16): 31, (8, 32): 31, (8, 64): 61, (6, 128): 61, (32, 64): 61}.items():
        assert lib.kmx_lloyd_kernel_variant(100_000, d, k, 0, 0) == variant, (d, k)
    X, w, init = _blobs(5_000, 4, 20, seed=11)
    labels, c_out, sizes, status, variant, rechecked = _one_iteration(X, w, init, cuda, flags=0)
    assert variant == 31 and rechecked == 0
    _check_against_oracle(X, w, init, labels, c_out, sizes, status)


def test_fp32_matrix_core_step_selected_by_flag(cuda):
    """KMX_FLAG_LABELS_F32 selects the all-fp32 kernel (variant 31); both give the oracle's labels."""
    X, w, init = _blobs(30_000, 14, 127, seed=5)
    got = {}
    for mode in ("screen", "f32"):
        labels, c_out, sizes, status, variant, rechecked = _one_iteration(
            X, w, init, cuda, flags=SCREEN if mode == "screen" else ALL_F32)
        assert variant == (61 if mode == "screen" else 31)
        if mode == "f32":
            assert rechecked == 0
        _check_against_oracle(X, w, init, labels, c_out, sizes, status)
        got[mode] = labels
    # the two kernels may only differ at fp64 near-ties
    assert_labels_match(got["screen"], got["f32"], X, init)


@pytest.mark.parametrize("d", [14, 24, 40, 64])
def test_duplicate_centroids_take_the_lowest_index(cuda, d):
    """Two pairs of identical centroids: exact ties, none of them certifiable; the reference's
    strict '<' in increasing centroid order keeps the lower index.  Whole 32-sample columns are
    redone in fp32 here, with one to four K steps of 16 features."""
    X, w, init = _blobs(20_000, d, 64, seed=21)
    init[40] = init[3]
    init[63] = init[17]
    labels, c_out, sizes, status, variant, rechecked = _one_iteration(X, w, init, cuda)
    assert variant == 61
    assert not np.any(labels == 40) and not np.any(labels == 63)
    ref = ok.assign_labels(X, init)
    assert_labels_match(labels, ref, X, init)
    # every sample of the duplicated clusters went through the fp32 evaluation
    assert rechecked >= int(np.count_nonzero((ref == 3) | (ref == 17)))
    assert status.n_empty == 2 and status.state == 4


@pytest.mark.parametrize("d", [14, 30, 48, 57])
def test_all_centroids_identical(cuda, d):
    """No sample can be certified: every label comes from the fp32 evaluation and is 0."""
    X, w, init = _blobs(5_000, d, 16, seed=22)
    init[:] = init[0]
    labels, c_out, sizes, status, variant, rechecked = _one_iteration(X, w, init, cuda)
    assert variant == 61
    assert np.all(labels == 0)
    assert rechecked == X.shape[0]
    assert status.n_empty == 15


def test_samples_on_the_bisector(cuda):
    """Samples at exactly the same fp32 distance from two centroids (mirror images in the
    first coordinate): the lower index wins; the other samples follow the oracle."""
    rng = np.random.default_rng(23)
    n, d, k = 8_192, 14, 32
    init = rng.uniform(-4, 4, (k, d)).astype(np.float32)
    init[1] = init[0]
    init[1, 0] = -init[0, 0]                       # centroid 1 mirrors centroid 0
    X = (init[rng.integers(0, k, n)] + 0.3 * rng.standard_normal((n, d))).astype(np.float32)
    on = np.arange(0, n, 7)
    X[on] = init[0] + 0.05 * rng.standard_normal((on.size, d)).astype(np.float32)
    X[on, 0] = 0.0                                 # on the bisector of centroids 0 and 1
    w = np.ones(n, dtype=np.float32)
    labels, c_out, sizes, status, variant, rechecked = _one_iteration(X, w, init, cuda)
    assert variant == 61
    ref = ok.assign_labels(X, init)
    assert np.all(ref[on] <= 1)
    assert np.all(labels[on] == 0)
    assert_labels_match(labels, ref, X, init)
    assert rechecked >= on.size


def test_more_uncertain_samples_than_the_queue_holds(cuda):
    """Two samples of every 32-sample column lie on the bisector of centroids 0 and 1: too few
    for the column to be redone as a whole, so they go to the workgroup's queue, and with
    512 of them per workgroup the queue (256 entries at most) overflows.  Labels, weighted sums
    and sizes must come out the same whichever route a sample took."""
    rng = np.random.default_rng(29)
    n, d, k = 1 << 21, 4, 16
    init = rng.uniform(-4, 4, (k, d)).astype(np.float32)
    init[1] = init[0]
    init[1, 0] = -init[0, 0]
    X = (init[rng.integers(0, k, n)] + 0.3 * rng.standard_normal((n, d))).astype(np.float32)
    on = np.arange(0, n, 16)
    X[on] = init[0] + 0.05 * rng.standard_normal((on.size, d)).astype(np.float32)
    X[on, 0] = 0.0
    w = rng.uniform(0.5, 1.5, n).astype(np.float32)
    labels, c_out, sizes, status, variant, rechecked = _one_iteration(X, w, init, cuda)
    assert variant == 61
    assert np.all(labels[on] == 0)
    assert rechecked >= on.size
    _check_against_oracle(X, w, init, labels, c_out, sizes, status)


def test_features_of_very_different_scale(cuda):
    """One feature 1e6 times larger than the one that separates the clusters: the fp16 parts
    of the small feature are far below those of the large one."""
    rng = np.random.default_rng(24)
    n, d, k = 20_000, 6, 24
    centers = rng.uniform(-1, 1, (k, d))
    X = centers[rng.integers(0, k, n)] + 0.05 * rng.standard_normal((n, d))
    scales = np.array([1e3, 1e-3, 1.0, 30.0, 1e-2, 5.0])
    X = (X * scales).astype(np.float32)
    init = X[rng.choice(n, k, replace=False)].copy()
    w = rng.uniform(0.5, 1.5, n).astype(np.float32)
    labels, c_out, sizes, status, variant, rechecked = _one_iteration(X, w, init, cuda)
    assert variant == 61
    _check_against_oracle(X, w, init, labels, c_out, sizes, status)


@pytest.mark.parametrize("offset,scale", [(1000.0, 1.0), (-3.0e4, 10.0), (0.0, 1e-12), (0.0, 1e12)])
def test_offsets_and_extreme_magnitudes(cuda, offset, scale):
    """Data far from the origin (the gaps between scores are tiny next to ||x|| ||c||, so many
    samples need the fp32 evaluation) and data near the ends of the fp32 range."""
    X, w, init = _blobs(10_000, 8, 20, seed=25, offset=offset, scale=scale)
    labels, c_out, sizes, status, variant, rechecked = _one_iteration(X, w, init, cuda)
    assert variant == 61
    k = init.shape[0]
    assert labels.min() >= 0 and labels.max() < k
    # fp32 itself cannot separate clusters whose distance differences drown in ||x||^2: the
    # oracle evaluates the same fp32 formula, and labels may differ where fp64 says near-tie
    ref = ok.assign_labels(X, init)
    dist_scale = 1.0
    if offset != 0.0:
        # accept the labels the fp32 formula can justify: compare through fp64 distances with
        # the fp32 resolution of 0.5||c||^2 - <x, c> as tolerance
        X64, C64 = X.astype(np.float64), init.astype(np.float64)
        dd = ((X64[:, None, :] - C64[None, :, :]) ** 2).sum(axis=2)
        got_d = dd[np.arange(len(labels)), labels]
        best_d = dd.min(axis=1)
        resolution = 64 * np.finfo(np.float32).eps * (np.abs(X64).max() ** 2) * X.shape[1]
        assert np.all(got_d - best_d <= resolution * dist_scale)
    else:
        assert_labels_match(labels, ref, X, init)
    sums, ref_sizes = ok.weighted_sums(X, w, labels, k)
    np.testing.assert_allclose(sizes, ref_sizes, rtol=1e-5)


def test_all_zero_data(cuda):
    X = np.zeros((4_096, 14), dtype=np.float32)
    w = np.ones(4_096, dtype=np.float32)
    init = np.zeros((16, 14), dtype=np.float32)
    labels, c_out, sizes, status, variant, rechecked = _one_iteration(X, w, init, cuda)
    assert variant == 61
    assert np.all(labels == 0)
    assert sizes[0] == 4_096 and status.n_empty == 15


@pytest.mark.parametrize("shape,iterations", [((50_000, 14, 127), 10), ((60_000, 9, 45), 25),
                                              # accumulators and operands fill the LDS: no room for the list of
                                              # samples that change cluster, little for the queue
                                              ((20_000, 16, 512), 15), ((30_000, 14, 600), 15),
                                              # three and four K steps
                                              ((30_000, 40, 127), 15), ((30_000, 64, 100), 15),
                                              # two K steps' worth of features on the three-step kernel
                                              ((30_000, 20, 300), 15), ((30_000, 32, 256), 12)])
def test_iterations_stay_in_lockstep_with_the_oracle(cuda, shape, iterations):
    """Iterations through the driver-level loop of the C ABI; every iteration is compared from
    the centroids the GPU started it with - labels against the oracle's, centroids against the
    weighted means of the labels the GPU wrote, whichever way the step brought its sums up to
    date (rebuilt, corrected tile by tile, corrected from the list) - and the count of fp32
    evaluations stays small."""
    import torch

    from sklearn_numba_dpex_amd import _capi
    from sklearn_numba_dpex_amd._capi import lib, ptr

    X, w, init = _blobs(*shape, seed=26)
    if shape[1] > 16:
        # overlapping blobs: no cluster runs empty and the labels keep moving for many iterations
        rng = np.random.default_rng(26)
        n_, d_, k_ = shape
        X = (rng.uniform(-1.5, 1.5, (k_, d_))[rng.integers(0, k_, n_)] + rng.standard_normal((n_, d_))).astype(np.float32)
        init = X[rng.choice(n_, k_, replace=False)].copy()
    n, d = X.shape
    k = init.shape[0]
    dev = lambda a: torch.as_tensor(np.ascontiguousarray(a), device=cuda)
    X_t, w_d = dev(X.T), dev(w)
    cent = [dev(init.T), torch.empty(d, k, dtype=torch.float32, device=cuda)]
    labels = [torch.zeros(n, dtype=torch.int32, device=cuda) for _ in range(2)]
    sizes = torch.empty(k, dtype=torch.float32, device=cuda)
    empty = torch.empty(k, dtype=torch.int32, device=cuda)
    plan = _capi.lloyd_plan(n, d, k, 0, SCREEN)
    ws_bytes = plan.workspace_bytes
    ws = torch.empty(ws_bytes, dtype=torch.uint8, device=cuda)
    stream = _capi.current_stream()
    assert plan.variant == 61
    _capi.check(lib.kmx_lloyd_init(plan, ptr(ws), ws_bytes, ptr(X_t), ptr(w_d), ptr(cent[0]), 100, 0.0, stream), "init")
    status = _capi.LloydStatus()
    rechecked = ctypes.c_uint32(0)
    for it in range(iterations):
        a, b = it % 2, (it + 1) % 2
        c_in = cent[a].cpu().numpy().T.copy()
        _capi.check(lib.kmx_lloyd_iter(plan, ptr(X_t), None, ptr(w_d), ptr(cent[a]), ptr(cent[b]), ptr(labels[a]),
                                       ptr(labels[b]), ptr(sizes), ptr(empty), ptr(ws), ws_bytes, stream), "iter")
        _capi.check(lib.kmx_lloyd_status_read(ptr(ws), status, stream), "status")
        _capi.check(lib.kmx_lloyd_recheck_count(plan, ptr(ws), ctypes.byref(rechecked), stream), "recheck")
        got = labels[b].cpu().numpy().astype(np.int64)
        assert_labels_match(got, ok.assign_labels(X, c_in), X, c_in)
        assert rechecked.value <= n // 50
        if status.n_empty or status.state != _capi.KMX_RUNNING:
            break
        sums, ref_sizes = ok.weighted_sums(X, w, got, k)
        assert_centers_close(cent[b].cpu().numpy().T, sums / ref_sizes[:, None], np.float32)
        assert status.n_iter == it + 1


@pytest.mark.parametrize("shape,direct", [((20_000, 4, 1_100), True),     # few sums: finished by one workgroup
                                          ((30_000, 14, 700), True),
                                          ((9_001, 8, 1_024), True),
                                          ((20_000, 64, 256), True),
                                          ((12_345, 48, 300), True),
                                          ((40_000, 16, 1_140), False)])  # accumulators beyond the LDS: sums per bucket
def test_screened_labels_with_separate_sums_run_to_convergence(cuda, shape, direct):
    """Shapes whose operands fit the screened kernel but whose accumulators do not fit beside them:
    labels by the screened kernel, sums by a kernel of their own (every cluster's fixed-point
    accumulators in LDS where they fit, else per bucket of samples).  Uneven weights with zeros
    among them; every iteration is compared with the oracle from the centroids it started with,
    and the run must stop exactly when an iteration changes no label (60 iterations at most)."""
    import torch

    from sklearn_numba_dpex_amd import _capi
    from sklearn_numba_dpex_amd._capi import lib, ptr

    n, d, k = shape
    rng = np.random.default_rng(n + d + k)
    # (wide samples: blobs that overlap, or the second iteration already changes nothing)
    noise = 0.3 if d <= 16 else 1.0
    X = (rng.uniform(-2, 2, (k, d))[rng.integers(0, k, n)] + noise * rng.standard_normal((n, d))).astype(np.float32)
    w = rng.uniform(0.5, 2.0, n).astype(np.float32)
    w[rng.integers(0, n, n // 50)] = 0.0
    chosen = rng.choice(n, k, replace=False)
    w[chosen] = 1.0  # (a cluster of one sample of weight zero would be empty at once)
    init = X[chosen].copy()
    dev = lambda a: torch.as_tensor(np.ascontiguousarray(a), device=cuda)
    X_t, w_d = dev(X.T), dev(w)
    cent = [dev(init.T), torch.empty(d, k, dtype=torch.float32, device=cuda)]
    labels = [torch.full((n,), k, dtype=torch.int32, device=cuda) for _ in range(2)]
    sizes = torch.empty(k, dtype=torch.float32, device=cuda)
    empty = torch.empty(k, dtype=torch.int32, device=cuda)
    plan = _capi.lloyd_plan(n, d, k, 0, 0)
    assert plan.variant == 63
    ws_bytes = plan.workspace_bytes
    ws = torch.empty(ws_bytes, dtype=torch.uint8, device=cuda)
    stream = _capi.current_stream()
    _capi.check(lib.kmx_lloyd_init(plan, ptr(ws), ws_bytes, ptr(X_t), ptr(w_d), ptr(cent[0]), 200, 0.0, stream), "init")
    status = _capi.LloydStatus()
    previous = None
    for it in range(60):
        a, b = it % 2, (it + 1) % 2
        c_in = cent[a].cpu().numpy().T.copy()
        _capi.check(lib.kmx_lloyd_iter(plan, ptr(X_t), None, ptr(w_d), ptr(cent[a]), ptr(cent[b]), ptr(labels[a]),
                                       ptr(labels[b]), ptr(sizes), ptr(empty), ptr(ws), ws_bytes, stream), "iter")
        _capi.check(lib.kmx_lloyd_status_read(ptr(ws), status, stream), "status")
        got = labels[b].cpu().numpy().astype(np.int64)
        assert_labels_match(got, ok.assign_labels(X, c_in), X, c_in)
        sums, ref_sizes = ok.weighted_sums(X, w, got, k)
        np.testing.assert_allclose(sizes.cpu().numpy(), ref_sizes, rtol=1e-5)
        if status.n_empty:
            assert status.state == _capi.KMX_NEED_RELOCATION
            break
        assert_centers_close(cent[b].cpu().numpy().T, sums / ref_sizes[:, None], np.float32)
        assert status.n_iter == it + 1
        if previous is not None and np.array_equal(got, previous):
            assert status.state == _capi.KMX_CONVERGED_STRICT
            break
        assert status.state == _capi.KMX_RUNNING, (it, status.state)
        previous = got
    assert it >= 1, (it, status.state, status.n_empty)


def _screen_scores(X, C, cuda):
    import torch

    from sklearn_numba_dpex_amd import _capi
    from sklearn_numba_dpex_amd._capi import lib, ptr

    n, d = X.shape
    k = C.shape[0]
    dev = lambda a: torch.as_tensor(np.ascontiguousarray(a), device=cuda)
    X_t, C_t = dev(X.T), dev(C.T)
    scores = torch.empty(k, n, dtype=torch.float32, device=cuda)
    bounds = torch.empty(n, dtype=torch.float32, device=cuda)
    half = torch.empty(k, dtype=torch.float32, device=cuda)
    scale = torch.empty(1, dtype=torch.float32, device=cuda)
    scratch = torch.zeros(64, dtype=torch.int32, device=cuda)
    _capi.check(lib.kmx_screen_scores(ptr(X_t), ptr(C_t), ptr(scores), ptr(bounds), ptr(half), ptr(scale),
                                      ptr(scratch), n, d, k, _capi.current_stream()), "screen_scores")
    torch.cuda.synchronize()
    return scores.cpu().numpy(), bounds.cpu().numpy(), half.cpu().numpy(), float(scale.cpu().numpy()[0])


def _screen_cases():
    rng = np.random.default_rng(31)
    cases = {}
    X, _, C = _blobs(4_000, 14, 127, seed=32)
    cases["blobs d=14 k=127"] = (X, C)
    X, _, C = _blobs(3_000, 32, 64, seed=33)
    cases["blobs d=32 k=64"] = (X, C)
    # centroids are samples: <x, c> - 0.5||c||^2 cancels to 0.5||x||^2 - 0.5||x - c||^2
    X = rng.standard_normal((2_048, 16)).astype(np.float32) * 3 + 50
    cases["offset 50, centroids = samples"] = (X, X[:64].copy())
    # every mantissa bit in use, alternating signs, wide range of magnitudes inside a row
    X = (rng.uniform(1, 2, (2_048, 31)) * rng.choice([-1, 1], (2_048, 31)) *
         np.exp2(rng.integers(-12, 12, (2_048, 31)))).astype(np.float32)
    C = (rng.uniform(1, 2, (48, 31)) * rng.choice([-1, 1], (48, 31)) *
         np.exp2(rng.integers(-12, 12, (48, 31)))).astype(np.float32)
    cases["random exponents d=31"] = (X, C)
    # one feature only, tiny and huge data
    cases["d=1"] = (rng.standard_normal((1_000, 1)).astype(np.float32), rng.standard_normal((16, 1)).astype(np.float32))
    cases["tiny values"] = ((rng.standard_normal((1_000, 8)) * 1e-18).astype(np.float32),
                            (rng.standard_normal((20, 8)) * 1e-18).astype(np.float32))
    cases["huge values"] = ((rng.standard_normal((1_000, 8)) * 1e16).astype(np.float32),
                            (rng.standard_normal((20, 8)) * 1e16).astype(np.float32))
    # the wide path's shapes: 16 K steps, centroids = samples (maximal cancellation), and noise
    X = (rng.standard_normal((1_024, 256)) * 2 + rng.standard_normal(256) * 5).astype(np.float32)
    cases["d=256, centroids = samples"] = (X, X[:32].copy())
    cases["d=200 random"] = (rng.standard_normal((1_024, 200)).astype(np.float32) * 7,
                             rng.standard_normal((32, 200)).astype(np.float32) * 7)
    cases["d=70"] = (rng.standard_normal((1_024, 70)).astype(np.float32), rng.standard_normal((64, 70)).astype(np.float32))
    # three and four K steps of the narrow kernel
    X, _, C = _blobs(3_000, 48, 64, seed=34)
    cases["blobs d=48 k=64"] = (X, C)
    X = (rng.standard_normal((2_048, 64)) * 2 + rng.standard_normal(64) * 5).astype(np.float32)
    cases["d=64, centroids = samples"] = (X, X[:48].copy())
    return cases


@pytest.mark.parametrize("name", list(_screen_cases().keys()))
def test_error_bound_of_the_screen_holds_on_the_hardware(cuda, name):
    """The certificate of variant 61 rests on |approximate score - exact score| <= E(x).  The
    scores the matrix cores really produce are compared with fp64 here (the bound assumes at
    most one ulp of error per accumulation inside an MFMA, which no document guarantees)."""
    X, C = _screen_cases()[name]
    scores, bounds, half, scale = _screen_scores(X, C, cuda)
    assert np.log2(scale) == np.round(np.log2(scale))            # a power of two
    # the fused step of narrow shapes keeps its scaled data below 2^13 (so that -0.5||c||^2 over
    # 2^15 fits fp16 in the spare feature slot), the wide path's label kernel below 2^15
    top = 13 if X.shape[1] <= 32 else 15
    assert 2.0 ** (top - 1) <= np.abs(X).max() * scale < 2.0 ** top
    Xs, Cs = X.astype(np.float64) * scale, C.astype(np.float64) * scale
    np.testing.assert_allclose(half, 0.5 * (Cs ** 2).sum(axis=1), rtol=1e-5)
    exact = Cs @ Xs.T - half.astype(np.float64)[:, None]           # from the fp32 half norms the step uses
    err = np.abs(scores.astype(np.float64) - exact)
    assert np.all(np.isfinite(scores))
    ratio = (err / bounds[None, :].astype(np.float64)).max()
    print(f"{name}: largest error / bound = {ratio:.3f}")
    assert ratio <= 1.0
    # and the bound is not vacuous: far below the typical score
    typical = np.median(np.abs(exact))
    assert np.median(bounds) <= 1e-3 * max(typical, np.abs(exact).max() * 1e-3)


@pytest.mark.parametrize("shape", [(60_000, 14, 127), (30_001, 9, 45), (40_000, 16, 64), (60_000, 20, 60),
                                   (40_000, 48, 40), (40_000, 64, 30)])
def test_sums_corrected_for_label_changes_equal_rebuilt_sums(cuda, shape):
    """Once few labels change per iteration the screened step no longer rebuilds the fixed-point
    sums but takes every sample that changes cluster off its old cluster and adds it to the new
    one.  Integer sums make that exact: run next to the all-fp32 step (variant 31, which rebuilds
    its sums every iteration) from the same centroids, an iteration whose labels agree must give
    bit-identical centroids and sizes, however many iterations the correction has been running."""
    import torch

    from sklearn_numba_dpex_amd import _capi
    from sklearn_numba_dpex_amd._capi import lib, ptr

    n, d, k = shape
    X, w, init = _blobs(n, d, k, seed=n + d + 7)
    if d > 16:
        # overlapping blobs: no cluster runs empty and the labels keep moving for many iterations
        rng = np.random.default_rng(n + d)
        X = (rng.uniform(-1.5, 1.5, (k, d))[rng.integers(0, k, n)] + rng.standard_normal((n, d))).astype(np.float32)
        init = X[rng.choice(n, k, replace=False)].copy()
    dev = lambda a: torch.as_tensor(np.ascontiguousarray(a), device=cuda)
    X_t, w_d = dev(X.T), dev(w)
    stream = _capi.current_stream()
    runs = {}
    for name, flags in (("screen", SCREEN), ("f32", ALL_F32)):
        plan = _capi.lloyd_plan(n, d, k, 0, flags)
        assert plan.variant == (61 if name == "screen" else 31)
        ws = torch.empty(plan.workspace_bytes, dtype=torch.uint8, device=cuda)
        runs[name] = dict(plan=plan, ws=ws, cent=[dev(init.T), torch.empty(d, k, dtype=torch.float32, device=cuda)],
                          labels=[torch.zeros(n, dtype=torch.int32, device=cuda) for _ in range(2)],
                          sizes=torch.empty(k, dtype=torch.float32, device=cuda),
                          empty=torch.empty(k, dtype=torch.int32, device=cuda), status=_capi.LloydStatus())
        _capi.check(lib.kmx_lloyd_init(plan, ptr(ws), plan.workspace_bytes, ptr(X_t), ptr(w_d), ptr(runs[name]["cent"][0]),
                                       200, 0.0, stream), "init")
    corrected = identical = 0
    for it in range(60):
        a, b = it % 2, (it + 1) % 2
        # both runs start every iteration from the screened run's centroids (the all-fp32 run's
        # packed copy is refreshed by giving it the same array to finalise into next time)
        for name, r in runs.items():
            _capi.check(lib.kmx_lloyd_iter(r["plan"], ptr(X_t), None, ptr(w_d), ptr(r["cent"][a]), ptr(r["cent"][b]),
                                           ptr(r["labels"][a]), ptr(r["labels"][b]), ptr(r["sizes"]), ptr(r["empty"]),
                                           ptr(r["ws"]), r["plan"].workspace_bytes, stream), "iter")
            _capi.check(lib.kmx_lloyd_status_read(ptr(r["ws"]), r["status"], stream), "status")
        s61, s31 = runs["screen"]["status"], runs["f32"]["status"]
        if s61.state != _capi.KMX_RUNNING or s31.state != _capi.KMX_RUNNING:
            break
        lab61 = runs["screen"]["labels"][b].cpu().numpy()
        lab31 = runs["f32"]["labels"][b].cpu().numpy()
        c61 = runs["screen"]["cent"][b].cpu().numpy()
        c31 = runs["f32"]["cent"][b].cpu().numpy()
        if it >= 1 and s61.reserved[1] * 64 <= n:
            corrected += 1   # the NEXT iteration of the screened run corrects its sums
        if np.array_equal(lab61, lab31):
            identical += 1
            np.testing.assert_array_equal(c61, c31)
            np.testing.assert_array_equal(runs["screen"]["sizes"].cpu().numpy(), runs["f32"]["sizes"].cpu().numpy())
        else:
            # a near-tie went the other way in one of the two kernels: the trajectories part here
            assert_labels_match(lab61, lab31, X, runs["screen"]["cent"][a].cpu().numpy().T)
            break
        # and against the oracle's sums for these labels
        sums, ref_sizes = ok.weighted_sums(X, w, lab61.astype(np.int64), k)
        if np.all(ref_sizes > 0):
            assert_centers_close(c61.T, sums / ref_sizes[:, None], np.float32)
    print(f"{shape}: {identical} iterations with identical labels, {corrected} of them after few label changes")
    assert identical >= 8
    assert corrected >= 3, "the data were meant to reach the regime in which sums are corrected"


@pytest.mark.parametrize("shape", [(6_000, 128, 64), (3_000, 256, 200), (4_097, 40, 400), (2_500, 70, 1024),
                                   (3_001, 67, 300), (2_000, 33, 300), (1_500, 255, 96)])
def test_wide_screened_step_matches_oracle(cuda, shape):
    """The wide fp32 path (variant 42) screens its labels the same way; what it cannot certify
    goes through the all-fp32 matrix-core kernel."""
    n, d, k = shape
    X, w, init = _blobs(n, d, k, seed=n + d)
    labels, c_out, sizes, status, variant, rechecked = _one_iteration(X, w, init, cuda, flags=SCREEN | WIDE)
    assert variant == 42
    _check_against_oracle(X, w, init, labels, c_out, sizes, status)
    assert rechecked <= 8 + n // 10


@pytest.mark.parametrize("shape", [(6_000, 128, 64), (3_000, 256, 200), (4_097, 40, 400), (2_500, 70, 1024),
                                   (3_001, 67, 300), (1_500, 255, 96)])
def test_wide_screened_labels_only_match_oracle(cuda, shape):
    """kmx_assign_labels for wide shapes: screened in fp16 when the workspace has room for the list
    of uncertified samples (kmx_assign_workspace_bytes_for), all fp32 with the minimal workspace;
    both must give the oracle's labels."""
    from sklearn_numba_dpex_amd._capi import lib

    n, d, k = shape
    X, _, init = _blobs(n, d, k, seed=n + d + 2)
    assert lib.kmx_assign_workspace_bytes_for(n, d, k, 0, SCREEN | WIDE) > lib.kmx_assign_workspace_bytes(d, k, 0)
    ref = ok.assign_labels(X, init)
    for roomy in (True, False):
        labels = _labels_only(X, init, cuda, roomy=roomy, flags=SCREEN | WIDE)
        assert labels.min() >= 0 and labels.max() < k
        assert_labels_match(labels, ref, X, init)


def test_wide_labels_only_with_samples_far_from_the_centroids(cuda):
    """Scale taken from the centroids: samples a thousand times larger overflow fp16, are all
    listed and evaluated in fp32; duplicated centroids give the lowest index."""
    rng = np.random.default_rng(41)
    n, d, k = 3_000, 96, 128
    C = rng.standard_normal((k, d)).astype(np.float32)
    C[7] = C[3]
    X = (1000.0 * rng.standard_normal((n, d))).astype(np.float32)
    labels = _labels_only(X, C, cuda, flags=SCREEN | WIDE)
    assert not np.any(labels == 7)
    assert_labels_match(labels, ok.assign_labels(X, C), X, C)


def test_wide_duplicate_centroids_take_the_lowest_index(cuda):
    X, w, init = _blobs(8_000, 128, 96, seed=41)
    init[70] = init[5]
    init[95] = init[64]
    labels, c_out, sizes, status, variant, rechecked = _one_iteration(X, w, init, cuda, flags=SCREEN | WIDE)
    assert variant == 42
    assert not np.any(labels == 70) and not np.any(labels == 95)
    ref = ok.assign_labels(X, init)
    assert_labels_match(labels, ref, X, init)
    assert rechecked >= int(np.count_nonzero((ref == 5) | (ref == 64)))
    assert status.n_empty == 2


def test_wide_all_centroids_identical(cuda):
    X, w, init = _blobs(3_000, 96, 64, seed=42)
    init[:] = init[0]
    labels, c_out, sizes, status, variant, rechecked = _one_iteration(X, w, init, cuda, flags=SCREEN | WIDE)
    assert variant == 42
    assert np.all(labels == 0)
    assert rechecked == X.shape[0]
    assert status.n_empty == 63


def test_wide_screen_switched_off_by_flag(cuda):
    X, w, init = _blobs(5_000, 128, 64, seed=43)
    labels, c_out, sizes, status, variant, rechecked = _one_iteration(X, w, init, cuda, flags=ALL_F32 | WIDE)
    assert variant == 42 and rechecked == 0
    _check_against_oracle(X, w, init, labels, c_out, sizes, status)


def test_many_ties_stay_affordable(cuda):
    """Columns with several uncertifiable samples are redone on the fp32 matrix cores: with every
    sample of a large input failing the screen, an iteration must stay within a small multiple
    of the usual time (the per-sample route alone would take tens of times longer)."""
    import time

    import torch

    from sklearn_numba_dpex_amd import _capi
    from sklearn_numba_dpex_amd._capi import lib, ptr

    n, d, k = 1_000_000, 14, 127
    X_t = torch.randn(d, n, device=cuda)
    w = torch.ones(n, device=cuda)

    def one_iteration_ms(c_in):
        c_out = torch.empty_like(c_in)
        lab0 = torch.zeros(n, dtype=torch.int32, device=cuda)
        lab1 = torch.empty(n, dtype=torch.int32, device=cuda)
        sizes = torch.empty(k, device=cuda)
        empty = torch.empty(k, dtype=torch.int32, device=cuda)
        plan = _capi.lloyd_plan(n, d, k, 0, SCREEN)
        wsb = plan.workspace_bytes
        ws = torch.empty(wsb, dtype=torch.uint8, device=cuda)
        st = _capi.current_stream()
        best = 1e9
        for _ in range(3):
            _capi.check(lib.kmx_lloyd_init(plan, ptr(ws), wsb, ptr(X_t), ptr(w), ptr(c_in), 10, 0.0, st), "init")
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            _capi.check(lib.kmx_lloyd_iter(plan, ptr(X_t), None, ptr(w), ptr(c_in), ptr(c_out), ptr(lab0), ptr(lab1),
                                           ptr(sizes), ptr(empty), ptr(ws), wsb, st), "iter")
            torch.cuda.synchronize()
            best = min(best, (time.perf_counter() - t0) * 1e3)
        return best, lab1

    usual, _ = one_iteration_ms(torch.randn(d, k, device=cuda))
    tied, labels = one_iteration_ms(torch.randn(d, 1, device=cuda).repeat(1, k).contiguous())
    assert int(labels.max()) == 0
    print(f"usual {usual:.3f} ms, every sample tied {tied:.3f} ms")
    assert tied < 10 * usual + 0.5


@pytest.mark.parametrize("shape", [(60_001, 14, 127, np.float32), (20_000, 16, 64, np.float32), (9_000, 20, 40, np.float32),
                                   (5_000, 1, 16, np.float32), (70_000, 9, 300, np.float32),
                                   (4_000, 40, 20, np.float32), (3_000, 7, 5, np.float32), (6_000, 12, 30, np.float64),
                                   (9_001, 48, 64, np.float32), (9_000, 64, 100, np.float32)])
@pytest.mark.parametrize("weighted", [True, False])
def test_labels_and_inertia_in_one_call(cuda, shape, weighted):
    """kmx_assign_labels_inertia: the labels of kmx_assign_labels and the inertia of kmx_inertia on
    them, on shapes the screened kernel takes in one pass over X (one and two K steps, odd d, d = 1,
    a ragged last tile, more than 64 KB of LDS) and on shapes that fall back to the two calls (wide,
    tiny k, fp64); samples the screen cannot certify (duplicate centroids) included."""
    import torch

    from sklearn_numba_dpex_amd.kmeans import drivers

    def _dev(a, device):
        return torch.as_tensor(np.ascontiguousarray(a), device=device)

    n, d, k, dtype = shape
    rng = np.random.default_rng(n + d + k)
    centers = rng.normal(size=(k, d)).astype(dtype) * 3
    centers[1] = centers[0]  # every sample of these two clusters is tied: the fp32 route
    X = (centers[rng.integers(0, k, n)] + rng.normal(size=(n, d))).astype(dtype)
    w = rng.uniform(0.5, 2.0, n).astype(dtype) if weighted else None
    X_t, C_t = _dev(X.T, cuda), _dev(centers.T, cuda)
    w_d = _dev(w, cuda) if weighted else None

    labels = torch.empty(n, dtype=torch.int32, device=cuda)
    total = drivers._assign_with_inertia(X_t, w_d, C_t, labels)
    assert total.shape == (1,) and total.dtype == dtype

    ref_labels = torch.empty(n, dtype=torch.int32, device=cuda)
    drivers._assign(X_t, C_t, ref_labels)
    np.testing.assert_array_equal(labels.cpu().numpy(), ref_labels.cpu().numpy())
    two_calls = drivers._inertia_array(X_t, w_d, C_t, ref_labels)
    rtol = 1e-5 if dtype == np.float32 else 1e-12
    np.testing.assert_allclose(total[0], two_calls[0], rtol=rtol)
    got = labels.cpu().numpy().astype(np.int64)
    exact = ((X.astype(np.float64) - centers.astype(np.float64)[got]) ** 2).sum(axis=1)
    exact = float((exact * (w.astype(np.float64) if weighted else 1.0)).sum())
    np.testing.assert_allclose(float(total[0]), exact, rtol=rtol)


@pytest.mark.parametrize("shape", [(4_000, 100, 100), (3_001, 300, 40), (2_000, 784, 130), (5_000, 70, 20)])
def test_tiled_product_screened_on_request(cuda, shape):
    """KMX_FLAG_LABELS_SCREEN on shapes of the tiled matrix-core product: its fp16-screened version
    (the uncertified samples through the listed all-fp32 pass) gives the oracle's labels, through
    kmx_assign_labels with both workspace sizes and through one Lloyd iteration; samples far
    larger than the centroids (labels only: the scale comes from the centroids) overflow fp16
    and are all listed."""
    n, d, k = shape
    X, w, init = _blobs(n, d, k, seed=n + d + 3)
    ref = ok.assign_labels(X, init)
    for roomy in (True, False):
        labels = _labels_only(X, init, cuda, roomy=roomy, flags=SCREEN)
        assert_labels_match(labels, ref, X, init)
    labels, c_out, sizes, status, variant, rechecked = _one_iteration(X, w, init, cuda, flags=SCREEN)
    assert variant == 63 and 0 < rechecked < n // 2
    _check_against_oracle(X, w, init, labels, c_out, sizes, status)
    big = (X * 1000.0).astype(np.float32)
    labels = _labels_only(big, init, cuda, roomy=True, flags=SCREEN)
    assert_labels_match(labels, ok.assign_labels(big, init), big, init)


# ------------------------------------------------------------------------------------------
# fp64 inputs: the same screen on the inputs rounded to fp32 (kernel variant 71); the samples it
# cannot certify are evaluated on the fp64 matrix cores, the sums are taken from the fp64 inputs


def _blobs64(n, d, k, seed, spread=1.0):
    rng = np.random.default_rng(seed)
    centers = rng.uniform(-10, 10, (k, d))
    X = centers[rng.integers(0, k, n)] + spread * rng.standard_normal((n, d))
    init = X[rng.choice(n, k, replace=False)].copy()
    w = rng.uniform(0.5, 1.5, n)
    return X, w, init


@pytest.mark.parametrize("shape", [(20_000, 32, 64), (10_003, 9, 45), (4_096, 16, 16), (3_001, 17, 40), (777, 1, 20),
                                   (64, 31, 16), (6_000, 33, 16), (6_000, 48, 64), (5_003, 64, 64), (7_001, 63, 20),
                                   (20_000, 16, 256), (9_000, 14, 300)])
def test_fp64_screened_step_matches_oracle(cuda, shape):
    n, d, k = shape
    X, w, init = _blobs64(n, d, k, seed=n + d)
    labels, c_out, sizes, status, variant, rechecked = _one_iteration(X, w, init, cuda, flags=0)
    assert variant == 71
    _check_against_oracle(X, w, init, labels, c_out, sizes, status)
    assert rechecked <= 8 + n // 10


def test_fp64_screen_switched_off_by_flag(cuda):
    X, w, init = _blobs64(20_000, 32, 64, seed=3)
    labels, c_out, sizes, status, variant, rechecked = _one_iteration(X, w, init, cuda, flags=ALL_F32)
    assert variant == 51 and rechecked == 0
    _check_against_oracle(X, w, init, labels, c_out, sizes, status)


@pytest.mark.parametrize("d", [14, 32, 40, 64])
def test_fp64_duplicate_and_identical_centroids(cuda, d):
    X, w, init = _blobs64(20_000, d, 64, seed=41)
    dup = init.copy()
    dup[40] = dup[3]
    dup[63] = dup[17]
    labels, c_out, sizes, status, variant, rechecked = _one_iteration(X, w, dup, cuda, flags=0)
    assert variant == 71
    assert not np.any(labels == 40) and not np.any(labels == 63)
    ref = ok.assign_labels(X, dup)
    assert_labels_match(labels, ref, X, dup)
    assert rechecked >= int(np.count_nonzero((ref == 3) | (ref == 17)))
    same = init.copy()
    same[:] = same[0]
    labels, c_out, sizes, status, variant, rechecked = _one_iteration(X, w, same, cuda, flags=0)
    assert np.all(labels == 0) and rechecked == X.shape[0] and status.n_empty == 63


def test_fp64_more_uncertain_samples_than_the_list_holds(cuda):
    """One workgroup per compute unit and identical centroids: every sample is uncertain, 8192 per
    workgroup, twice what its list of noted samples holds; the rest is evaluated where it turns
    up.  Labels, sums and sizes must not depend on the route."""
    rng = np.random.default_rng(43)
    n, d, k = 1 << 21, 4, 16
    # (off the origin: the 64-bit fixed-point sums resolve 2^-61 of n max|w| max|x|, which is 1e-12 of
    # a cluster's sum unless that sum all but cancels)
    X = 3.0 + rng.standard_normal((n, d))
    w = rng.uniform(0.5, 1.5, n)
    init = np.tile(X[5], (k, 1))
    labels, c_out, sizes, status, variant, rechecked = _one_iteration(X, w, init, cuda, flags=1 << 8)
    assert variant == 71
    assert np.all(labels == 0) and rechecked == n
    assert status.n_empty == k - 1
    sums, ref_sizes = ok.weighted_sums(X, w, labels, k)
    np.testing.assert_allclose(sizes, ref_sizes, rtol=1e-12)
    assert_centers_close(c_out, sums, np.float64)


def test_fp64_initial_centroids_far_outside_the_data(cuda):
    """A quarter of the initial centroids at +1e3 in every coordinate (as in the configuration with
    forced empty clusters): they set the fp16 scale and have huge norms, and must cost neither the
    other centroids' scores their precision nor the samples their certificate."""
    X, w, init = _blobs64(60_000, 32, 64, seed=47, spread=0.5)
    init[48:] = 1e3 + np.arange(16)[:, None]
    labels, c_out, sizes, status, variant, rechecked = _one_iteration(X, w, init, cuda, flags=0)
    assert variant == 71
    assert labels.max() < 48 and status.n_empty >= 16
    assert_labels_match(labels, ok.assign_labels(X, init), X, init)
    assert rechecked <= X.shape[0] // 2


@pytest.mark.parametrize("spread", [1.0, 300.0])
@pytest.mark.parametrize("d,k", [(32, 64), (14, 20), (48, 33)])
def test_fp64_certificate_passes_no_label_that_fp64_would_not_give(cuda, d, k, spread):
    """Samples at distances from a bisector spread over twelve decades (gaps between the two best
    squared distances from 1e-14 to 1e-2 of their size): whatever the screen certifies must be
    the fp64 arg-min - labels may differ from an extended-precision evaluation only where fp64
    itself cannot tell, far below anything fp32 or fp16 resolves."""
    rng = np.random.default_rng(53 + d)
    n = 40_000
    C = rng.uniform(-10, 10, (k, d))
    # (spread > 1: centroids whose norms differ by that factor - the part of the bound that is kept
    # per centroid spans five orders of magnitude, and the far centroids set the fp16 scale)
    C *= spread ** rng.uniform(0.0, 1.0, (k, 1))
    a = rng.integers(0, k, n)
    b = (a + 1 + rng.integers(0, k - 1, n)) % k
    mid = 0.5 * (C[a] + C[b])
    axis = C[b] - C[a]
    axis /= np.linalg.norm(axis, axis=1, keepdims=True)
    ortho = 0.01 * rng.standard_normal((n, d))
    ortho -= (ortho * axis).sum(axis=1, keepdims=True) * axis
    offset = 10.0 ** rng.uniform(-14, -2, n) * rng.choice([-1.0, 1.0], n)
    X = mid + ortho + offset[:, None] * axis * np.linalg.norm(C[b] - C[a], axis=1, keepdims=True)
    w = np.ones(n)
    labels, c_out, sizes, status, variant, rechecked = _one_iteration(X, w, C, cuda, flags=0)
    assert variant == 71
    XL, CL = X.astype(np.longdouble), C.astype(np.longdouble)
    dist = ((XL[:, None, :] - CL[None, :, :]) ** 2).sum(axis=2)
    ref = dist.argmin(axis=1)
    bad = np.flatnonzero(labels != ref)
    gap = (dist[bad, labels[bad]] - dist[bad, ref[bad]]) / dist[bad].max(axis=1)
    assert np.all(gap <= 1e-14), f"{bad.size} labels differ, worst relative gap {gap.max():.3e}"
    # (most of these samples cannot be certified; with spread centroids a third, smaller centroid is
    # often nearer than the pair whose bisector the sample was put on, and fewer stay uncertain)
    assert rechecked > (n // 4 if spread == 1.0 else n // 20)
    # the same kernel without the update (kmx_assign_labels on fp64 inputs): the same bar
    import torch

    from sklearn_numba_dpex_amd.kmeans import drivers

    X_t = torch.as_tensor(np.ascontiguousarray(X.T), device=cuda)
    C_t = torch.as_tensor(np.ascontiguousarray(C.T), device=cuda)
    assigned = torch.full((n,), -1, dtype=torch.int32, device=cuda)
    drivers._assign(X_t, C_t, assigned)
    got = assigned.cpu().numpy().astype(np.int64)
    bad = np.flatnonzero(got != ref)
    gap = (dist[bad, got[bad]] - dist[bad, ref[bad]]) / dist[bad].max(axis=1)
    assert np.all(gap <= 1e-14), f"assign: {bad.size} labels differ, worst relative gap {gap.max():.3e}"
