"""GPU parity of the Lloyd path (fused step, reduction/finalisation, full run, labels,
inertia) against the CPU oracle, through the C ABI and through the drivers."""

import ctypes

import numpy as np
import pytest

from oracle import datasets
from oracle import kmeans as ok
from tests._parity import RTOL, assert_centers_close, assert_labels_match

pytestmark = pytest.mark.gpu


def _dev(a, cuda):
    import torch

    return torch.as_tensor(np.ascontiguousarray(a), device=cuda)


def _small_configs():
    return {
        "C1": lambda: datasets.config1(n=100_000),
        "C2": lambda: datasets.config2(n=200_000),
        "C3": lambda: datasets.config3(n=20_000, d=256, k=1024),
        "C3s": lambda: datasets.config3(n=30_001, d=70, k=50),
        "C3m": lambda: datasets.config3(n=30_001, d=100, k=300),
        "C3w": lambda: datasets.config3(n=9_000, d=300, k=70),
        "C5": lambda: datasets.config5(n=100_000),
        "odd": lambda: _odd_config(),
        # shapes off the fast paths of the matrix-core kernels: n not a multiple of the tile or
        # of 4 (no 128-bit accesses), odd d, k not a multiple of the centroid block
        "F64a": lambda: _blob_config(10_007, 13, 37, np.float64, 11),
        "F64b": lambda: _blob_config(4_100, 30, 100, np.float64, 12),
        "F64c": lambda: _blob_config(50, 32, 16, np.float64, 13),
        "M32a": lambda: _blob_config(10_003, 9, 45, np.float32, 14),
        "M32b": lambda: _blob_config(5_000, 40, 20, np.float32, 15),
        "M32c": lambda: _blob_config(33, 14, 16, np.float32, 16),
        # wide fp32 path with very unequal clusters (bucket sizes from 0 to a third of n)
        "C3k": lambda: dict(_blob_config(40_000, 128, 64, np.float32, 17, skew=True), flags=0x3, variant=42),
        "C3k2": lambda: dict(_blob_config(40_000, 128, 64, np.float32, 17, skew=True), variant=63),
        # few features, many clusters: accumulators and centroid copies need more than 64 KB of
        # LDS, which only the screened step (one workgroup per compute unit) may take
        "M32d": lambda: dict(_blob_config(20_000, 14, 600, np.float32, 18), variant=61),
        # the same with the screen switched off, and a shape whose accumulators exceed what any
        # kernel keeps in LDS: the wide path with one chunk of features (d <= 32)
        "M32e": lambda: dict(_blob_config(20_000, 14, 600, np.float32, 18), flags=0x10, variant=42),
        # beyond the LDS of the fused screened step: its labels-only form with sums per bucket of
        # samples; the wide path on request
        "M32f": lambda: dict(_blob_config(20_000, 14, 700, np.float32, 20), variant=63),
        "M32g": lambda: dict(_blob_config(20_000, 14, 700, np.float32, 20), flags=0x3, variant=42),
        # accumulators beyond LDS off the wide fp32 path: a labels-only kernel (fp64 matrix cores
        # where the centroids fit, else vector ALU) and sums per bucket of samples
        "F64d": lambda: dict(_blob_config(20_000, 32, 500, np.float64, 19), variant=53),
        "B64a": lambda: dict(_blob_config(20_001, 100, 100, np.float64, 25), variant=63),
        "B64b": lambda: dict(_blob_config(30_000, 8, 5000, np.float64, 26), variant=63),
        "B64d": lambda: dict(_blob_config(30_000, 8, 5000, np.float64, 26), flags=0x2, variant=13),
        "B64e": lambda: dict(_blob_config(10_000, 100, 100, np.float64, 30), flags=0x1, variant=3),
        "B32a": lambda: dict(_blob_config(9_001, 300, 40, np.float32, 27, skew=True), variant=63),
        "B32b": lambda: dict(_blob_config(3_000, 784, 130, np.float32, 28), variant=63),
        "B64c": lambda: dict(_blob_config(2_999, 70, 260, np.float64, 29), variant=63),
        # the tiled product with one tile of 32 / 64 centroids
        "B32c": lambda: dict(_blob_config(5_001, 300, 20, np.float32, 31), variant=63),
        "B64f": lambda: dict(_blob_config(4_000, 100, 24, np.float64, 32), variant=63),
        "B64g": lambda: dict(_blob_config(4_003, 90, 50, np.float64, 33), variant=63),
        # cluster counts either side of where the tiled product widens its centroid tile (32, 64)
        "B32d": lambda: dict(_blob_config(3_001, 300, 32, np.float32, 68), variant=63),
        "B32e": lambda: dict(_blob_config(3_001, 300, 33, np.float32, 69), variant=63),
        "B32f": lambda: dict(_blob_config(2_000, 200, 64, np.float32, 70), variant=63),
        "B32g": lambda: dict(_blob_config(2_000, 200, 65, np.float32, 71), variant=63),
        "B64i": lambda: dict(_blob_config(2_001, 150, 32, np.float64, 72), variant=63),
        "B64j": lambda: dict(_blob_config(2_001, 150, 33, np.float64, 73), variant=63),
        "B64k": lambda: dict(_blob_config(1_500, 100, 64, np.float64, 74), variant=63),
        "B64l": lambda: dict(_blob_config(1_500, 100, 65, np.float64, 75), variant=63),
        # few clusters of wide fp64 samples: the finalisation with 64 lanes per cluster
        "B64h": lambda: dict(_blob_config(3_001, 300, 18, np.float64, 67, skew=True), variant=63),
        # few clusters: the register-resident and the streaming vector-ALU steps
        "R64a": lambda: dict(_blob_config(5_003, 50, 7, np.float64, 34), variant=11),
        "R32a": lambda: dict(_blob_config(5_003, 40, 8, np.float32, 35), variant=11),
        "S64a": lambda: dict(_blob_config(5_002, 90, 16, np.float64, 36), flags=0x1, variant=1),
        # (fp64 below a million samples leaves the streaming step to the tiled product by itself)
        "S64c": lambda: dict(_blob_config(5_002, 90, 16, np.float64, 36), variant=63),
        "S32a": lambda: dict(_blob_config(300_000, 70, 5, np.float32, 37), flags=0x1, variant=1),
        # enough samples for four (fp32) / two (fp64) consecutive samples per thread
        "S32b": lambda: dict(_blob_config(600_000, 70, 5, np.float32, 38), flags=0x1, variant=1),
        # fp32, up to 16 clusters, more than 64 features: a tile of samples in LDS serves the labels
        # and the sums (one read of X); tiles of 64, 32 and 16 samples, every unrolling of the
        # kernel, n below a tile, n not a multiple of 4, one cluster
        "K32a": lambda: dict(_blob_config(7_001, 784, 10, np.float32, 48), variant=81),
        "K32b": lambda: dict(_blob_config(20_000, 100, 10, np.float32, 49), variant=81),
        "K32c": lambda: dict(_blob_config(5_003, 65, 16, np.float32, 50), variant=81),
        "K32d": lambda: dict(_blob_config(3_002, 1216, 3, np.float32, 51), variant=81),
        "K32e": lambda: dict(_blob_config(40, 300, 2, np.float32, 52), variant=81),
        "K32f": lambda: dict(_blob_config(9_000, 257, 7, np.float32, 53), variant=81),
        "K32g": lambda: dict(_blob_config(300_000, 70, 5, np.float32, 37), variant=81),
        "K32h": lambda: dict(_blob_config(6_000, 513, 1, np.float32, 54), variant=81),
        "K32i": lambda: dict(_blob_config(8_000, 200, 12, np.float32, 55, skew=True), variant=81),
        # up to 128 features (a multiple of 4) with the row-major copy: every wave on tiles of its own
        "K32j": lambda: dict(_blob_config(50_001, 128, 16, np.float32, 56), variant=81),
        "K32k": lambda: dict(_blob_config(10_000, 68, 3, np.float32, 57), variant=81),
        "K32l": lambda: dict(_blob_config(30_003, 112, 9, np.float32, 58, skew=True), variant=81),
        # tiles that arrive in LDS directly (row-major copy, a multiple of 4 features beyond 128): four
        # waves per workgroup up to 512 features, eight beyond; fewer samples than a tile; rows of
        # exactly one, two and more than two load instructions of 64 pieces
        "K32m": lambda: dict(_blob_config(2_501, 384, 6, np.float32, 59), variant=81),
        "K32n": lambda: dict(_blob_config(9, 640, 4, np.float32, 60), variant=81),
        "K32o": lambda: dict(_blob_config(4_100, 512, 16, np.float32, 61), variant=81),
        "K32p": lambda: dict(_blob_config(1_030, 832, 5, np.float32, 62, skew=True), variant=81),
        "K32q": lambda: dict(_blob_config(777, 256, 11, np.float32, 63), variant=81),
        # the widest samples of this step: one workgroup per compute unit, with and without the row-major copy
        "K32r": lambda: dict(_blob_config(1_500, 1792, 4, np.float32, 64), variant=81),
        "K32s": lambda: dict(_blob_config(2_003, 1500, 16, np.float32, 65), variant=81),
        # enough samples for the labels-only kernel with a tile per wave, n odd (no 128-bit accesses)
        "K32t": lambda: dict(_blob_config(270_001, 96, 7, np.float32, 66), variant=81),
        "S64b": lambda: dict(_blob_config(300_000, 70, 5, np.float64, 39), flags=0x1, variant=1),
        # extremes of the tiled product: thousands of features (many passes of the bucketed sums),
        # more clusters than the bucket counts hold in LDS and than the wide path takes
        "X32a": lambda: dict(_blob_config(1_500, 3_000, 20, np.float32, 40), variant=63),
        "X32b": lambda: dict(_blob_config(30_000, 8, 9_000, np.float32, 41), variant=63),
        "X64a": lambda: dict(_blob_config(12_000, 3, 5_000, np.float64, 42), variant=63),
        # the tiled product screened on the fp16 matrix cores (on request), the uncertified
        # samples through the listed fp32 pass
        "G32s": lambda: dict(_blob_config(6_001, 100, 100, np.float32, 43), flags=0x20, variant=63),
        "G32t": lambda: dict(_blob_config(3_000, 784, 40, np.float32, 44, skew=True), flags=0x20, variant=63),
        "G32u": lambda: dict(_blob_config(5_000, 70, 20, np.float32, 45), flags=0x20, variant=63),
        # fp64 on the matrix cores beyond 32 features (no rows in flight for the next tile) and
        # with accumulators that need most of a compute unit's LDS
        # (fp64 inputs up to 64 features: labels screened on the fp16 matrix cores, the rest in
        # fp64 - variant 71; with the screen switched off the all-fp64 matrix-core step, 51)
        "F64e": lambda: dict(_blob_config(20_003, 48, 64, np.float64, 21), variant=71),
        # (64 features x 100 clusters: the fp64 and fp32 copies of the centroids do not both fit the LDS)
        "F64f": lambda: dict(_blob_config(8_000, 64, 100, np.float64, 22), variant=51),
        "F64g": lambda: dict(_blob_config(20_000, 32, 300, np.float64, 23), variant=51),
        "F64h": lambda: dict(_blob_config(6_001, 61, 33, np.float64, 24), variant=71),
        "F64e1": lambda: dict(_blob_config(20_003, 48, 64, np.float64, 21), flags=0x10, variant=51),
        "F64h1": lambda: dict(_blob_config(6_001, 61, 33, np.float64, 24), flags=0x10, variant=51),
        "C5f": lambda: dict(datasets.config5(n=100_000), flags=0x10, variant=51),
        # fp64 screened step, one K step of 16 features with and without a spare slot
        "F64i": lambda: dict(_blob_config(30_000, 16, 127, np.float64, 46), variant=71),
        "F64j": lambda: dict(_blob_config(30_004, 14, 127, np.float64, 47), variant=71),
    }


def _blob_config(n, d, k, dtype, seed, skew=False):
    rng = np.random.default_rng(seed)
    centers = rng.uniform(-10, 10, (k, d))
    p = rng.dirichlet(np.full(k, 0.15)) if skew else np.full(k, 1.0 / k)
    y = rng.choice(k, size=n, p=p)
    X = (centers[y] + rng.standard_normal((n, d))).astype(dtype)
    init = X[rng.choice(n, k, replace=False)].copy()
    w = rng.uniform(0.5, 1.5, n).astype(dtype)
    return dict(X=X, init=init, sample_weight=w, k=k, max_iter=20, tol=0.0, name=f"blob{seed}")


def _odd_config():
    """Ragged shapes: n not a multiple of anything, d = 3, k = 5, fp64."""
    rng = np.random.default_rng(7)
    X = rng.normal(size=(1237, 3))
    init = X[rng.choice(1237, 5, replace=False)].copy()
    return dict(X=X, init=init, sample_weight=rng.uniform(0.5, 2, 1237), k=5, max_iter=50, tol=0.0, name="odd")


@pytest.mark.parametrize("rowmajor", [False, True])
@pytest.mark.parametrize("name", ["C1", "C2", "C3", "C3s", "C3m", "C3w", "C5", "odd", "F64a", "F64b", "F64c",
                                  "M32a", "M32b", "M32c", "C3k", "M32d", "M32e", "M32f", "M32g", "F64d", "F64e", "F64f",
                                  "F64g", "F64h", "F64e1", "F64h1", "C5f", "F64i", "F64j", "B64a", "B64b", "B32a", "B32b", "B64c", "B64d", "B64e", "C3k2", "B32c", "B64f", "B64g", "B64h", "B32d", "B32e", "B32f", "B32g", "B64i", "B64j", "B64k", "B64l", "R64a", "R32a", "S64a", "S64c", "S32a", "S32b", "S64b", "X32a", "X32b", "X64a", "G32s", "G32t", "G32u",
                                  "K32a", "K32b", "K32c", "K32d", "K32e", "K32f", "K32g", "K32h", "K32i",
                                  "K32j", "K32k", "K32l", "K32m", "K32n", "K32o", "K32p", "K32q", "K32r", "K32s"])
def test_single_iteration_through_c_abi(cuda, name, rowmajor):
    import torch

    from sklearn_numba_dpex_amd import _capi
    from sklearn_numba_dpex_amd._capi import lib, ptr

    cfg = _small_configs()[name]()
    X, init, w, k = cfg["X"], cfg["init"], cfg["sample_weight"], cfg["k"]
    n, d = X.shape
    dc = _capi.dtype_code(X.dtype)
    X_t = _dev(X.T, cuda)
    w_d = _dev(w, cuda)
    c_in = _dev(init.T, cuda)
    c_out = torch.empty_like(c_in)
    labels_prev = torch.zeros(n, dtype=torch.int32, device=cuda)
    labels = torch.empty(n, dtype=torch.int32, device=cuda)
    sizes = torch.empty(k, dtype=X_t.dtype, device=cuda)
    empty = torch.empty(k, dtype=torch.int32, device=cuda)
    plan = _capi.lloyd_plan(n, d, k, dc, cfg.get("flags", 0))
    if "variant" in cfg:
        assert plan.variant == cfg["variant"]
    ws_bytes = plan.workspace_bytes
    ws = torch.empty(ws_bytes, dtype=torch.uint8, device=cuda)
    stream = _capi.current_stream()
    _capi.check(lib.kmx_lloyd_init(plan, ptr(ws), ws_bytes, ptr(X_t), ptr(w_d), ptr(c_in), 100, 0.0, stream), "init")
    if rowmajor and plan.variant not in (42, 3, 13, 53, 63, 81):
        pytest.skip("the row-major copy is only used by the wide fp32 path, the bucketed sums and the few-cluster step")
    X_rm = _dev(X, cuda) if rowmajor else None
    _capi.check(lib.kmx_lloyd_iter(plan, ptr(X_t), ptr(X_rm), ptr(w_d), ptr(c_in), ptr(c_out), ptr(labels_prev),
                                   ptr(labels), ptr(sizes), ptr(empty), ptr(ws), ws_bytes, stream), "iter")
    status = _capi.LloydStatus()
    _capi.check(lib.kmx_lloyd_status_read(ptr(ws), status, stream), "status")

    ref_labels = ok.assign_labels(X, init)
    n_ties = assert_labels_match(labels.cpu().numpy(), ref_labels, X, init)
    got_labels = labels.cpu().numpy().astype(np.int64)
    sums, ref_sizes = ok.weighted_sums(X, w, got_labels, k)
    n_empty = int(np.count_nonzero(ref_sizes == 0))
    assert status.n_empty == n_empty
    np.testing.assert_allclose(sizes.cpu().numpy(), ref_sizes, rtol=RTOL[X.dtype])
    if n_empty:
        assert status.state == _capi.KMX_NEED_RELOCATION
        assert status.n_iter == 0
        np.testing.assert_array_equal(empty.cpu().numpy()[:n_empty], np.flatnonzero(ref_sizes == 0))
        got = c_out.cpu().numpy().T
        assert_centers_close(got, sums, X.dtype)
    else:
        assert status.state == _capi.KMX_RUNNING
        assert status.n_iter == 1
        ref_centers = sums / ref_sizes[:, None]
        assert_centers_close(c_out.cpu().numpy().T, ref_centers, X.dtype)
        shift = float(np.sum((np.asarray(init, np.float64) - ref_centers.astype(np.float64)) ** 2))
        assert status.shift_sum == pytest.approx(shift, rel=1e-4)
        expected_changed = int(np.count_nonzero(got_labels != 0))
        assert status.reserved[1] == expected_changed
    print(f"{name}: near-tie label differences: {n_ties}")


@pytest.mark.parametrize("name", ["C2", "M32a", "M32b", "C3", "C3s", "C5", "C5f", "F64j", "F64d", "B64a", "B64d", "B64e", "odd", "S64a", "K32a", "K32b"])
def test_duplicate_and_identical_centroids_on_every_kernel_family(cuda, name):
    """Exact ties: with two centroids duplicated no sample may take the copy with the higher
    index, with all centroids identical every label is 0 (the reference's strict '<' in
    increasing centroid order), whichever label kernel the shape selects."""
    import torch

    from sklearn_numba_dpex_amd import _capi
    from sklearn_numba_dpex_amd._capi import lib, ptr

    cfg = _small_configs()[name]()
    X, w, k = cfg["X"], cfg["sample_weight"], cfg["k"]
    n, d = X.shape
    dc = _capi.dtype_code(X.dtype)
    X_t, w_d = _dev(X.T, cuda), _dev(w, cuda)
    labels_prev = torch.zeros(n, dtype=torch.int32, device=cuda)
    labels = torch.empty(n, dtype=torch.int32, device=cuda)
    sizes = torch.empty(k, dtype=X_t.dtype, device=cuda)
    empty = torch.empty(k, dtype=torch.int32, device=cuda)
    plan = _capi.lloyd_plan(n, d, k, dc, cfg.get("flags", 0))
    ws = torch.empty(plan.workspace_bytes, dtype=torch.uint8, device=cuda)
    stream = _capi.current_stream()

    def one_iteration(init):
        c_in = _dev(init.T, cuda)
        c_out = torch.empty_like(c_in)
        _capi.check(lib.kmx_lloyd_init(plan, ptr(ws), plan.workspace_bytes, ptr(X_t), ptr(w_d), ptr(c_in), 100, 0.0,
                                       stream), "init")
        _capi.check(lib.kmx_lloyd_iter(plan, ptr(X_t), None, ptr(w_d), ptr(c_in), ptr(c_out), ptr(labels_prev),
                                       ptr(labels), ptr(sizes), ptr(empty), ptr(ws), plan.workspace_bytes, stream),
                    "iter")
        return labels.cpu().numpy().astype(np.int64)

    init = cfg["init"].copy()
    init[k - 1] = init[0]
    init[k // 2] = init[1]
    got = one_iteration(init)
    assert not np.any(got == k - 1) and not np.any(got == k // 2)
    assert_labels_match(got, ok.assign_labels(X, init), X, init)

    init = cfg["init"].copy()
    init[:] = init[0]
    assert np.all(one_iteration(init) == 0)


@pytest.mark.parametrize("name", ["C1", "C2", "C3s", "C3w", "odd", "F64a", "F64b", "M32a", "M32b", "C3k", "M32d", "M32e", "F64d",
                                  "F64e", "F64f", "F64g", "F64h", "F64e1", "F64h1", "C5f", "F64i", "F64j", "B64a", "B64b", "B32a", "B32b", "B64c", "B64d", "B64e", "C3k2", "B32c", "B64f", "B64g", "B64h", "R64a", "R32a", "S64a", "S32a", "G32s", "G32t",
                                  # (not K32d: with 1216 features two fp32 evaluations of a score differ by up
                                  # to 2e-6 of its size, more than the near-tie rule's 1e-6 - one label in ten
                                  # iterations of 3002 samples)
                                  "K32a", "K32b", "K32c", "K32f", "K32i", "K32m", "K32o", "K32q"])
def test_lockstep_iterations_match_oracle(cuda, name):
    """Ten iterations, each compared from identical inputs: the oracle repeats every GPU
    iteration from the centroids the GPU started it with (a Lloyd trajectory at tol = 0 is
    chaotic, so free-running trajectories may only be compared until the first near-tie)."""
    import torch

    from sklearn_numba_dpex_amd import _capi
    from sklearn_numba_dpex_amd._capi import lib, ptr

    cfg = _small_configs()[name]()
    X, init, w, k = cfg["X"], cfg["init"], cfg["sample_weight"], cfg["k"]
    n, d = X.shape
    dc = _capi.dtype_code(X.dtype)
    X_t, w_d = _dev(X.T, cuda), _dev(w, cuda)
    cent = [_dev(init.T, cuda), None]
    cent[1] = torch.empty_like(cent[0])
    labels = [torch.zeros(n, dtype=torch.int32, device=cuda) for _ in range(2)]
    sizes = torch.empty(k, dtype=X_t.dtype, device=cuda)
    empty = torch.empty(k, dtype=torch.int32, device=cuda)
    plan = _capi.lloyd_plan(n, d, k, dc, cfg.get("flags", 0))
    ws_bytes = plan.workspace_bytes
    ws = torch.empty(ws_bytes, dtype=torch.uint8, device=cuda)
    stream = _capi.current_stream()
    status = _capi.LloydStatus()
    _capi.check(lib.kmx_lloyd_init(plan, ptr(ws), ws_bytes, ptr(X_t), ptr(w_d), ptr(cent[0]), 100, 0.0, stream), "init")
    prev = None
    for it in range(10):
        a, b = it % 2, (it + 1) % 2
        c_in = cent[a].cpu().numpy().T.copy()
        _capi.check(lib.kmx_lloyd_iter(plan, ptr(X_t), None, ptr(w_d), ptr(cent[a]), ptr(cent[b]), ptr(labels[a]),
                                       ptr(labels[b]), ptr(sizes), ptr(empty), ptr(ws), ws_bytes, stream),
                    "iter")
        _capi.check(lib.kmx_lloyd_status_read(ptr(ws), status, stream), "status")
        got = labels[b].cpu().numpy().astype(np.int64)
        assert_labels_match(got, ok.assign_labels(X, c_in), X, c_in)
        sums, ref_sizes = ok.weighted_sums(X, w, got, k)
        if status.n_empty > 0:
            # an empty cluster appeared: the iteration waits for the host's relocation
            assert status.state == _capi.KMX_NEED_RELOCATION and status.n_iter == it
            assert status.n_empty == int(np.count_nonzero(ref_sizes == 0))
            break
        assert status.n_iter == it + 1
        assert_centers_close(cent[b].cpu().numpy().T, sums / ref_sizes[:, None], X.dtype)
        if prev is not None:
            assert status.reserved[1] == int(np.count_nonzero(got != prev))
        prev = got
        if status.state != _capi.KMX_RUNNING:
            assert status.state == _capi.KMX_CONVERGED_STRICT and np.array_equal(got, prev)
            break


@pytest.mark.parametrize("name", ["C1", "C2", "C3s", "C3m", "C5", "odd"])
def test_full_lloyd_run_matches_oracle(cuda, name):
    from sklearn_numba_dpex_amd.kmeans import drivers

    cfg = _small_configs()[name]()
    if name == "C2":
        cfg = datasets.config2(n=50_000)
    X, init, w, k = cfg["X"], cfg["init"], cfg["sample_weight"], cfg["k"]
    max_iter = min(cfg["max_iter"], 30)
    Xc = X - X.mean(axis=0).astype(X.dtype)
    initc = init - X.mean(axis=0).astype(X.dtype)
    tol = 0.0
    labels, inertia, centers_t, n_iter = drivers.lloyd(
        _dev(Xc.T, cuda), _dev(w, cuda), _dev(initc.T, cuda), False, max_iter=max_iter, tol=tol
    )
    ref_labels, ref_inertia, ref_centers, ref_n_iter = ok.lloyd(Xc, w, initc, max_iter=max_iter, tol=tol)
    assert n_iter == ref_n_iter
    centers = centers_t.cpu().numpy().T
    got = labels.cpu().numpy().astype(np.int64)
    # the returned labels are the argmin for the returned centroids, whatever the trajectory
    assert_labels_match(got, ok.assign_labels(Xc, centers), Xc, centers)
    assert float(inertia) == pytest.approx(float(ok.inertia(Xc, w, centers, got)), rel=1e-5)
    if np.array_equal(got, ref_labels.astype(np.int64)):
        # same final partition: centroids must agree to rounding
        # (ten roundings of 1e-5 / 1e-12: the two runs agree iteration by iteration, each
        # within the per-iteration tolerance, and the iterations contract towards the fixed point)
        assert_centers_close(centers, ref_centers, X.dtype, scale_rtol=RTOL[X.dtype] * 10)
        assert float(inertia) == pytest.approx(float(ref_inertia), rel=1e-5)
    else:
        # a near-tie flipped somewhere along the run: a few samples at a boundary, not another
        # clustering (per-iteration parity is what the lockstep test above asserts)
        assert np.count_nonzero(got != ref_labels.astype(np.int64)) <= max(1, n_samples_differ_cap(X))
        assert float(inertia) == pytest.approx(float(ref_inertia), rel=1e-4)


def _converging_configs():
    """Cases whose Lloyd run at tol = 0 reaches strict convergence (an iteration that changes no
    label) well below max_iter = 100.  Per case: the data, the kernel variant the plan must
    choose, and the iteration count of the oracle (found on the CPU; scikit-learn's Cython loop
    takes the same number when run on 8 threads, but its own count moves with its thread count
    - 43 instead of 39 on C1 with 4 threads - because its per-thread partial sums round
    differently and a Lloyd trajectory at tol = 0 amplifies every flipped near-tie)."""
    return {
        # BASELINE configs[0] at full size (fused screened step, sums corrected per moved sample)
        "C1": (lambda: datasets.config1(), 61, 39),
        # configs[1] (weighted, unequal blobs, one cluster empties and is relocated) and
        # configs[4] (fp64, sixteen clusters that empty on the first iteration) on fewer samples
        "C2_30k": (lambda: datasets.config2(n=30_000), 61, 38),
        "C5_100k": (lambda: datasets.config5(n=100_000), 71, 67),
        # screened labels with the sums taken straight from the labels, and with sums per bucket
        "direct": (lambda: _blob_config(20_000, 14, 700, np.float32, 20), 63, 8),
        "bucket": (lambda: _blob_config(20_000, 32, 500, np.float64, 19), 53, 8),
    }


@pytest.mark.parametrize("name", ["C1", "C2_30k", "C5_100k", "direct", "bucket"])
def test_n_iter_at_real_strict_convergence(cuda, name):
    """n_iter must be identical at tol = 0: whole runs with max_iter = 100 that stop because an
    iteration changed no label, not because of the cap, against the oracle, and against
    scikit-learn's own Lloyd loop wherever that one stayed on the oracle's trajectory."""
    from sklearn.cluster._kmeans import _kmeans_single_lloyd

    from sklearn_numba_dpex_amd import _capi
    from sklearn_numba_dpex_amd.kmeans import drivers

    make, variant, expected_n_iter = _converging_configs()[name]
    cfg = make()
    X, init, w, k = cfg["X"], cfg["init"], cfg["sample_weight"], cfg["k"]
    n, d = X.shape
    assert _capi.lloyd_plan(n, d, k, _capi.dtype_code(X.dtype), 0).variant == variant
    mean = X.mean(axis=0).astype(X.dtype)
    Xc, initc = X - mean, init - mean
    max_iter = 100
    labels, inertia, centers_t, n_iter = drivers.lloyd(
        _dev(Xc.T, cuda), _dev(w, cuda), _dev(initc.T, cuda), False, max_iter=max_iter, tol=0.0
    )
    ref_labels, ref_inertia, ref_centers, ref_n_iter = ok.lloyd(Xc, w, initc, max_iter=max_iter, tol=0.0)
    # the case is not decided by the cap
    assert ref_n_iter == expected_n_iter < max_iter
    assert n_iter == ref_n_iter
    centers = centers_t.cpu().numpy().T
    got = labels.cpu().numpy().astype(np.int64)
    # strict convergence: the returned labels are those of the last iteration and the argmin for
    # the returned centroids
    assert_labels_match(got, ok.assign_labels(Xc, centers), Xc, centers)
    assert float(inertia) == pytest.approx(float(ok.inertia(Xc, w, centers, got)), rel=RTOL[X.dtype] * 10)
    n_diff = np.count_nonzero(got != ref_labels.astype(np.int64))
    if n_diff == 0:
        # same final partition: the centroids are the same weighted means, 1e-5 / 1e-12
        assert_centers_close(centers, ref_centers, X.dtype)
        assert float(inertia) == pytest.approx(float(ref_inertia), rel=RTOL[X.dtype] * 10)
    else:
        # a near-tie went the other way in some iteration and the run ended in a neighbouring
        # fixed point after the same number of iterations: a few boundary samples (iteration by
        # iteration parity from identical inputs is what the lockstep tests assert)
        assert n_diff <= n_samples_differ_cap(X)
        assert float(inertia) == pytest.approx(float(ref_inertia), rel=1e-4)
    sk_labels, sk_inertia, sk_centers, sk_n_iter = _kmeans_single_lloyd(
        Xc, w, initc.copy(), max_iter=max_iter, tol=0.0, n_threads=8
    )
    if np.array_equal(sk_labels, ref_labels):
        # scikit-learn ended in the oracle's partition: it took the oracle's path
        assert n_iter == sk_n_iter
    assert float(inertia) == pytest.approx(float(sk_inertia), rel=1e-3)


def test_lockstep_to_strict_convergence_where_free_runs_part_ways(cuda):
    """configs[1] on 100 000 samples: at iteration 3 one sample lies within 4e-9 (relative) of a
    bisector, the kernel and the oracle label it differently, and from there the two free runs
    (and scikit-learn's) follow different trajectories: 69, 84 and 84 iterations.  What can be
    pinned there is every single iteration up to the end: the oracle repeats each iteration from
    the centroids the GPU started it with, through the relocation of the cluster that empties, and
    the run must stop at the first iteration whose labels equal the previous ones."""
    import torch

    from sklearn_numba_dpex_amd import _capi
    from sklearn_numba_dpex_amd._capi import lib, ptr
    from sklearn_numba_dpex_amd.kmeans import drivers

    cfg = datasets.config2(n=100_000)
    X, init, w, k = cfg["X"], cfg["init"], cfg["sample_weight"], cfg["k"]
    mean = X.mean(axis=0).astype(X.dtype)
    X, init = X - mean, init - mean
    n, d = X.shape
    dc = _capi.dtype_code(X.dtype)
    X_t, w_d = _dev(X.T, cuda), _dev(w, cuda)
    cent = [_dev(init.T, cuda), None]
    cent[1] = torch.empty_like(cent[0])
    labels = [torch.zeros(n, dtype=torch.int32, device=cuda) for _ in range(2)]
    sizes = torch.empty(k, dtype=X_t.dtype, device=cuda)
    empty = torch.empty(k, dtype=torch.int32, device=cuda)
    plan = _capi.lloyd_plan(n, d, k, dc, 0)
    assert plan.variant == 61
    ws_bytes = plan.workspace_bytes
    ws = torch.empty(ws_bytes, dtype=torch.uint8, device=cuda)
    stream = _capi.current_stream()
    status = _capi.LloydStatus()
    _capi.check(lib.kmx_lloyd_init(plan, ptr(ws), ws_bytes, ptr(X_t), ptr(w_d), ptr(cent[0]), 100, 0.0, stream), "init")
    prev = None
    n_relocations = 0
    for it in range(100):
        a, b = it % 2, (it + 1) % 2
        c_in = cent[a].cpu().numpy().T.copy()
        _capi.check(lib.kmx_lloyd_iter(plan, ptr(X_t), None, ptr(w_d), ptr(cent[a]), ptr(cent[b]), ptr(labels[a]),
                                       ptr(labels[b]), ptr(sizes), ptr(empty), ptr(ws), ws_bytes, stream), "iter")
        _capi.check(lib.kmx_lloyd_status_read(ptr(ws), status, stream), "status")
        got = labels[b].cpu().numpy().astype(np.int64)
        assert_labels_match(got, ok.assign_labels(X, c_in), X, c_in)
        sums, ref_sizes = ok.weighted_sums(X, w, got, k)
        if status.state == _capi.KMX_NEED_RELOCATION:
            n_relocations += 1
            assert status.n_empty == int(np.count_nonzero(ref_sizes == 0)) and status.n_iter == it
            drivers._relocate_empty_clusters(status.n_empty, X_t, w_d, cent[b], sizes, labels[b], empty, cent[a])
            _capi.check(lib.kmx_lloyd_finalize(plan, ptr(cent[a]), ptr(cent[b]), ptr(sizes), ptr(ws), ws_bytes, stream),
                        "finalize")
            _capi.check(lib.kmx_lloyd_status_read(ptr(ws), status, stream), "status")
            ok.relocate_empty_clusters(X, w, sums, ref_sizes, got, ok.sq_dist_to_assigned(X, c_in, got))
        assert status.n_iter == it + 1
        assert_centers_close(cent[b].cpu().numpy().T, sums / ref_sizes[:, None], X.dtype)
        strict = prev is not None and np.array_equal(got, prev)
        assert (status.state == _capi.KMX_CONVERGED_STRICT) == strict
        if strict:
            break
        assert status.state == _capi.KMX_RUNNING
        prev = got
    assert status.state == _capi.KMX_CONVERGED_STRICT and n_relocations >= 1
    # the driver's own loop (iterations enqueued ahead) stops at the same iteration
    n_iter = drivers.lloyd(X_t, w_d, _dev(init.T, cuda), False, max_iter=100, tol=0.0)[3]
    assert n_iter == status.n_iter


def n_samples_differ_cap(X):
    return X.shape[0] // 1000


@pytest.mark.parametrize("name", ["C3s", "C3w", "C3k2", "F64d", "F64e", "F64h", "F64i", "F64j", "C5", "B64a", "B64b", "B32a", "B32b", "B64c", "odd", "B32c", "B64f", "B64g", "B64h", "B32d", "B32e", "B32f", "B32g", "B64i", "B64j", "B64k", "B64l", "R64a", "R32a", "S64a", "S32a",
                                  # few clusters on wide samples: the labels-only matrix-core kernel that reads
                                  # the feature-major array directly (tiles of 32 and of 64 samples, every width
                                  # of its centroid registers, n odd, n below a tile) and the inertia summed
                                  # with the features split over workgroups
                                  "K32a", "K32b", "K32d", "K32e", "K32f", "K32g", "K32j", "K32m", "K32n", "K32o", "K32p", "K32r", "K32s", "K32t"])
def test_labels_and_score_paths_on_every_label_kernel(cuda, name):
    """kmx_assign_labels, labels + inertia in one call and the distances on the shapes of the
    tiled matrix-core product, of the labels-only fp64 matrix-core kernel, of the vector-ALU
    kernels and of the few-cluster kernels, against the oracle."""
    import torch

    from sklearn_numba_dpex_amd.kmeans import drivers

    cfg = _small_configs()[name]()
    X, init, w = cfg["X"], cfg["init"], cfg["sample_weight"]
    n = X.shape[0]
    X_t, C_t, w_d = _dev(X.T, cuda), _dev(init.T, cuda), _dev(w, cuda)
    ref = ok.assign_labels(X, init)
    labels = torch.full((n,), -1, dtype=torch.int32, device=cuda)
    drivers._assign(X_t, C_t, labels)
    got = labels.cpu().numpy().astype(np.int64)
    assert_labels_match(got, ref, X, init)
    labels2, inertia = drivers.get_labels_inertia(X_t, C_t, w_d, True)
    np.testing.assert_array_equal(labels2.cpu().numpy().astype(np.int64), got)
    assert float(inertia[0]) == pytest.approx(float(ok.inertia(X, w, init, got)), rel=RTOL[X.dtype] * 5)
    dist = drivers.get_euclidean_distances(X_t[:, :512].contiguous(), C_t).cpu().numpy()
    exact = np.sqrt(((X[:512].astype(np.float64)[:, None, :] - init.astype(np.float64)[None, :, :]) ** 2).sum(axis=2))
    np.testing.assert_allclose(dist, exact, rtol=RTOL[X.dtype] * 2, atol=RTOL[X.dtype])
