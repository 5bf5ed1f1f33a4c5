"""The C-ABI library without a GPU: it loads, exports every function the header declares,
answers the size queries and rejects bad arguments before touching the device."""

import ctypes
import os
import re

import numpy as np
import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "mi355x_kmeans.h")


def _declared_functions():
    text = open(HEADER).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(kmx_[a-z0-9_]+)\s*\(", text)))


def test_library_exports_every_declared_function():
    from sklearn_numba_dpex_amd import _capi

    declared = _declared_functions()
    assert len(declared) >= 35
    raw = ctypes.CDLL(_capi.LIB_PATH)
    for name in declared:
        assert hasattr(raw, name), f"{name} is declared in the header but not exported"
    assert sorted(_capi.SIGNATURES) == declared, "ctypes signatures and header disagree"
    assert _capi.lib.kmx_abi_version() == 3


def test_header_cites_the_reference_for_every_entry_point():
    text = open(HEADER).read()
    # every declaration block mentions the reference file it replaces, or says it has none
    for name in _declared_functions():
        if name in ("kmx_abi_version", "kmx_error_string") or name.endswith("_workspace_bytes") \
                or name.endswith("_ptr") or name in ("kmx_lloyd_status_read", "kmx_lloyd_kernel_variant"):
            continue
        idx = text.index(name + "(")
        comment = text[text.rfind("/*", 0, idx):idx]
        assert re.search(r"\.py:\d+|no\s+counterpart", comment), f"{name}: no reference citation"


def test_error_strings_and_codes():
    from sklearn_numba_dpex_amd import _capi

    assert _capi.error_string(0) == "ok"
    assert "null" in _capi.error_string(-1)
    assert "workspace" in _capi.error_string(-4)
    with pytest.raises(_capi.KmxError) as e:
        _capi.check(-2, "somewhere")
    assert e.value.code == -2 and "somewhere" in str(e.value)


def test_workspace_queries():
    from sklearn_numba_dpex_amd import _capi
    from sklearn_numba_dpex_amd._capi import lib

    small = lib.kmx_lloyd_workspace_bytes(100_000, 14, 127, 0, 0)
    assert 0 < small < 64 << 20
    # the screened fp32 step keeps ||x_i|| per sample: 4 bytes per sample
    assert abs(lib.kmx_lloyd_workspace_bytes(5_000_000, 14, 127, 0, 0) - small - 4 * 4_900_000) < 256
    # and so does the screened fp64 step; the all-fp64 matrix-core step (screen switched off) keeps nothing per sample
    assert abs(lib.kmx_lloyd_workspace_bytes(5_000_000, 14, 127, 1, 0)
               - lib.kmx_lloyd_workspace_bytes(100_000, 14, 127, 1, 0) - 4 * 4_900_000) < 256
    assert (lib.kmx_lloyd_workspace_bytes(5_000_000, 14, 127, 1, 0x10)
            == lib.kmx_lloyd_workspace_bytes(100_000, 14, 127, 1, 0x10))
    assert lib.kmx_lloyd_kernel_variant(2_000_000, 32, 64, 1, 0) == 71
    assert lib.kmx_lloyd_kernel_variant(2_000_000, 32, 64, 1, 0x10) == 51
    # sums beyond LDS off the wide path: sample order and ranks (2 n words) + one copy of the sums;
    # the screened tiled product (on request) adds its list (n words)
    assert 8_000_000 + 4 * 301 * 1024 < lib.kmx_lloyd_workspace_bytes(1_000_000, 300, 1024, 0, 0) < (16 << 20)
    assert (lib.kmx_lloyd_workspace_bytes(1_000_000, 300, 1024, 0, 0x20)
            >= lib.kmx_lloyd_workspace_bytes(1_000_000, 300, 1024, 0, 0) + 4_000_000)
    assert lib.kmx_lloyd_kernel_variant(1_000_000, 300, 1024, 0, 0) == 63
    # the second (row-major) copy of X: read by the wide step and by the sums per bucket, not by the
    # fused steps nor by the sums taken straight from the labels
    for (n_, d_, k_, dt_), reads in {(1_000_000, 256, 1024, 0): 1, (1_000_000, 300, 1024, 0): 1,
                                     (1_000_000, 100, 100, 1): 1, (5_000_000, 14, 127, 0): 0,
                                     (1_000_000, 14, 700, 0): 0, (2_000_000, 32, 64, 1): 0}.items():
        assert lib.kmx_lloyd_plan_reads_rowmajor(_capi.lloyd_plan(n_, d_, k_, dt_, 0)) == reads, (n_, d_, k_, dt_)
    assert lib.kmx_lloyd_kernel_variant(1_000_000, 48, 64, 1, 0) == 71
    assert lib.kmx_lloyd_kernel_variant(1_000_000, 48, 64, 1, 0x10) == 51
    assert lib.kmx_lloyd_kernel_variant(1_000_000, 64, 100, 1, 0) == 51  # (both copies of the centroids: beyond the LDS)
    assert lib.kmx_lloyd_kernel_variant(1_000_000, 32, 500, 1, 0) == 53
    assert lib.kmx_lloyd_workspace_bytes(0, 14, 127, 0, 0) == 0
    assert lib.kmx_lloyd_workspace_bytes(10, 14, 127, 7, 0) == 0
    assert lib.kmx_assign_workspace_bytes(14, 127, 0) > 127 * 16 * 4
    # the roomy variant only grows for wide fp32 shapes (a list of sample indices)
    assert lib.kmx_assign_workspace_bytes_for(1000, 14, 127, 0, 0) == lib.kmx_assign_workspace_bytes(14, 127, 0)
    assert lib.kmx_assign_workspace_bytes_for(1000, 256, 1024, 1, 0) == lib.kmx_assign_workspace_bytes(256, 1024, 1)
    assert (lib.kmx_assign_workspace_bytes_for(1000, 256, 1024, 0, 0)
            >= lib.kmx_assign_workspace_bytes(256, 1024, 0) + 1000 * 4)
    assert lib.kmx_kpp_workspace_bytes(1_000_000, 64, 256, 7, 0) >= 7 * 4_000_000
    assert lib.kmx_kpp_workspace_bytes(1000, 4, 8, 17, 0) == 0  # more trials than supported
    assert lib.kmx_topk_workspace_bytes(1000, 10) > 0
    assert lib.kmx_topk_workspace_bytes(5, 10) == 0
    one_row = lib.kmx_topk_rows_workspace_bytes(1, 1000, 10, 0)
    assert 0 < one_row <= lib.kmx_topk_workspace_bytes(1000, 10)
    assert lib.kmx_topk_rows_workspace_bytes(7, 1000, 10, 0) == 7 * one_row
    assert lib.kmx_topk_rows_workspace_bytes(7, 1000, 10, 5) == 0
    assert lib.kmx_sum_workspace_bytes(7, 1_000_000) >= 7 * 256 * 8


def test_kernel_variant_selection():
    from sklearn_numba_dpex_amd._capi import lib

    assert lib.kmx_lloyd_kernel_variant(5_000_000, 14, 127, 0, 0) == 61   # fp16-screened MFMA + LDS accumulators
    assert lib.kmx_lloyd_kernel_variant(5_000_000, 40, 127, 0, 0) == 61   # three K steps of the screen
    assert lib.kmx_lloyd_kernel_variant(5_000_000, 64, 120, 0, 0) == 61   # four, all of a compute unit's LDS
    assert lib.kmx_lloyd_kernel_variant(5_000_000, 40, 127, 0, 0x10) == 31  # fp32 MFMA + LDS accumulators
    assert lib.kmx_lloyd_kernel_variant(5_000_000, 4, 127, 0, 0) == 31    # too few features for the screen to pay
    assert lib.kmx_lloyd_kernel_variant(5_000_000, 8, 64, 0, 0) == 61
    assert lib.kmx_lloyd_kernel_variant(5_000_000, 8, 32, 0, 0) == 31
    assert lib.kmx_lloyd_kernel_variant(2_000_000, 32, 64, 1, 0) == 71    # fp64: fp16-screened labels, fp64 sums in LDS
    assert lib.kmx_lloyd_kernel_variant(2_000_000, 32, 64, 1, 0x10) == 51  # screen off: fp64 matrix cores + LDS
    assert lib.kmx_lloyd_kernel_variant(1_000_000, 64, 128, 1, 0) == 51    # with all of a compute unit's LDS
    assert lib.kmx_lloyd_kernel_variant(2_000_000, 32, 500, 1, 0) == 53    # labels on the matrix cores, bucketed sums
    assert lib.kmx_lloyd_kernel_variant(2_000_000, 32, 1024, 1, 0) == 63   # centroids too big for LDS as well: tiled product
    assert lib.kmx_lloyd_kernel_variant(2_000_000, 32, 1024, 1, 0x2) == 13  # vector-ALU labels when asked for
    assert lib.kmx_lloyd_kernel_variant(2_000_000, 100, 100, 1, 0) == 63     # tiled matrix-core labels, bucketed sums
    assert lib.kmx_lloyd_kernel_variant(2_000_000, 100, 100, 1, 0x1) == 3     # vector-ALU labels when asked for
    assert lib.kmx_lloyd_kernel_variant(1 << 31, 100, 100, 1, 0) == 2      # too many samples for 32-bit buckets
    assert lib.kmx_lloyd_kernel_variant(1_000_000, 256, 1024, 0, 0) == 42  # wide MFMA + global sums
    assert lib.kmx_lloyd_kernel_variant(1_000_000, 300, 1024, 0, 0) == 63  # tiled matrix-core labels + bucketed sums
    assert lib.kmx_lloyd_kernel_variant(1000, 3, 5, 0, 0) == 11           # too few clusters for MFMA
    # fp64, few clusters of wide samples: streamed twice from a million samples on, else the tiled product
    assert lib.kmx_lloyd_kernel_variant(2_000_000, 100, 10, 1, 0) == 1
    assert lib.kmx_lloyd_kernel_variant(200_000, 100, 10, 1, 0) == 63
    assert lib.kmx_lloyd_kernel_variant(200_000, 100, 10, 1, 0x1) == 1
    assert lib.kmx_lloyd_kernel_variant(2_000_000, 100, 64, 0, 0) == 63    # the wide path only beyond 256 clusters
    assert lib.kmx_lloyd_kernel_variant(2_000_000, 100, 300, 0, 0) == 42
    assert lib.kmx_lloyd_kernel_variant(2_000_000, 100, 10, 0, 0) == 81    # few clusters, wide samples: one read of X
    assert lib.kmx_lloyd_kernel_variant(100_000, 784, 10, 0, 0) == 81
    assert lib.kmx_lloyd_kernel_variant(2_000_000, 100, 10, 0, 0x1) == 1   # on request: the fused vector-ALU step
    assert lib.kmx_lloyd_kernel_variant(100_000, 784, 10, 0, 0x4) == 63    # or the tiled product with sums per bucket
    assert lib.kmx_lloyd_kernel_variant(100_000, 1300, 10, 0, 0) == 81
    assert lib.kmx_lloyd_kernel_variant(100_000, 1800, 10, 0, 0) == 63     # a tile of such samples does not fit the LDS
    assert lib.kmx_lloyd_kernel_variant(2_000_000, 100, 10, 1, 0) == 1     # fp64: as before
    assert lib.kmx_lloyd_kernel_variant(5_000_000, 14, 127, 0, 0x4) == 63  # the tiled product on request
    assert lib.kmx_lloyd_kernel_variant(0, 3, 5, 0, 0) == -2
    assert lib.kmx_lloyd_kernel_variant(10, 3, 5, 4, 0) == -3
    # the caller's flags, and nothing else, move the choice
    F32, SCREEN, REGISTER, STREAM = 0x10, 0x20, 0x2, 0x1
    assert lib.kmx_lloyd_kernel_variant(5_000_000, 14, 127, 0, F32) == 31
    assert lib.kmx_lloyd_kernel_variant(5_000_000, 4, 127, 0, SCREEN) == 61
    assert lib.kmx_lloyd_kernel_variant(5_000_000, 14, 127, 0, REGISTER) == 11
    assert lib.kmx_lloyd_kernel_variant(5_000_000, 14, 127, 0, STREAM) == 1
    assert lib.kmx_lloyd_kernel_variant(1_000_000, 256, 1024, 0, F32) == 42   # same path, labels all fp32
    assert lib.kmx_lloyd_kernel_variant(10, 3, 5, 0, 0x30) == -5    # both label switches
    assert lib.kmx_lloyd_kernel_variant(10, 3, 5, 0, 0x8000) == -5  # unknown bit
    assert lib.kmx_lloyd_kernel_variant(10, 3, 5, 0, 0x3000) == -5  # three sample columns


def test_environment_does_not_reach_the_library(monkeypatch):
    """The library reads no environment variable: only the flags select a kernel.  (The Python
    binding turns the variables into default flags once, when it is imported.)"""
    from sklearn_numba_dpex_amd import _capi
    from sklearn_numba_dpex_amd._capi import lib

    before = lib.kmx_lloyd_kernel_variant(5_000_000, 14, 127, 0, 0)
    monkeypatch.setenv("KMX_LLOYD_ASSIGN", "f32")
    monkeypatch.setenv("KMX_LLOYD_VARIANT", "stream")
    assert lib.kmx_lloyd_kernel_variant(5_000_000, 14, 127, 0, 0) == before == 61
    assert _capi.lloyd_plan(5_000_000, 14, 127, 0, 0).variant == 61
    assert _capi._flags_from_environment() == (_capi.FLAG_LABELS_F32 | _capi.FLAG_PATH_STREAM)
    # no getenv in any source of the library
    import glob
    import os
    for path in glob.glob(os.path.join(os.path.dirname(_capi.__file__), "csrc", "*")):
        assert "getenv" not in open(path).read(), path


def test_lloyd_plan_is_validated():
    """A plan carries shape, flags, variant and workspace size; the calls that take one reject a
    plan they did not make, an edited one, and a workspace smaller than the plan's."""
    from sklearn_numba_dpex_amd import _capi
    from sklearn_numba_dpex_amd._capi import lib

    buf = ctypes.create_string_buffer(1 << 16)
    p = ctypes.addressof(buf)
    plan = _capi.lloyd_plan(1000, 14, 127, 0, 0)
    assert (plan.n, plan.d, plan.k, plan.dtype, plan.flags) == (1000, 14, 127, 0, 0)
    assert plan.variant == 61 and plan.workspace_bytes == lib.kmx_lloyd_workspace_bytes(1000, 14, 127, 0, 0)
    f32 = _capi.lloyd_plan(1000, 14, 127, 0, _capi.FLAG_LABELS_F32)
    assert f32.variant == 31 and f32.workspace_bytes < plan.workspace_bytes   # no per-sample norms
    # a workspace sized for the other variant is too small for this plan
    assert lib.kmx_lloyd_init(plan, p, f32.workspace_bytes, p, p, p, 10, 0.0, None) == -4
    assert lib.kmx_lloyd_iter(plan, p, None, p, p, p, p, p, p, p, p, f32.workspace_bytes, None) == -4
    # flags changed behind the library's back: variant and layout would no longer match
    edited = _capi.LloydPlan.from_buffer_copy(plan)
    edited.flags = _capi.FLAG_LABELS_F32
    assert lib.kmx_lloyd_iter(edited, p, None, p, p, p, p, p, p, p, p, 1 << 16, None) == _capi.KMX_ERR_BAD_PLAN
    edited = _capi.LloydPlan.from_buffer_copy(plan)
    edited.variant = 31
    assert lib.kmx_lloyd_init(edited, p, 1 << 16, p, p, p, 10, 0.0, None) == _capi.KMX_ERR_BAD_PLAN
    edited = _capi.LloydPlan.from_buffer_copy(plan)
    edited.n = 2000
    assert lib.kmx_lloyd_finalize(edited, p, p, p, p, 1 << 16, None) == _capi.KMX_ERR_BAD_PLAN
    assert lib.kmx_lloyd_iter(_capi.LloydPlan(), p, None, p, p, p, p, p, p, p, p, 1 << 16, None) == _capi.KMX_ERR_BAD_PLAN
    assert lib.kmx_lloyd_iter(None, p, None, p, p, p, p, p, p, p, p, 1 << 16, None) == -1
    rechecked = ctypes.c_uint32(7)
    assert lib.kmx_lloyd_recheck_count(edited, p, ctypes.byref(rechecked), None) == _capi.KMX_ERR_BAD_PLAN
    assert "plan" in _capi.error_string(_capi.KMX_ERR_BAD_PLAN)


def test_bad_arguments_are_rejected_without_a_device():
    from sklearn_numba_dpex_amd._capi import lib

    buf = ctypes.create_string_buffer(4096)
    p = ctypes.addressof(buf)
    NULL = None
    from sklearn_numba_dpex_amd import _capi

    plan = _capi.LloydPlan()
    assert lib.kmx_lloyd_plan_init(plan, 0, 2, 2, 0, 0) == -2
    assert lib.kmx_lloyd_plan_init(plan, 10, 2, 2, 9, 0) == -3
    assert lib.kmx_lloyd_plan_init(None, 10, 2, 2, 0, 0) == -1
    assert lib.kmx_lloyd_plan_init(plan, 10, 2, 2, 0, 0) == 0
    assert lib.kmx_lloyd_init(plan, NULL, 0, p, p, p, 10, 0.0, NULL) == -1
    assert lib.kmx_lloyd_init(plan, p, 4096, p, p, p, -1, 0.0, NULL) == -2
    assert lib.kmx_lloyd_init(plan, p, 16, p, p, p, 10, 0.0, NULL) == -4
    assert lib.kmx_lloyd_iter(plan, p, NULL, p, p, p, p, p, p, p, p, 16, NULL) == -4
    assert lib.kmx_lloyd_iter(plan, p, NULL, NULL, p, p, p, p, p, p, p, 4096, NULL) == -1
    assert lib.kmx_assign_labels(p, p, NULL, p, 4096, 10, 2, 2, 0, 0, NULL) == -1
    assert lib.kmx_assign_labels(p, p, p, p, 4096, 10, 2, 2, 0, 0x30, NULL) == -5
    assert lib.kmx_per_sample_inertia(p, NULL, p, p, p, 0, 2, 2, 0, NULL) == -2
    assert lib.kmx_inertia(p, NULL, p, p, p, p, 8, 0, 2, 2, 0, NULL) == -2
    assert lib.kmx_inertia(p, NULL, p, p, p, NULL, 1 << 20, 10, 2, 2, 0, NULL) == -1
    assert lib.kmx_assign_labels_inertia(p, NULL, p, p, p, p, 16, 1000, 14, 127, 0, 0, NULL) == -4
    assert lib.kmx_assign_labels_inertia(p, NULL, p, p, NULL, p, 1 << 30, 1000, 14, 127, 0, 0, NULL) == -1
    assert lib.kmx_assign_inertia_workspace_bytes(1000, 14, 127, 0, 0) > lib.kmx_assign_workspace_bytes_for(1000, 14, 127, 0, 0)
    assert lib.kmx_euclidean_distances(p, p, p, 10, 2, 2, 5, NULL) == -3
    assert lib.kmx_topk_idx(p, p, 5, 10, p, 4096, 0, NULL) == -5      # k > n
    assert lib.kmx_topk_idx(p, p, 50, 10, p, 8, 0, NULL) == -4
    assert lib.kmx_topk_idx_rows(p, p, 0, 50, 10, p, 1 << 20, 0, NULL) == -2   # no rows
    assert lib.kmx_topk_idx_rows(p, NULL, 3, 50, 10, p, 1 << 20, 0, NULL) == -1
    assert lib.kmx_topk_values(p, p, 3, 50, 10, p, 8, 1, NULL) == -4
    assert lib.kmx_topk_values(p, p, 3, 50, 10, p, 1 << 20, 7, NULL) == -3     # unknown dtype
    assert lib.kmx_broadcast_rows(p, p, 2, 2, 3, 0, NULL) == -5       # unknown op
    assert lib.kmx_kpp_init(p, p, 20, p, p, p, 1 << 20, 10, 2, 2, 2, 0, 0, NULL) in (-4, -5)
    assert lib.kmx_kpp_run(p, p, p, 0, p, p, p, 16, 10, 2, 2, 2, 0, 0, NULL) == -4
    assert lib.kmx_kpp_step(p, p, 1, p, p, p, 16, 10, 2, 2, 99, 0, 0, NULL) == -6  # too many trials
    assert lib.kmx_relocate_empty_clusters(p, p, p, p, p, 3, NULL, p, p, 10, 2, 2, 0, NULL) == -2
    assert lib.kmx_sum_rows(p, p, 0, 5, 0, p, 4096, 0, NULL) == -2
    assert lib.kmx_matmul(p, p, NULL, 2, 2, 2, 0, NULL) == -1
    assert lib.kmx_matmul_fused(p, p, p, 2, 2, 2, 3, 0, 0.0, 0, NULL) == -5   # unknown multiply
    assert lib.kmx_matmul_fused(p, p, p, 2, 2, 2, 0, 3, 0.0, 0, NULL) == -5   # unknown output function
    assert lib.kmx_argmin(p, p, 0, 0, NULL) == -2


def test_engine_surface_and_host_checks_without_gpu():
    from sklearn.cluster import KMeans as SkKMeans

    from sklearn_numba_dpex_amd.kmeans.engine import KMeansEngine, NotSupportedByEngineError
    from sklearn_numba_dpex_amd.kmeans.estimator import KMeans

    for method in ["accepts", "prepare_fit", "init_centroids", "kmeans_single", "is_same_clustering",
                   "count_distinct_clusters", "unshift_centers", "prepare_prediction", "get_labels",
                   "get_score", "prepare_transform", "get_euclidean_distances", "convert_to_sklearn_types"]:
        assert callable(getattr(KMeansEngine, method))
    assert KMeansEngine.engine_name == "kmeans"
    engine = KMeansEngine(SkKMeans(algorithm="elkan"))
    assert engine.accepts(np.zeros((3, 2)), None, None) is False
    engine = KMeansEngine(SkKMeans(algorithm="lloyd"))
    assert engine.accepts(np.zeros((3, 2)), None, None) is True
    import scipy.sparse as sp

    assert engine.accepts(sp.csr_matrix(np.eye(3)), None, None) is False
    assert issubclass(KMeans, SkKMeans)
    assert issubclass(NotSupportedByEngineError, Exception)


def test_testing_mode_env_is_validated(monkeypatch):
    from sklearn.cluster import KMeans as SkKMeans

    from sklearn_numba_dpex_amd.kmeans.engine import KMeansEngine, NotSupportedByEngineError

    monkeypatch.setenv("SKLEARN_NUMBA_DPEX_TESTING_MODE", "2")
    with pytest.raises(ValueError, match="SKLEARN_NUMBA_DPEX_TESTING_MODE"):
        KMeansEngine(SkKMeans())
    monkeypatch.setenv("SKLEARN_NUMBA_DPEX_TESTING_MODE", "1")
    with pytest.raises(NotSupportedByEngineError):
        KMeansEngine(SkKMeans(algorithm="elkan")).accepts(np.zeros((3, 2)), None, None)


def test_missing_gpu_fails_loudly():
    import torch

    if torch.cuda.is_available():
        pytest.skip("a GPU is present")
    from sklearn_numba_dpex_amd.kmeans import drivers

    with pytest.raises(RuntimeError, match="needs a ROCm GPU"):
        drivers.get_labels_inertia(torch.zeros(2, 3), torch.zeros(2, 2), torch.ones(3), False)


def test_plans_for_arrays_past_32_bit_limits():
    """Which kernel a plan chooses follows from what the kernel can address: the screened fused
    step numbers tiles and samples with 32 bits (n < 2^29) and takes its fast path only while
    d * n * 4 < 2^32 (decided per launch); the bucketed sums and the wide path keep 32-bit sample
    orders (n <= INT32_MAX); past that only the fused vector-ALU kernels and the all-fp32 / fp64
    matrix-core steps, whose index arithmetic is 64-bit throughout, are planned.  The other entry
    points refuse what they cannot address."""
    from sklearn_numba_dpex_amd._capi import lib

    big = 1 << 31
    assert lib.kmx_lloyd_kernel_variant((1 << 29) - 1, 14, 127, 0, 0) == 61
    assert lib.kmx_lloyd_kernel_variant(1 << 29, 14, 127, 0, 0) == 31          # all-fp32 step, 64-bit tiles
    assert lib.kmx_lloyd_kernel_variant(big, 14, 127, 0, 0) == 31
    assert lib.kmx_lloyd_kernel_variant(1 << 29, 256, 512, 0, 0) == 42         # wide, screen off (n >= 2^29)
    assert lib.kmx_lloyd_kernel_variant(big, 14, 1270, 0, 0) in (2, 12)        # no 32-bit sample order past 2^31
    assert lib.kmx_lloyd_kernel_variant(big, 300, 3000, 0, 0) == 2
    assert lib.kmx_lloyd_kernel_variant(big, 32, 64, 1, 0) == 51
    assert lib.kmx_lloyd_kernel_variant(3_000_000_000, 8, 5000, 1, 0) == 12
    # forcing the tiled product or the wide path on such an input does not produce a plan that uses them
    assert lib.kmx_lloyd_kernel_variant(big, 300, 3000, 0, 0x4) == 2
    assert lib.kmx_lloyd_kernel_variant(big, 14, 1270, 0, 0x3) in (2, 12)
    # arrays past 2^31 ELEMENTS with fewer samples keep the fast kernels
    assert lib.kmx_lloyd_kernel_variant(4_300_000, 512, 300, 0, 0) == 63
    assert lib.kmx_lloyd_kernel_variant(8_500_000, 256, 512, 0, 0) == 42
    assert lib.kmx_lloyd_kernel_variant(34_000_000, 64, 64, 0, 0) == 61
    # kmeans++ and top-k address samples with 32 bits
    assert lib.kmx_kpp_workspace_bytes(big, 8, 4, 3, 0) > 0
    p = ctypes.c_void_p(4096)
    assert lib.kmx_kpp_init(p, p, 0, p, p, p, 1 << 62, big, 8, 4, 3, 0, 0, None) == -2
    assert lib.kmx_argmin(p, p, big, 0, None) == -2
