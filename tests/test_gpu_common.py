"""GPU parity of the shared kernels (sums, argmin, top-k, elementwise, matmul, label helpers),
restating the reference's common/tests and kmeans/tests cases against numpy."""

import numpy as np
import pytest

from oracle import kmeans as ok

pytestmark = pytest.mark.gpu

DTYPES = [np.float32, np.float64]


def _dev(a, cuda):
    import torch

    return torch.as_tensor(np.ascontiguousarray(a), device=cuda)


# reference common/tests/test_reductions.py:16-68
@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("axis", [0, 1])
@pytest.mark.parametrize("shape", [(1, 1), (1, 3), (3, 1), (3, 5), (5, 3), (3, 4), (4, 3), (3, 9), (7, 20011)])
def test_sum_reduction_2d(cuda, shape, axis, dtype):
    from sklearn_numba_dpex_amd.common.reductions import sum_reduction

    a = np.arange(shape[0] * shape[1], dtype=dtype).reshape(shape) % 1000
    got = sum_reduction(_dev(a, cuda), axis=axis).cpu().numpy()
    np.testing.assert_allclose(got, a.sum(axis=axis, dtype=np.float64), rtol=1e-6)


@pytest.mark.parametrize("dtype", DTYPES)
def test_sum_reduction_1d_square_and_determinism(cuda, dtype):
    from sklearn_numba_dpex_amd.common.reductions import sum_reduction

    for length, expected in [(4, 6), (5, 10)]:
        assert sum_reduction(_dev(np.arange(length, dtype=dtype), cuda)).cpu().numpy()[0] == pytest.approx(expected)
    rng = np.random.default_rng(0)
    v = rng.normal(size=3_000_017).astype(dtype)
    d = _dev(v, cuda)
    s1 = sum_reduction(d, square=True).cpu().numpy()[0]
    s2 = sum_reduction(d, square=True).cpu().numpy()[0]
    assert s1 == s2  # fixed summation order
    assert s1 == pytest.approx(float(np.sum(v.astype(np.float64) ** 2)), rel=1e-6)


# reference common/tests/test_reductions.py:109-133
@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("values, expected", [([3.0, 1.0, 0.0, 2.0], 2), ([0.0, 1.0, 3.0, 2.0], 0),
                                              ([3.0, 1.0, 2.0, -1.0, -2.0], 4), ([5.0, 1.0, 1.0, 7.0], 1)])
def test_argmin(cuda, values, expected, dtype):
    import torch

    from sklearn_numba_dpex_amd.common.reductions import argmin_reduction

    out = argmin_reduction(_dev(np.array(values, dtype=dtype), cuda))
    assert out.dtype == torch.int32
    assert int(out.cpu()[0]) == expected
    rng = np.random.default_rng(1)
    big = rng.normal(size=50_000).astype(dtype)
    big[[123, 40_000]] = -100.0
    assert int(argmin_reduction(_dev(big, cuda)).cpu()[0]) == 123


TOPK_CASES = [
    [0, 1, -2, -3, 4, -5, 6, 7, 8, -9, 10],
    [0, 8, -2, -3, 4, -5, 6, 7, 8, -9, 10],
    [0, 8, -2, -3, 4, -5, 6, 7, 8, -9, 8],
    [0, 8, 8, -3, 4, -5, 6, 7, 8, -9, 10],
    [0, 8, 8, -3, 4, -5, 6, 7, 8, -9, 8],
    [8, 8, 8, 8, 8, 8, 8, 8, 8, 8, 8],
]


# reference common/tests/test_topk.py:28-59 (+ our deterministic order policy)
@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("k", [1, 3, 11])
@pytest.mark.parametrize("case", range(len(TOPK_CASES)))
def test_topk_handcrafted(cuda, case, k, dtype):
    from sklearn_numba_dpex_amd.common.topk import topk, topk_idx

    a = np.array(TOPK_CASES[case], dtype=dtype)
    idx = topk_idx(_dev(a, cuda), k).cpu().numpy()
    np.testing.assert_array_equal(idx, ok.top_k_indices(a, k))  # descending value, ascending index
    np.testing.assert_array_equal(np.sort(a[idx]), np.sort(a)[-k:])
    np.testing.assert_array_equal(np.sort(topk(_dev(a, cuda), k).cpu().numpy()), np.sort(a)[-k:])


@pytest.mark.parametrize("dtype", DTYPES)
def test_topk_multirow_and_random(cuda, dtype):
    from sklearn_numba_dpex_amd.common.topk import topk, topk_idx

    a = np.array(TOPK_CASES, dtype=dtype)
    got = topk(_dev(a, cuda), 3).cpu().numpy()
    np.testing.assert_array_equal(got, -np.sort(-a, axis=1)[:, :3])  # descending
    rng = np.random.default_rng(123)
    # the reference's random case (common/tests/test_topk.py:62-80): 1000 rows of 1000 values;
    # 1001 columns here so that most rows start off a 16-byte boundary
    big = rng.normal(size=(1000, 1001)).astype(dtype)
    d_big = _dev(big, cuda)
    for k in (1, 3, 40):
        idx = topk_idx(d_big, k).cpu().numpy()
        assert idx.shape == (1000, k) and idx.dtype == np.int64
        want = np.stack([ok.top_k_indices(big[r], k) for r in range(big.shape[0])])
        np.testing.assert_array_equal(idx, want)
        vals = topk(d_big, k).cpu().numpy()
        np.testing.assert_array_equal(vals, np.take_along_axis(big, want, axis=1))


@pytest.mark.parametrize("dtype", DTYPES)
def test_topk_dense_threshold_bucket_and_signed_zeros(cuda, dtype):
    """Rows whose largest values share their leading digits: more candidates than the side
    buffer holds (all of [1, 1.25) and a constant row), a quarter-full one (uniform [0, 1)),
    and -0.0 / +0.0, which rank as equal (lowest index first)."""
    from sklearn_numba_dpex_amd.common.topk import topk, topk_idx

    rng = np.random.default_rng(77)
    n = 300_001
    rows = np.stack([
        rng.uniform(1.0, 1.25, n),
        np.full(n, 3.0),
        rng.uniform(0.0, 1.0, n),
        -rng.uniform(1.0, 1.25, n),
    ]).astype(dtype)
    d_rows = _dev(rows, cuda)
    for k in (1, 7, 2000):
        idx = topk_idx(d_rows, k).cpu().numpy()
        want = np.stack([ok.top_k_indices(rows[r], k) for r in range(rows.shape[0])])
        np.testing.assert_array_equal(idx, want)
        np.testing.assert_array_equal(topk(d_rows, k).cpu().numpy(), np.take_along_axis(rows, want, axis=1))
    z = np.array([-1.0, -0.0, 0.0, -0.0, 0.0, -2.0], dtype=dtype)
    np.testing.assert_array_equal(topk_idx(_dev(z, cuda), 3).cpu().numpy(), [1, 2, 3])
    got = topk(_dev(z, cuda), 3).cpu().numpy()
    np.testing.assert_array_equal(np.signbit(got), [True, False, True])  # the stored values, bit for bit


@pytest.mark.parametrize("dtype", DTYPES)
def test_topk_edges(cuda, dtype):
    """k = n, a single value, infinities, and more rows than one grid dimension holds."""
    from sklearn_numba_dpex_amd.common.topk import topk, topk_idx

    rng = np.random.default_rng(9)
    v = rng.normal(size=37).astype(dtype)
    np.testing.assert_array_equal(topk_idx(_dev(v, cuda), 37).cpu().numpy(), ok.top_k_indices(v, 37))
    np.testing.assert_array_equal(topk_idx(_dev(v[:1], cuda), 1).cpu().numpy(), [0])
    w = v.copy()
    w[[3, 20]] = np.inf
    w[[5, 6]] = -np.inf
    np.testing.assert_array_equal(topk_idx(_dev(w, cuda), 4).cpu().numpy(), ok.top_k_indices(w, 4))
    np.testing.assert_array_equal(topk(_dev(w, cuda), 37).cpu().numpy()[-2:], [-np.inf, -np.inf])
    many = rng.normal(size=(70_000, 5)).astype(dtype)  # 70 000 rows: two slices of the grid
    got = topk_idx(_dev(many, cuda), 2).cpu().numpy()
    want = np.argsort(-many, axis=1, kind="stable")[:, :2]
    np.testing.assert_array_equal(got, want)


@pytest.mark.parametrize("dtype", DTYPES)
def test_topk_large_with_ties_and_negatives(cuda, dtype):
    from sklearn_numba_dpex_amd.common.topk import topk_idx

    rng = np.random.default_rng(5)
    v = rng.normal(size=1_000_003).astype(dtype)
    v[rng.choice(v.size, 5000, replace=False)] = np.float32(2.5)  # many ties at the threshold
    v[::7] *= -1
    for k in (1, 16, 300):
        idx = topk_idx(_dev(v, cuda), k).cpu().numpy()
        np.testing.assert_array_equal(idx, ok.top_k_indices(v, k))
    with pytest.raises(ValueError, match="Expected k to be greater than or equal"):
        topk_idx(_dev(v[:5], cuda), 6)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("n", [1, 63, 1_024, 4_097, 65_537, 262_145, 1_048_577, 4_200_003, 16_000_001])
def test_topk_of_one_row_for_small_k(cuda, dtype, n):
    """One row and k <= 64 take the path that reads the row once (per workgroup the k largest via
    the thread maxima, then one workgroup over the workgroups' results): every tier of elements
    per thread, rows that are sorted either way (all the large values in one thread or one in
    each), constant rows and rows of few distinct values (ties everywhere: lowest index first)."""
    from sklearn_numba_dpex_amd.common.topk import topk, topk_idx

    rng = np.random.default_rng(n)
    rows = {
        "random": rng.normal(size=n),
        "ascending": np.arange(n, dtype=np.float64),
        "descending": -np.arange(n, dtype=np.float64),
        "constant": np.full(n, -1.5),
        "few values": rng.integers(0, 3, n).astype(np.float64),
    }
    for name, v in rows.items():
        v = v.astype(dtype)
        d_v = _dev(v, cuda)
        for k in (1, 16, 64):
            if k > n:
                continue
            want = ok.top_k_indices(v, k)
            np.testing.assert_array_equal(topk_idx(d_v, k).cpu().numpy(), want, err_msg=f"{name}, k={k}")
        k = min(5, n)
        np.testing.assert_array_equal(topk(d_v, k).cpu().numpy(), v[ok.top_k_indices(v, k)], err_msg=name)


@pytest.mark.parametrize("dtype", DTYPES)
def test_elementwise_kernels(cuda, dtype):
    from sklearn_numba_dpex_amd.common import kernels

    rng = np.random.default_rng(2)
    a = rng.normal(size=(5, 1003)).astype(dtype)
    v_rows = rng.normal(size=5).astype(dtype)
    v_cols = rng.uniform(1, 2, 1003).astype(dtype)
    d = _dev(a, cuda)
    np.testing.assert_array_equal(kernels.half_l2_norm(d).cpu().numpy().shape, (1003,))
    np.testing.assert_allclose(kernels.half_l2_norm(d).cpu().numpy(), ok.half_sq_norms(a.T), rtol=1e-6)
    kernels.broadcast_rows(d, _dev(v_rows, cuda), "minus")
    np.testing.assert_array_equal(d.cpu().numpy(), a - v_rows[:, None])
    kernels.broadcast_rows(d, _dev(v_rows, cuda), "plus")
    np.testing.assert_allclose(d.cpu().numpy(), a, atol=1e-6)
    d = _dev(a, cuda)
    kernels.broadcast_division(d, _dev(v_cols, cuda))
    np.testing.assert_array_equal(d.cpu().numpy(), a / v_cols[None, :])
    d = _dev(a, cuda)
    kernels.divide_by(d, 7.0)
    np.testing.assert_array_equal(d.cpu().numpy(), a / dtype(7.0))
    b = rng.normal(size=(5, 1003)).astype(dtype)
    np.testing.assert_allclose(kernels.centroid_shifts(_dev(a, cuda), _dev(b, cuda)).cpu().numpy(),
                               ((a - b) ** 2).sum(axis=0), rtol=1e-6)
    kernels.initialize_to_zeros(d)
    assert float(d.abs().sum()) == 0.0


# reference common/tests/test_matmul.py:71-127
@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("shape", [(1, 1, 1), (3, 5, 2), (16, 16, 16), (65, 17, 130), (1999, 661, 563), (128, 4, 128),
                                   (257, 33, 129), (300, 70, 200), (1024, 256, 512)])
def test_matmul(cuda, shape, dtype):
    from sklearn_numba_dpex_amd.common.matmul import matmul

    m, p, q = shape
    rng = np.random.default_rng(0)
    X = rng.normal(size=(m, p)).astype(dtype)
    Y_t = rng.normal(size=(q, p)).astype(dtype)
    got = matmul(_dev(X, cuda), _dev(Y_t, cuda)).cpu().numpy()
    np.testing.assert_allclose(got, X.astype(np.float64) @ Y_t.astype(np.float64).T,
                               rtol=1e-4 if dtype == np.float32 else 1e-11, atol=1e-4 if dtype == np.float32 else 1e-11)


# the reference's small shapes with `arange` operands (common/tests/test_matmul.py:13-16,71-104)
@pytest.mark.parametrize("shapes", [((1, 1), (1, 1)), ((4, 4), (4, 4)), ((5, 5), (5, 5)), ((1, 4), (4, 1)),
                                    ((1, 5), (5, 1)), ((4, 1), (1, 4)), ((5, 1), (1, 5)), ((4, 5), (5, 4)),
                                    ((5, 4), (4, 5)), ((5, 4), (4, 8)), ((5, 4), (4, 10)), ((4, 5), (5, 10)),
                                    ((10, 4), (4, 5)), ((5, 10), (10, 4)), ((1999, 661), (661, 563))])
def test_matmul_arange(cuda, shapes):
    from sklearn_numba_dpex_amd.common.matmul import matmul

    (m, p), (_, q) = shapes
    X = np.arange(m * p, dtype=np.float32).reshape(m, p)
    Y = np.arange(p * q, dtype=np.float32).reshape(p, q)
    got = matmul(_dev(X, cuda), _dev(np.ascontiguousarray(Y.T), cuda)).cpu().numpy()
    np.testing.assert_allclose(got, np.matmul(X, Y), rtol=1e-5)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("shape", [(3, 5, 2), (65, 17, 130), (257, 33, 129), (1000, 70, 300)])
def test_matmul_fused_functions(cuda, shape, dtype):
    """multiply_fn and out_fused_elementwise_fn of make_matmul_2d_kernel (reference
    common/matmul.py:55-66) for the functions the reference predefines (common/_utils.py:17-33)."""
    from sklearn_numba_dpex_amd.common import _utils
    from sklearn_numba_dpex_amd.common.matmul import matmul

    m, p, q = shape
    rng = np.random.default_rng(3)
    X = rng.normal(size=(m, p)).astype(dtype)
    Y_t = rng.normal(size=(q, p)).astype(dtype)
    X64, Y64 = X.astype(np.float64), Y_t.astype(np.float64)
    tol = dict(rtol=1e-4, atol=1e-4) if dtype == np.float32 else dict(rtol=1e-11, atol=1e-11)
    dX, dY = _dev(X, cuda), _dev(Y_t, cuda)
    prod = X64 @ Y64.T
    np.testing.assert_allclose(matmul(dX, dY, out_fused_elementwise_fn=_utils._square).cpu().numpy(), prod**2, **tol)
    np.testing.assert_allclose(matmul(dX, dY, out_fused_elementwise_fn=_utils._divide_by(4.0)).cpu().numpy(),
                               prod / 4.0, **tol)
    minus = X64.sum(axis=1)[:, None] - Y64.sum(axis=1)[None, :]
    plus = X64.sum(axis=1)[:, None] + Y64.sum(axis=1)[None, :]
    np.testing.assert_allclose(matmul(dX, dY, multiply_fn=_utils._minus).cpu().numpy(), minus, **tol)
    np.testing.assert_allclose(matmul(dX, dY, multiply_fn=_utils._plus).cpu().numpy(), plus, **tol)
    np.testing.assert_allclose(
        matmul(dX, dY, multiply_fn=_utils._minus, out_fused_elementwise_fn=_utils._square).cpu().numpy(),
        minus**2, rtol=tol["rtol"] * 10, atol=tol["atol"] * 10)
    with pytest.raises(NotImplementedError, match="predefined functions"):
        matmul(dX, dY, multiply_fn=lambda x, y: x * y + 1)


def test_label_helpers(cuda):
    from sklearn_numba_dpex_amd.kmeans import drivers

    # reference kmeans/tests/test_kmeans.py:448-457
    labels = _dev(np.array([0, 1, 0, 2, 2, 7, 6, 5, 3, 3], dtype=np.int32), cuda)
    assert int(drivers.get_nb_distinct_clusters(labels, 8)) == 7
    rng = np.random.default_rng(0)
    a = rng.integers(0, 50, 200_000).astype(np.int32)
    perm = rng.permutation(50).astype(np.int32)
    b = perm[a]
    c = b.copy()
    c[77_777] = (c[77_777] + 1) % 50
    assert drivers.is_same_clustering(_dev(a, cuda), _dev(b, cuda), 50) is True
    assert drivers.is_same_clustering(_dev(a, cuda), _dev(c, cuda), 50) is False
    assert int(drivers.get_nb_distinct_clusters(_dev(a, cuda), 50)) == len(np.unique(a))


# every instantiation of the distance and inertia kernels (register / tiled distances,
# centroids in LDS or not, 128-bit or scalar accesses) against numpy in fp64
@pytest.mark.parametrize("shape", [(1003, 14, 127, np.float32), (4096, 32, 7, np.float32), (777, 33, 5, np.float32),
                                   (1001, 16, 9, np.float64), (500, 17, 3, np.float64), (1000, 300, 50, np.float32),
                                   (3, 2, 2, np.float64), (1000, 70, 130, np.float64), (1028, 100, 64, np.float32),
                                   (515, 129, 67, np.float32), (1026, 48, 66, np.float64),
                                   # few clusters of wide samples: centroid tiles of 16 (one, two), then of 64
                                   (1001, 784, 10, np.float32), (1030, 200, 20, np.float64),
                                   (1000, 65, 32, np.float32), (1000, 65, 33, np.float32)])
def test_distances_and_inertia_kernels(cuda, shape):
    import torch

    from sklearn_numba_dpex_amd.kmeans import drivers

    n, d, k, dtype = shape
    rng = np.random.default_rng(n + d)
    X = rng.normal(size=(n, d)).astype(dtype)
    C = rng.normal(size=(k, d)).astype(dtype)
    w = rng.uniform(0.5, 2.0, n).astype(dtype)
    labels = rng.integers(0, k, n).astype(np.int32)
    X_t, C_t = _dev(X.T, cuda), _dev(C.T, cuda)
    rtol = 2e-5 if dtype == np.float32 else 1e-12
    exact = np.sqrt(((X.astype(np.float64)[:, None, :] - C.astype(np.float64)[None, :, :]) ** 2).sum(axis=2))
    got = drivers.get_euclidean_distances(X_t, C_t).cpu().numpy()
    assert got.shape == (n, k)
    np.testing.assert_allclose(got, exact, rtol=rtol, atol=rtol)
    per_sample = (exact[np.arange(n), labels] ** 2)
    lab_d = torch.as_tensor(labels, device=cuda)
    got_w = drivers._per_sample_inertia(X_t, _dev(w, cuda), C_t, lab_d).cpu().numpy()
    np.testing.assert_allclose(got_w, per_sample * w.astype(np.float64), rtol=rtol * 5, atol=rtol)
    # unit weights through the NULL-weights entry (what the relocation ranks samples by)
    from sklearn_numba_dpex_amd import _capi
    from sklearn_numba_dpex_amd._capi import lib, ptr

    out = torch.empty(n, dtype=X_t.dtype, device=cuda)
    _capi.check(lib.kmx_per_sample_inertia(ptr(X_t), None, ptr(C_t), ptr(lab_d), ptr(out), n, d, k,
                                           _capi.dtype_code(X.dtype), _capi.current_stream()), "inertia")
    np.testing.assert_allclose(out.cpu().numpy(), per_sample, rtol=rtol * 5, atol=rtol)
    # the same kernel with the sum folded in (no per-sample values written)
    total = drivers._inertia_array(X_t, _dev(w, cuda), C_t, lab_d)
    assert total.shape == (1,) and total.dtype == dtype
    np.testing.assert_allclose(total[0], (per_sample * w.astype(np.float64)).sum(), rtol=rtol)
    total_unit = drivers._inertia_array(X_t, None, C_t, lab_d)
    np.testing.assert_allclose(total_unit[0], per_sample.sum(), rtol=rtol)


def test_distances_with_few_samples_split_the_centroids(cuda):
    """With few samples the centroid range is split over the second grid dimension (ragged last
    share, k not a multiple of 4), and exact zeros / tiny distances go through the square root."""
    from sklearn_numba_dpex_amd.kmeans import drivers

    rng = np.random.default_rng(5)
    n, d, k = 2000, 14, 127
    X = rng.normal(size=(n, d)).astype(np.float32)
    C = rng.normal(size=(k, d)).astype(np.float32)
    C[3] = X[10]            # distance exactly 0
    C[4] = X[11] + 1e-20    # below the fast path's range
    exact = np.sqrt(((X.astype(np.float64)[:, None, :] - C.astype(np.float64)[None, :, :]) ** 2).sum(axis=2))
    got = drivers.get_euclidean_distances(_dev(X.T, cuda), _dev(C.T, cuda)).cpu().numpy()
    np.testing.assert_allclose(got, exact, rtol=1e-5, atol=1e-6)
    assert got[10, 3] == 0.0 and np.isfinite(got).all()


@pytest.mark.parametrize("shape", [(5_000, 14), (14, 5_000), (1, 1), (64, 64), (65, 129), (300, 1), (1, 300), (1_000, 784)])
@pytest.mark.parametrize("dtype", [np.float32, np.float64])
def test_transposed_copy(cuda, shape, dtype):
    import torch

    from sklearn_numba_dpex_amd.common.kernels import transposed_copy

    a = np.arange(shape[0] * shape[1], dtype=dtype).reshape(shape)
    got = transposed_copy(_dev(a, cuda))
    assert got.is_contiguous() and tuple(got.shape) == (shape[1], shape[0])
    np.testing.assert_array_equal(got.cpu().numpy(), a.T)
