"""GPU parity of kmeans++ seeding: each kernel family through the C ABI against the oracle's
exact sampler, the whole seeding against the oracle, and the reference's known answer."""

import ctypes

import numpy as np
import pytest

from oracle import datasets
from oracle import kmeans as ok
from oracle import rng as orng

pytestmark = pytest.mark.gpu


def _dev(a, cuda):
    import torch

    return torch.as_tensor(np.ascontiguousarray(a), device=cuda)


def _cases():
    rng = np.random.default_rng(11)
    Xw = rng.normal(size=(5003, 5))
    return {
        "C4": (datasets.config4(n=40_000, d=64, k=24)["X"], None, 24, 3),
        "weighted_f64": (Xw, rng.uniform(0.1, 3.0, 5003), 9, 1),
        "tiny_f32": (rng.normal(size=(37, 2)).astype(np.float32), None, 4, 0),
        "weighted_f32": (rng.normal(size=(4099, 9)).astype(np.float32), rng.uniform(0.1, 3.0, 4099), 17, 6),
        "wide_f32": (rng.normal(size=(3000, 150)).astype(np.float32), None, 5, 2),
        # 2 + floor(ln 3000) = 10 local trials: the 16-trial instantiation of the kernels
        "many_trials_f32": (rng.normal(size=(6001, 7)).astype(np.float32), None, 3000, 4),
        # more than 4 x 256 blocks of 1024 samples: the sampler re-reads its block sums
        "many_blocks_f64": (rng.normal(size=(1_100_003, 2)), None, 6, 5),
        # few samples of many features: the step with the features split over a workgroup's
        # waves, at 1, 2 and 4 samples per thread, with and without a ragged last block
        "short_wide_f32": (rng.normal(size=(70_001, 96)).astype(np.float32), None, 6, 7),
        "short_wide_f64": (rng.normal(size=(100_000, 70)), rng.uniform(0.1, 3.0, 100_000), 5, 8),
        "short_wide_4_f32": (rng.normal(size=(200_000, 64)).astype(np.float32), None, 7, 9),
        "short_wide_4_ragged_f32": (rng.normal(size=(140_003, 65)).astype(np.float32), rng.uniform(0.1, 3.0, 140_003), 4, 10),
        "short_wide_1_f64": (rng.normal(size=(2_049, 333)), None, 12, 12),
    }


@pytest.mark.parametrize("sampler", ["scan", "literal"])
@pytest.mark.parametrize("name", ["C4", "weighted_f64", "tiny_f32", "wide_f32", "many_trials_f32", "many_blocks_f64", "weighted_f32",
                                  "short_wide_f32", "short_wide_f64", "short_wide_4_f32", "short_wide_4_ragged_f32",
                                  "short_wide_1_f64"])
def test_whole_seeding_matches_oracle(cuda, name, sampler):
    """Both samplers of the library against their counterparts in the oracle: the fp64 scan
    (default) and the reference's running sum in the compute dtype (`KMX_KPP_SAMPLER_LITERAL`)."""
    from sklearn_numba_dpex_amd.kmeans import drivers

    X, w, k, seed = _cases()[name]
    w = np.ones(len(X), X.dtype) if w is None else w.astype(X.dtype)
    centers_t, idx = drivers.kmeans_plusplus(_dev(X.T, cuda), _dev(w, cuda), k, np.random.RandomState(seed),
                                             sampler=sampler)
    seed64 = orng.seed_from_random_state(np.random.RandomState(seed))
    ref_centers, ref_idx = ok.kmeans_plusplus(X, w, k, seed64, sampler="exact" if sampler == "scan" else "literal")
    idx = idx.cpu().numpy()
    np.testing.assert_array_equal(idx, ref_idx)
    np.testing.assert_array_equal(centers_t.cpu().numpy().T, X[idx])
    assert idx.dtype == np.int32 and np.all((idx >= 0) & (idx < len(X)))


# (n, d, local trials): the plain step; then few samples of many features, where a workgroup's
# waves share the features - more than 8 trials at 2 samples per thread (fp32; fp64 keeps the
# plain step there) and at 1, and 4 samples per thread (fp32 only)
@pytest.mark.parametrize("sampler", ["scan", "literal"])
@pytest.mark.parametrize("dtype", [np.float32, np.float64])
@pytest.mark.parametrize("n,d", [(65_536, 64), (65_537, 64), (131_072, 64), (131_073, 65), (262_144, 64), (262_145, 64),
                                 (70_000, 63), (1, 64), (63, 64), (65, 80)])
def test_seeding_at_the_limits_of_the_feature_split_step(cuda, n, d, dtype, sampler):
    """Sample counts either side of where the step changes its samples per thread (65 536,
    131 072, 262 144; fp64 stops one earlier), one feature short of the split, and arrays of one
    sample, of less than a wave and of one more than a wave: indices equal to the oracle's."""
    from sklearn_numba_dpex_amd.kmeans import drivers

    rng = np.random.default_rng(n + d)
    X = rng.normal(size=(n, d)).astype(dtype)
    w = rng.uniform(0.5, 1.5, n).astype(dtype)
    k = min(3, n)
    centers_t, idx = drivers.kmeans_plusplus(_dev(X.T, cuda), _dev(w, cuda), k, np.random.RandomState(n % 97), sampler=sampler)
    seed64 = orng.seed_from_random_state(np.random.RandomState(n % 97))
    ref_idx = ok.kmeans_plusplus(X, w, k, seed64, sampler="exact" if sampler == "scan" else "literal")[1]
    np.testing.assert_array_equal(idx.cpu().numpy(), ref_idx)
    np.testing.assert_array_equal(centers_t.cpu().numpy().T, X[ref_idx])


@pytest.mark.parametrize("shape", [(10_007, 6, 4), (66_001, 64, 12), (3_001, 70, 10), (140_000, 65, 3)])
@pytest.mark.parametrize("dtype", [np.float32, np.float64])
def test_step_kernels_through_c_abi(cuda, dtype, shape):
    """init -> sample -> step with the same uniforms as the oracle: candidates, potentials and
    the updated closest-distance array all match."""
    import torch

    from sklearn_numba_dpex_amd import _capi
    from sklearn_numba_dpex_amd._capi import lib, ptr

    rng = np.random.default_rng(3)
    (n, d, tn), k = shape, 8 if shape[0] < 20_000 else 4
    X = rng.normal(size=(n, d)).astype(dtype)
    w = rng.uniform(0.5, 1.5, n).astype(dtype)
    dc = _capi.dtype_code(dtype)
    X_t, w_d = _dev(X.T, cuda), _dev(w, cuda)
    centers_t = torch.zeros((d, k), dtype=X_t.dtype, device=cuda)
    indices = torch.full((k,), -1, dtype=torch.int32, device=cuda)
    ws_bytes = lib.kmx_kpp_workspace_bytes(n, d, k, tn, dc)
    ws = torch.zeros(ws_bytes, dtype=torch.uint8, device=cuda)
    st = _capi.current_stream()
    start = 4242 % n
    _capi.check(lib.kmx_kpp_init(ptr(X_t), ptr(w_d), start, ptr(centers_t), ptr(indices), ptr(ws), ws_bytes,
                                 n, d, k, tn, dc, 0, st), "kpp_init")
    closest = (((X - X[start]) ** 2).sum(axis=1, dtype=dtype) * w).astype(dtype)
    rows_ptr = lib.kmx_kpp_closest_ptr(ptr(ws), n, d, k, tn, dc)
    off = rows_ptr - ws.data_ptr()
    itemsize = np.dtype(dtype).itemsize

    def row(r):
        return ws[off + r * n * itemsize: off + (r + 1) * n * itemsize].view(X_t.dtype).cpu().numpy()

    np.testing.assert_allclose(row(0), closest, rtol=1e-5 if dtype == np.float32 else 1e-12)
    closest = row(0).copy()  # continue from the device's own values: later comparisons are exact
    assert int(indices.cpu()[0]) == start
    np.testing.assert_array_equal(centers_t.cpu().numpy()[:, 0], X[start])

    best_row = 0
    for c in range(1, k):
        u = rng.random(tn)
        u[0] = 0.0 if c == 1 else u[0]            # rv == 0 -> first sample (reference would give -1)
        u[1] = 1.0 - 2.0**-53 if c == 2 else u[1]  # top of the range -> last crossing, clipped to n - 1
        cand = torch.empty(tn, dtype=torch.int32, device=cuda)
        # the reference's own sampler first (its candidates are overwritten by the default one):
        # running sum in T; rv <= 0 leaves -1 there, read as an index from the end
        u_T = u.astype(dtype).astype(np.float64)
        _capi.check(lib.kmx_kpp_sample_candidates(ptr(X_t), ptr(_dev(u_T, cuda)), ptr(cand), ptr(ws), ws_bytes, n, d, k,
                                                  tn, dc, _capi.KMX_KPP_SAMPLER_LITERAL, st), "kpp_sample literal")
        total_T = dtype(closest.sum(dtype=np.float64))
        literal = np.array([ok._sample_literal(closest, total_T, dtype(uu)) % n for uu in u_T])
        np.testing.assert_array_equal(cand.cpu().numpy(), literal)
        assert lib.kmx_kpp_sample_candidates(ptr(X_t), ptr(_dev(u, cuda)), ptr(cand), ptr(ws), ws_bytes, n, d, k, tn,
                                             dc, 2, st) == -5
        _capi.check(lib.kmx_kpp_sample_candidates(ptr(X_t), ptr(_dev(u, cuda)), ptr(cand), ptr(ws), ws_bytes, n, d, k, tn,
                                                  dc, _capi.KMX_KPP_SAMPLER_SCAN, st), "kpp_sample")
        expected = np.array([ok._sample_exact(closest, uu) for uu in u])
        np.testing.assert_array_equal(cand.cpu().numpy(), expected)
        _capi.check(lib.kmx_kpp_step(ptr(X_t), ptr(w_d), c, ptr(centers_t), ptr(indices), ptr(ws), ws_bytes,
                                     n, d, k, tn, dc, 0, st), "kpp_step")
        rows = np.stack([np.minimum((((X - X[i]) ** 2).sum(axis=1, dtype=dtype) * w).astype(dtype), closest)
                         for i in expected])
        pots_ptr = lib.kmx_kpp_potentials_ptr(ptr(ws), n, d, k, tn, dc)
        poff = pots_ptr - ws.data_ptr()
        pots = ws[poff: poff + tn * 8].view(torch.float64).cpu().numpy()
        for t in range(tn):
            np.testing.assert_allclose(row(t), rows[t], rtol=1e-5 if dtype == np.float32 else 1e-12)
        got_rows = np.stack([row(t) for t in range(tn)])
        np.testing.assert_allclose(pots, got_rows.sum(axis=1, dtype=np.float64), rtol=1e-12)
        best_row = int(np.argmin(pots))
        assert int(indices.cpu()[c]) == expected[best_row]
        np.testing.assert_array_equal(centers_t.cpu().numpy()[:, c], X[expected[best_row]])
        closest = got_rows[best_row].copy()


@pytest.mark.parametrize("dtype", [np.float32, np.float64])
def test_known_answer_through_the_engine(cuda, dtype):
    """reference kmeans/tests/test_kmeans.py:251-325: mean score over seeds 0..9 of the
    engine's kmeans++ initialisation is -865.257501."""
    from sklearn.cluster import KMeans as SkKMeans
    from sklearn.cluster.tests.test_k_means import X as X_sk, n_clusters

    from sklearn_numba_dpex_amd.kmeans.engine import KMeansEngine

    X = X_sk.astype(dtype)
    kmeans = SkKMeans(n_clusters=n_clusters, init="k-means++")
    kmeans._n_threads = 1
    scores = []
    for random_state in range(10):
        kmeans.set_params(random_state=random_state)
        engine = KMeansEngine(kmeans)
        X_prepared, _, sample_weight = engine.prepare_fit(X)
        centers_t = engine.init_centroids(X_prepared, sample_weight)
        centers = centers_t.T
        engine.unshift_centers(X_prepared, centers)
        kmeans.cluster_centers_ = np.ascontiguousarray(centers.cpu().numpy())
        scores.append(kmeans.score(X))
    np.testing.assert_allclose(np.mean(scores), -865.257501, rtol=1e-7)


def test_output_sanity_and_data_order(cuda):
    """reference kmeans/tests/test_kmeans.py:328-392."""
    from sklearn.cluster import KMeans as SkKMeans
    from sklearn.cluster.tests.test_k_means import X as X_sk, n_clusters

    from sklearn_numba_dpex_amd.kmeans.engine import KMeansEngine

    for dtype in (np.float32, np.float64):
        X = X_sk.astype(dtype)
        sample_weight = np.random.default_rng(42).random(X.shape[0], dtype=dtype)
        est = SkKMeans(init="k-means++", n_clusters=n_clusters, random_state=42)
        engine = KMeansEngine(est)
        X_prepared, _, sw = engine.prepare_fit(X, sample_weight=sample_weight)
        centers_t, indices = engine._kmeans_plusplus(X_prepared, sw)
        centers = centers_t.T
        engine.unshift_centers(X_prepared, centers)
        centers, indices = centers.cpu().numpy(), indices.cpu().numpy()
        assert indices.shape[0] == n_clusters and (indices >= 0).all() and (indices < X.shape[0]).all()
        assert (centers.max(axis=0) <= X.max(axis=0) + 1e-5).all() and (centers.min(axis=0) >= X.min(axis=0) - 1e-5).all()
        np.testing.assert_allclose(X[indices], centers, rtol=1e-5, atol=1e-6)

    est = SkKMeans(init="k-means++", n_clusters=n_clusters, random_state=42)
    engine = KMeansEngine(est)
    Xp, _, sw = engine.prepare_fit(X_sk)
    centers_c = engine.init_centroids(Xp, sw).T.cpu().numpy()
    engine = KMeansEngine(est)
    Xp, _, sw = engine.prepare_fit(np.asfortranarray(X_sk))
    centers_f = engine.init_centroids(Xp, sw).T.cpu().numpy()
    np.testing.assert_allclose(centers_c, centers_f)
