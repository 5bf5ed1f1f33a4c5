"""The engine behind the estimator, against scikit-learn: the reference's integration tests
(sklearn_numba_dpex/kmeans/tests/test_kmeans.py) restated for this engine, plus the forced
empty-cluster configuration and input/ error handling."""

import numpy as np
import pytest
from numpy.testing import assert_array_equal
from sklearn.base import clone
from sklearn.cluster import KMeans as SkKMeans
from sklearn.cluster._kmeans import _is_same_clustering
from sklearn.datasets import make_blobs
from sklearn.utils._testing import assert_allclose

from oracle import datasets
from oracle import kmeans as ok
from tests._parity import assert_centers_close, assert_labels_match

pytestmark = pytest.mark.gpu

DTYPES = [np.float32, np.float64]


def _np(v):
    return v.cpu().numpy() if hasattr(v, "cpu") else np.asarray(v)


def _as_cuda(a, dtype):
    import torch

    return torch.as_tensor(np.asarray(a, dtype=dtype), device="cuda")


# reference test_kmeans.py:28-110
@pytest.mark.parametrize("kind", ["numpy", "torch_cuda", "torch_cuda+convert", "numpy_fortran"])
@pytest.mark.parametrize("dtype", DTYPES)
def test_kmeans_same_results(cuda, dtype, kind):
    from sklearn_numba_dpex_amd.kmeans.estimator import KMeans, config_context

    X, _ = make_blobs(random_state=42)
    X = X.astype(dtype)
    X_array = {"numpy": X, "numpy_fortran": np.asfortranarray(X)}.get(kind)
    if X_array is None:
        X_array = _as_cuda(X, dtype)
    convert = "sklearn_types" if kind.endswith("+convert") else None

    kmeans_truth = SkKMeans(random_state=42, algorithm="lloyd", max_iter=2, n_init=2, init="random")
    kmeans_engine = KMeans(**kmeans_truth.get_params())
    kmeans_truth.fit(X)
    with config_context(engine_attributes=convert):
        kmeans_engine.fit(X_array)
    if convert:
        assert isinstance(kmeans_engine.labels_, np.ndarray) and isinstance(kmeans_engine.cluster_centers_, np.ndarray)

    def same_fit():
        assert_array_equal(kmeans_truth.labels_, _np(kmeans_engine.labels_))
        assert_allclose(kmeans_truth.cluster_centers_, _np(kmeans_engine.cluster_centers_))
        assert_allclose(kmeans_truth.inertia_, kmeans_engine.inertia_)
        assert kmeans_truth.n_iter_ == kmeans_engine.n_iter_

    same_fit()
    assert_array_equal(kmeans_truth.fit_predict(X), _np(kmeans_engine.fit_predict(X_array)))
    same_fit()
    assert_allclose(kmeans_truth.fit_transform(X), _np(kmeans_engine.fit_transform(X_array)))
    same_fit()
    assert_array_equal(kmeans_truth.predict(X), _np(kmeans_engine.predict(X_array)))
    assert_allclose(kmeans_truth.score(X), kmeans_engine.score(X_array))
    assert_allclose(kmeans_truth.transform(X), _np(kmeans_engine.transform(X_array)))


# reference test_kmeans.py:113-122
@pytest.mark.parametrize("dtype", DTYPES)
def test_kmeans_predict_centers(cuda, dtype):
    from sklearn_numba_dpex_amd.kmeans.estimator import KMeans

    kmeans = KMeans(n_clusters=10)
    centers = kmeans.cluster_centers_ = _as_cuda(np.arange(100).reshape(10, 10), dtype)
    kmeans.n_features_in_ = 10
    assert_array_equal(_np(kmeans.predict(centers)), np.arange(10))


# reference test_kmeans.py:125-158
@pytest.mark.parametrize("dtype", DTYPES)
def test_kmeans_relocated_clusters(cuda, dtype):
    from sklearn_numba_dpex_amd.kmeans.estimator import KMeans

    X = np.array([[0, 0], [0.5, 0], [0.5, 1], [1, 1]], dtype=dtype)
    init_centers = np.array([[0.5, 0.5], [3, 3]], dtype=dtype)
    kmeans = KMeans(n_clusters=2, n_init=1, init=init_centers).fit(X)
    assert_allclose(kmeans.inertia_, 0.25)
    assert kmeans.n_iter_ == 3
    labels, centers = _np(kmeans.labels_), _np(kmeans.cluster_centers_)
    if labels[0] == 0:
        assert_array_equal(labels, [0, 0, 1, 1])
        assert_allclose(centers, [[0.25, 0], [0.75, 1]])
    else:
        assert_array_equal(labels, [1, 1, 0, 0])
        assert_allclose(centers, [[0.75, 1.0], [0.25, 0.0]])


# reference test_kmeans.py:161-179
@pytest.mark.parametrize("dtype", DTYPES)
def test_euclidean_distance(cuda, dtype):
    from sklearn_numba_dpex_amd.kmeans.engine import KMeansEngine

    rng = np.random.default_rng(42)
    a = rng.random(size=(1, 100), dtype=dtype)
    b = rng.standard_normal((1, 100), dtype=dtype)
    estimator = SkKMeans(n_clusters=len(b))
    estimator.cluster_centers_ = b
    estimator.n_features_in_ = 100
    result = KMeansEngine(estimator).get_euclidean_distances(a)
    assert tuple(result.shape) == (1, 1)
    assert_allclose(_np(result), np.sqrt(((a - b) ** 2).sum()), rtol=1e-4 if dtype == np.float32 else 1e-7)


# reference test_kmeans.py:182-205 (signed weights)
@pytest.mark.parametrize("dtype", DTYPES)
def test_inertia(cuda, dtype):
    from sklearn_numba_dpex_amd.kmeans.engine import KMeansEngine

    rng = np.random.default_rng(42)
    X = rng.random((100, 10), dtype=dtype)
    sample_weight = rng.standard_normal(100, dtype=dtype)
    centers = rng.standard_normal((5, 10), dtype=dtype)
    estimator = SkKMeans(n_clusters=len(centers))
    estimator.cluster_centers_ = _as_cuda(centers, dtype)
    estimator.n_features_in_ = 10
    engine = KMeansEngine(estimator)
    X_prepared, sw = engine.prepare_prediction(X, sample_weight)
    labels = _np(engine.get_labels(X_prepared, sw))
    expected = float(np.sum(((X - centers[labels]) ** 2).sum(axis=1) * sample_weight))
    inertia = engine.get_score(X_prepared, sw)
    assert_allclose(float(inertia), expected, rtol=1e-4 if dtype == np.float32 else 1e-6)


# reference test_kmeans.py:208-248
@pytest.mark.parametrize("dtype", DTYPES)
def test_relocate_empty_clusters(cuda, dtype):
    from sklearn_numba_dpex_amd.kmeans.estimator import KMeans

    X = np.array([-10.0, -9.5, -9.0, -8.5, -8.0, -1.0, 1.0, 9.0, 9.5, 10.0], dtype=dtype).reshape(-1, 1)
    init_centers = np.array([-10.0, -10.0, -10.0]).reshape(-1, 1)
    kmeans_truth = SkKMeans(n_clusters=3, n_init=1, max_iter=1, init=init_centers, algorithm="lloyd")
    kmeans_engine = KMeans(**kmeans_truth.get_params())
    kmeans_truth.fit(X)
    kmeans_engine.fit(X)
    truth_labels = kmeans_truth.labels_
    engine_labels = _np(kmeans_engine.labels_).astype(np.int32)
    assert kmeans_truth.n_iter_ == 1 and kmeans_engine.n_iter_ == 1
    assert _is_same_clustering(truth_labels, engine_labels, n_clusters=3)
    assert _is_same_clustering(truth_labels, np.asarray([0, 0, 0, 0, 0, 0, 0, 2, 2, 1], dtype=np.int32), n_clusters=3)
    assert_allclose(kmeans_truth.cluster_centers_[truth_labels], _np(kmeans_engine.cluster_centers_)[engine_labels])
    assert_allclose(kmeans_truth.inertia_, kmeans_engine.inertia_)


def test_forced_empty_clusters_config5(cuda):
    """fp64, 16 of 64 initial centroids far away: they empty on iteration 1 and are relocated
    onto the farthest samples by the radix select; compared with the oracle iteration by
    iteration until the first relocation is through, then on the final result."""
    import torch

    from sklearn_numba_dpex_amd.kmeans import drivers

    cfg = datasets.config5(n=60_000)
    X, init, w, k = cfg["X"], cfg["init"], cfg["sample_weight"], cfg["k"]
    mean = X.mean(axis=0)
    Xc, initc = X - mean, init - mean
    tol = float(np.mean(np.var(Xc, axis=0)) * cfg["tol"])
    X_t = torch.as_tensor(np.ascontiguousarray(Xc.T), device=cuda)
    w_d = torch.as_tensor(w, device=cuda)
    for relocation in ("sklearn", "literal"):
        labels, inertia, centers_t, n_iter = drivers.lloyd(
            X_t, w_d, torch.as_tensor(np.ascontiguousarray(initc.T), device=cuda), True,
            max_iter=1, tol=tol, relocation=relocation)
        it = next(ok.lloyd_iterations(Xc, w, initc, max_iter=1, tol=tol, relocation=relocation))
        assert it["n_empty"] == 16 and n_iter == 1
        assert_centers_close(centers_t.cpu().numpy().T, it["centers"], np.float64, scale_rtol=1e-11)
    labels, inertia, centers_t, n_iter = drivers.lloyd(
        X_t, w_d, torch.as_tensor(np.ascontiguousarray(initc.T), device=cuda), True, max_iter=100, tol=tol)
    ref_labels, ref_inertia, ref_centers, ref_n_iter = ok.lloyd(Xc, w, initc, max_iter=100, tol=tol)
    assert n_iter == ref_n_iter
    assert_labels_match(labels.cpu().numpy(), ref_labels, Xc, ref_centers)
    assert_centers_close(centers_t.cpu().numpy().T, ref_centers, np.float64, scale_rtol=1e-10)
    assert float(inertia) == pytest.approx(float(ref_inertia), rel=1e-12)
    assert len(np.unique(labels.cpu().numpy())) == 64


@pytest.mark.parametrize("d", [100, 784])
def test_forced_empty_clusters_few_clusters_on_wide_samples(cuda, d):
    """fp32, 10 clusters on wide samples (the step that keeps a tile of samples on chip): two of
    the initial centroids lie far away, empty on iteration 1 and are relocated; compared with the
    oracle after that iteration and on the final result."""
    import torch

    from sklearn_numba_dpex_amd import _capi
    from sklearn_numba_dpex_amd.kmeans import drivers

    rng = np.random.default_rng(d)
    n, k = 6_000, 10
    centers = rng.uniform(-1.0, 1.0, (k, d)) * (8.0 / np.sqrt(d))
    X = (centers[rng.integers(0, k, n)] + rng.standard_normal((n, d))).astype(np.float32)
    X -= X.mean(axis=0)
    w = rng.uniform(0.5, 1.5, n).astype(np.float32)
    init = X[rng.choice(n, k, replace=False)].copy()
    init[3] += 100.0
    init[7] -= 100.0
    assert _capi.lloyd_plan(n, d, k, _capi.dtype_code(np.float32), 0).variant == 81
    X_t = torch.as_tensor(np.ascontiguousarray(X.T), device=cuda)
    w_d = torch.as_tensor(w, device=cuda)
    init_t = torch.as_tensor(np.ascontiguousarray(init.T), device=cuda)
    labels, inertia, centers_t, n_iter = drivers.lloyd(X_t, w_d, init_t, True, max_iter=1, tol=0.0)
    it = next(ok.lloyd_iterations(X, w, init, max_iter=1, tol=0.0))
    assert it["n_empty"] == 2 and n_iter == 1
    assert_centers_close(centers_t.cpu().numpy().T, it["centers"], np.float32)
    labels, inertia, centers_t, n_iter = drivers.lloyd(X_t, w_d, init_t, True, max_iter=30, tol=0.0)
    ref_labels, ref_inertia, ref_centers, ref_n_iter = ok.lloyd(X, w, init, max_iter=30, tol=0.0)
    assert n_iter == ref_n_iter
    assert_labels_match(labels.cpu().numpy(), ref_labels, X, ref_centers)
    assert_centers_close(centers_t.cpu().numpy().T, ref_centers, np.float32)
    assert float(inertia) == pytest.approx(float(ref_inertia), rel=1e-5)
    assert len(np.unique(labels.cpu().numpy())) == k


def test_more_clusters_than_distinct_points(cuda):
    from sklearn_numba_dpex_amd.kmeans.estimator import KMeans

    X = np.repeat(np.array([[0.0, 0.0], [1.0, 1.0]]), 5, axis=0)
    init = np.array([[0.0, 0.0], [1.0, 1.0], [5.0, 5.0]])
    with pytest.warns(Warning, match="distinct clusters"):
        km = KMeans(n_clusters=3, n_init=1, init=init).fit(X)
    assert np.isfinite(_np(km.cluster_centers_)).all()
    assert km.inertia_ == pytest.approx(0.0, abs=1e-12)


@pytest.mark.parametrize("dtype", DTYPES)
def test_kmeans_plusplus_fit_quality_and_weights(cuda, dtype):
    from sklearn_numba_dpex_amd.kmeans.estimator import KMeans

    X, y = make_blobs(n_samples=3000, n_features=5, centers=6, cluster_std=0.6, random_state=3)
    X = X.astype(dtype)
    w = np.random.default_rng(0).uniform(0.5, 1.5, 3000).astype(dtype)
    km = KMeans(n_clusters=6, init="k-means++", n_init=1, random_state=0).fit(X, sample_weight=w)
    sk = SkKMeans(n_clusters=6, init="k-means++", n_init=3, random_state=0).fit(X, sample_weight=w)
    assert km.inertia_ <= sk.inertia_ * 1.05
    # uniform scalar weight == no weight
    a = KMeans(n_clusters=6, init=X[:6].copy(), n_init=1).fit(X)
    b = KMeans(n_clusters=6, init=X[:6].copy(), n_init=1).fit(X, sample_weight=np.full(3000, 1.0))
    assert_array_equal(_np(a.labels_), _np(b.labels_))


def test_verbose_output_and_callable_init(cuda, capsys):
    from sklearn_numba_dpex_amd.kmeans.estimator import KMeans

    X, _ = make_blobs(n_samples=500, centers=4, random_state=0)

    def init(X_, n_clusters, random_state):
        return X_[:n_clusters]  # rows of the (centred, device-resident) data the engine passes in

    km = KMeans(n_clusters=4, init=init, n_init=1, verbose=1, max_iter=50).fit(X)
    out = capsys.readouterr().out
    assert "Iteration 0, inertia" in out
    assert "Converged at iteration" in out
    sk = SkKMeans(n_clusters=4, init=X[:4].copy(), n_init=1, max_iter=50).fit(X)
    assert km.n_iter_ == sk.n_iter_
    assert_allclose(_np(km.cluster_centers_), sk.cluster_centers_)


def test_copy_x_false_restores_a_device_input(cuda):
    import torch

    from sklearn_numba_dpex_amd.kmeans.estimator import KMeans

    X, _ = make_blobs(n_samples=400, centers=3, random_state=1)
    X = X + 50.0
    X_dev = torch.as_tensor(np.asfortranarray(X).T.copy(), device=cuda).T  # F-ordered device tensor
    before = X_dev.cpu().numpy().copy()
    KMeans(n_clusters=3, init=X[:3].copy(), n_init=1, copy_x=False).fit(X_dev)
    np.testing.assert_allclose(X_dev.cpu().numpy(), before, rtol=1e-12, atol=1e-9)
    X_np = X.copy()
    KMeans(n_clusters=3, init=X[:3].copy(), n_init=1, copy_x=True).fit(X_np)
    assert_array_equal(X_np, X)
    # copy_x=True on a device tensor that could be centred in place: one copy is made, and the
    # caller's buffer is never written
    KMeans(n_clusters=3, init=X[:3].copy(), n_init=1, copy_x=True).fit(X_dev)
    assert_array_equal(X_dev.cpu().numpy(), before)


def test_input_validation_errors(cuda):
    import scipy.sparse as sp

    from sklearn_numba_dpex_amd.kmeans.engine import KMeansEngine, NotSupportedByEngineError
    from sklearn_numba_dpex_amd.kmeans.estimator import KMeans

    X, _ = make_blobs(n_samples=50, centers=3, random_state=1)
    with pytest.raises(ValueError, match="should be >= n_clusters"):
        KMeans(n_clusters=60, n_init=1).fit(X)
    with pytest.raises(ValueError, match="sample_weight.shape"):
        KMeans(n_clusters=3, n_init=1).fit(X, sample_weight=np.ones(49))
    with pytest.raises(ValueError, match="NaN|infinity"):
        bad = X.copy()
        bad[3, 1] = np.nan
        KMeans(n_clusters=3, n_init=1).fit(bad)
    with pytest.raises(ValueError, match="does not match the number of clusters"):
        KMeans(n_clusters=3, n_init=1, init=X[:4].copy()).fit(X)
    km = KMeans(n_clusters=3, n_init=1, random_state=0).fit(X)
    with pytest.raises(ValueError, match="features"):
        km.predict(X[:, :1])
    with pytest.raises(NotSupportedByEngineError):
        KMeansEngine(SkKMeans())._validate_data(sp.csr_matrix(X))
    # elkan is not accepted: the estimator falls back to scikit-learn
    ek = KMeans(n_clusters=3, n_init=1, algorithm="elkan", random_state=0).fit(X)
    assert isinstance(ek.labels_, np.ndarray)


def test_integer_and_float16_inputs_are_converted(cuda):
    from sklearn_numba_dpex_amd.kmeans.estimator import KMeans

    X, _ = make_blobs(n_samples=300, centers=3, random_state=2)
    Xi = np.round(X * 10).astype(np.int64)
    km = KMeans(n_clusters=3, init=Xi[:3].astype(np.float64), n_init=1).fit(Xi)
    sk = SkKMeans(n_clusters=3, init=Xi[:3].astype(np.float64), n_init=1).fit(Xi)
    assert_array_equal(_np(km.labels_), sk.labels_)
    assert_allclose(_np(km.cluster_centers_), sk.cluster_centers_)


# reference benchmark/kmeans.py:137-207: every provider runs max_iter iterations from the same
# centroids and returns the same clustering
def test_benchmark_cli_consistency(cuda, capsys):
    from sklearn_numba_dpex_amd.benchmark import kmeans as bench_cli

    rc = bench_cli.main(["--dataset", "config1", "--n-data-samples", "30000", "--n-clusters", "31",
                         "--max-iter", "5", "--run-consistency-checks"])
    assert rc == 0
    out = capsys.readouterr().out
    assert "KMeansEngine ... done" in out and "consistency:" in out


class _DLPackOnly:
    """An array that offers nothing but the DLPack protocol (stands for dpnp / cupy arrays)."""

    def __init__(self, tensor):
        self._t = tensor

    def __dlpack__(self, stream=None):
        return self._t.__dlpack__()

    def __dlpack_device__(self):
        return self._t.__dlpack_device__()


# reference test_kmeans.py:28-37: the engine takes device arrays of another library
@pytest.mark.parametrize("dtype", [np.float32, np.float64])
def test_dlpack_inputs_give_the_same_fit(cuda, dtype):
    import torch

    from sklearn_numba_dpex_amd.kmeans.estimator import KMeans, config_context

    rng = np.random.default_rng(5)
    X = rng.normal(size=(500, 6)).astype(dtype)
    w = rng.uniform(0.5, 2.0, 500).astype(dtype)
    init = X[:7].copy()
    with config_context(engine_attributes="sklearn_types"):
        a = KMeans(n_clusters=7, init=init, n_init=1, max_iter=20, tol=0).fit(X, sample_weight=w)
        b = KMeans(n_clusters=7, init=init, n_init=1, max_iter=20, tol=0).fit(
            _DLPackOnly(torch.as_tensor(X, device=cuda)), sample_weight=_DLPackOnly(torch.as_tensor(w, device=cuda)))
    np.testing.assert_array_equal(a.labels_, b.labels_)
    # this small shape runs the vector-ALU kernel, whose sums go through floating-point LDS
    # atomics in an order that varies from run to run (only the matrix-core fp32 kernels, with
    # their fixed-point sums, are bit-reproducible: tests/test_gpu_full_size.py checks that)
    if dtype == np.float32:
        np.testing.assert_allclose(a.cluster_centers_, b.cluster_centers_, rtol=2e-6, atol=1e-6)
    else:
        np.testing.assert_allclose(a.cluster_centers_, b.cluster_centers_, rtol=1e-12, atol=1e-13)
    assert a.n_iter_ == b.n_iter_


def test_numpy_inputs_are_uploaded_through_pinned_staging(cuda):
    """Large numpy inputs travel through two pinned staging buffers (several chunks, a ragged
    last one); the device copy is bit-identical to the host array, for every dtype and for
    sizes below the staging threshold (plain copy)."""
    import torch

    from sklearn_numba_dpex_amd.common import _buffers

    rng = np.random.default_rng(5)
    for shape, dtype in (((3_000_017, 7), np.float32), ((1_100_003, 9), np.float64), ((4_000_001,), np.float32),
                         ((1000, 3), np.float32), ((9_000_001,), np.int32)):
        a = rng.standard_normal(shape).astype(dtype) if np.issubdtype(dtype, np.floating) \
            else rng.integers(-5, 5, shape).astype(dtype)
        t = _buffers.upload(a, cuda)
        assert t.device.type == "cuda" and tuple(t.shape) == shape
        np.testing.assert_array_equal(t.cpu().numpy(), a)
    assert _buffers._stage is not None and _buffers._stage[0][0].is_pinned()
    # and the engine takes that route: a fit from numpy equals a fit from a device tensor
    X = rng.standard_normal((400_000, 6)).astype(np.float32) + rng.integers(0, 4, (400_000, 1)).astype(np.float32) * 5
    w = rng.uniform(0.5, 1.5, 400_000).astype(np.float32)
    init = X[:4].copy()
    from sklearn_numba_dpex_amd.kmeans.estimator import KMeans

    a = KMeans(n_clusters=4, init=init, n_init=1, max_iter=5, tol=0).fit(X, sample_weight=w)
    b = KMeans(n_clusters=4, init=init, n_init=1, max_iter=5, tol=0).fit(torch.as_tensor(X, device=cuda),
                                                                       sample_weight=torch.as_tensor(w, device=cuda))
    # (four clusters: the vector-ALU step with floating-point atomics, reproducible to rounding only)
    # (one blob sits at the origin: its centroid's coordinates are noise around zero, hence the absolute term)
    np.testing.assert_allclose(_np(a.cluster_centers_), _np(b.cluster_centers_), rtol=1e-5, atol=1e-5)


# The same estimator-level comparison (reference test_kmeans.py:28-110) on shapes that take every
# family of label kernels: screened / all-fp32 / fp64 matrix-core steps, the wide path, the tiled
# product with bucketed sums, the fp64 matrix-core labels with bucketed sums and the vector-ALU
# steps.  A fit from the same explicit centres must follow scikit-learn's iterations: same number
# of iterations, the same labels up to samples on a boundary, inertia and centres to rounding.
@pytest.mark.parametrize("shape", [(20_000, 14, 127, np.float32, 61), (20_000, 4, 30, np.float32, 31), (20_000, 40, 30, np.float32, 61),
                                   (20_000, 32, 64, np.float64, 71), (20_000, 64, 100, np.float64, 51),
                                   (6_000, 70, 300, np.float32, 42),
                                   (6_000, 300, 40, np.float32, 63), (6_000, 100, 100, np.float64, 63),
                                   (20_000, 32, 400, np.float64, 53), (20_000, 100, 10, np.float32, 81),
                                   (20_000, 100, 10, np.float64, 63), (1_000_000, 66, 4, np.float64, 1),
                                   (20_000, 20, 8, np.float64, 11), (1_500, 784, 10, np.float32, 81),
                                   (6_000, 300, 20, np.float32, 63)])
def test_fit_follows_scikit_learn_on_every_kernel_family(cuda, shape):
    from sklearn_numba_dpex_amd import _capi
    from sklearn_numba_dpex_amd.kmeans.estimator import KMeans

    n, d, k, dtype, variant = shape
    assert _capi.lloyd_plan(n, d, k, _capi.dtype_code(dtype), None).variant == variant
    rng = np.random.default_rng(n + d + k)
    centers = (rng.uniform(-1.0, 1.0, (k, d)) * (6.0 / np.sqrt(d))).astype(dtype)
    X = centers[rng.integers(0, k, n)] + rng.standard_normal((n, d)).astype(dtype)
    init = X[rng.choice(n, k, replace=False)].copy()
    truth = SkKMeans(n_clusters=k, init=init, n_init=1, max_iter=8, tol=0.0, algorithm="lloyd").fit(X)
    engine = KMeans(n_clusters=k, init=init, n_init=1, max_iter=8, tol=0.0).fit(X)
    assert engine.n_iter_ == truth.n_iter_
    differ = int(np.count_nonzero(_np(engine.labels_) != truth.labels_))
    assert differ <= n // 1000, f"{differ} labels differ"
    rtol = 1e-4 if dtype == np.float32 else 1e-9
    assert_allclose(engine.inertia_, truth.inertia_, rtol=rtol)
    if differ == 0:
        assert_allclose(_np(engine.cluster_centers_), truth.cluster_centers_, rtol=rtol, atol=rtol)
    assert_array_equal(_np(engine.predict(X)), _np(engine.labels_))
    assert_allclose(_np(engine.transform(X[:256])), truth.transform(X[:256]) if differ == 0 else
                    np.sqrt(((X[:256, None, :].astype(np.float64) - _np(engine.cluster_centers_)[None]) ** 2).sum(2)),
                    rtol=rtol * 10, atol=rtol * 10)


@pytest.mark.parametrize("bad", [np.nan, np.inf, -np.inf])
@pytest.mark.parametrize("kind", ["numpy", "torch_cuda"])
def test_non_finite_input_is_refused_like_scikit_learn(cuda, kind, bad):
    """The finiteness check runs on the device; the error is scikit-learn's."""
    from sklearn_numba_dpex_amd.kmeans.estimator import KMeans

    X, _ = make_blobs(n_samples=300, random_state=1)
    X = X.astype(np.float32)
    km = KMeans(n_clusters=3, n_init=1, random_state=0).fit(X)
    X_bad = X.copy()
    X_bad[17, 1] = bad
    expected = None
    try:
        SkKMeans(n_clusters=3, n_init=1).fit(X_bad)
    except ValueError as e:
        expected = str(e)
    assert expected is not None
    arg = X_bad if kind == "numpy" else _as_cuda(X_bad, np.float32)
    for call in (lambda: KMeans(n_clusters=3, n_init=1).fit(arg), lambda: km.predict(arg), lambda: km.transform(arg),
                 lambda: km.score(arg)):
        with pytest.raises(ValueError) as err:
            call()
        assert str(err.value) == expected


def test_finite_input_whose_sum_overflows_is_accepted(cuda):
    """The check sums the array first; finite values whose sum overflows must still pass."""
    from sklearn_numba_dpex_amd.kmeans.estimator import KMeans

    X, _ = make_blobs(n_samples=300, random_state=1)
    X = X.astype(np.float32)
    km = KMeans(n_clusters=3, n_init=1, random_state=0).fit(X)
    X_big = X.copy()
    X_big[5, 0] = X_big[9, 0] = 3e38
    with np.errstate(over="ignore"):
        assert not np.isfinite(X_big.sum(dtype=np.float32))
    keep = np.ones(300, dtype=bool)
    keep[[5, 9]] = False
    for arg in (X_big, _as_cuda(X_big, np.float32)):
        assert_array_equal(_np(km.predict(arg))[keep], _np(km.predict(X))[keep])
