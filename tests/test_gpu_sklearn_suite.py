"""scikit-learn's own KMeans tests, routed through the engine.

The reference's CI runs `sklearn/cluster/tests/test_k_means.py` with the plugin selected and
SKLEARN_NUMBA_DPEX_TESTING_MODE=1 (reference .github/workflows/run_tests.yaml:51-52,
README.md:285-287; the conversions of that mode: kmeans/engine.py:108-115,219-225), expecting
the cases the engine does not cover to fail with NotSupportedByEngineError.  Released
scikit-learn cannot select an engine, so here the module's `KMeans` name is replaced by the
estimator subclass that drives KMeansEngine, and every estimator-level case of the installed
scikit-learn's test module that needs only the public API is called with its own
parametrisation:

  * cases for MiniBatchKMeans, bisecting or the private Cython helpers are not the engine's;
  * `algorithm="elkan"` and sparse inputs must raise NotSupportedByEngineError (asserted, then
    reported as xfail, the reference's convention);
  * everything else must pass unchanged.
"""

import itertools
import os

import numpy as np
import pytest
from _pytest.mark.structures import ParameterSet

pytestmark = pytest.mark.gpu

# Test functions of sklearn.cluster.tests.test_k_means that exercise KMeans through its public
# API (fit / predict / score / transform / fit_* and fitted attributes).
SELECTED = [
    "test_kmeans_results",
    "test_kmeans_relocated_clusters",
    "test_kmeans_convergence",
    "test_all_init",
    "test_kmeans_init_auto_with_initial_centroids",
    "test_fortran_aligned_data",
    "test_kmeans_verbose",
    "test_warning_n_init_precomputed_centers",
    "test_kmeans_copyx",
    "test_score_max_iter",
    "test_kmeans_predict",
    "test_dense_sparse",
    "test_predict_dense_sparse",
    "test_integer_input",
    "test_transform",
    "test_fit_transform",
    "test_n_init",
    "test_float_precision",
    "test_centers_not_mutated",
    "test_kmeans_init_fitted_centers",
    "test_kmeans_warns_less_centers_than_unique_points",
    "test_weighted_vs_repeated",
    "test_unit_weights_vs_no_weights",
    "test_scaled_weights",
    "test_kmeans_empty_cluster_relocated",
    "test_k_means_1_iteration",
    "test_n_init_auto",
    "test_sample_weight_unchanged",
    "test_wrong_params",
    "test_kmeans_with_array_like_or_np_scalar_init",
    "test_feature_names_out",
    "test_predict_does_not_change_cluster_centers",
    "test_sample_weight_init",
    "test_sample_weight_zero",
    "test_relocating_with_duplicates",
]

# Cases whose expectation is tied to scikit-learn's own implementation rather than to the
# estimator's contract; each with the reason it is not asserted here.
NOT_APPLICABLE = {
    "test_kmeans_verbose": "asserts the exact progress text of scikit-learn's Cython loop (the engine prints the "
                           "reference's own messages, kmeans/drivers.py:304-352, covered by tests/test_gpu_engine.py)",
    "test_result_equal_in_diff_n_threads": "thread count of the Cython kernels",
}


def _sk_module():
    import sklearn.cluster.tests.test_k_means as sk

    return sk


def _cases():
    """(function name, kwargs, id) for every parametrisation of the selected functions."""
    sk = _sk_module()
    out = []
    for name in SELECTED:
        fn = getattr(sk, name, None)
        if fn is None:  # another scikit-learn version
            continue
        marks = [m for m in getattr(fn, "pytestmark", []) if m.name == "parametrize"]
        axes = []
        for m in marks:
            argnames = [a.strip() for a in m.args[0].split(",")] if isinstance(m.args[0], str) else list(m.args[0])
            values = []
            for v in m.args[1]:
                is_param = isinstance(v, ParameterSet)  # pytest.param(...)
                vals = v.values if is_param else v
                if len(argnames) == 1 and not is_param:
                    vals = (vals,)
                values.append(dict(zip(argnames, vals)))
            axes.append(values)
        for combo in itertools.product(*axes) if axes else [()]:
            kwargs = {}
            for part in combo:
                kwargs.update(part)
            ident = name + "[" + "-".join(_ident(v) for v in kwargs.values()) + "]"
            out.append(pytest.param(name, kwargs, id=ident))
    return out


def _ident(v):
    if isinstance(v, type) or callable(v):
        return getattr(v, "__name__", repr(v))
    if isinstance(v, np.ndarray):
        return f"ndarray{v.shape}"
    return str(v)[:24]


@pytest.fixture()
def engine_suite(monkeypatch, cuda):
    """The scikit-learn test module with its KMeans replaced by the engine-driven estimator,
    in the plugin's testing mode (numpy in, numpy out)."""
    from sklearn_numba_dpex_amd.kmeans import estimator

    sk = _sk_module()
    monkeypatch.setenv("SKLEARN_NUMBA_DPEX_TESTING_MODE", "1")
    original = sk.KMeans
    monkeypatch.setattr(sk, "KMeans", estimator.KMeans)
    return sk, original, estimator.KMeans


@pytest.mark.parametrize("name, kwargs", _cases())
def test_scikit_learn_kmeans_case(engine_suite, name, kwargs, capsys):
    import inspect

    import scipy.sparse as sp
    from sklearn.cluster import MiniBatchKMeans

    from sklearn_numba_dpex_amd.kmeans.engine import NotSupportedByEngineError

    sk, stock_kmeans, engine_kmeans = engine_suite
    if name in NOT_APPLICABLE:
        pytest.skip(NOT_APPLICABLE[name])
    kwargs = dict(kwargs)
    for key, value in list(kwargs.items()):
        if value is MiniBatchKMeans:
            pytest.skip("MiniBatchKMeans is not an engine of the reference")
        if value is stock_kmeans:
            kwargs[key] = engine_kmeans
    fn = getattr(sk, name)
    wanted = inspect.signature(fn).parameters
    if "global_random_seed" in wanted:
        kwargs["global_random_seed"] = 42
    if "global_dtype" in wanted:
        kwargs["global_dtype"] = np.float64
    if "capsys" in wanted:
        kwargs["capsys"] = capsys

    unsupported = None
    if kwargs.get("algo") == "elkan" or kwargs.get("algorithm") == "elkan":
        unsupported = "algorithm='elkan'"
    for key in ("array_constr", "X_csr", "csr_container", "input_data"):
        v = kwargs.get(key)
        if v is not None and (sp.issparse(v) or (isinstance(v, type) and issubclass(v, sp.spmatrix))
                              or getattr(v, "__name__", "").startswith(("csr_", "csc_", "coo_"))):
            unsupported = "sparse input"
    if name in ("test_dense_sparse", "test_predict_dense_sparse"):
        unsupported = "sparse input"

    if unsupported is not None:
        try:
            fn(**kwargs)
        except BaseException as exc:  # noqa: BLE001  (pytest's own Failed is a BaseException)
            # the engine's refusal, possibly wrapped by a `pytest.warns` / `pytest.raises` block of
            # the scikit-learn test that was open when it was raised
            chain, seen = exc, []
            while chain is not None and not isinstance(chain, NotSupportedByEngineError):
                seen.append(chain)
                chain = chain.__cause__ or chain.__context__
            if chain is None:
                raise
            pytest.xfail(f"{unsupported}: NotSupportedByEngineError, as for the reference's engine")
        pytest.fail(f"{unsupported} must be refused with NotSupportedByEngineError")
    fn(**kwargs)
