"""KMeansEngine: the scikit-learn engine-API plugin class for KMeans, same method surface as
the reference's sklearn_numba_dpex/kmeans/engine.py:36-392, computing on one MI355X through
the HIP library.

Device arrays are torch ROCm tensors.  As in the reference (engine.py:88-98) the engine keeps
X in "F order": the (n_samples, n_features) tensor it hands back is the transposed view of a
C-contiguous (n_features, n_samples) buffer, which is the layout the kernels read.

scikit-learn releases without the engine API (no `KMeansCythonEngine`, no
`NotSupportedByEngineError`) are supported through small stand-ins; with the engine-API
branch installed the real base class is used and the entry point
`sklearn_engines: kmeans = sklearn_numba_dpex_amd.kmeans.engine:KMeansEngine` makes the
engine selectable with `sklearn.config_context(engine_provider="sklearn_numba_dpex_amd")`.
"""

import numbers
import os
from typing import Any, Dict

import numpy as np
import scipy.sparse as sp
import torch
from sklearn.utils import check_array, check_random_state
from sklearn.utils.validation import _is_arraylike_not_scalar

try:  # scikit-learn feature/engine-api branch
    from sklearn.cluster._kmeans import KMeansCythonEngine as _EngineBase
    from sklearn.exceptions import NotSupportedByEngineError
except ImportError:  # stock scikit-learn

    class NotSupportedByEngineError(NotImplementedError):
        """The engine cannot run the requested configuration."""

    class _EngineBase:
        def __init__(self, estimator):
            self.estimator = estimator


from ..common._buffers import require_cuda, upload
from ..common.kernels import transposed_copy
from .drivers import (
    get_euclidean_distances,
    get_labels_inertia,
    get_nb_distinct_clusters,
    is_same_clustering,
    kmeans_plusplus,
    lloyd,
    prepare_data_for_lloyd,
    restore_data_after_lloyd,
)

_ACCEPTED_DTYPES = (np.float64, np.float32)
_TORCH_FLOAT = {torch.float32, torch.float64}


def _to_numpy(value):
    if isinstance(value, torch.Tensor):
        return value.detach().cpu().numpy()
    return np.asarray(value)


class KMeansEngine(_EngineBase):
    """GPU implementation of Lloyd's k-means for scikit-learn's engine API.

    Public methods override those of scikit-learn's `KMeansCythonEngine`; the others are
    private to this implementation (same convention as the reference, engine.py:65-68).
    """

    # Test hook, as in the reference (engine.py:70-75): {"device": "cuda:0"} pins the device.
    _CONFIG: Dict[str, Any] = dict()

    engine_name = "kmeans"

    @staticmethod
    def convert_to_sklearn_types(name, value):
        if name in ["cluster_centers_", "labels_"]:
            value = _to_numpy(value)
            if name == "labels_":
                value = value.astype(np.int32, copy=False)
        return value

    def __init__(self, estimator):
        self.device = torch.device(self._CONFIG.get("device", "cuda"))
        order = self._CONFIG.get("order", "F")
        if order != "F":
            raise ValueError("The kernels read X in the Fortran memory layout only.")
        self.order = order
        self.estimator = estimator

        mode = os.getenv("SKLEARN_NUMBA_DPEX_TESTING_MODE", "0")
        if mode not in {"0", "1"}:
            raise ValueError(
                "If the environment variable SKLEARN_NUMBA_DPEX_TESTING_MODE is set, it is "
                f'expected to take values in {{"0", "1"}}, but got {mode} instead.'
            )
        self._is_in_testing_mode = mode == "1"

    # ------------------------------------------------------------------ fit

    def accepts(self, X, y, sample_weight):
        if (algorithm := self.estimator.algorithm) not in ("lloyd", "auto", "full"):
            if self._is_in_testing_mode:
                raise NotSupportedByEngineError(
                    "The sklearn_numba_dpex_amd engine for KMeans only support the Lloyd "
                    f"algorithm, {algorithm} is not supported."
                )
            return False
        if sp.issparse(X):
            return self._is_in_testing_mode
        return True

    def prepare_fit(self, X, y=None, sample_weight=None):
        estimator = self.estimator
        X = self._validate_data(X)
        self._check_params_vs_input(X)
        sample_weight = self._check_sample_weight(sample_weight, X)

        init = estimator.init
        if _is_arraylike_not_scalar(init) or isinstance(init, torch.Tensor):
            init = self._check_init(init, X)

        X_t, X_mean, self.init, self.tol, self.sample_weight_is_uniform = prepare_data_for_lloyd(
            X.T, init, estimator.tol, sample_weight, estimator.copy_x and not self._owns_X
        )
        if self._is_in_testing_mode and X_mean is not None:
            X_mean = _to_numpy(X_mean)
        self.X_mean = X_mean
        self.random_state = check_random_state(estimator.random_state)
        return X_t.T, y, sample_weight

    def unshift_centers(self, X, best_centers):
        if (X_mean := self.X_mean) is None:
            return
        if isinstance(best_centers, np.ndarray):  # testing mode hands numpy centres around
            best_centers += _to_numpy(X_mean)
            if not self.estimator.copy_x:
                restore_data_after_lloyd(X.T, None, self._as_device(X_mean, X.dtype), copy_x=False)
            return
        restore_data_after_lloyd(X.T, best_centers.T, self._as_device(X_mean, X.dtype), self.estimator.copy_x)

    def init_centroids(self, X, sample_weight):
        init = self.init
        n_clusters = self.estimator.n_clusters

        if isinstance(init, torch.Tensor):
            centers_t = init
        elif isinstance(init, str) and init == "k-means++":
            centers_t, _ = self._kmeans_plusplus(X, sample_weight)
        elif callable(init):
            centers = init(X, n_clusters, random_state=self.random_state)
            centers_t = self._check_init(centers, X)
        else:
            # sampling without replacement is sequential: done on the host with the same
            # numpy call as scikit-learn, so a given seed picks the same rows
            sample_weight_numpy = _to_numpy(sample_weight)
            p = sample_weight_numpy / sample_weight_numpy.sum()
            centers_idx = self.random_state.choice(X.shape[0], size=n_clusters, replace=False, p=p)
            idx = torch.as_tensor(centers_idx, dtype=torch.int64, device=X.device)
            centers_t = torch.index_select(X.T, 1, idx).contiguous()
        return centers_t

    def _kmeans_plusplus(self, X, sample_weight):
        return kmeans_plusplus(X.T, sample_weight, self.estimator.n_clusters, self.random_state)

    def kmeans_single(self, X, sample_weight, centers_init_t):
        assignments_idx, inertia, best_centroids_t, n_iteration = lloyd(
            X.T,
            sample_weight,
            centers_init_t,
            self.sample_weight_is_uniform,
            self.estimator.max_iter,
            self.estimator.verbose,
            self.tol,
        )
        if self._is_in_testing_mode:
            assignments_idx = _to_numpy(assignments_idx).astype(np.int32)
            best_centroids_t = np.asfortranarray(_to_numpy(best_centroids_t)).astype(
                getattr(self.estimator, "_output_dtype", np.float64)
            )
        return assignments_idx, inertia, best_centroids_t.T, n_iteration

    def is_same_clustering(self, labels, best_labels, n_clusters):
        if isinstance(labels, np.ndarray):
            labels = torch.as_tensor(labels.astype(np.int32), device=self.device)
            best_labels = torch.as_tensor(np.asarray(best_labels).astype(np.int32), device=self.device)
        return is_same_clustering(labels, best_labels, n_clusters)

    def count_distinct_clusters(self, best_labels):
        if isinstance(best_labels, np.ndarray):
            best_labels = torch.as_tensor(best_labels.astype(np.int32), device=self.device)
        return get_nb_distinct_clusters(best_labels, self.estimator.n_clusters)

    # ------------------------------------------------------------------ predict / score / transform

    def prepare_prediction(self, X, sample_weight):
        X = self._validate_data(X, reset=False)
        sample_weight = self._check_sample_weight(sample_weight, X)
        return X, sample_weight

    def get_labels(self, X, sample_weight):
        labels, _ = self._get_labels_inertia(X, sample_weight, with_inertia=False)
        if self._is_in_testing_mode:
            labels = _to_numpy(labels).astype(np.int32)
        return labels

    def get_score(self, X, sample_weight):
        _, inertia = self._get_labels_inertia(X, sample_weight, with_inertia=True)
        return inertia

    def _get_labels_inertia(self, X, sample_weight, with_inertia=True):
        cluster_centers = self._check_init(self.estimator.cluster_centers_, X, copy=False)
        assignments_idx, inertia = get_labels_inertia(X.T, cluster_centers, sample_weight, with_inertia)
        if with_inertia:
            inertia = inertia[0]
        return assignments_idx, inertia

    def prepare_transform(self, X):
        return X

    def get_euclidean_distances(self, X):
        X = self._validate_data(X, reset=False)
        cluster_centers = self._check_init(self.estimator.cluster_centers_, X, copy=False)
        euclidean_distances = get_euclidean_distances(X.T, cluster_centers)
        if self._is_in_testing_mode:
            euclidean_distances = _to_numpy(euclidean_distances).astype(
                getattr(self.estimator, "_output_dtype", np.float64)
            )
        return euclidean_distances

    # ------------------------------------------------------------------ validation (private)

    def _as_device(self, array, dtype):
        if not isinstance(array, (torch.Tensor, np.ndarray)) and hasattr(array, "__dlpack__"):
            array = torch.from_dlpack(array)
        if isinstance(array, torch.Tensor):
            return array.to(device=self.device, dtype=dtype)
        return torch.as_tensor(np.asarray(array), device=self.device).to(dtype)

    def _assert_all_finite(self, X_t, X_host):
        """scikit-learn's check of the input (check_array(ensure_all_finite=True), as the
        reference's engine runs it: kmeans/engine.py:293-302), taken on the device: one pass at
        memory speed instead of a single-threaded host pass that costs more than the upload.
        Non-finite data then get scikit-learn's own error from the host copy.  As in
        scikit-learn, the sum goes first (one read, nothing written): a NaN or an infinity
        anywhere makes it non-finite, and so may an overflow of finite values, which the
        element-wise test then clears."""
        if bool(torch.isfinite(X_t.sum())) or bool(torch.isfinite(X_t).all()):
            return
        from sklearn.utils.validation import _assert_all_finite

        host = X_host if X_host is not None else X_t.T.cpu().numpy()
        _assert_all_finite(host, input_name="X", estimator_name=type(self.estimator).__name__)

    def _validate_data(self, X, reset=True):
        """Returns X on the device as the transposed view of a contiguous (d, n) buffer, dtype
        float64 or float32 (other dtypes are converted to float64, as scikit-learn does)."""
        require_cuda()
        estimator = self.estimator
        if sp.issparse(X):
            raise NotSupportedByEngineError("A sparse matrix was passed, but dense data is required.")

        if not isinstance(X, (torch.Tensor, np.ndarray)) and hasattr(X, "__dlpack__"):
            # any array library that speaks DLPack (the counterpart of the reference taking
            # dpctl / dpnp arrays, engine.py:293-302): device arrays are used without a copy
            X = torch.from_dlpack(X)

        if isinstance(X, torch.Tensor):
            if X.dim() != 2:
                raise ValueError(f"Expected 2D array, got {X.dim()}D array instead.")
            if X.shape[0] < 1 or X.shape[1] < 1:
                raise ValueError(f"Found array with shape {tuple(X.shape)}: at least one sample and "
                                 "one feature are required.")
            out_dtype = X.dtype if X.dtype in _TORCH_FLOAT else torch.float64
            n_features = X.shape[1]
            X_dev = X.to(device=self.device, dtype=out_dtype)
            # (d, n) contiguous; already the case for an F-ordered tensor
            X_t = X_dev.T
            owns_copy = X_dev.data_ptr() != X.data_ptr()
            if not X_t.is_contiguous():
                X_t = transposed_copy(X_dev) if X_dev.is_contiguous() else X_t.contiguous()
                owns_copy = True
            self._assert_all_finite(X_t, None)
        else:
            owns_copy = True  # the upload below is this engine's own device copy
            X_np = check_array(
                X,
                accept_sparse=False,
                dtype=list(_ACCEPTED_DTYPES),
                order=None,
                copy=False,
                ensure_all_finite=False,  # checked on the device below: the host pass costs more than the upload
                estimator=estimator,
                input_name="X",
            )
            n_features = X_np.shape[1]
            # upload, then transpose on the device: (d, n) contiguous
            # (through pinned staging buffers when the array is large)
            X_t = upload(np.ascontiguousarray(X_np.T) if X_np.flags.f_contiguous else X_np, self.device)
            X_t = X_t if X_np.flags.f_contiguous else transposed_copy(X_t)
            self._assert_all_finite(X_t, X_np)

        # prepare_fit centres the data in place when this buffer is not the caller's (or copy_x is off)
        self._owns_X = owns_copy
        if reset:
            estimator.n_features_in_ = n_features
            if self._is_in_testing_mode:
                estimator._output_dtype = np.float64 if X_t.dtype == torch.float64 else np.float32
        elif hasattr(estimator, "n_features_in_") and n_features != estimator.n_features_in_:
            raise ValueError(
                f"X has {n_features} features, but {estimator.__class__.__name__} is expecting "
                f"{estimator.n_features_in_} features as input."
            )
        return X_t.T

    def _check_params_vs_input(self, X):
        """The checks of scikit-learn's KMeans._check_params_vs_input that need the data."""
        estimator = self.estimator
        if X.shape[0] < estimator.n_clusters:
            raise ValueError(f"n_samples={X.shape[0]} should be >= n_clusters={estimator.n_clusters}.")
        n_init = estimator.n_init
        if n_init == "auto":
            init = estimator.init
            if isinstance(init, str) and init == "k-means++":
                n_init = 1
            elif isinstance(init, str) and init == "random":
                n_init = 10
            elif callable(init):
                n_init = 10
            else:
                n_init = 1
        if (_is_arraylike_not_scalar(estimator.init) or isinstance(estimator.init, torch.Tensor)) and n_init != 1:
            import warnings

            warnings.warn(
                "Explicit initial center position passed: performing only one init in "
                f"{estimator.__class__.__name__} instead of n_init={n_init}.",
                RuntimeWarning,
                stacklevel=2,
            )
            n_init = 1
        estimator._n_init = n_init
        estimator._algorithm = "lloyd"

    def _check_sample_weight(self, sample_weight, X):
        n_samples = X.shape[0]
        if sample_weight is None:
            return torch.ones(n_samples, dtype=X.dtype, device=X.device)
        if isinstance(sample_weight, numbers.Number):
            return torch.full((n_samples,), float(sample_weight), dtype=X.dtype, device=X.device)
        if not isinstance(sample_weight, (torch.Tensor, np.ndarray)) and hasattr(sample_weight, "__dlpack__"):
            sample_weight = torch.from_dlpack(sample_weight)
        if isinstance(sample_weight, torch.Tensor):
            sample_weight = sample_weight.to(device=X.device, dtype=X.dtype).contiguous()
        else:
            sample_weight = check_array(
                sample_weight,
                accept_sparse=False,
                order="C",
                dtype=np.float64 if X.dtype == torch.float64 else np.float32,
                ensure_all_finite=True,
                ensure_2d=False,
                allow_nd=False,
                estimator=self.estimator,
                input_name="sample_weight",
            )
            sample_weight = upload(sample_weight, X.device)
        if sample_weight.dim() != 1:
            raise ValueError("Sample weights must be 1D array or scalar")
        if tuple(sample_weight.shape) != (n_samples,):
            raise ValueError(
                "sample_weight.shape == {}, expected {}!".format(tuple(sample_weight.shape), (n_samples,))
            )
        return sample_weight

    def _check_init(self, init, X, copy=False):
        """Initial (or fitted) centres as a fresh C-contiguous (d, k) device tensor of X's dtype."""
        if isinstance(init, torch.Tensor):
            if init.dim() != 2:
                raise ValueError(f"Expected 2D array, got {init.dim()}D array instead.")
            init_dev = init.to(device=X.device, dtype=X.dtype)
        else:
            init_np = check_array(
                init,
                dtype=np.float64 if X.dtype == torch.float64 else np.float32,
                accept_sparse=False,
                copy=False,
                order="C",
                ensure_all_finite=True,
                ensure_2d=True,
                estimator=self.estimator,
                input_name="init",
            )
            # check_array hands back the caller's own array when nothing had to change, and that
            # one may be read-only: wrap a private copy
            init_dev = torch.as_tensor(np.array(init_np, copy=True), device=X.device)
        self._validate_center_shape(X, init_dev)
        init_t = init_dev.T.contiguous()
        if init_t.data_ptr() == getattr(init, "data_ptr", lambda: None)():
            init_t = init_t.clone()
        return init_t

    def _validate_center_shape(self, X, centers):
        n_clusters = self.estimator.n_clusters
        if centers.shape[0] != n_clusters:
            raise ValueError(
                f"The shape of the initial centers {tuple(centers.shape)} does not "
                f"match the number of clusters {n_clusters}."
            )
        if centers.shape[1] != X.shape[1]:
            raise ValueError(
                f"The shape of the initial centers {tuple(centers.shape)} does not "
                f"match the number of features of the data {X.shape[1]}."
            )
