"""A KMeans estimator that drives KMeansEngine, for scikit-learn releases without the
engine API.

scikit-learn's `feature/engine-api` branch calls a plugin engine from `KMeans.fit`,
`predict`, `score` and `transform`; released versions cannot.  This subclass reproduces
that call order (the sequence the reference's engine.py overrides and its tests exercise:
accepts -> prepare_fit -> n_init x [init_centroids, kmeans_single, is_same_clustering] ->
unshift_centers -> count_distinct_clusters; prepare_prediction -> get_labels / get_score;
prepare_transform -> get_euclidean_distances) so the engine is a drop-in either way.
"""

import contextlib
import warnings

import numpy as np
from sklearn.cluster import KMeans as _SklearnKMeans
from sklearn.exceptions import ConvergenceWarning
from sklearn.utils.validation import check_is_fitted

from .engine import KMeansEngine

_config = {"engine_attributes": None}


@contextlib.contextmanager
def config_context(engine_attributes=None):
    """`engine_attributes="sklearn_types"` converts fitted attributes to numpy, like the
    option of the same name in the engine-API branch's `sklearn.config_context`."""
    old = dict(_config)
    _config["engine_attributes"] = engine_attributes
    try:
        yield
    finally:
        _config.update(old)


class KMeans(_SklearnKMeans):
    """scikit-learn KMeans whose computations run in KMeansEngine (one MI355X)."""

    def _engine(self):
        return KMeansEngine(self)

    def _convert(self, name, value):
        if _config["engine_attributes"] == "sklearn_types":
            return KMeansEngine.convert_to_sklearn_types(name, value)
        return value

    def fit(self, X, y=None, sample_weight=None):
        self._validate_params()
        engine = self._engine()
        if not engine.accepts(X, y, sample_weight):
            return super().fit(X, y, sample_weight=sample_weight)

        X, y, sample_weight = engine.prepare_fit(X, y, sample_weight)
        best_inertia, best_labels = None, None
        for _ in range(self._n_init):
            centers_init = engine.init_centroids(X, sample_weight)
            labels, inertia, centers, n_iter_ = engine.kmeans_single(X, sample_weight, centers_init)
            if best_inertia is None or (
                inertia < best_inertia and not engine.is_same_clustering(labels, best_labels, self.n_clusters)
            ):
                best_labels, best_centers, best_inertia, best_n_iter = labels, centers, inertia, n_iter_

        engine.unshift_centers(X, best_centers)
        distinct_clusters = engine.count_distinct_clusters(best_labels)
        if distinct_clusters < self.n_clusters:
            warnings.warn(
                f"Number of distinct clusters ({distinct_clusters}) found smaller than "
                f"n_clusters ({self.n_clusters}). Possibly due to duplicate points in X.",
                ConvergenceWarning,
                stacklevel=2,
            )
        self.cluster_centers_ = self._convert("cluster_centers_", best_centers)
        self._n_features_out = self.cluster_centers_.shape[0]
        self.labels_ = self._convert("labels_", best_labels)
        self.inertia_ = best_inertia
        self.n_iter_ = best_n_iter
        return self

    def fit_predict(self, X, y=None, sample_weight=None):
        return self.fit(X, sample_weight=sample_weight).labels_

    def fit_transform(self, X, y=None, sample_weight=None):
        return self.fit(X, sample_weight=sample_weight).transform(X)

    def predict(self, X):
        check_is_fitted(self)
        engine = self._engine()
        X, sample_weight = engine.prepare_prediction(X, None)
        return self._convert("labels_", engine.get_labels(X, sample_weight))

    def score(self, X, y=None, sample_weight=None):
        check_is_fitted(self)
        engine = self._engine()
        X, sample_weight = engine.prepare_prediction(X, sample_weight)
        return -engine.get_score(X, sample_weight)

    def transform(self, X):
        check_is_fitted(self)
        engine = self._engine()
        X = engine.prepare_transform(X)
        return engine.get_euclidean_distances(X)
