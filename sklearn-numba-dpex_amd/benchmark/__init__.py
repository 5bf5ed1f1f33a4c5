"""Command-line benchmark of the KMeans estimators (python -m sklearn_numba_dpex_amd.benchmark.kmeans)."""
