"""MI355X-native KMeans engine for scikit-learn's engine API.

Layout
------
csrc/        HIP kernels for gfx950 and the C ABI (include/mi355x_kmeans.h)
_capi.py     ctypes binding of libmi355x_kmeans.so
common/      host wrappers of the shared kernels (sums, argmin, top-k, RNG, matmul)
kmeans/      drivers (Lloyd loop, kmeans++, labels/inertia, distances) and the KMeansEngine

The package mirrors the operator surface of soda-inria/sklearn-numba-dpex for the KMeans
path; the compute path is the HIP library only (no CPU or PyTorch fallback).
"""

__version__ = "0.1.0"
