"""Test bench for KMeans: scikit-learn's CPU Lloyd next to the MI355X engine.

Same protocol and flags as the reference's bench (benchmark/kmeans.py:137-207, 262-361):
every provider fits the same data from the same initial centroids with n_init=1, tol=0 and
algorithm="lloyd", after a dry run with max_iter=1; the timed fit must run exactly max_iter
iterations; --run-consistency-checks compares labels, centres and inertia between providers.
The data is synthetic (Gaussian blobs; there is no network for the reference's OpenML set):
--dataset picks one of the frozen configurations, --n-data-samples / --n-features resample it
the way the reference resamples its dataset (:210-252).

    python -m sklearn_numba_dpex_amd.benchmark.kmeans --dataset config2 --max-iter 100
"""

from argparse import ArgumentParser
from time import perf_counter

import numpy as np


def _resample(X, n_samples, n_features, rng):
    """n_samples rows and n_features columns drawn from X, repeating some when more are asked
    for than exist (benchmark/kmeans.py:210-252)."""
    n, d = X.shape
    if n_features is not None and n_features != d:
        cols = rng.choice(d, size=n_features, replace=n_features > d)
        X = X[:, cols]
    if n_samples is not None and n_samples != n:
        rows = rng.choice(n, size=n_samples, replace=n_samples > n)
        X = X[rows]
    return np.ascontiguousarray(X)


def _blobs(name, dtype):
    # same generators as the parity tests and the throughput benchmark
    from sklearn_numba_dpex_amd import datasets

    cfg = getattr(datasets, name)()
    return cfg["X"].astype(dtype, copy=False)


def _providers(skip_cpu, skip_gpu, selected):
    from sklearn.cluster import KMeans as SklearnKMeans

    out = []
    if not skip_cpu and "scikit-learn" in selected:
        out.append(("scikit-learn (OpenMP Cython Lloyd)", "cpu", SklearnKMeans))
    if not skip_gpu and "mi355x" in selected:
        from sklearn_numba_dpex_amd.kmeans.estimator import KMeans as EngineKMeans

        out.append(("sklearn_numba_dpex_amd KMeansEngine", "gpu", EngineKMeans))
    return out


def main(argv=None):
    ap = ArgumentParser(description=__doc__.split("\n\n")[0])
    ap.add_argument("--sample-weight", default="random", choices=["unary", "random", "None"])
    ap.add_argument("--init", default="random", choices=["k-means++", "random"])
    ap.add_argument("--n-clusters", default=127, type=int)
    ap.add_argument("--max-iter", default=100, type=int)
    ap.add_argument("--dataset", default="config1", choices=["config1", "config2", "config3", "config4", "config5"],
                    help="synthetic Gaussian-blob configuration the samples are drawn from")
    ap.add_argument("--n-data-samples", default=None, type=int)
    ap.add_argument("--n-features", default=None, type=int)
    ap.add_argument("--dtype", default="float32", choices=["float32", "float64"])
    ap.add_argument("--random-state", default=123, type=int)
    ap.add_argument("--run-consistency-checks", action="store_true")
    ap.add_argument("--engine-providers", nargs="+", choices=["scikit-learn", "mi355x"],
                    default=["scikit-learn", "mi355x"])
    ap.add_argument("--skip-cpu", action="store_true")
    ap.add_argument("--skip-gpu", action="store_true")
    args = ap.parse_args(argv)

    dtype = np.dtype(args.dtype).type
    rng = np.random.default_rng(args.random_state)
    X = _resample(_blobs(args.dataset, dtype), args.n_data_samples, args.n_features, rng)
    n, d = X.shape
    if args.sample_weight == "None":
        sample_weight = None
    elif args.sample_weight == "unary":
        sample_weight = np.ones(n, dtype=dtype)
    else:
        sample_weight = rng.random(n).astype(dtype)

    k = args.n_clusters
    if args.init == "random":
        centers_init = X[rng.choice(n, size=k, replace=False)].copy()
    else:
        from sklearn.cluster import kmeans_plusplus

        centers_init, _ = kmeans_plusplus(X, k, random_state=args.random_state, sample_weight=sample_weight)
        centers_init = centers_init.astype(dtype)
    print(f"data {n} x {d} {np.dtype(dtype).name}, n_clusters={k}, max_iter={args.max_iter}, "
          f"init={args.init}, sample_weight={args.sample_weight}")

    reference = None
    for name, device, cls in _providers(args.skip_cpu, args.skip_gpu, args.engine_providers):
        kwargs = dict(n_clusters=k, init=centers_init.copy(), n_init=1, max_iter=args.max_iter, tol=0,
                      random_state=args.random_state, copy_x=True, algorithm="lloyd")
        print(f"\nRunning {name} on device {device}...")
        cls(**kwargs).set_params(max_iter=1).fit(X.copy(), sample_weight=sample_weight)  # dry run
        est = cls(**kwargs)
        t0 = perf_counter()
        est.fit(X.copy(), sample_weight=sample_weight)
        t1 = perf_counter()
        n_iter = int(est.n_iter_)
        print(f"Running {name} ... done in {t1 - t0:.3f} s ({n_iter} iterations, "
              f"{n_iter / (t1 - t0):.1f} iter/s, inertia {float(est.inertia_):.6g})")
        if n_iter != args.max_iter:
            raise RuntimeError(
                f"The estimator {name} only ran {n_iter} iterations instead of max_iter={args.max_iter} "
                "iterations. It is expected for all estimators in the benchmark to run the same number of "
                "iterations and return the same results.")
        if args.run_consistency_checks:
            got = dict(labels=np.asarray(_to_numpy(est.labels_)), centers=np.asarray(_to_numpy(est.cluster_centers_)),
                       inertia=float(est.inertia_))
            if reference is None:
                reference = got
            else:
                _check_same_fit(X, reference, got, dtype, args.max_iter)
    return 0


def _check_same_fit(X, reference, got, dtype, n_iter):
    """Two providers ran the same iterations from the same centres: inertia within 1e-5 (fp32) /
    1e-12 (fp64), centres within that tolerance per iteration run (relative to the coordinate,
    with the centroid's largest coordinate as floor), and labels equal except where the two
    nearest centres of the reference fit are tied to within ten times the centre tolerance.
    (The reference compares labels exactly and everything else with assert_allclose's default,
    and calls its own check unreliable: benchmark/kmeans.py:172-206, 326-327.)"""
    rtol = 1e-5 if np.dtype(dtype) == np.float32 else 1e-12
    centres_rtol = rtol * max(1, n_iter)
    ref_c = np.asarray(reference["centers"], dtype=np.float64)
    got_c = np.asarray(got["centers"], dtype=np.float64)
    n = reference["labels"].shape[0]
    differ = np.flatnonzero(reference["labels"] != got["labels"])
    print(f"consistency: {differ.size} of {n} labels differ, "
          f"inertia {reference['inertia']:.8g} vs {got['inertia']:.8g}")
    np.testing.assert_allclose(got["inertia"], reference["inertia"], rtol=rtol * max(1, n_iter))
    scale = np.abs(ref_c).max(axis=1, keepdims=True)
    bound = centres_rtol * np.maximum(np.abs(ref_c), scale)
    worst = float(np.max(np.abs(got_c - ref_c) / np.maximum(bound, 1e-300)))
    if worst > 1.0:
        raise AssertionError(f"cluster centres differ: largest error is {worst:.2f} x the bound (rtol {centres_rtol:g})")
    if differ.size:
        if differ.size > max(1, n // 1000):
            raise AssertionError(f"{differ.size} of {n} labels differ")
        rows = np.asarray(X, dtype=np.float64)[differ]
        dist = ((rows[:, None, :] - ref_c[None, :, :]) ** 2).sum(axis=2)
        at = np.arange(differ.size)
        gap = np.abs(dist[at, reference["labels"][differ].astype(np.int64)]
                     - dist[at, got["labels"][differ].astype(np.int64)])
        if not np.all(gap <= 10.0 * centres_rtol * dist.max(axis=1)):
            raise AssertionError(f"{differ.size} labels differ and not all of them are ties between two centres")


def _to_numpy(value):
    return value.cpu().numpy() if hasattr(value, "cpu") else value


if __name__ == "__main__":
    raise SystemExit(main())
