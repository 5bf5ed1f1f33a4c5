"""The plugin packaging: the `sklearn_engines` entry point scikit-learn's engine API looks
plugins up by (reference: pyproject.toml:55-56) resolves to this build's KMeansEngine, and the
built package is importable under its installed name without the in-tree import shim."""

import importlib.metadata
import os
import subprocess
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _setup_py(args, tmp_path):
    env = dict(os.environ, PYTHONDONTWRITEBYTECODE="1")
    proc = subprocess.run([sys.executable, os.path.join(ROOT, "setup.py"), "-q", *args], cwd=ROOT, env=env,
                          capture_output=True, text=True, timeout=300)
    if proc.returncode != 0:
        pytest.skip(f"setuptools cannot build metadata offline here: {proc.stderr[-400:]}")


def test_entry_point_resolves_to_the_engine(tmp_path):
    _setup_py(["egg_info", "--egg-base", str(tmp_path)], tmp_path)
    dists = list(importlib.metadata.distributions(path=[str(tmp_path)]))
    assert len(dists) == 1 and dists[0].metadata["Name"] == "sklearn-numba-dpex-amd"
    eps = [ep for ep in dists[0].entry_points if ep.group == "sklearn_engines"]
    assert [(ep.name, ep.value) for ep in eps] == [("kmeans", "sklearn_numba_dpex_amd.kmeans.engine:KMeansEngine")]
    engine_class = eps[0].load()
    from sklearn_numba_dpex_amd.kmeans.engine import KMeansEngine

    assert engine_class is KMeansEngine and engine_class.engine_name == "kmeans"


def test_built_package_imports_under_its_installed_name(tmp_path):
    lib = os.path.join(ROOT, "sklearn-numba-dpex_amd", "libmi355x_kmeans.so")
    if not os.path.exists(lib):
        pytest.skip("the HIP library has not been built")
    build_lib = tmp_path / "lib"
    _setup_py(["build_py", "--build-lib", str(build_lib)], tmp_path)
    pkg = build_lib / "sklearn_numba_dpex_amd"
    assert (pkg / "libmi355x_kmeans.so").exists(), "the HIP library must ship as package data"
    assert (pkg / "kmeans" / "engine.py").exists() and (pkg / "common" / "topk.py").exists()
    # a fresh interpreter that sees only the built tree (not the repository root with its shim)
    code = ("import sys; sys.path[:] = [p for p in sys.path if p not in ('', %r)]; "
            "import sklearn_numba_dpex_amd as m; from sklearn_numba_dpex_amd.kmeans.engine import KMeansEngine; "
            "from sklearn_numba_dpex_amd import _capi; "
            "print(m.__file__); print(_capi.lib.kmx_abi_version(), KMeansEngine.engine_name)" % ROOT)
    env = {k: v for k, v in os.environ.items() if k != "PYTHONPATH"}
    env["PYTHONPATH"] = str(build_lib)
    proc = subprocess.run([sys.executable, "-c", code], cwd=str(tmp_path), env=env, capture_output=True, text=True,
                          timeout=300)
    assert proc.returncode == 0, proc.stderr[-800:]
    lines = proc.stdout.strip().splitlines()
    assert lines[0].startswith(str(pkg)), lines
    assert lines[1].split() == [str(__import__("sklearn_numba_dpex_amd._capi", fromlist=["x"]).ABI_VERSION), "kmeans"]


def test_benchmark_consistency_rule():
    """The benchmark's check between two providers: centres and inertia at 1e-5 per iteration,
    labels equal except at ties between two centres."""
    import numpy as np
    import pytest

    from sklearn_numba_dpex_amd.benchmark.kmeans import _check_same_fit

    rng = np.random.default_rng(0)
    centers = np.array([[0.0, 0.0], [4.0, 0.0], [0.0, 4.0]], dtype=np.float32)
    X = (centers[rng.integers(0, 3, 300)] + 0.3 * rng.standard_normal((300, 2))).astype(np.float32)
    X[0] = [2.0, 0.0]  # exactly between the first two centres
    labels = ((X[:, None, :] - centers[None]) ** 2).sum(axis=2).argmin(axis=1).astype(np.int32)
    ref = dict(labels=labels, centers=centers, inertia=10.0)
    same = dict(labels=labels.copy(), centers=centers * (1 + 2e-6), inertia=10.0 * (1 + 2e-6))
    _check_same_fit(X, ref, same, np.float32, 1)
    tie = dict(same, labels=labels.copy())
    tie["labels"][0] = 1 - labels[0]
    _check_same_fit(X, ref, tie, np.float32, 1)
    wrong = dict(same, labels=labels.copy())
    wrong["labels"][5] = (labels[5] + 1) % 3
    with pytest.raises(AssertionError, match="not all of them are ties"):
        _check_same_fit(X, ref, wrong, np.float32, 1)
    with pytest.raises(AssertionError, match="cluster centres differ"):
        _check_same_fit(X, ref, dict(same, centers=centers + np.float32(1e-3)), np.float32, 1)
    with pytest.raises(AssertionError):
        _check_same_fit(X, ref, dict(same, inertia=10.01), np.float32, 1)
