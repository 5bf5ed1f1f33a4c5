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
