"""Import shim: makes the package in `sklearn-numba-dpex_amd/` (whose directory name is not a
valid Python identifier) importable as `sklearn_numba_dpex_amd`."""
import os as _os

__path__ = [_os.path.join(_os.path.dirname(_os.path.abspath(__file__)), "sklearn-numba-dpex_amd")]
with open(_os.path.join(__path__[0], "__init__.py")) as _f:
    exec(compile(_f.read(), _os.path.join(__path__[0], "__init__.py"), "exec"))
del _os, _f
