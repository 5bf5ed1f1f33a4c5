"""Scalar functions that the shared kernels accept as fused operations (reference:
sklearn_numba_dpex/common/_utils.py:17-33).  The reference compiles arbitrary Python functions
into its kernels; the HIP kernels here are compiled ahead of time, so they accept exactly these
predefined functions, recognised by identity (or, for `_divide_by`, by the closure's attribute).
"""


def _square(x):
    return x * x


def _minus(x, y):
    return x - y


def _plus(x, y):
    return x + y


def _multiply(x, y):
    return x * y


def _divide_by(divisor):
    def _divide_closure(x):
        return x / divisor

    _divide_closure.divisor = divisor
    return _divide_closure
