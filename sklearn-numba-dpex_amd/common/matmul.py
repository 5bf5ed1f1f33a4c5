"""Dense matmul (reference: sklearn_numba_dpex/common/matmul.py)."""

import torch

from .. import _capi
from .._capi import check, lib, ptr
from . import _utils
from ._buffers import contiguous, dcode

MULTIPLY, MINUS, PLUS = 0, 1, 2
OUT_IDENTITY, OUT_SQUARE, OUT_DIVIDE_BY = 0, 1, 2


def _multiply_code(fn):
    if fn is None or fn is _utils._multiply:
        return MULTIPLY
    if fn is _utils._minus:
        return MINUS
    if fn is _utils._plus:
        return PLUS
    raise NotImplementedError(
        "multiply_fn must be one of the predefined functions of common._utils (_multiply, _minus, _plus): "
        "the kernels are compiled ahead of time"
    )


def _out_code(fn):
    if fn is None:
        return OUT_IDENTITY, 0.0
    if fn is _utils._square:
        return OUT_SQUARE, 0.0
    if hasattr(fn, "divisor"):
        return OUT_DIVIDE_BY, float(fn.divisor)
    raise NotImplementedError(
        "out_fused_elementwise_fn must be one of the predefined functions of common._utils (_square, "
        "_divide_by(divisor)): the kernels are compiled ahead of time"
    )


def matmul(X, Y_t, multiply_fn=None, out_fused_elementwise_fn=None):
    """out[i, j] = out_fn(sum_k multiply_fn(X[i, k], Y_t[j, k])) for X (m, p) and Y_t (q, p): the
    operand convention and the two fused functions of make_matmul_2d_kernel
    (common/matmul.py:13-70).  The plain product runs on the matrix cores (fp32 and fp64)."""
    X = contiguous(X)
    Y_t = contiguous(Y_t)
    m, p = X.shape
    q, p2 = Y_t.shape
    if p != p2:
        raise ValueError(f"inner dimensions differ: {p} and {p2}")
    if X.dtype != Y_t.dtype:
        raise ValueError(f"operand dtypes differ: {X.dtype} and {Y_t.dtype}")
    mul = _multiply_code(multiply_fn)
    out_op, out_param = _out_code(out_fused_elementwise_fn)
    out = torch.empty((m, q), dtype=X.dtype, device=X.device)
    check(lib.kmx_matmul_fused(ptr(X), ptr(Y_t), ptr(out), m, p, q, mul, out_op, out_param, dcode(X),
                               _capi.current_stream()), "kmx_matmul_fused")
    return out
