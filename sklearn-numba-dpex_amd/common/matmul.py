"""Dense matmul (reference: sklearn_numba_dpex/common/matmul.py)."""

import torch

from .. import _capi
from .._capi import check, lib, ptr
from ._buffers import contiguous, dcode


def matmul(X, Y_t):
    """X (m, p) @ Y_t (q, p)^T -> (m, q), the operand convention of make_matmul_2d_kernel
    (common/matmul.py:13-70)."""
    X = contiguous(X)
    Y_t = contiguous(Y_t)
    m, p = X.shape
    q, p2 = Y_t.shape
    if p != p2:
        raise ValueError(f"inner dimensions differ: {p} and {p2}")
    out = torch.empty((m, q), dtype=X.dtype, device=X.device)
    check(lib.kmx_matmul(ptr(X), ptr(Y_t), ptr(out), m, p, q, dcode(X), _capi.current_stream()), "kmx_matmul")
    return out
