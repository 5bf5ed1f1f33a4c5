"""Sum and argmin reductions (reference: sklearn_numba_dpex/common/reductions.py)."""

import torch

from .. import _capi
from .._capi import check, lib, ptr
from ._buffers import contiguous, dcode, workspace


def sum_reduction(array, axis=1, square=False):
    """Sum of a 1-D array (returns shape (1,)) or of a 2-D array along `axis`.

    axis=1 -> (rows,), axis=0 -> (cols,).  `square` sums x**2 instead (the reference's
    fused_elementwise_func=_square, applied once).  Mirrors make_sum_reduction_2d_kernel
    (common/reductions.py:214-460).
    """
    a = contiguous(array)
    if a.dim() == 1:
        a = a.reshape(1, -1)
        axis = 1
    rows, cols = a.shape
    ws_bytes = lib.kmx_sum_workspace_bytes(rows, cols)
    ws = workspace(ws_bytes, a.device, tag="sum")
    stream = _capi.current_stream()
    if axis == 1:
        out = torch.empty(rows, dtype=a.dtype, device=a.device)
        check(lib.kmx_sum_rows(ptr(a), ptr(out), rows, cols, int(bool(square)), ptr(ws), ws_bytes,
                               dcode(a), stream), "kmx_sum_rows")
    elif axis == 0:
        if square:
            raise ValueError("square is only supported with axis=1")
        out = torch.empty(cols, dtype=a.dtype, device=a.device)
        check(lib.kmx_sum_cols(ptr(a), ptr(out), rows, cols, ptr(ws), ws_bytes, dcode(a), stream),
              "kmx_sum_cols")
    else:
        raise ValueError(f"axis must be 0 or 1, got {axis}")
    return out


def argmin_reduction(values):
    """Index (int32, shape (1,)) of the smallest value, lowest index on ties
    (make_argmin_reduction_1d_kernel, common/reductions.py:17-209)."""
    v = contiguous(values)
    out = torch.empty(1, dtype=torch.int32, device=v.device)
    check(lib.kmx_argmin(ptr(v), ptr(out), v.numel(), dcode(v), _capi.current_stream()), "kmx_argmin")
    return out
