"""Top-k selection (reference: sklearn_numba_dpex/common/topk.py)."""

import torch

from .. import _capi
from .._capi import check, lib, ptr
from ._buffers import contiguous, dcode, workspace


def _prepare(array_in, k):
    a = contiguous(array_in)
    if a.dim() not in (1, 2):
        raise ValueError("expected a 1-D or 2-D array")
    rows, n = (1, a.shape[0]) if a.dim() == 1 else a.shape
    if n < k:
        raise ValueError(
            "Expected k to be greater than or equal to the number of items in the search space, "
            f"but got k={k} and {n} items in the search space."
        )
    if a.dtype not in (torch.float32, torch.float64):
        raise ValueError(f"topk currently only supports float32 and float64, got dtype={a.dtype} .")
    ws_bytes = lib.kmx_topk_rows_workspace_bytes(rows, n, k, dcode(a))
    return a, rows, n, workspace(ws_bytes, a.device, tag="topk"), ws_bytes


def topk_idx(array_in, k):
    """Indices (int64) of the k greatest values of a 1-D array, or of each row of a 2-D one.

    Unlike the reference (common/topk.py:194-227) the output is deterministic: descending
    value, ties by ascending index.
    """
    k = int(k)
    a, rows, n, ws, ws_bytes = _prepare(array_in, k)
    out = torch.empty((k,) if a.dim() == 1 else (rows, k), dtype=torch.int64, device=a.device)
    if rows == 0 or k == 0:
        return out
    check(lib.kmx_topk_idx_rows(ptr(a), ptr(out), rows, n, k, ptr(ws), ws_bytes, dcode(a), _capi.current_stream()),
          "kmx_topk_idx_rows")
    return out


def topk(array_in, k):
    """The k greatest values (descending) of a 1-D array, or of each row of a 2-D one
    (reference common/topk.py:112-191, where the order is undefined)."""
    k = int(k)
    a, rows, n, ws, ws_bytes = _prepare(array_in, k)
    out = torch.empty((k,) if a.dim() == 1 else (rows, k), dtype=a.dtype, device=a.device)
    if rows == 0 or k == 0:
        return out
    check(lib.kmx_topk_values(ptr(a), ptr(out), rows, n, k, ptr(ws), ws_bytes, dcode(a), _capi.current_stream()),
          "kmx_topk_values")
    return out
