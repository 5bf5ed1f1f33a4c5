"""Top-k selection (reference: sklearn_numba_dpex/common/topk.py)."""

import torch

from .. import _capi
from .._capi import check, lib, ptr
from ._buffers import contiguous, dcode, workspace


def topk_idx(array_in, k):
    """Indices (int64) of the k greatest values of a 1-D array, or of each row of a 2-D one.

    Unlike the reference (common/topk.py:194-227) the output is deterministic: descending
    value, ties by ascending index.
    """
    a = contiguous(array_in)
    if a.dim() == 1:
        return _topk_idx_row(a, k)
    if a.dim() != 2:
        raise ValueError("expected a 1-D or 2-D array")
    return torch.stack([_topk_idx_row(a[r], k) for r in range(a.shape[0])])


def _topk_idx_row(row, k):
    n = row.numel()
    if n < k:
        raise ValueError(
            "Expected k to be greater than or equal to the number of items in the search space, "
            f"but got k={k} and {n} items in the search space."
        )
    if row.dtype not in (torch.float32, torch.float64):
        raise ValueError(f"topk currently only supports float32 and float64, got dtype={row.dtype} .")
    ws_bytes = lib.kmx_topk_workspace_bytes(n, k)
    ws = workspace(ws_bytes, row.device)
    out = torch.empty(k, dtype=torch.int64, device=row.device)
    check(lib.kmx_topk_idx(ptr(row), ptr(out), n, k, ptr(ws), ws_bytes, dcode(row), _capi.current_stream()),
          "kmx_topk_idx")
    return out


def topk(array_in, k):
    """The k greatest values (descending); gathered through topk_idx."""
    idx = topk_idx(array_in, k)
    a = contiguous(array_in)
    if a.dim() == 1:
        return a[idx]
    return torch.gather(a, 1, idx)
