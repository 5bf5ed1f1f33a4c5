"""Elementwise and broadcast kernels (reference: sklearn_numba_dpex/common/kernels.py)."""

import torch

from .. import _capi
from .._capi import check, lib, ptr
from ._buffers import dcode


def _require_contiguous(t):
    if not t.is_contiguous():
        raise ValueError("in-place kernels need a contiguous array")


def half_l2_norm(data_t):
    """(sum over rows of data**2) / 2 per column (common/kernels.py:116-145)."""
    _require_contiguous(data_t)
    rows, cols = data_t.shape
    out = torch.empty(cols, dtype=data_t.dtype, device=data_t.device)
    check(lib.kmx_half_sq_norms(ptr(data_t), ptr(out), rows, cols, dcode(data_t), _capi.current_stream()),
          "kmx_half_sq_norms")
    return out


def broadcast_rows(array, vector, op):
    """array[r, c] = array[r, c] (op) vector[r], in place; op is "minus" or "plus"
    (make_broadcast_ops_1d_2d_axis1_kernel, common/kernels.py:85-113)."""
    _require_contiguous(array)
    rows, cols = array.shape
    code = {"minus": 0, "plus": 1}[op]
    check(lib.kmx_broadcast_rows(ptr(array), ptr(vector), rows, cols, code, dcode(array),
                                 _capi.current_stream()), "kmx_broadcast_rows")


def broadcast_division(array, divisor):
    """array[r, c] /= divisor[c], in place (common/kernels.py:60-82)."""
    _require_contiguous(array)
    rows, cols = array.shape
    check(lib.kmx_broadcast_div_cols(ptr(array), ptr(divisor), rows, cols, dcode(array),
                                     _capi.current_stream()), "kmx_broadcast_div_cols")


def divide_by(data, divisor):
    """data /= divisor, in place (make_apply_elementwise_func with _divide_by)."""
    _require_contiguous(data)
    check(lib.kmx_divide_by(ptr(data), data.numel(), float(divisor), dcode(data), _capi.current_stream()),
          "kmx_divide_by")


def transposed_copy(array):
    """A C-contiguous copy of array.T for a C-contiguous 2-d fp32 / fp64 array (the reference
    leaves these copies to the array library: kmeans/engine.py:88-98)."""
    _require_contiguous(array)
    rows, cols = array.shape
    out = torch.empty((cols, rows), dtype=array.dtype, device=array.device)
    check(lib.kmx_transpose(ptr(array), ptr(out), rows, cols, dcode(array), _capi.current_stream()),
          "kmx_transpose")
    return out


def initialize_to_zeros(data):
    """Zero fill, in place (common/kernels.py:38-57)."""
    _require_contiguous(data)
    check(lib.kmx_fill_zero(ptr(data), data.numel() * data.element_size(), _capi.current_stream()),
          "kmx_fill_zero")


def centroid_shifts(centroids_t, new_centroids_t):
    """Squared shift per centroid (kmeans/kernels/utils.py:79-110)."""
    d, k = centroids_t.shape
    out = torch.empty(k, dtype=centroids_t.dtype, device=centroids_t.device)
    check(lib.kmx_centroid_shifts(ptr(centroids_t), ptr(new_centroids_t), ptr(out), d, k,
                                  dcode(centroids_t), _capi.current_stream()), "kmx_centroid_shifts")
    return out
