"""Device-buffer helpers: torch tensors serve only as HIP allocations."""

import numpy as np
import torch

from .. import _capi


def require_cuda():
    if not torch.cuda.is_available():
        raise RuntimeError("sklearn_numba_dpex_amd needs a ROCm GPU (torch.cuda.is_available() is False)")


def torch_dtype(dtype):
    if isinstance(dtype, torch.dtype):
        return dtype
    return {np.dtype(np.float32): torch.float32, np.dtype(np.float64): torch.float64}[np.dtype(dtype)]


def workspace(n_bytes, device):
    return torch.empty(max(int(n_bytes), 1), dtype=torch.uint8, device=device)


def dcode(t):
    return _capi.dtype_code(t.dtype)


def contiguous(t):
    return t if t.is_contiguous() else t.contiguous()
