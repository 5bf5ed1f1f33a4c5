"""Device-buffer helpers: torch tensors serve only as HIP allocations."""

import threading

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


_workspaces = {}
_workspaces_lock = threading.Lock()
# a kept buffer larger than this is not kept (the list of uncertified samples of a wide label
# call is 4 bytes per sample)
_WORKSPACE_KEEP_BYTES = 64 << 20


def workspace(n_bytes, device, tag=None):
    """Scratch bytes for one library call.  With a `tag` the buffer is kept and handed out again
    to the next call with the same tag by the same host thread on the same device and stream
    (one thread's work on one stream is ordered, so those calls cannot overlap; two threads
    that share a stream each get a buffer of their own).  A kept buffer only grows, up to
    64 MiB: a larger one is made for the call and released with it.  `release_workspaces()`
    drops them all."""
    n_bytes = max(int(n_bytes), 1)
    if tag is None or n_bytes > _WORKSPACE_KEEP_BYTES:
        return torch.empty(n_bytes, dtype=torch.uint8, device=device)
    device = torch.device(device)
    key = (tag, device.index if device.index is not None else torch.cuda.current_device(),
           _capi.current_stream(), threading.get_ident())
    with _workspaces_lock:
        buf = _workspaces.get(key)
        if buf is None or buf.numel() < n_bytes:
            buf = torch.empty(max(n_bytes, 4096), dtype=torch.uint8, device=device)
            _workspaces[key] = buf
    return buf


def release_workspaces():
    """Forgets every kept scratch buffer (their memory goes back to the allocator once the
    calls that use them have run)."""
    with _workspaces_lock:
        _workspaces.clear()


def dcode(t):
    return _capi.dtype_code(t.dtype)


def contiguous(t):
    return t if t.is_contiguous() else t.contiguous()


# ---------------------------------------------------------------------------- host -> device

# Large numpy inputs go to the device through two pinned staging buffers: while one chunk
# travels by DMA the host fills the other, instead of the runtime bouncing a pageable array
# through its own small staging area.  (The counterpart of the reference's host -> device
# conversion, kmeans/engine.py:293-302.)  The buffers are allocated pinned (registering existing
# memory is not available everywhere) once per process and kept.
_STAGE_BYTES = 32 << 20
_STAGE_MIN_BYTES = 4 << 20   # below this a plain copy is as fast
_stage = None
_stage_lock = threading.Lock()   # one upload at a time: the two buffers and their events are shared


def _staging():
    global _stage
    if _stage is None:
        _stage = [(torch.empty(_STAGE_BYTES, dtype=torch.uint8, pin_memory=True), torch.cuda.Event())
                  for _ in range(2)]
    return _stage


def upload(array, device):
    """A C-contiguous numpy array as a device tensor of the same shape and dtype."""
    array = np.ascontiguousarray(array)
    if array.nbytes < _STAGE_MIN_BYTES or not array.dtype.isnative or array.dtype.kind not in "fiub":
        return torch.as_tensor(array, device=device)
    dev = torch.device(device)
    out = torch.empty(array.shape, dtype=torch.from_numpy(array[:0].reshape(-1)).dtype, device=dev)
    src = torch.from_numpy(array.reshape(-1).view(np.uint8))
    dst = out.view(-1).view(torch.uint8)
    with _stage_lock, torch.cuda.device(dev):
        stage = _staging()
        for turn, lo in enumerate(range(0, src.numel(), _STAGE_BYTES)):
            hi = min(lo + _STAGE_BYTES, src.numel())
            buf, busy = stage[turn % 2]
            if turn >= 2:
                busy.synchronize()   # the DMA that last read this buffer
            buf[: hi - lo].copy_(src[lo:hi])            # host copy (torch spreads it over its threads)
            dst[lo:hi].copy_(buf[: hi - lo], non_blocking=True)
            busy.record()
        # the staging buffers are reused by the next call: leave none of them in flight
        for _, busy in stage:
            busy.synchronize()
    return out
