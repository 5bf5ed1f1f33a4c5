"""The allocation-free row sum (kmx_sum_rows_static) against kmx_sum_rows, through the C ABI."""

import numpy as np
import pytest

pytestmark = pytest.mark.gpu


def _both(x, square, cuda):
    import torch

    from sklearn_numba_dpex_amd import _capi
    from sklearn_numba_dpex_amd._capi import lib, ptr

    rows, cols = x.shape
    dc = _capi.dtype_code(x.dtype)
    stream = _capi.current_stream()
    ws_bytes = lib.kmx_sum_workspace_bytes(rows, cols)
    ws = torch.empty(ws_bytes, dtype=torch.uint8, device=cuda)
    ref = torch.empty(rows, dtype=x.dtype, device=cuda)
    got = torch.full((rows,), float("nan"), dtype=x.dtype, device=cuda)
    _capi.check(lib.kmx_sum_rows(ptr(x), ptr(ref), rows, cols, square, ptr(ws), ws_bytes, dc, stream), "sum_rows")
    # warm-up call: the one-time address lookup of the scratch array and the module load stay
    # outside the window that is checked
    _capi.check(lib.kmx_sum_rows_static(ptr(x), ptr(got), rows, cols, square, dc, stream), "sum_rows_static")
    got.fill_(float("nan"))
    torch.cuda.synchronize()
    # torch's counters see torch's allocator only; the device's free bytes (hipMemGetInfo) also
    # move when the library itself allocates device memory
    before = torch.cuda.memory_allocated(), torch.cuda.memory_reserved(), torch.cuda.mem_get_info()[0]
    _capi.check(lib.kmx_sum_rows_static(ptr(x), ptr(got), rows, cols, square, dc, stream), "sum_rows_static")
    torch.cuda.synchronize()
    after = torch.cuda.memory_allocated(), torch.cuda.memory_reserved(), torch.cuda.mem_get_info()[0]
    assert after == before
    return got.cpu().numpy(), ref.cpu().numpy()


@pytest.mark.parametrize("dtype", ["float32", "float64"])
def test_static_row_sum_equals_workspace_row_sum_on_two_calls_in_a_row(cuda, dtype):
    """Same kernels, same fixed summation order: the results are bit-identical.  The second call
    is smaller than the first, so it meets the first call's leftovers in the shared scratch."""
    import torch

    tdt = getattr(torch, dtype)
    g = torch.Generator(device=cuda)
    g.manual_seed(3)
    big = torch.randn(7, 1_000_003, device=cuda, generator=g).to(tdt)
    small = torch.randn(3, 1_001, device=cuda, generator=g).to(tdt)
    for x, square in ((big, 0), (small, 1)):
        got, ref = _both(x, square, cuda)
        np.testing.assert_array_equal(got, ref)
        x64 = x.double().cpu().numpy()
        exact = (x64 * x64).sum(axis=1) if square else x64.sum(axis=1)
        np.testing.assert_allclose(got, exact, rtol=1e-5 if dtype == "float32" else 1e-12, atol=1e-3 if dtype == "float32" else 1e-9)


def test_static_row_sum_rejects_what_its_scratch_cannot_hold(cuda):
    import torch

    from sklearn_numba_dpex_amd import _capi
    from sklearn_numba_dpex_amd._capi import lib, ptr

    x = torch.ones(65, 128, device=cuda)
    out = torch.empty(65, device=cuda)
    st = _capi.current_stream()
    assert lib.kmx_sum_rows_static(ptr(x), ptr(out), 65, 128, 0, 0, st) == -6
    assert lib.kmx_sum_rows_static(ptr(x), ptr(out), 64, 128, 0, 0, st) == 0
    torch.cuda.synchronize()
    assert torch.all(out[:64] == 128)
    assert lib.kmx_sum_rows_static(None, ptr(out), 1, 128, 0, 0, st) == -1
    assert lib.kmx_sum_rows_static(ptr(x), ptr(out), 0, 128, 0, 0, st) == -2
