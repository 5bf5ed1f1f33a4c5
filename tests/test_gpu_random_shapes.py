"""Lloyd iterations on shapes drawn at random (seeded) against the CPU oracle: sample counts
around the tile sizes, feature counts around the K steps of the matrix-core kernels, cluster
counts around the centroid blocks, both dtypes, with and without the row-major copy - a net
under the named shapes of the other files."""

import numpy as np
import pytest

from oracle import kmeans as ok

pytestmark = pytest.mark.gpu

D_CHOICES = [1, 2, 3, 5, 8, 13, 14, 16, 17, 24, 31, 32, 33, 40, 47, 48, 49, 63, 64, 65, 70, 100, 128, 130, 200, 257]
K_CHOICES = [1, 2, 3, 7, 15, 16, 17, 31, 32, 33, 50, 64, 65, 100, 127, 128, 129, 200, 256, 257, 300, 500]
N_CHOICES = [63, 64, 65, 100, 1000, 1023, 1025, 4096, 5000, 10007, 20000]


def _case(seed):
    rng = np.random.default_rng(seed)
    dtype = np.float32 if rng.random() < 0.6 else np.float64
    d, k = int(rng.choice(D_CHOICES)), int(rng.choice(K_CHOICES))
    n = max(int(rng.choice(N_CHOICES + [k, k + 1])), k)
    spread = rng.choice([0.5, 3.0, 10.0])
    centers = rng.uniform(-spread, spread, (k, d))
    X = (centers[rng.integers(0, k, n)] + rng.standard_normal((n, d))).astype(dtype)
    init = X[rng.choice(n, k, replace=False)].copy()
    w = (rng.uniform(0.5, 1.5, n) if rng.random() < 0.7 else np.ones(n)).astype(dtype)
    return X, w, init, bool(rng.random() < 0.5)


@pytest.mark.parametrize("block", range(4))
def test_iterations_on_random_shapes_match_the_oracle(cuda, block):
    import torch

    from sklearn_numba_dpex_amd import _capi
    from sklearn_numba_dpex_amd._capi import lib, ptr

    dev = lambda a: torch.as_tensor(np.ascontiguousarray(a), device=cuda)
    stream = _capi.current_stream()
    for seed in range(1000 + 12 * block, 1000 + 12 * (block + 1)):
        X, w, init, rowmajor = _case(seed)
        n, d = X.shape
        k = init.shape[0]
        what = f"seed {seed}: n={n} d={d} k={k} {X.dtype}"
        X_t, w_d = dev(X.T), dev(w)
        cent = [dev(init.T), torch.empty(d, k, dtype=X_t.dtype, device=cuda)]
        labels = [torch.zeros(n, dtype=torch.int32, device=cuda) for _ in range(2)]
        sizes = torch.empty(k, dtype=X_t.dtype, device=cuda)
        empty = torch.empty(k, dtype=torch.int32, device=cuda)
        plan = _capi.lloyd_plan(n, d, k, _capi.dtype_code(X.dtype), 0)
        ws = torch.empty(plan.workspace_bytes, dtype=torch.uint8, device=cuda)
        status = _capi.LloydStatus()
        _capi.check(lib.kmx_lloyd_init(plan, ptr(ws), plan.workspace_bytes, ptr(X_t), ptr(w_d), ptr(cent[0]), 100,
                                       0.0, stream), "init")
        X_rm = dev(X) if rowmajor and plan.variant in (42, 3, 13, 53, 63) else None
        tie = 1e-6 if X.dtype == np.float32 else 1e-13
        for it in range(3):
            a, b = it % 2, (it + 1) % 2
            c_in = cent[a].cpu().numpy().T.copy()
            _capi.check(lib.kmx_lloyd_iter(plan, ptr(X_t), ptr(X_rm), ptr(w_d), ptr(cent[a]), ptr(cent[b]),
                                           ptr(labels[a]), ptr(labels[b]), ptr(sizes), ptr(empty), ptr(ws),
                                           plan.workspace_bytes, stream), "iter")
            _capi.check(lib.kmx_lloyd_status_read(ptr(ws), status, stream), "status")
            got = labels[b].cpu().numpy().astype(np.int64)
            assert got.min() >= 0 and got.max() < k, what
            bad = np.flatnonzero(got != ok.assign_labels(X, c_in))
            if bad.size:  # equal except where two centroids are equally near
                D = ((X[bad, None, :].astype(np.float64) - c_in[None].astype(np.float64)) ** 2).sum(-1)
                gap = (D[np.arange(bad.size), got[bad]] - D.min(1)) / np.maximum(D.max(1), 1e-300)
                assert np.all(gap <= tie), f"{what}, variant {plan.variant}, iteration {it}: {gap.max():.2e}"
            sums, ref_sizes = ok.weighted_sums(X, w, got, k)
            np.testing.assert_allclose(sizes.cpu().numpy(), ref_sizes, rtol=1e-5 if X.dtype == np.float32 else 1e-12,
                                       err_msg=what)
            assert status.n_empty == int(np.count_nonzero(ref_sizes == 0)), what
            if status.n_empty or status.state != _capi.KMX_RUNNING:
                break
            ref = sums / ref_sizes[:, None]
            err = np.abs(cent[b].cpu().numpy().T - ref).max() / max(np.abs(ref).max(), 1e-30)
            assert err <= (2e-5 if X.dtype == np.float32 else 1e-11), f"{what}, variant {plan.variant}: {err:.2e}"
