"""The benchmark configurations at their FULL sizes, through properties that do not need a CPU
run of the same size: conservation of the weighted sums, labels against exact distances on a
random slice, monotone inertia, run-to-run reproducibility, and the kmeans++ output contract.
(The oracle comparisons proper run on reduced sizes in the other test files.)"""

import numpy as np
import pytest

from oracle import kmeans as ok
from sklearn_numba_dpex_amd import datasets
from tests._parity import assert_labels_match

pytestmark = pytest.mark.gpu


def _run_iterations(cuda, cfg, n_iter):
    """n_iter Lloyd iterations through the C ABI; returns per-iteration (centroids_t, labels,
    sizes) as device tensors plus the inputs on the device."""
    import torch

    from sklearn_numba_dpex_amd import _capi
    from sklearn_numba_dpex_amd._capi import lib, ptr

    X, init, w, k = cfg["X"], cfg["init"], cfg["sample_weight"], cfg["k"]
    n, d = X.shape
    dc = _capi.dtype_code(X.dtype)
    X_rm = torch.as_tensor(X, device=cuda)
    X_t = X_rm.T.contiguous()
    plan = _capi.lloyd_plan(n, d, k, dc, 0)
    if plan.variant not in (42, 63, 53, 13, 3):  # the variants that sum rows of a row-major copy
        X_rm = None
    w_d = torch.as_tensor(w, device=cuda)
    cent = [torch.as_tensor(np.ascontiguousarray(init.T), device=cuda), None]
    cent[1] = torch.empty_like(cent[0])
    labels = [torch.zeros(n, dtype=torch.int32, device=cuda) for _ in range(2)]
    sizes = torch.empty(k, dtype=X_t.dtype, device=cuda)
    empty = torch.empty(k, dtype=torch.int32, device=cuda)
    ws_bytes = plan.workspace_bytes
    ws = torch.empty(ws_bytes, dtype=torch.uint8, device=cuda)
    stream = _capi.current_stream()
    status = _capi.LloydStatus()
    _capi.check(lib.kmx_lloyd_init(plan, ptr(ws), ws_bytes, ptr(X_t), ptr(w_d), ptr(cent[0]), 1000, 0.0,
                                   stream), "init")
    out = []
    for it in range(n_iter):
        a, b = it % 2, (it + 1) % 2
        _capi.check(lib.kmx_lloyd_iter(plan, ptr(X_t), ptr(X_rm), ptr(w_d), ptr(cent[a]), ptr(cent[b]),
                                       ptr(labels[a]), ptr(labels[b]), ptr(sizes), ptr(empty), ptr(ws), ws_bytes,
                                       stream), "iter")
        _capi.check(lib.kmx_lloyd_status_read(ptr(ws), status, stream), "status")
        out.append(dict(inp=cent[a].clone(), new=cent[b].clone(), labels=labels[b].clone(), sizes=sizes.clone(),
                        state=status.state, n_empty=status.n_empty, n_iter=status.n_iter))
        if status.state != _capi.KMX_RUNNING:
            break
    return X_t, w_d, out


def _check_iteration(X, X_t, w_d, rec, k, rtol, rng):
    import torch

    n = X.shape[0]
    labels = rec["labels"].long()
    assert int(labels.min()) >= 0 and int(labels.max()) < k
    # conservation: the sizes are the weights per label, and sum_c size_c * centroid_c = sum_i w_i x_i
    w64 = w_d.double()
    sizes_ref = torch.zeros(k, dtype=torch.float64, device=X_t.device).index_add_(0, labels, w64)
    np.testing.assert_allclose(rec["sizes"].double().cpu().numpy(), sizes_ref.cpu().numpy(), rtol=rtol)
    assert float(rec["sizes"].double().sum()) == pytest.approx(float(w64.sum()), rel=rtol)
    if rec["state"] == 0:  # centroids were finalised (no empty cluster)
        total = (rec["new"].double() * rec["sizes"].double()[None, :]).sum(dim=1)
        ref_total = (X_t.double() * w64[None, :]).sum(dim=1)
        scale = float((X_t.double().abs() * w64[None, :]).sum(dim=1).max())
        np.testing.assert_allclose(total.cpu().numpy(), ref_total.cpu().numpy(), atol=10 * rtol * scale)
    # labels against exact fp64 distances to the centroids they were computed from, on a slice
    rows = np.sort(rng.choice(n, size=20_000, replace=False))
    cin = rec["inp"].T.cpu().numpy()
    got = rec["labels"].cpu().numpy()[rows]
    return assert_labels_match(got, ok.assign_labels(X[rows], cin), X[rows], cin)


@pytest.mark.parametrize("name", ["config2", "config3", "config5"])
def test_lloyd_properties_at_full_size(cuda, name):
    import torch

    from sklearn_numba_dpex_amd.kmeans import drivers

    cfg = getattr(datasets, name)()
    X, k = cfg["X"], cfg["k"]
    rtol = 1e-5 if X.dtype == np.float32 else 1e-12
    rng = np.random.default_rng(0)
    X_t, w_d, recs = _run_iterations(cuda, cfg, 3)
    ties = sum(_check_iteration(X, X_t, w_d, rec, k, rtol, rng) for rec in recs)
    print(f"{name}: {len(recs)} iterations, near-tie label differences on the slices: {ties}")
    if name == "config5":
        # 16 centroids start far away: empty after the first assignment, relocation required
        assert recs[0]["n_empty"] == 16 and recs[0]["state"] != 0
    else:
        # (config 3 loses clusters on its own in the second iteration: the loop then stops
        # there and waits for the host's relocation)
        assert all(r["state"] == 0 for r in recs[:-1]) and (len(recs) == 3 or recs[-1]["n_empty"] > 0)
        # inertia of successive (labels, centroids they were computed from) never increases
        inertias = [float(drivers._inertia(X_t, w_d, r["inp"], r["labels"])) for r in recs]
        assert all(b <= a * (1 + 1e-6) for a, b in zip(inertias, inertias[1:])), inertias
    if X.dtype == np.float32:
        # integer (fixed-point) sums: a second run gives the same bits
        _, _, again = _run_iterations(cuda, cfg, len(recs))
        for r, r2 in zip(recs, again):
            assert torch.equal(r["labels"], r2["labels"]) and torch.equal(r["new"], r2["new"])


def test_full_lloyd_run_with_relocation_at_full_size(cuda):
    import torch

    from sklearn_numba_dpex_amd.kmeans import drivers

    cfg = datasets.config5()
    X, k = cfg["X"], cfg["k"]
    X_t = torch.as_tensor(X, device=cuda).T.contiguous()
    w_d = torch.as_tensor(cfg["sample_weight"], device=cuda)
    c0 = torch.as_tensor(np.ascontiguousarray(cfg["init"].T), device=cuda)
    labels, inertia, cent_t, n_iter = drivers.lloyd(X_t, w_d, c0, max_iter=cfg["max_iter"], tol=0.0)
    assert 1 <= n_iter <= cfg["max_iter"]
    counts = torch.bincount(labels.long(), minlength=k)
    assert int(counts.min()) > 0, "a cluster stayed empty after relocation"
    # the returned labels are the arg-min for the returned centroids and the inertia is theirs
    rows = np.sort(np.random.default_rng(1).choice(X.shape[0], size=20_000, replace=False))
    C = cent_t.T.cpu().numpy()
    assert_labels_match(labels.cpu().numpy()[rows], ok.assign_labels(X[rows], C), X[rows], C)
    ref_inertia = float(drivers._inertia(X_t, w_d, cent_t, labels))
    assert float(inertia) == pytest.approx(ref_inertia, rel=1e-12)


def test_kmeanspp_contract_at_full_size(cuda):
    import torch

    from sklearn_numba_dpex_amd.kmeans import drivers

    cfg = datasets.config4()
    X, k = cfg["X"], cfg["k"]
    X_t = torch.as_tensor(X, device=cuda).T.contiguous()
    w_d = torch.as_tensor(cfg["sample_weight"], device=cuda)
    runs = [drivers.kmeans_plusplus(X_t, w_d, k, np.random.RandomState(cfg["seed"])) for _ in range(2)]
    idx = runs[0][1].cpu().numpy()
    assert idx.shape == (k,) and idx.min() >= 0 and idx.max() < X.shape[0]
    assert len(np.unique(idx)) == k  # a centre has zero distance to itself: never drawn twice
    np.testing.assert_array_equal(runs[0][0].cpu().numpy().T, X[idx])
    np.testing.assert_array_equal(idx, runs[1][1].cpu().numpy())  # same draws, same centres
    # 256 well separated blobs: seeding must reach (nearly) all of them
    dist = drivers.get_euclidean_distances(X_t[:, :50_000].contiguous(), runs[0][0])
    assert float(dist.min(dim=1).values.max()) < 30.0


@pytest.mark.parametrize("sampler", ["scan", "literal"])
def test_kmeanspp_first_centres_match_oracle_at_full_n(cuda, sampler):
    """The first 12 centres on the full 1,000,000 x 64 data against the oracle's sampler fed
    with the same uniform draws (the whole 256-centre seeding would take the oracle minutes):
    the default fp64 scan against the oracle's exact sampler, and the reference's own running
    sum in fp32 (`KMX_KPP_SAMPLER_LITERAL`, kmeans/kernels/kmeans_plusplus.py:79-100) against the
    oracle's literal one - at this size the two samplers pick different samples for most draws."""
    import torch

    from oracle import rng as orng
    from sklearn_numba_dpex_amd.kmeans import drivers

    cfg = datasets.config4()
    X, k = cfg["X"], 12
    w = cfg["sample_weight"]
    X_t = torch.as_tensor(X, device=cuda).T.contiguous()
    _, idx = drivers.kmeans_plusplus(X_t, torch.as_tensor(w, device=cuda), k, np.random.RandomState(cfg["seed"]),
                                     sampler=sampler)
    seed64 = orng.seed_from_random_state(np.random.RandomState(cfg["seed"]))
    _, ref_idx = ok.kmeans_plusplus(X, w, k, seed64, sampler="exact" if sampler == "scan" else "literal")
    np.testing.assert_array_equal(idx.cpu().numpy(), ref_idx)


def test_score_path_and_topk_at_full_size(cuda):
    """configs[1] at full size: labels and inertia in one pass equal the two-pass results (labels
    bit for bit, inertia to 1e-5 and to an exact fp64 sum on a slice-free formula), and the
    top-k of the 5e6 per-sample values - unique values, then heavy ties - equals a host sort."""
    import torch

    from sklearn_numba_dpex_amd.common.topk import topk, topk_idx
    from sklearn_numba_dpex_amd.kmeans import drivers

    cfg = datasets.config2()
    X, init, w = cfg["X"], cfg["init"], cfg["sample_weight"]
    n = X.shape[0]
    X_t = torch.as_tensor(X, device=cuda).T.contiguous()
    C_t = torch.as_tensor(np.ascontiguousarray(init.T), device=cuda)
    w_d = torch.as_tensor(w, device=cuda)
    labels = torch.empty(n, dtype=torch.int32, device=cuda)
    total = drivers._assign_with_inertia(X_t, w_d, C_t, labels)
    ref = torch.empty(n, dtype=torch.int32, device=cuda)
    drivers._assign(X_t, C_t, ref)
    assert torch.equal(labels, ref)
    per_sample = drivers._per_sample_inertia(X_t, w_d, C_t, ref)
    exact = float(per_sample.double().sum())
    assert abs(float(total[0]) - exact) <= 1e-5 * exact
    assert abs(float(drivers._inertia_array(X_t, w_d, C_t, ref)[0]) - exact) <= 1e-5 * exact

    host = per_sample.cpu().numpy()
    for k in (1, 16, 127):
        want = ok.top_k_indices(host, k)
        np.testing.assert_array_equal(topk_idx(per_sample, k).cpu().numpy(), want)
        np.testing.assert_array_equal(topk(per_sample, k).cpu().numpy(), host[want])
    tied = torch.floor(per_sample)  # a few hundred distinct values: every threshold is a tie
    host = tied.cpu().numpy()
    for k in (16, 1000):
        np.testing.assert_array_equal(topk_idx(tied, k).cpu().numpy(), ok.top_k_indices(host, k))


@pytest.mark.parametrize("shape", [(2_000_000, 100, 100, np.float64, 63), (1_000_000, 32, 500, np.float64, 53),
                                   (500_000, 300, 300, np.float32, 63), (2_000_000, 100, 10, np.float32, 81),
                                   (2_000_000, 100, 10, np.float64, 1), (300_000, 784, 10, np.float32, 81),
                                   (2_000_000, 48, 64, np.float32, 61), (1_000_000, 64, 128, np.float64, 51),
                                   (2_000_000, 48, 64, np.float64, 71),
                                   # the tiled product with centroid tiles of 32 and stages of twice the features
                                   (1_000_000, 200, 24, np.float32, 63), (500_000, 200, 10, np.float64, 63)])
def test_large_shapes_off_the_benchmark_configurations(cuda, shape):
    """The same properties on large inputs of the other kernel families: the tiled matrix-core
    product and the fp64 matrix-core labels with bucketed sums, the few-cluster step (per-wave and
    per-workgroup tiles), the streaming vector-ALU step, the screened step with three K steps on
    fp32 and fp64 inputs, the fp64 step with a compute unit's whole LDS."""
    from sklearn_numba_dpex_amd import _capi
    from sklearn_numba_dpex_amd.kmeans import drivers

    n, d, k, dtype, variant = shape
    assert _capi.lloyd_plan(n, d, k, _capi.dtype_code(dtype), 0).variant == variant
    rng = np.random.default_rng(n + d + k)
    centers = (rng.uniform(-1.0, 1.0, (k, d)) * (6.0 / np.sqrt(d))).astype(dtype)
    X = centers[rng.integers(0, k, n)]
    X += rng.standard_normal((n, d), dtype=dtype)
    cfg = dict(X=X, init=X[rng.choice(n, k, replace=False)].copy(), sample_weight=rng.uniform(0.5, 1.5, n).astype(dtype), k=k)
    rtol = 1e-5 if dtype == np.float32 else 1e-12
    X_t, w_d, recs = _run_iterations(cuda, cfg, 3)
    ties = sum(_check_iteration(X, X_t, w_d, rec, k, rtol, rng) for rec in recs)
    print(f"{shape}: {len(recs)} iterations, near-tie label differences on the slices: {ties}")
    assert len(recs) == 3 and all(r["state"] == 0 for r in recs)
    inertias = [float(drivers._inertia(X_t, w_d, r["inp"], r["labels"])) for r in recs]
    assert all(b <= a * (1 + 1e-6) for a, b in zip(inertias, inertias[1:])), inertias


@pytest.mark.parametrize("n,d,k,variant", [(4_300_000, 512, 300, 63), (8_500_000, 256, 512, 42), (2_800_000, 784, 10, 81)])
def test_array_past_two_to_the_31_elements(cuda, n, d, k, variant):
    """4 300 000 x 512 (tiled product + sums per bucket), 8 500 000 x 256 with 512 clusters (the
    wide path: labels screened in fp16, fp32 pass over the uncertified samples, bucketed
    accumulation) and 2 800 000 x 784 with 10 clusters (the few-cluster step: tiles loaded from the
    row-major copy straight into LDS; its labels-only kernel and the inertia split over the
    features at the end) in fp32: 2.2e9 elements, 8.8 GB, generated on the device.  Feature rows from
    125 on start more than 2^31 bytes into the array and the last samples of the last row lie
    past element 2^31: three Lloyd iterations through the C ABI (tiled matrix-core labels, sums
    per bucket of samples from the row-major copy), checked through size-independent properties
    - conservation of the weighted sums, labels against exact fp64 distances on slices at the
    start, in the middle and at the very end, inertia that does not rise - then labels + inertia
    as the end of a fit takes them."""
    import torch

    from sklearn_numba_dpex_amd import _capi
    from sklearn_numba_dpex_amd._capi import lib, ptr
    from sklearn_numba_dpex_amd.kmeans import drivers

    assert n * d > 2**31
    g = torch.Generator(device=cuda)
    g.manual_seed(5)
    centers = torch.randn(k, d, device=cuda, generator=g) * 2.0
    X_t = torch.empty((d, n), dtype=torch.float32, device=cuda)
    chunk = 100_000
    for lo in range(0, n, chunk):
        hi = min(lo + chunk, n)
        y = torch.randint(0, k, (hi - lo,), device=cuda, generator=g)
        X_t[:, lo:hi] = (centers[y] + torch.randn(hi - lo, d, device=cuda, generator=g)).T
    w = torch.rand(n, device=cuda, generator=g) + 0.5
    # (one initial centroid near every blob: random rows leave some blobs without one, and a
    # cluster then empties in the second iteration, which is the host's relocation path)
    init = centers + 0.5 * torch.randn(k, d, device=cuda, generator=g)
    cent = [init.T.contiguous(), torch.empty((d, k), dtype=torch.float32, device=cuda)]
    dc = 0
    plan = _capi.lloyd_plan(n, d, k, dc, 0)
    assert plan.variant == variant and lib.kmx_lloyd_plan_reads_rowmajor(plan) == 1
    X_rm = X_t.T.contiguous()
    ws = torch.empty(plan.workspace_bytes, dtype=torch.uint8, device=cuda)
    labels = [torch.zeros(n, dtype=torch.int32, device=cuda) for _ in range(2)]
    sizes = torch.empty(k, dtype=torch.float32, device=cuda)
    empty = torch.empty(k, dtype=torch.int32, device=cuda)
    stream = _capi.current_stream()
    status = _capi.LloydStatus()
    _capi.check(lib.kmx_lloyd_init(plan, ptr(ws), plan.workspace_bytes, ptr(X_t), ptr(w), ptr(cent[0]), 10, 0.0, stream), "init")

    slices = [slice(0, 3000), slice(n // 2 + 1, n // 2 + 3001), slice(n - 3000, n)]

    def exact_labels(c_t, sl):
        Xs = X_t[:, sl].double()
        dist = (Xs * Xs).sum(0)[:, None] - 2.0 * Xs.T @ c_t.double() + (c_t.double() ** 2).sum(0)[None, :]
        return dist

    w64_total = float(w.double().sum())
    wx = torch.stack([(X_t[f].double() * w.double()).sum() for f in range(0, d, 37)])   # every 37th feature
    inertias = []
    for it in range(3):
        a, b = it % 2, (it + 1) % 2
        print(f"large array: iteration {it}", flush=True)
        _capi.check(lib.kmx_lloyd_iter(plan, ptr(X_t), ptr(X_rm), ptr(w), ptr(cent[a]), ptr(cent[b]), ptr(labels[a]),
                                       ptr(labels[b]), ptr(sizes), ptr(empty), ptr(ws), plan.workspace_bytes, stream),
                    "iter")
        _capi.check(lib.kmx_lloyd_status_read(ptr(ws), status, stream), "status")
        assert status.n_empty == 0 and status.n_iter == it + 1, (status.n_empty, status.n_iter, status.state)
        for sl in slices:
            dist = exact_labels(cent[a], sl)
            got = labels[b][sl].long()
            best = dist.argmin(dim=1)
            bad = torch.nonzero(got != best).flatten()
            if bad.numel():
                gap = dist[bad, got[bad]] - dist[bad, best[bad]]
                assert bool(torch.all(gap <= 1e-6 * dist[bad].max(dim=1).values)), (sl, int(bad.numel()))
        assert float(sizes.double().sum()) == pytest.approx(w64_total, rel=1e-5)
        got_wx = (cent[b][::37].double() * sizes.double()[None, :]).sum(dim=1)
        assert torch.allclose(got_wx, wx, rtol=1e-4, atol=1e-4 * float(wx.abs().max()))
        inertias.append(float(drivers._inertia(X_t, w, cent[b], labels[b])))
        last = b
        if status.state != _capi.KMX_RUNNING:
            # well separated blobs: the second iteration changes no label
            assert status.state == _capi.KMX_CONVERGED_STRICT and it >= 1
            break
    assert all(later <= earlier * (1 + 1e-6) for earlier, later in zip(inertias, inertias[1:]))
    # the end of a fit: labels for the final centroids and their inertia, in one library call
    final = torch.empty(n, dtype=torch.int32, device=cuda)
    inertia = drivers._assign_with_inertia(X_t, w, cent[last], final)[0]
    for sl in slices:
        dist = exact_labels(cent[last], sl)
        got = final[sl].long()
        bad = torch.nonzero(got != dist.argmin(dim=1)).flatten()
        if bad.numel():
            gap = dist[bad, got[bad]] - dist[bad].min(dim=1).values
            assert bool(torch.all(gap <= 1e-6 * dist[bad].max(dim=1).values))
    assert float(inertia) <= inertias[-1] * (1 + 1e-5)
