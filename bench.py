#!/usr/bin/env python3
"""Lloyd throughput of the MI355X KMeans engine on one GPU.

Workload (the second of the frozen configurations, configs[1]): fp32 X of shape 5,000,000 x 14 from 127 Gaussian blobs
(seed 1), k = 127, random-row init, sample weights uniform in [0.5, 1.5], tol = 0.
A "step" is one Lloyd iteration (fused assignment + partial sums, reduction, finalisation)
with X, the weights and the centroids already resident in HBM.

Prints ONE JSON line: iterations/s, plus
  roofline      the fused-step kernel against the roofline it has to approach, from HIP events
                recorded around that kernel on its stream (kmx_lloyd_iter_timed): HBM for the
                kernel that screens the labels on the fp16 matrix cores (variant 61), the fp32
                MFMA peak for the all-fp32 kernel (variant 31, KMX_FLAG_LABELS_F32);
  roofline_other_bound  the same kernel's fp32-equivalent rate (variant 61) or HBM fraction (31);
  cpu_baseline  scikit-learn's OpenMP/Cython Lloyd on the same data on this host's cores (the
                inner routine, and the estimator-level fit of the reference's benchmark protocol);
  kmeanspp_ms   kmeans++ seeding time on configs[3] (1,000,000 x 64, k = 256), with
                cpu_baseline_kmeanspp (scikit-learn's seeding on the same data) and the default
                sampler's picks against the reference's own sampler beside it.
"""

import argparse
import ctypes
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0       # MI355X HBM3E
FP32_PEAK_TFLOPS = 157.3    # MI355X fp32, vector and matrix
RAMP_MS = 60.0              # untimed iterations before every timed region, for the GPU clocks
FLAG_LABELS_F32 = 0x10      # KMX_FLAG_LABELS_F32: every product of the fp32 paths in fp32
REGIONS = 3                 # timed regions of --steps iterations; the median one is reported


def log(*a):
    print(*a, file=sys.stderr, flush=True)


def lloyd_bytes(n, d, s):
    # read X once, read weight, read previous label, write new label
    return n * (s * d + s + 4 + 4)


def lloyd_flops(n, d, k):
    return 2.0 * n * d * k + 2.0 * n * d


def check_labels(labels, X, centers, chunk=20_000):
    """Labels against the arg-min of exact fp64 squared distances; a difference is accepted
    only at a near-tie, |d1 - d2| <= 1e-6 * max_c d(x, c).  Returns the number of near-ties."""
    C = np.asarray(centers, dtype=np.float64)
    ties = 0
    for lo in range(0, X.shape[0], chunk):
        Xc = np.asarray(X[lo:lo + chunk], dtype=np.float64)
        dist = (Xc * Xc).sum(axis=1)[:, None] - 2.0 * Xc @ C.T + (C * C).sum(axis=1)[None, :]
        got = labels[lo:lo + chunk].astype(np.int64)
        bad = np.flatnonzero(got != dist.argmin(axis=1))
        if bad.size:
            exact = ((Xc[bad, None, :] - C[None, :, :]) ** 2).sum(axis=2)
            gap = exact[np.arange(bad.size), got[bad]] - exact.min(axis=1)
            if np.any(gap > 1e-6 * exact.max(axis=1)):
                raise RuntimeError(f"{bad.size} labels differ from the exact arg-min beyond the near-tie bound")
            ties += int(np.count_nonzero(gap > 0))
    return ties


def gpu_lloyd(cfg, steps, warmup, flags=0, gates=True):
    """Times `steps` Lloyd iterations of one fit: a throw-away run first brings the GPU clocks
    up (at least RAMP_MS of iterations, whatever --warmup says), then the fit restarts from the
    initial centroids, runs `warmup` untimed iterations and `steps` timed ones, i.e. the timed
    region is iterations warmup + 1 .. warmup + steps of a fit."""
    import torch

    from sklearn_numba_dpex_amd import _capi
    from sklearn_numba_dpex_amd._capi import lib, ptr

    dev = torch.device("cuda:0")
    X, init, w, k = cfg["X"], cfg["init"], cfg["sample_weight"], cfg["k"]
    n, d = X.shape
    dc = _capi.dtype_code(X.dtype)
    X_t = torch.as_tensor(X, device=dev).T.contiguous()
    w_d = torch.as_tensor(w, device=dev)
    cent = [torch.as_tensor(np.ascontiguousarray(init.T), device=dev), None]
    cent[1] = torch.empty_like(cent[0])
    labels = [torch.zeros(n, dtype=torch.int32, device=dev) for _ in range(2)]
    sizes = torch.empty(k, dtype=X_t.dtype, device=dev)
    empty = torch.empty(k, dtype=torch.int32, device=dev)
    plan = _capi.lloyd_plan(n, d, k, dc, flags)
    ws_bytes = plan.workspace_bytes
    ws = torch.empty(ws_bytes, dtype=torch.uint8, device=dev)
    stream = _capi.current_stream()
    status = _capi.LloydStatus()
    cent_init = cent[0].clone()
    # At tol = 0 the run stops by itself once no label changes (iteration 851 on configs[1]);
    # kernels enqueued after that are no-ops.  So that every timed launch does its work for
    # any --steps, the run restarts from the initial centroids every RESTART iterations (one
    # tiny copy + kmx_lloyd_init, inside the timed region when it happens).
    RESTART = 600
    it = 0          # iterations since the last (re)start
    done = 0        # iterations that must have done work, over all restarts
    checked = 0

    def restart():
        nonlocal it, checked
        if it:
            _capi.check(lib.kmx_lloyd_status_read(ptr(ws), status, stream), "status")
            if status.n_iter != it:
                raise RuntimeError(f"only {status.n_iter} of {it} iterations did work (state {status.state}): "
                                   "the timed region would include no-op launches")
            checked += it
        cent[0].copy_(cent_init)
        _capi.check(lib.kmx_lloyd_init(plan, ptr(ws), ws_bytes, ptr(X_t), ptr(w_d), ptr(cent[0]),
                                       RESTART + 8, 0.0, stream), "init")
        it = 0

    def enqueue(ms=None):
        nonlocal it, done
        if it >= RESTART:
            restart()
        a, b = it % 2, (it + 1) % 2
        args = (plan, ptr(X_t), None, ptr(w_d), ptr(cent[a]), ptr(cent[b]), ptr(labels[a]), ptr(labels[b]),
                ptr(sizes), ptr(empty), ptr(ws), ws_bytes, stream)
        if ms is None:
            _capi.check(lib.kmx_lloyd_iter(*args), "iter")
        else:
            _capi.check(lib.kmx_lloyd_iter_timed(*args, ms), "iter_timed")
        it += 1
        done += 1

    # clock ramp: the GPU clocks need tens of milliseconds of load to come up; a throw-away
    # run provides them, then the fit proper starts over from the initial centroids
    restart()
    ramp_iters = 0
    t_ramp = time.perf_counter()
    while (time.perf_counter() - t_ramp) * 1e3 < RAMP_MS and ramp_iters < RESTART - 50:
        for _ in range(50):
            enqueue()
        ramp_iters += 50
        torch.cuda.synchronize()
    restart()
    for _ in range(warmup):
        enqueue()
    # REGIONS timed regions of `steps` iterations each, one after the other in the same fit; the
    # median region is the one reported
    regions = []
    region_event_ms = []
    for _ in range(REGIONS):
        # (HIP events on the launch stream - torch's current stream is the one the library is
        # given - around the whole region: two event records per region, not per launch)
        ev0, ev1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        ev0.record()
        for _ in range(steps):
            enqueue()
        ev1.record()
        torch.cuda.synchronize()
        regions.append(time.perf_counter() - t0)
        region_event_ms.append(ev0.elapsed_time(ev1))
    elapsed = float(np.median(regions))
    launch_period_ms = float(np.median(region_event_ms)) / steps

    # per-kernel durations from HIP events on the launch stream: a stream of back-to-back
    # iterations, every one with events around its kernels (kmx_lloyd_iter_traced enqueues and
    # does not wait), read after the last one.  Iterations that each wait for the host, as
    # kmx_lloyd_iter_timed does, leave the GPU idle in between, and on some machines the kernels
    # that follow such a gap run for 20 us longer than in a fit.
    def enqueue_traced():
        nonlocal it, done
        if it >= RESTART:
            restart()
        a, b = it % 2, (it + 1) % 2
        _capi.check(lib.kmx_lloyd_iter_traced(plan, ptr(X_t), None, ptr(w_d), ptr(cent[a]), ptr(cent[b]),
                                              ptr(labels[a]), ptr(labels[b]), ptr(sizes), ptr(empty), ptr(ws),
                                              ws_bytes, stream), "iter_traced")
        it += 1
        done += 1

    ms = (ctypes.c_float * 3)()
    ms_min = (ctypes.c_float * 3)()
    n_traced = ctypes.c_int32(0)
    for _ in range(10):
        enqueue()
    timed = 100
    for _ in range(timed):
        enqueue_traced()
    _capi.check(lib.kmx_lloyd_trace_collect(ms, ms_min, ctypes.byref(n_traced)), "trace_collect")
    if n_traced.value != timed:
        raise RuntimeError(f"{n_traced.value} traced launches, expected {timed}")
    kernel_ms = np.array(list(ms), dtype=np.float64)
    _capi.check(lib.kmx_lloyd_status_read(ptr(ws), status, stream), "status")
    if status.n_iter != it or checked + it != done:
        raise RuntimeError(f"only {status.n_iter} of {it} iterations did work (state {status.state})")

    # samples the last iteration evaluated in fp32 because its fp16 screen could not certify them
    rechecked = ctypes.c_uint32(0)
    _capi.check(lib.kmx_lloyd_recheck_count(plan, ptr(ws), ctypes.byref(rechecked), stream), "recheck_count")
    if not gates:
        return elapsed, kernel_ms, 0, plan.variant, int(rechecked.value), ramp_iters, regions, launch_period_ms

    # parity gate 1: the labels the last Lloyd iteration wrote, against exact fp64 distances to
    # the centroids it started from, on a slice
    m = min(n, 200_000)
    prev_c = cent[(it - 1) % 2].T.cpu().numpy()
    ties_iter = check_labels(labels[it % 2][:m].cpu().numpy(), X[:m], prev_c)
    # parity gate 2: kmx_assign_labels for the centroids the last iteration produced
    cur = cent[it % 2].T.cpu().numpy()
    lab = torch.empty(n, dtype=torch.int32, device=dev)
    aws = lib.kmx_assign_workspace_bytes_for(n, d, k, dc, flags)
    aws_t = torch.empty(aws, dtype=torch.uint8, device=dev)
    _capi.check(lib.kmx_assign_labels(ptr(X_t), ptr(X_t.new_tensor(cur.T.copy())), ptr(lab), ptr(aws_t), aws,
                                      n, d, k, dc, flags, stream), "assign")
    ties = ties_iter + check_labels(lab[:m].cpu().numpy(), X[:m], cur)
    return elapsed, kernel_ms, ties, plan.variant, int(rechecked.value), ramp_iters, regions, launch_period_ms


def gpu_measured_peaks():
    """What this GPU reaches on the simplest kernels (probe kernels of the library, HIP events on
    the launch stream): a 1 GiB device-to-device copy, a read-only pass over 1 GiB, and streams
    of independent fp32 / fp16 / fp64 matrix-core instructions."""
    import torch

    from sklearn_numba_dpex_amd import _capi
    from sklearn_numba_dpex_amd._capi import lib, ptr

    dev = torch.device("cuda:0")
    stream = _capi.current_stream()
    nbytes = 1 << 30
    src = torch.empty(nbytes // 4, dtype=torch.float32, device=dev).normal_()
    dst = torch.empty_like(src)
    scratch = torch.zeros(1 << 20, dtype=torch.uint8, device=dev)

    def timed(fn, reps):
        for _ in range(3):
            fn()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(reps):
            fn()
        e1.record()
        e1.synchronize()
        return e0.elapsed_time(e1) * 1e-3 / reps

    t_copy = timed(lambda: _capi.check(lib.kmx_probe_copy(ptr(src), ptr(dst), nbytes, stream), "probe_copy"), 10)
    t_read = timed(lambda: _capi.check(lib.kmx_probe_read(ptr(src), nbytes, ptr(scratch), stream), "probe_read"), 10)
    out = {"what": "probe kernels of the library on this GPU: 1 GiB copy (read + written bytes), 1 GiB read-only "
                   "stream, independent MFMA chains (two waves per SIMD)",
           "copy_GBps": 2 * nbytes / t_copy / 1e9, "read_GBps": nbytes / t_read / 1e9}
    flops = ctypes.c_double(0.0)
    for kind, name in ((0, "mfma_f32_TFLOPs"), (1, "mfma_f16_TFLOPs"), (2, "mfma_f64_TFLOPs")):
        t = timed(lambda: _capi.check(lib.kmx_probe_mfma(kind, 20000, ptr(scratch), ctypes.byref(flops), stream),
                                      "probe_mfma"), 3)
        out[name] = flops.value / t / 1e12
    # issue slots: ns per loop round (two MFMAs + 2 V vector-ALU instructions per wave, three waves per SIMD)
    iters = 20000
    issue = {}
    for kind, name in ((2, "valu_only"), (0, "mfma_f16"), (1, "mfma_f32")):
        for v in (0, 8, 16, 32):
            if kind == 2 and v == 0:
                continue
            t = timed(lambda: _capi.check(lib.kmx_probe_issue(kind, v, iters, ptr(scratch), stream), "probe_issue"), 3)
            issue[f"{name}_valu{v}"] = t * 1e9 / iters
    per_valu = issue["valu_only_valu32"] / (3 * 64)   # 3 waves x 64 instructions per round
    out["issue"] = {
        "what": "ns per loop round of 3 waves on one SIMD, each issuing two MFMAs and 2 V independent v_max3_f32 "
                "(valuV); hidden = share of the MFMA-only time that disappears when the vector work is added",
        "ns_per_round": issue,
        "ns_per_valu_instruction": per_valu,
        "ns_per_mfma_f16": issue["mfma_f16_valu0"] / 6, "ns_per_mfma_f32": issue["mfma_f32_valu0"] / 6,
        "mfma_f16_hidden_at_valu16": 1.0 - (issue["mfma_f16_valu16"] - issue["valu_only_valu16"]) / issue["mfma_f16_valu0"],
        "mfma_f16_hidden_at_valu8": 1.0 - (issue["mfma_f16_valu8"] - issue["valu_only_valu8"]) / issue["mfma_f16_valu0"],
        "mfma_f32_hidden_at_valu16": 1.0 - (issue["mfma_f32_valu16"] - issue["valu_only_valu16"]) / issue["mfma_f32_valu0"],
    }
    del src, dst
    return out


def gpu_lloyd_step_time(cfg, reps, consecutive=False, flags=0):
    """Per-kernel times of a Lloyd iteration, mean ms of (fused step, reduce, finalize).

    ONE iteration from the configuration's initial centroids, the state re-initialised before
    every repetition (so relocation or convergence never turns a timed launch into a no-op).
    consecutive=True additionally returns the wall time per iteration of iterations 6 .. 5 + reps
    of the host driver's loop (relocation of empty clusters included), as the difference of two
    runs from the same centroids."""
    import torch

    from sklearn_numba_dpex_amd import _capi
    from sklearn_numba_dpex_amd._capi import lib, ptr

    dev = torch.device("cuda:0")
    X, init, w, k = cfg["X"], cfg["init"], cfg["sample_weight"], cfg["k"]
    n, d = X.shape
    dc = _capi.dtype_code(X.dtype)
    plan = _capi.lloyd_plan(n, d, k, dc, flags)
    variant = plan.variant
    X_rm = torch.as_tensor(X, device=dev)
    X_t = X_rm.T.contiguous()
    if lib.kmx_lloyd_plan_reads_rowmajor(plan) != 1:  # (only some kernels sum rows of a row-major copy)
        X_rm = None
    w_d = torch.as_tensor(w, device=dev)
    cent = [torch.as_tensor(np.ascontiguousarray(init.T), device=dev), None]
    cent[1] = torch.empty_like(cent[0])
    labels = [torch.zeros(n, dtype=torch.int32, device=dev) for _ in range(2)]
    sizes = torch.empty(k, dtype=X_t.dtype, device=dev)
    empty = torch.empty(k, dtype=torch.int32, device=dev)
    ws_bytes = plan.workspace_bytes
    ws = torch.empty(ws_bytes, dtype=torch.uint8, device=dev)
    stream = _capi.current_stream()
    ms = (ctypes.c_float * 3)()
    acc = np.zeros(3)
    if consecutive:
        # the loop as a fit runs it (relocation of empty clusters included): two runs of the
        # driver from the same centroids, the difference isolates the later iterations
        from sklearn_numba_dpex_amd.kmeans import drivers

        def run(max_iter):
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            n_iter = drivers.lloyd(X_t, w_d, cent[0], max_iter=max_iter, tol=0.0, flags=flags)[3]
            torch.cuda.synchronize()
            return time.perf_counter() - t0, int(n_iter)

        run(2)
        t_short, it_short = run(5)
        t_long, it_long = run(5 + reps)
        if it_long <= it_short:
            raise RuntimeError(f"the run converged after {it_long} iterations: nothing to time")
        wall_ms = (t_long - t_short) / (it_long - it_short) * 1e3
    for rep in range(reps + 2):
        _capi.check(lib.kmx_lloyd_init(plan, ptr(ws), ws_bytes, ptr(X_t), ptr(w_d), ptr(cent[0]), 10, 0.0,
                                       stream), "init")
        _capi.check(lib.kmx_lloyd_iter_timed(plan, ptr(X_t), ptr(X_rm), ptr(w_d), ptr(cent[0]), ptr(cent[1]),
                                             ptr(labels[0]), ptr(labels[1]), ptr(sizes), ptr(empty), ptr(ws),
                                             ws_bytes, stream, ms), "iter_timed")
        if rep >= 2:
            acc += np.array(list(ms))
    if consecutive:
        return acc / reps, int(variant), wall_ms
    return acc / reps, int(variant)


def gpu_lloyd_later_step_time(cfg, start_iter, reps, flags=0):
    """Mean ms of the fused step over iterations start_iter + 3 .. start_iter + 2 + reps of a run:
    the driver's loop (relocation of empty clusters included) runs start_iter iterations from the
    configuration's initial centroids, then the iterations are timed one by one through the C ABI
    (the first two rebuild the sums, as after every re-initialisation, and are left out).  Also
    returns the samples per iteration that the label screen could not certify."""
    import torch

    from sklearn_numba_dpex_amd import _capi
    from sklearn_numba_dpex_amd._capi import lib, ptr
    from sklearn_numba_dpex_amd.kmeans import drivers

    dev = torch.device("cuda:0")
    X, init, w, k = cfg["X"], cfg["init"], cfg["sample_weight"], cfg["k"]
    n, d = X.shape
    plan = _capi.lloyd_plan(n, d, k, _capi.dtype_code(X.dtype), flags)
    X_rm = torch.as_tensor(X, device=dev)
    X_t = X_rm.T.contiguous()
    if lib.kmx_lloyd_plan_reads_rowmajor(plan) != 1:
        X_rm = None
    w_d = torch.as_tensor(w, device=dev)
    c0 = torch.as_tensor(np.ascontiguousarray(init.T), device=dev)
    cent = [drivers.lloyd(X_t, w_d, c0, max_iter=start_iter, tol=0.0, flags=flags)[2].clone(), None]
    cent[1] = torch.empty_like(cent[0])
    labels = [torch.zeros(n, dtype=torch.int32, device=dev) for _ in range(2)]
    sizes = torch.empty(k, dtype=X_t.dtype, device=dev)
    empty = torch.empty(k, dtype=torch.int32, device=dev)
    ws = torch.empty(plan.workspace_bytes, dtype=torch.uint8, device=dev)
    stream = _capi.current_stream()
    ms = (ctypes.c_float * 3)()
    status = _capi.LloydStatus()
    count = ctypes.c_uint32(0)
    _capi.check(lib.kmx_lloyd_init(plan, ptr(ws), plan.workspace_bytes, ptr(X_t), ptr(w_d), ptr(cent[0]), 1000, 0.0,
                                   stream), "init")
    fused, uncertain = [], []
    for it in range(reps + 2):
        a, b = it % 2, (it + 1) % 2
        _capi.check(lib.kmx_lloyd_iter_timed(plan, ptr(X_t), ptr(X_rm), ptr(w_d), ptr(cent[a]), ptr(cent[b]),
                                             ptr(labels[a]), ptr(labels[b]), ptr(sizes), ptr(empty), ptr(ws),
                                             plan.workspace_bytes, stream, ms), "iter_timed")
        _capi.check(lib.kmx_lloyd_status_read(ptr(ws), status, stream), "status")
        _capi.check(lib.kmx_lloyd_recheck_count(plan, ptr(ws), ctypes.byref(count), stream), "recheck")
        if status.state != _capi.KMX_RUNNING:
            break
        if it >= 2:
            fused.append(float(ms[0]))
            uncertain.append(int(count.value))
    if not fused:
        raise RuntimeError("the run ended before an iteration could be timed")
    return float(np.mean(fused)), int(np.mean(uncertain)), len(fused)


def extra_configs():
    """Configs 3 (fp32, d=256, k=1024: matrix-core bound) and 5 (fp64, forced empty clusters)."""
    from sklearn_numba_dpex_amd import datasets

    out = {}
    t0 = time.time()
    c3 = datasets.config3()
    n, d = c3["X"].shape
    kms, variant, wall_ms = gpu_lloyd_step_time(c3, 10, consecutive=True)
    # the same step with every product in fp32 on the matrix cores (the label kernel the default
    # path falls back to for the samples its fp16 screen cannot certify): MFMA utilisation
    kms32, _ = gpu_lloyd_step_time(c3, 5, flags=FLAG_LABELS_F32)
    flops = lloyd_flops(n, d, c3["k"])
    out["config3"] = {
        "workload": f"configs[2]: Lloyd n={n} d={d} k={c3['k']} fp32; ms_per_iter over iterations 6-15 of the "
                    "driver's loop, kernel_ms of the first iteration",
        "kernel_variant": variant, "ms_per_iter": wall_ms, "iters_per_sec": 1e3 / wall_ms,
        "labels": "fp16 matrix-core screen, certified per sample, all-fp32 matrix-core kernel where not certified",
        "kernel_ms": {"fused_step": float(kms[0]), "reduce": float(kms[1]), "finalize": float(kms[2])},
        "fused_step_fp32_equivalent_TFLOPs": flops / (kms[0] * 1e-3) / 1e12,
        "all_fp32": {"switch": "KMX_FLAG_LABELS_F32", "fused_step_ms": float(kms32[0]),
                     "fused_step_TFLOPs": flops / (kms32[0] * 1e-3) / 1e12,
                     "fused_step_frac_of_fp32_peak": flops / (kms32[0] * 1e-3) / 1e12 / FP32_PEAK_TFLOPS},
    }
    log(f"[bench] config 3: {out['config3']['ms_per_iter']:.3f} ms/iter (fused step {kms[0]:.3f} ms); with every "
        f"product in fp32: fused step {kms32[0]:.3f} ms = "
        f"{out['config3']['all_fp32']['fused_step_frac_of_fp32_peak']:.3f} of fp32 peak ({time.time() - t0:.1f}s incl. data)")
    del c3
    t0 = time.time()
    c5 = datasets.config5()
    n, d = c5["X"].shape
    kms, variant, wall_ms = gpu_lloyd_step_time(c5, 10, consecutive=True)
    later_ms, later_uncertain, later_n = gpu_lloyd_later_step_time(c5, 4, 8)
    # the same with the fp16 screen switched off: every product on the fp64 matrix cores
    kms64, variant64, wall64_ms = gpu_lloyd_step_time(c5, 10, consecutive=True, flags=FLAG_LABELS_F32)
    flops = lloyd_flops(n, d, c5["k"])
    nbytes = lloyd_bytes(n, d, 8)
    out["config5"] = {
        "workload": f"configs[4]: Lloyd n={n} d={d} k={c5['k']} fp64 (16 clusters that empty on the first iteration); "
                    "ms_per_iter over iterations 6-15 of the driver's loop, kernel_ms of the first iteration "
                    "(sums rebuilt from every sample), later_iterations: iterations 7-14 (sums corrected)",
        "kernel_variant": variant, "ms_per_iter": wall_ms, "iters_per_sec": 1e3 / wall_ms,
        "labels": "fp16 matrix-core screen on the rows rounded to fp32, certified per sample, fp64 matrix cores "
                  "where not certified; sums from the fp64 rows",
        "kernel_ms": {"fused_step": float(kms[0]), "reduce": float(kms[1]), "finalize": float(kms[2])},
        "later_iterations": {"fused_step_ms": later_ms, "iterations": later_n,
                             "samples_not_certified": later_uncertain,
                             "fused_step_frac_of_hbm_peak": nbytes / (later_ms * 1e-3) / 1e9 / HBM_PEAK_GBS},
        "fused_step_frac_of_hbm_peak": nbytes / (kms[0] * 1e-3) / 1e9 / HBM_PEAK_GBS,
        "all_fp64": {"switch": "KMX_FLAG_LABELS_F32", "kernel_variant": variant64, "ms_per_iter": wall64_ms,
                     "fused_step_ms": float(kms64[0]),
                     "fused_step_frac_of_fp64_peak": flops / (kms64[0] * 1e-3) / 1e12 / 78.6},
    }
    log(f"[bench] config 5: {wall_ms:.3f} ms/iter (fused step: first iteration {kms[0]:.3f} ms, later {later_ms:.3f} ms, "
        f"{later_uncertain} samples not certified); all fp64: {wall64_ms:.3f} ms/iter, fused step {kms64[0]:.3f} ms "
        f"({time.time() - t0:.1f}s incl. data)")
    del c5
    out["other_shapes"] = other_shapes()
    return out


def other_shapes():
    """Shapes off the specialised kernels, as users bring them: few clusters of wide samples,
    fp64 with sums beyond LDS, more than 256 features.  Overlapping blobs (the labels keep
    changing), wall time per iteration over iterations 6-13 of the driver's loop."""
    return [one_shape(*spec) for spec in (("70000 x 784, 10 clusters, fp32", 70_000, 784, 10, np.float32),
                                          ("70000 x 784, 24 clusters, fp32", 70_000, 784, 24, np.float32),
                                          ("70000 x 784, 10 clusters, fp64", 70_000, 784, 10, np.float64),
                                          ("2e6 x 100, 10 clusters, fp32", 2_000_000, 100, 10, np.float32),
                                          ("1e6 x 100, 100 clusters, fp64", 1_000_000, 100, 100, np.float64),
                                          ("1e6 x 48, 64 clusters, fp64", 1_000_000, 48, 64, np.float64),
                                          ("1e5 x 300, 300 clusters, fp32", 100_000, 300, 300, np.float32))]


def seeding_ms(X, k, reps=3):
    """Median wall time of a whole kmeans++ seeding (default sampler) of k centres, unit weights."""
    import torch

    from sklearn_numba_dpex_amd.kmeans import drivers

    dev = torch.device("cuda:0")
    X_t = torch.as_tensor(X, device=dev).T.contiguous()
    w_d = torch.ones(X.shape[0], dtype=X_t.dtype, device=dev)
    ts = []
    for rep in range(reps + 1):
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        drivers.kmeans_plusplus(X_t, w_d, k, np.random.RandomState(rep))
        torch.cuda.synchronize()
        ts.append(time.perf_counter() - t0)
    return float(np.median(ts[1:])) * 1e3


def one_shape(name, n, d, k, dtype, reps=8):
    """Overlapping Gaussian blobs of the given shape: wall time per iteration over iterations
    6 .. 5 + reps of the driver's loop and the kernel times of a first iteration."""
    t0 = time.time()
    rng = np.random.default_rng(n + d + k)
    centers = (rng.uniform(-1.0, 1.0, (k, d)) * (4.0 / np.sqrt(d))).astype(dtype)  # overlapping blobs
    X = centers[rng.integers(0, k, n)]
    X += rng.standard_normal((n, d), dtype=dtype)
    cfg = {"X": X, "init": X[rng.choice(n, k, replace=False)].copy(), "sample_weight": np.ones(n, dtype=dtype), "k": k}
    kms, variant, wall_ms = gpu_lloyd_step_time(cfg, reps, consecutive=True)
    s = np.dtype(dtype).itemsize
    log(f"[bench] {name}: variant {variant}, {wall_ms:.3f} ms/iter ({time.time() - t0:.1f}s incl. data)")
    return {"shape": name, "kernel_variant": variant, "ms_per_iter": wall_ms, "kmeanspp_ms": seeding_ms(X, k),
            "label_and_sum_kernels_ms": float(kms[0]), "reduce_and_finalize_ms": float(kms[1] + kms[2]),
            "TFLOPs": lloyd_flops(n, d, k) / (wall_ms * 1e-3) / 1e12,
            "X_bytes_per_iter_TBs": n * d * s / (wall_ms * 1e-3) / 1e12,
            "frac_of_hbm_peak": n * d * s / (wall_ms * 1e-3) / 1e9 / HBM_PEAK_GBS}


def gpu_components(cfg):
    """Times of the other kernels of the path on the same data (configs[1]), each with its
    algorithmic bytes: labels, inertia, labels + inertia as `predict`/`score` run them,
    euclidean distances (on a slice: the output is n x k), radix top-k, sums, centering."""
    import torch

    from sklearn_numba_dpex_amd.common.reductions import sum_reduction
    from sklearn_numba_dpex_amd.common.topk import topk_idx
    from sklearn_numba_dpex_amd.kmeans import drivers

    dev = torch.device("cuda:0")
    X, init, w, k = cfg["X"], cfg["init"], cfg["sample_weight"], cfg["k"]
    n, d = X.shape
    X_t = torch.as_tensor(X, device=dev).T.contiguous()
    w_d = torch.as_tensor(w, device=dev)
    cent_t = torch.as_tensor(np.ascontiguousarray(init.T), device=dev)
    labels = torch.empty(n, dtype=torch.int32, device=dev)
    s = 4

    def timed(fn, reps=5):
        fn()
        ts = []
        for _ in range(reps):
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            fn()
            torch.cuda.synchronize()
            ts.append(time.perf_counter() - t0)
        return float(np.median(ts))

    out = {}

    def put(name, seconds, nbytes, note):
        out[name] = {"ms": seconds * 1e3, "algorithmic_MB": nbytes / 1e6, "GBps": nbytes / seconds / 1e9,
                     "hbm_frac": nbytes / seconds / 1e9 / HBM_PEAK_GBS, "what": note}

    t = timed(lambda: drivers._assign(X_t, cent_t, labels))
    put("assign_labels", t, n * (s * d + 4), "kmx_assign_labels (pack + labels kernel); fp32 contraction bound")
    out["assign_labels"]["TFLOPs"] = 2.0 * n * d * k / t / 1e12
    per_sample = torch.empty(n, dtype=X_t.dtype, device=dev)
    t = timed(lambda: drivers._per_sample_inertia(X_t, w_d, cent_t, labels, out=per_sample))
    put("per_sample_inertia", t, n * (s * d + 4 + 2 * s), "kmx_per_sample_inertia")
    t = timed(lambda: sum_reduction(per_sample))
    put("sum_1d", t, n * s, "kmx_sum_rows over n values (launches + workspace allocation included)")
    t = timed(lambda: drivers.get_labels_inertia(X_t, cent_t, w_d, True))
    put("get_labels_inertia", t, n * (2 * s * d + 8 + 3 * s),
        "labels + inertia + sum + scalar read-back, as score() runs it")
    m = min(n, 500_000)
    Xs_t = X_t[:, :m].contiguous()
    t = timed(lambda: drivers.get_euclidean_distances(Xs_t, cent_t))
    put("euclidean_distances", t, m * (s * d + s * k),
        f"kmx_euclidean_distances on {m} samples (output {m}x{k}, allocation included)")
    t = timed(lambda: topk_idx(per_sample, 16))
    put("topk_idx_16", t, 2 * n * s,
        "radix select of the 16 largest of n values: two reads of the values (first digit, then winners + "
        "candidates), the remaining digits on the few candidates; six launches whose ends wait on each other")
    t = timed(lambda: sum_reduction(X_t, axis=1))
    put("sum_rows_d_by_n", t, n * d * s, "kmx_sum_rows over X_t (d, n): the feature sums of the centering")
    from sklearn_numba_dpex_amd.common.matmul import matmul

    A = torch.randn(4096, 4096, device=dev)
    B = torch.randn(4096, 4096, device=dev)
    t = timed(lambda: matmul(A, B))
    put("matmul_4096", t, 3 * 4096 * 4096 * s, "kmx_matmul fp32 4096 x 4096 x 4096 on the matrix cores (contraction bound)")
    out["matmul_4096"]["TFLOPs"] = 2.0 * 4096**3 / t / 1e12
    out["matmul_4096"]["fp32_peak_frac"] = out["matmul_4096"]["TFLOPs"] / FP32_PEAK_TFLOPS
    A64, B64 = A.double(), B.double()
    t = timed(lambda: matmul(A64, B64))
    put("matmul_4096_f64", t, 3 * 4096 * 4096 * 8, "kmx_matmul fp64 4096 x 4096 x 4096 (v_mfma_f64_16x16x4_f64)")
    out["matmul_4096_f64"]["TFLOPs"] = 2.0 * 4096**3 / t / 1e12
    out["matmul_4096_f64"]["fp64_peak_frac"] = out["matmul_4096_f64"]["TFLOPs"] / 78.6
    del A, B, A64, B64
    Xc = X_t.clone()
    t = timed(lambda: drivers.prepare_data_for_lloyd(Xc, cent_t.clone(), 1e-4, w_d, copy_x=False))
    put("prepare_data_for_lloyd", t, 4 * n * d * s,
        "mean, centering in place, variance for tol, uniform-weight test (3 reads + 1 write of X)")
    return out


def gpu_kmeanspp(cfg):
    import torch

    from sklearn_numba_dpex_amd.kmeans import drivers

    dev = torch.device("cuda:0")
    X_t = torch.as_tensor(cfg["X"], device=dev).T.contiguous()
    w = torch.as_tensor(cfg["sample_weight"], device=dev)
    times = []
    for rep in range(3):
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        centers_t, idx = drivers.kmeans_plusplus(X_t, w, cfg["k"], np.random.RandomState(cfg["seed"]))
        torch.cuda.synchronize()
        times.append((time.perf_counter() - t0) * 1e3)
    return float(np.median(times)), idx.cpu().numpy()


def kpp_sampler_report(cfg):
    """The default sampler (search of the fp64 inclusive scan) against the reference's own
    (running sum in the compute dtype, KMX_KPP_SAMPLER_LITERAL) on the same seeding: for every
    centre both samplers draw their candidates from the same closest-distance array with the
    same uniforms, then the seeding goes on with the default sampler's.  Reports how many draws
    pick another sample and how far apart the picks are in cumulative probability."""
    import torch

    from sklearn_numba_dpex_amd import _capi
    from sklearn_numba_dpex_amd._capi import lib, ptr
    from sklearn_numba_dpex_amd.kmeans import drivers

    dev = torch.device("cuda:0")
    X_t = torch.as_tensor(cfg["X"], device=dev).T.contiguous()
    w = torch.as_tensor(cfg["sample_weight"], device=dev)
    d, n = X_t.shape
    k, tn = cfg["k"], cfg["n_local_trials"]
    dc = _capi.dtype_code(X_t.dtype)
    start_raw, table = drivers.kpp_uniforms(k, tn, np.random.RandomState(cfg["seed"]), np.float32)
    uniforms = torch.from_numpy(table).to(dev)
    centers_t = torch.empty((d, k), dtype=X_t.dtype, device=dev)
    indices = torch.full((k,), -1, dtype=torch.int32, device=dev)
    ws_bytes = lib.kmx_kpp_workspace_bytes(n, d, k, tn, dc)
    ws = torch.empty(ws_bytes, dtype=torch.uint8, device=dev)
    st = _capi.current_stream()
    _capi.check(lib.kmx_kpp_init(ptr(X_t), ptr(w), int(start_raw % n), ptr(centers_t), ptr(indices), ptr(ws), ws_bytes,
                                 n, d, k, tn, dc, 0, st), "kpp_init")
    rows_off = lib.kmx_kpp_closest_ptr(ptr(ws), n, d, k, tn, dc) - ws.data_ptr()
    cand_lit = torch.empty(tn, dtype=torch.int32, device=dev)
    cand_scan = torch.empty(tn, dtype=torch.int32, device=dev)
    draws = differ = 0
    shift_samples = []
    gap_prob = []
    lit_ms = 0.0
    for c in range(1, k):
        u = uniforms[c - 1]
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        _capi.check(lib.kmx_kpp_sample_candidates(ptr(X_t), ptr(u), ptr(cand_lit), ptr(ws), ws_bytes, n, d, k, tn, dc,
                                                  _capi.KMX_KPP_SAMPLER_LITERAL, st), "kpp_sample literal")
        torch.cuda.synchronize()
        lit_ms += (time.perf_counter() - t0) * 1e3
        _capi.check(lib.kmx_kpp_sample_candidates(ptr(X_t), ptr(u), ptr(cand_scan), ptr(ws), ws_bytes, n, d, k, tn, dc,
                                                  _capi.KMX_KPP_SAMPLER_SCAN, st), "kpp_sample")
        a, b = cand_lit.cpu().numpy().astype(np.int64), cand_scan.cpu().numpy().astype(np.int64)
        draws += tn
        if np.any(a != b):
            best_row = int(ws[:4].view(torch.int32).item())
            lo = rows_off + best_row * n * 4
            closest = ws[lo:lo + n * 4].view(torch.float32).cpu().numpy()
            cum = np.cumsum(closest.astype(np.float64))
            rv = table[c - 1] * cum[-1]
            for t in np.flatnonzero(a != b):
                differ += 1
                shift_samples.append(abs(int(a[t]) - int(b[t])))
                gap_prob.append(abs(rv[t] - cum[a[t]]) / cum[-1])
        _capi.check(lib.kmx_kpp_step(ptr(X_t), ptr(w), c, ptr(centers_t), ptr(indices), ptr(ws), ws_bytes, n, d, k, tn,
                                     dc, 0, st), "kpp_step")
    return {
        "what": "default sampler (fp64 inclusive scan) against the reference's running sum in fp32 "
                "(KMX_KPP_SAMPLER_LITERAL), same closest-distance array and uniforms for every draw of one seeding",
        "draws": draws, "draws_with_another_pick": differ,
        "index_shift_samples_median": float(np.median(shift_samples)) if shift_samples else 0.0,
        "index_shift_samples_max": int(max(shift_samples)) if shift_samples else 0,
        "max_gap_rv_minus_cum_at_literal_pick_over_total": float(max(gap_prob)) if gap_prob else 0.0,
        "literal_sampler_ms_per_centre": lit_ms / (k - 1),
    }


def cpu_kmeanspp_baseline(cfg):
    """scikit-learn's own seeding on the same data: wall clock of
    sklearn.cluster.kmeans_plusplus(X, k, random_state=seed), after a small warm-up call."""
    from sklearn.cluster import kmeans_plusplus
    from sklearn.utils._openmp_helpers import _openmp_effective_n_threads

    X = cfg["X"]
    kmeans_plusplus(X[:10_000], 8, random_state=0)
    t0 = time.perf_counter()
    kmeans_plusplus(X, cfg["k"], random_state=cfg["seed"])
    elapsed = time.perf_counter() - t0
    return elapsed * 1e3, _openmp_effective_n_threads()


def cpu_lloyd_baseline(cfg, max_iter):
    """scikit-learn's Lloyd (OpenMP Cython) on the same data, inner routine only."""
    from sklearn.cluster._kmeans import _kmeans_single_lloyd
    from sklearn.utils._openmp_helpers import _openmp_effective_n_threads

    X, init, w = cfg["X"], cfg["init"], cfg["sample_weight"]
    threads = _openmp_effective_n_threads()
    _kmeans_single_lloyd(X, w, init.copy(), max_iter=1, tol=0, n_threads=threads)  # warm-up
    t0 = time.perf_counter()
    _, _, _, n_iter = _kmeans_single_lloyd(X, w, init.copy(), max_iter=max_iter, tol=0, n_threads=threads)
    elapsed = time.perf_counter() - t0
    # the routine ends with one extra labelling pass; count it as the work it is
    return n_iter / elapsed, threads, n_iter, elapsed


def cpu_fit_baseline(cfg, max_iter):
    """The reference benchmark's own protocol (benchmark/kmeans.py:137-170) on stock
    scikit-learn: KMeans(init=<array>, n_init=1, tol=0, algorithm="lloyd", copy_x=True).fit
    timed with perf_counter after a max_iter=1 dry run; iterations per second = n_iter_ / elapsed."""
    from sklearn.cluster import KMeans

    X, init, w = cfg["X"], cfg["init"], cfg["sample_weight"]
    kwargs = dict(n_clusters=cfg["k"], init=init.copy(), n_init=1, max_iter=max_iter, tol=0, random_state=0,
                  copy_x=True, algorithm="lloyd")
    import warnings

    with warnings.catch_warnings():
        warnings.simplefilter("ignore")   # ConvergenceWarning: max_iter is the point
        KMeans(**kwargs).set_params(max_iter=1).fit(X, sample_weight=w)
        est = KMeans(**kwargs)
        t0 = time.perf_counter()
        est.fit(X, sample_weight=w)
        elapsed = time.perf_counter() - t0
    return est.n_iter_ / elapsed, int(est.n_iter_), elapsed


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=100)
    ap.add_argument("--warmup", type=int, default=5,
                    help="untimed iterations of the fit before the timed ones (the GPU clocks are brought up "
                         "by a separate throw-away run, whatever this is)")
    ap.add_argument("--n", type=int, default=5_000_000, help="samples (default: the full configuration)")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--no-kpp", action="store_true", help="skip the kmeans++ leg")
    ap.add_argument("--cpu-iters", type=int, default=20)
    ap.add_argument("--no-extra", action="store_true", help="skip the config 3 / config 5 legs")
    ap.add_argument("--shape", default=None, metavar="N,D,K,f32|f64",
                    help="only time Lloyd iterations on synthetic blobs of this shape (one JSON line) and exit")
    ap.add_argument("--copy-probe", action="store_true",
                    help="also run five 1 GiB device-to-device copies (calibration of HBM traffic counters)")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py measures one GPU: this build has no multi-GPU path (--gpus must be 1)")

    if args.shape:
        n_s, d_s, k_s, t_s = args.shape.split(",")
        print(json.dumps(one_shape(f"{n_s} x {d_s}, {k_s} clusters, {t_s}", int(n_s), int(d_s), int(k_s),
                                   np.float64 if t_s == "f64" else np.float32, reps=max(1, args.steps))), flush=True)
        return

    from sklearn_numba_dpex_amd import datasets

    t0 = time.time()
    cfg = datasets.config2(n=args.n)
    n, d = cfg["X"].shape
    k = cfg["k"]
    log(f"[bench] data {n}x{d} k={k} generated in {time.time() - t0:.1f}s")

    if args.copy_probe:
        import torch

        src = torch.empty(1 << 28, dtype=torch.float32, device="cuda:0").normal_()
        dst = torch.empty_like(src)
        for _ in range(5):
            dst.copy_(src)
        torch.cuda.synchronize()
        del src, dst

    elapsed, kernel_ms, ties, variant, rechecked, ramp_iters, regions, period_ms = gpu_lloyd(cfg, args.steps, args.warmup)
    ms_per_step = elapsed / args.steps * 1e3
    iters_per_s = args.steps / elapsed
    # Variant 61 is ONE kernel per iteration (its last workgroup finishes the iteration), so the
    # launch period of the back-to-back launches of a timed region - two HIP events around the
    # region on the launch stream, divided by the launches - is that kernel's duration plus the
    # gap to the next launch.  Event pairs around every single launch (kernel_ms) add the cost of
    # their own records to what they bracket, several microseconds per record on these machines.
    one_kernel = int(variant) == 61 and kernel_ms[1] + kernel_ms[2] < 0.5 * kernel_ms[0]
    fused_s = (period_ms if one_kernel else kernel_ms[0]) * 1e-3
    flops = lloyd_flops(n, d, k)
    nbytes = lloyd_bytes(n, d, 4)
    log(f"[bench] {ms_per_step:.4f} ms/iter; kernels (ms): fused {kernel_ms[0]:.4f} reduce "
        f"{kernel_ms[1]:.4f} finalize {kernel_ms[2]:.4f}; near-tie label differences on slices: {ties}; "
        f"samples evaluated in fp32 by the last iteration: {rechecked} ({rechecked / n:.2e} of n)")

    traffic = None
    traffic_source = None
    traffic_file = os.path.join(ROOT, "profiles", "lloyd_fused_step_c2_traffic.json")
    if os.path.exists(traffic_file) and n == 5_000_000:
        with open(traffic_file) as f:
            traffic = json.load(f).get("hbm_bytes_per_launch")
        traffic_source = ("profiles/lloyd_fused_step_c2_traffic.json: rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE of this "
                          "kernel on this workload, calibrated against a 1 GiB copy; a committed counter reading, "
                          "not taken in this run")

    mfma_roof = {
        "bound": "mfma",
        "achieved": flops / fused_s / 1e12,
        "peak": FP32_PEAK_TFLOPS,
        "unit": "TFLOP/s",
        "frac": flops / fused_s / 1e12 / FP32_PEAK_TFLOPS,
        "traffic": traffic,
        "traffic_source": traffic_source,
        "kernel": "fused Lloyd step",
        "flops_per_launch": flops,
    }
    hbm_roof = {
        "bound": "hbm",
        "achieved": nbytes / fused_s / 1e9,
        "peak": HBM_PEAK_GBS,
        "unit": "GB/s",
        "frac": nbytes / fused_s / 1e9 / HBM_PEAK_GBS,
        "traffic": traffic,
        "traffic_source": traffic_source,
        "kernel": "fused Lloyd step",
        "bytes_per_launch": nbytes,
        "launch_duration_ms": fused_s * 1e3,
        "launch_duration_from": ("HIP events around each timed region of back-to-back launches (one kernel per "
                                 "iteration) / launches: kernel plus the gap to the next launch"
                                 if one_kernel else "HIP events around every launch of the kernel"),
    }
    # Variant 61 screens the labels on the fp16 matrix cores: the fp32 contraction that bounded
    # variant 31 is gone, and what is left to approach is the HBM time of the algorithmic bytes.
    # Variant 31 (KMX_FLAG_LABELS_F32) multiplies in fp32 and is priced against the fp32 MFMA peak.
    roofline, roofline_other = (hbm_roof, mfma_roof) if int(variant) == 61 else (mfma_roof, hbm_roof)
    if int(variant) == 61:
        # this kernel multiplies on the fp16 matrix cores: the fp32 peak does not bound it, so the
        # rate of the exact contraction it replaces is reported as a rate, not as a fraction
        roofline_other = {
            "fp32_equivalent_TFLOPs": mfma_roof["achieved"],
            "flops_per_launch": flops,
            "kernel": "fused Lloyd step",
            "note": "2 n d k + 2 n d flops of the exact fp32 contraction over the kernel time, for comparison "
                    "with the all-fp32 kernel (all_fp32); this kernel runs 3 fp16 products per fp32 one "
                    "instead, so the fp32 MFMA peak (157.3 TFLOP/s) is no bound for it",
        }

    # the same fit with every product taken in fp32 (variant 31), timed the same way
    e32, kms32, _, variant32, _, _, _, _ = gpu_lloyd(cfg, args.steps, args.warmup, flags=FLAG_LABELS_F32, gates=False)
    all_fp32 = {
        "switch": "KMX_FLAG_LABELS_F32", "kernel_variant": int(variant32),
        "ms_per_step": e32 / args.steps * 1e3, "iters_per_sec": args.steps / e32,
        "fused_step_ms": float(kms32[0]),
        "fused_step_TFLOPs": flops / (kms32[0] * 1e-3) / 1e12,
        "frac_of_fp32_peak": flops / (kms32[0] * 1e-3) / 1e12 / FP32_PEAK_TFLOPS,
    }
    log(f"[bench] every product in fp32: {all_fp32['ms_per_step']:.4f} ms/iter, fused step "
        f"{kms32[0]:.4f} ms = {all_fp32['frac_of_fp32_peak']:.3f} of fp32 peak")
    peaks = gpu_measured_peaks()
    log("[bench] measured peaks: " + ", ".join(f"{k2} {v:.1f}" for k2, v in peaks.items() if isinstance(v, float)))
    hbm_roof["frac_of_measured_peak"] = hbm_roof["achieved"] / peaks["read_GBps"]
    if int(variant) != 61:
        mfma_roof["frac_of_measured_peak"] = mfma_roof["achieved"] / peaks["mfma_f32_TFLOPs"]
    all_fp32["frac_of_measured_fp32_peak"] = all_fp32["fused_step_TFLOPs"] / peaks["mfma_f32_TFLOPs"]

    out = {
        "metric": "lloyd_iterations_per_sec",
        "value": iters_per_s,
        "unit": "iter/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "clock_ramp_iters": int(ramp_iters),
        "timed_iterations": f"{REGIONS} regions of {args.steps} iterations, one after the other from iteration "
                            f"{args.warmup + 1} of a fit from the initial centroids; value and ms_per_step are the "
                            "median region's",
        "ms_per_step_regions": [r / args.steps * 1e3 for r in regions],
        "ms_per_step": ms_per_step,
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "f32",
        "data": "synthetic",
        "config": {"workload": f"configs[1]: Lloyd n={n} d={d} k={k} fp32, weighted, tol=0",
                   "kernel_variant": int(variant),
                   "labels": ("fp16 matrix-core screen, certified per sample, fp32 where not certified"
                              if int(variant) == 61 else "fp32 matrix cores"),
                   "sums": "fp32 inputs, 64-bit fixed point"},
        "samples_clusters_per_sec": iters_per_s * n * k,
        "kernel_ms": {"fused_step": float(kernel_ms[0]), "reduce": float(kernel_ms[1]),
                      "finalize": float(kernel_ms[2]),
                      "what": "HIP event pairs around every kernel of 100 back-to-back traced iterations "
                              "(kmx_lloyd_iter_traced); each interval includes the cost of an event record"},
        "launch_period_ms": period_ms,
        "roofline": roofline,
        "roofline_other_bound": roofline_other,
        "all_fp32": all_fp32,
        "measured_peaks": peaks,
        "fp32_evaluated_samples": {"count": int(rechecked), "fraction_of_n": rechecked / n},
        "parity": {"near_tie_label_differences": int(ties), "checked_samples": min(n, 200_000)},
    }

    if not args.no_kpp:
        t0 = time.time()
        c4 = datasets.config4()
        kpp_ms, _ = gpu_kmeanspp(c4)
        n4, d4 = c4["X"].shape
        tn = c4["n_local_trials"]
        kpp_bytes = (c4["k"] - 1) * (n4 * (4 * d4 + 8) + tn * n4 * 4)
        out["kmeanspp_ms"] = kpp_ms
        out["kmeanspp"] = {"workload": f"configs[3]: n={n4} d={d4} k={c4['k']} trials={tn}",
                           "ms": kpp_ms, "hbm_GBs": kpp_bytes / (kpp_ms * 1e-3) / 1e9,
                           "hbm_frac": kpp_bytes / (kpp_ms * 1e-3) / 1e9 / HBM_PEAK_GBS}
        log(f"[bench] kmeans++ {kpp_ms:.1f} ms ({time.time() - t0:.1f}s incl. data)")
        t0 = time.time()
        out["kmeanspp"]["sampler_vs_reference"] = kpp_sampler_report(c4)
        log(f"[bench] kmeans++ samplers: {out['kmeanspp']['sampler_vs_reference']} ({time.time() - t0:.1f}s)")
        if not args.no_cpu:
            cpu_kpp_ms, cpu_kpp_threads = cpu_kmeanspp_baseline(c4)
            out["cpu_baseline_kmeanspp"] = {
                "value": cpu_kpp_ms, "unit": "ms", "cores": int(cpu_kpp_threads), "kind": "reference",
                "impl": "sklearn.cluster.kmeans_plusplus(X, %d, random_state=%d), scikit-learn %s (numpy/BLAS "
                        "distances, one candidate batch per centre)" % (c4["k"], c4["seed"],
                                                                         __import__("sklearn").__version__),
                "sample": f"the whole seeding at full n={n4}, d={d4}",
            }
            log(f"[bench] sklearn CPU kmeans++: {cpu_kpp_ms:.0f} ms")
        del c4

    if not args.no_extra:
        out["components"] = gpu_components(cfg)
        log("[bench] components (ms): " + ", ".join(f"{k2} {v['ms']:.3f}" for k2, v in out["components"].items()))
        del cfg["X"]  # free host memory before the 1 GB configuration is generated
        out["other_configs"] = extra_configs()
        cfg = None

    if not args.no_cpu:
        if cfg is None:
            cfg = datasets.config2(n=args.n)
        cpu_ips, threads, cpu_iters, cpu_elapsed = cpu_lloyd_baseline(cfg, args.cpu_iters)
        fit_ips, fit_iters, fit_elapsed = cpu_fit_baseline(cfg, args.cpu_iters)
        try:
            from threadpoolctl import threadpool_info

            pools = [{key: p.get(key) for key in ("user_api", "internal_api", "prefix", "num_threads", "version")}
                     for p in threadpool_info()]
        except Exception as exc:  # the baseline does not depend on it
            pools = repr(exc)
        out["cpu_baseline"] = {
            "value": cpu_ips,
            "unit": "iter/s",
            "cores": int(threads),
            "kind": "reference",
            "impl": "scikit-learn %s _kmeans_single_lloyd (OpenMP Cython), the CPU engine the reference "
                    "plugin subclasses and falls back to" % __import__("sklearn").__version__,
            "sample": f"same data and init, {cpu_iters} iterations at full n={n} in {cpu_elapsed:.1f}s "
                      f"(os.cpu_count()={os.cpu_count()})",
            "estimator_fit": {"iters_per_sec": fit_ips, "n_iter": fit_iters, "seconds": fit_elapsed,
                              "what": "KMeans(init=array, n_init=1, tol=0, algorithm='lloyd', copy_x=True).fit(X, "
                                      "sample_weight) after a max_iter=1 dry run: input validation, centering "
                                      "and the final labelling included"},
            "threadpool_info": pools,
        }
        log(f"[bench] sklearn CPU Lloyd: {cpu_ips:.3f} iter/s on {threads} threads")

    print(json.dumps(out), flush=True)


if __name__ == "__main__":
    main()
