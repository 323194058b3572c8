#!/usr/bin/env python3
"""Benchmark of the index-tree kernel path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W]
                    [--workload headline|spmm|spgemm|tricount|spmv|ttgt|sddmm|coo2csr|copy|gather]

A step is one pass of the kernel over one batch of seeded synthetic input that is already
resident in HBM.  The default workload is the one the headline metric is quoted on: CSR SpMM,
A 500,000 x 500,000 with power-law rows (mean 16, cap 4096), B 500,000 x 64 fp64; the default run adds, under
"also", short runs of the other workloads the metric names (SpGEMM and masked SpGEMM at R-MAT scale 20) and of
SpMV and the TTGT contraction.  Prints ONE JSON line.  `roofline` describes the dominant kernel: algorithmic bytes (or flops)
per launch divided by that kernel's average duration, measured here with HIP events on the
library's stream.  `cpu_baseline` is the CPU checker (oracle/, a restatement of the loop nests
COMET generates) timed on this machine's host cores on a bounded sample of the same workload.
"""
import argparse
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0        # MI355X HBM3E, published
FP64_MFMA_PEAK_TFLOPS = 78.6  # MI355X dense fp64 matrix, published


def _sha12(path):
    import hashlib
    with open(os.path.join(ROOT, path), "rb") as f:
        return hashlib.sha256(f.read()).hexdigest()[:12]


def measured_traffic(workload):
    """HBM-side bytes per step from the rocprofv3 --pmc runs recorded in profiles/*.txt, or None.

    A profile summary carries one line per workload,
        TRAFFIC workload=<name> bytes=<per step> ... sources=<file>:<sha256[:12]>[,<file>:<sha>...]
    naming the kernel sources the counters were read on.  The figure is reported only while those files are
    unchanged: after any edit of a kernel source it is null until the counters are read again."""
    import glob
    for path in sorted(glob.glob(os.path.join(ROOT, "profiles", "*.txt"))):
        with open(path) as f:
            for line in f:
                if not line.startswith("TRAFFIC "):
                    continue
                kv = dict(tok.split("=", 1) for tok in line.split()[1:] if "=" in tok)
                if kv.get("workload") != workload:
                    continue
                try:
                    same = all(_sha12(src) == sha for src, sha in (t.rsplit(":", 1) for t in kv["sources"].split(",")))
                except (OSError, KeyError, ValueError):
                    same = False
                return (int(kv["bytes"]), os.path.basename(path)) if same else (None, os.path.basename(path) + " (stale: kernel sources changed since the counters were read)")
    return None, None


def mem_free(rt):
    import ctypes as C
    f, t = C.c_int64(), C.c_int64()
    rt._check(rt.lib().comet_hip_mem_info(C.byref(f), C.byref(t)), "comet_hip_mem_info")
    return f.value


def first_call(rt, fn):
    """Wall time of the first call of `fn` (device drained before and after) and the device memory it keeps:
    what a program that multiplies once pays on top of a steady-state step (plans cached in the handle,
    workspaces)."""
    rt.sync()
    free0 = mem_free(rt)
    t0 = time.perf_counter()
    fn()
    rt.sync()
    return (time.perf_counter() - t0) * 1e3, free0 - mem_free(rt)


_T0 = time.perf_counter()


def log(msg):
    """Progress line on stderr (the JSON result is the only thing printed on stdout)."""
    print(f"[bench {time.perf_counter() - _T0:7.1f}s] {msg}", file=sys.stderr, flush=True)


def host_threads():
    env = os.environ.get("OMP_NUM_THREADS")
    if env and env.isdigit():
        return int(env)
    try:
        return len(os.sched_getaffinity(0))
    except AttributeError:
        return os.cpu_count() or 1


def timed_steps(rt, fn, steps, warmup):
    for _ in range(warmup):
        fn()
    rt.sync()
    t0 = time.perf_counter()
    rt.timer_start()
    for _ in range(steps):
        fn()
    dev_ms = rt.timer_stop()
    rt.sync()
    wall_ms = (time.perf_counter() - t0) * 1e3
    return wall_ms / steps, dev_ms / steps


def kernel_times(rt, fn, steps):
    """Average duration per launch of every kernel `fn` starts, from event pairs."""
    rt.profile_reset()
    rt.profile_enable(True)
    for _ in range(steps):
        fn()
    rt.sync()
    rep = rt.profile_report()
    rt.profile_enable(False)
    return {k: {"launches": n, "avg_ms": ms / max(n, 1)} for k, (n, ms) in rep.items()}


def cpu_time(fn, budget_s=20.0, min_reps=1, max_reps=5):
    best = None
    t_start = time.perf_counter()
    reps = 0
    while reps < max_reps and (reps < min_reps or time.perf_counter() - t_start < budget_s):
        t0 = time.perf_counter()
        fn()
        dt = time.perf_counter() - t0
        best = dt if best is None else min(best, dt)
        reps += 1
        if dt > budget_s / 2:
            break
    return best, reps


# ----------------------------------------------------------------------------- workloads
def bench_spmm(rt, orc, gen, args):
    n, K = args.n or 500_000, 64
    pos, crd, val = gen.zipf_csr(n=n, mean=16.0, cap=4096, seed=2)
    nnz = len(crd)
    B = gen.dense((n, K), seed=3)
    A = rt.CsrMatrix.from_arrays((n, n), pos, crd, val)
    dB = rt.DeviceArray.from_numpy(B)
    dC = rt.DeviceArray((n, K))
    step = lambda: rt.spmm(A, dB, dC, accumulate=False)
    # the first product runs without a plan, the second one builds it (neither is timed as a step)
    first_ms, kept_first = first_call(rt, step)
    second_ms, kept_second = first_call(rt, step)
    kept_bytes = kept_first + kept_second
    wall_ms, dev_ms = timed_steps(rt, step, args.steps, args.warmup)
    kt = kernel_times(rt, step, args.steps)
    flops = 2.0 * nnz * K
    ib = 4
    alg_bytes = nnz * (8 + ib) + (n + 1) * ib + 8 * n * K + 8 * n * K
    # one product = several kernels (sweep, chunk kernel, the kernels that stitch rows together, fills); the
    # algorithmic bytes are those of the whole product, so the roofline is taken over the timed step
    dom = " + ".join(sorted(kt))
    dom_ms = dev_ms
    kernel_sum_ms = sum(v["avg_ms"] * v["launches"] for v in kt.values()) / args.steps
    traffic, traffic_src = measured_traffic("spmm_csr_zipf") if (n, K) == (500_000, 64) else (None, None)
    # parity of what was just timed, on a sample of rows (full check lives in tests/)
    got = dC.to_numpy()
    rows = np.random.default_rng(0).choice(n, 2000, replace=False)
    sub_pos = np.zeros(len(rows) + 1, dtype=np.int64)
    np.cumsum(pos[rows + 1] - pos[rows], out=sub_pos[1:])
    sel = np.concatenate([np.arange(pos[r], pos[r + 1]) for r in rows])
    want = orc.spmm(sub_pos, crd[sel], val[sel], B)
    bound = orc.spmm(sub_pos, crd[sel], np.abs(val[sel]), np.abs(B))
    parity_ok = bool(np.all(np.abs(got[rows] - want) <= 1e-12 * bound))
    cpu = None
    if not args.no_cpu:
        Cc = np.zeros((n, K))
        t, reps = cpu_time(lambda: orc.lib().oracle_spmm_csr(n, K, pos, crd, val, B, Cc), budget_s=20.0, min_reps=2)
        cpu = {"value": flops / t / 1e9, "unit": "GFLOP/s", "cores": host_threads(), "kind": "port",
               "sample": f"the full workload, best of {reps} runs, {t * 1e3:.1f} ms each (OpenMP over rows)"}
    lens = np.diff(pos)
    return {
        "metric": "CSR SpMM GFLOP/s (+ achieved HBM GB/s as % of roofline) on 1 MI355X",
        "value": flops / (dev_ms * 1e-3) / 1e9, "unit": "GFLOP/s", "ms_per_step": dev_ms,
        "dtype": "f64",
        "config": {"workload": "spmm_csr_zipf", "rows": n, "cols": n, "nnz": int(nnz), "dense_cols": K,
                   "row_lengths": "Zipf s=1.5 rescaled to mean 16, cap 4096 (untruncated draw, scale, clip)",
                   "max_row": int(lens.max()), "rows_len1_frac": float((lens == 1).mean()), "seed": 2,
                   "index_bytes": ib, "accumulate": False},
        "roofline": {"bound": "hbm", "achieved": alg_bytes / (dom_ms * 1e-3) / 1e9, "peak": HBM_PEAK_GBS,
                     "unit": "GB/s", "frac": alg_bytes / (dom_ms * 1e-3) / 1e9 / HBM_PEAK_GBS,
                     "traffic": traffic, "traffic_source": traffic_src,
                     "kernel": dom, "kernel_avg_ms": dom_ms, "kernel_sum_ms": kernel_sum_ms,
                     "algorithmic_bytes": int(alg_bytes),
                     "gather_inclusive_bytes": int(nnz * 8 * K + nnz * (8 + ib) + 8 * n * K)},
        "plan": {"first_call_ms": first_ms, "second_call_ms": second_ms, "plan_ms": max(second_ms - dev_ms, 0.0),
                 "kept_device_bytes": int(kept_bytes),
                 "note": "a matrix's first product runs without a plan (all rows through the chunk kernel), its second "
                         "one builds the plan: plan_ms = second product minus a steady-state one; bytes = device "
                         "memory the two calls keep (lists of the long rows, the other rows re-packed, workspaces)"},
        "cpu_baseline": cpu, "kernels": kt, "wall_ms_per_step": wall_ms, "parity_sample_ok": parity_ok,
    }


def bench_sddmm(rt, orc, gen, args):
    """A = B .* (C x D) on the SpMM matrix: B 500,000^2 CSR, C n x 64, D 64 x n."""
    n, K = args.n or 500_000, 64
    pos, crd, val = gen.zipf_csr(n=n, mean=16.0, cap=4096, seed=2)
    nnz = len(crd)
    Cm, D = gen.dense((n, K), seed=5), gen.dense((K, n), seed=6)
    B = rt.CsrMatrix.from_arrays((n, n), pos, crd, val)
    dC, dD = rt.DeviceArray.from_numpy(Cm), rt.DeviceArray.from_numpy(D)
    vals = rt.DeviceArray(nnz)               # A shares B's structure: the step writes its values
    step = lambda: rt.sddmm(B, dC, dD, out_values=vals)
    step()
    wall_ms, dev_ms = timed_steps(rt, step, args.steps, args.warmup)
    kt = kernel_times(rt, step, args.steps)
    rows = np.arange(0, n, max(1, n // 2000))            # the checker on a sample of rows
    lo, hi = pos[rows], pos[rows + 1]
    sel = np.concatenate([np.arange(a, b) for a, b in zip(lo, hi)])
    spos = np.concatenate([[0], np.cumsum(hi - lo)])
    parity_ok = bool(np.array_equal(vals.to_numpy()[sel],
                                    orc.sddmm(spos, crd[sel], val[sel], Cm[rows], D)))
    flops = 2.0 * nnz * K + nnz
    ib = 4
    alg_bytes = nnz * (8 + ib) + (n + 1) * ib + 8 * n * K * 2 + nnz * 8      # B, C and D once, A's values once
    dom = "sddmm_kernel"
    dom_ms = kt[dom]["avg_ms"]
    cpu = None
    if not args.no_cpu:
        res = np.zeros(nnz)
        t, reps = cpu_time(lambda: orc.lib().oracle_sddmm_csr(n, n, pos, crd, val, K, Cm, D, res), budget_s=20.0)
        cpu = {"value": flops / t / 1e9, "unit": "GFLOP/s", "cores": 1, "kind": "port",
               "sample": f"the full workload, best of {reps} runs, {t * 1e3:.0f} ms each (single thread)"}
    return {
        "metric": "SDDMM GFLOP/s (+ achieved HBM GB/s as % of roofline) on 1 MI355X",
        "value": flops / (dev_ms * 1e-3) / 1e9, "unit": "GFLOP/s", "ms_per_step": dev_ms, "dtype": "f64",
        "config": {"workload": "sddmm_csr_zipf", "rows": n, "cols": n, "nnz": int(nnz), "inner": K, "seed": 2,
                   "index_bytes": ib},
        "roofline": {"bound": "hbm", "achieved": alg_bytes / (dev_ms * 1e-3) / 1e9, "peak": HBM_PEAK_GBS,
                     "unit": "GB/s", "frac": alg_bytes / (dev_ms * 1e-3) / 1e9 / HBM_PEAK_GBS,
                     "traffic": measured_traffic("sddmm_csr_zipf")[0] if (n, K) == (500_000, 64) else None,
                     "kernel": dom + " (+ transpose of D: the whole step is timed)",
                     "kernel_avg_ms": dom_ms, "algorithmic_bytes": int(alg_bytes)},
        "cpu_baseline": cpu, "kernels": kt, "wall_ms_per_step": wall_ms, "parity_sample_ok": parity_ok,
    }


def bench_spmv(rt, orc, gen, args):
    n = args.n or 1_000_000
    pos, crd, val = gen.poisson_csr(n=n, mean=10.0, seed=1)
    nnz = len(crd)
    x = gen.dense(n, seed=4)
    A = rt.CsrMatrix.from_arrays((n, n), pos, crd, val)
    dx = rt.DeviceArray.from_numpy(x)
    dy = rt.DeviceArray(n)
    step = lambda: rt.spmv(A, dx, dy, accumulate=False)
    # the first product runs on the matrix as it is, the second one makes the column-blocked copy (neither is a step)
    first_ms, kept_first = first_call(rt, step)
    second_ms, kept_second = first_call(rt, step)
    kept_bytes = kept_first + kept_second
    wall_ms, dev_ms = timed_steps(rt, step, args.steps, args.warmup)
    kt = kernel_times(rt, step, args.steps)
    parity_ok = bool(np.array_equal(dy.to_numpy(), orc.spmv(pos, crd, val, x)))
    flops = 2.0 * nnz
    ib = 4
    alg_bytes = nnz * (8 + ib) + (n + 1) * ib + 8 * n + 8 * n
    # all column blocks of the plan in one launch, or (rows beyond what one resident grid holds) one launch per block
    dom = "spmv_csr_blocks" if "spmv_csr_blocks" in kt else "spmv_csr_stream"
    passes = kt[dom]["launches"] // args.steps
    # the step holds nothing but these launches, and an event pair per launch adds several microseconds of its own to
    # a kernel this short: the event pair around the timed steps is the kernel time
    dom_ms = dev_ms
    cpu = None
    if not args.no_cpu:
        y = np.zeros(n)
        t, reps = cpu_time(lambda: orc.lib().oracle_spmv_csr(n, pos, crd, val, x, y), budget_s=10.0, min_reps=3)
        cpu = {"value": flops / t / 1e9, "unit": "GFLOP/s", "cores": host_threads(), "kind": "port",
               "sample": f"the full workload, best of {reps} runs, {t * 1e3:.1f} ms each (OpenMP over rows)"}
    return {
        "metric": "CSR SpMV GFLOP/s (+ achieved HBM GB/s as % of roofline) on 1 MI355X",
        "value": flops / (dev_ms * 1e-3) / 1e9, "unit": "GFLOP/s", "ms_per_step": dev_ms, "dtype": "f64",
        "config": {"workload": "spmv_csr_poisson", "rows": n, "cols": n, "nnz": int(nnz), "seed": 1, "index_bytes": ib,
                   "launches_per_step": passes},
        "roofline": {"bound": "hbm", "achieved": alg_bytes / (dom_ms * 1e-3) / 1e9, "peak": HBM_PEAK_GBS,
                     "unit": "GB/s", "frac": alg_bytes / (dom_ms * 1e-3) / 1e9 / HBM_PEAK_GBS,
                     "traffic": measured_traffic("spmv_csr_poisson")[0] if n == 1_000_000 else None,
                     "kernel": dom, "kernel_avg_ms": dom_ms, "launches_per_step": passes,
                     "algorithmic_bytes": int(alg_bytes)},
        "plan": {"first_call_ms": first_ms, "second_call_ms": second_ms, "plan_ms": max(second_ms - dev_ms, 0.0),
                 "kept_device_bytes": int(kept_bytes),
                 "note": "a matrix's first product runs on its own arrays, its second one makes the column-blocked "
                         "copy: plan_ms = second product minus a steady-state one; bytes = that copy"},
        "cpu_baseline": cpu, "kernels": kt, "wall_ms_per_step": wall_ms, "parity_sample_ok": parity_ok,
    }


def bench_ttgt(rt, orc, gen, args):
    e = args.n or 64
    A = gen.dense((e,) * 4, seed=5)
    Bt = gen.dense((e,) * 4, seed=6)
    dA, dB = rt.DeviceArray.from_numpy(A), rt.DeviceArray.from_numpy(Bt)
    dC = rt.DeviceArray((e,) * 4, zero=True)
    plan = rt.ttgt_plan("aebf", "dfce", "abcd", {ch: e for ch in "abcdef"}, which=args.candidate)
    step = lambda: rt.ttgt_contract("aebf", "dfce", "abcd", dA, dB, dC, beta=0.0, plan=plan)
    step()
    wall_ms, dev_ms = timed_steps(rt, step, args.steps, args.warmup)
    kt = kernel_times(rt, step, args.steps)
    M = N = K = e * e
    flops = 2.0 * M * N * K
    dom = "dgemm_mfma_kernel"
    dom_ms = kt[dom]["avg_ms"]
    # parity on a slab of the output: C[a0,b0,:,:] against the checker's GEMM order is too slow at e = 64,
    # so compare with numpy's einsum on a few (a,b) pairs, tolerance relative to sum |a||b|
    got = dC.to_numpy()
    parity_ok = True
    for (a0, b0) in ((0, 0), (e // 2, 1), (e - 1, e - 1)):
        want = np.einsum("ef,dfce->cd", A[a0, :, b0, :], Bt)
        bound = np.einsum("ef,dfce->cd", np.abs(A[a0, :, b0, :]), np.abs(Bt))
        parity_ok &= bool(np.all(np.abs(got[a0, b0] - want) <= 1e-12 * bound))
    cpu = None
    if not args.no_cpu:
        # the default lowering runs a naive i-j-k loop nest; time it at a reduced extent and scale by flops
        m = 768
        Ac, Bc, Cc = gen.dense((m, m), seed=7), gen.dense((m, m), seed=8), np.zeros((m, m))
        t, reps = cpu_time(lambda: orc.lib().oracle_gemm_ijk(m, m, m, Ac, Bc, Cc), budget_s=15.0, min_reps=1)
        cpu = {"value": 2.0 * m ** 3 / t / 1e12, "unit": "TFLOP/s", "cores": host_threads(), "kind": "port",
               "sample": f"naive i-j-k GEMM {m}^3 (OpenMP over i), best of {reps} runs, {t:.2f} s each; the 4096^3 "
                         f"GEMM would take about {2.0 * 4096 ** 3 / (2.0 * m ** 3 / t):.0f} s at that rate"}
        # the strong baseline: the host BLAS numpy is linked against, on a size it finishes in about a second
        mb = 2048
        Ab, Bb = gen.dense((mb, mb), seed=9), gen.dense((mb, mb), seed=10)
        tb, repsb = cpu_time(lambda: Ab @ Bb, budget_s=6.0, min_reps=2)
        cpu["blas_dgemm"] = {"value": 2.0 * mb ** 3 / tb / 1e12, "unit": "TFLOP/s",
                             "sample": f"numpy matmul {mb}^3, best of {repsb} runs, {tb * 1e3:.0f} ms each, "
                                       f"{host_threads()} threads at most"}
    import ctypes as C
    peak = C.c_double(float("nan"))
    if not args.no_peak:        # the yardstick kernel; left out of a profiled run so that the trace holds the workload only
        rt._check(rt.lib().comet_hip_mfma_f64_peak(20000, C.byref(peak)), "comet_hip_mfma_f64_peak")
    perm_bytes = 2 * 8 * e ** 4 * (plan.transA + plan.transB + plan.transC)
    return {
        "metric": "TTGT contraction TFLOP/s (fp64 MFMA GEMM + LDS-tiled transposes) on 1 MI355X",
        "value": flops / (dev_ms * 1e-3) / 1e12, "unit": "TFLOP/s", "ms_per_step": dev_ms, "dtype": "f64",
        "config": {"workload": "ttgt_aebf_dfce_abcd", "extent": e, "gemm": [M, N, K], "candidate": plan.candidate,
                   "transposes": {"A": plan.transA, "B": plan.transB, "C": plan.transC}, "beta": 0.0},
        "roofline": {"bound": "mfma", "achieved": flops / (dom_ms * 1e-3) / 1e12, "peak": FP64_MFMA_PEAK_TFLOPS,
                     "unit": "TFLOP/s", "frac": flops / (dom_ms * 1e-3) / 1e12 / FP64_MFMA_PEAK_TFLOPS, "traffic": None,
                     "kernel": dom, "kernel_avg_ms": dom_ms, "transpose_bytes": int(perm_bytes),
                     "measured_peak": None if args.no_peak else peak.value,
                     "measured_peak_note": "back-to-back v_mfma_f64_16x16x4_f64 on registers, 8 wavefronts per CU",
                     "frac_of_measured_peak": None if args.no_peak else flops / (dom_ms * 1e-3) / 1e12 / peak.value},
        "cpu_baseline": cpu, "kernels": kt, "wall_ms_per_step": wall_ms, "parity_sample_ok": parity_ok,
    }


def _row_products(pos, crd):
    """Products per output row of A*A: sum over k in A_i of nnz(A_k)."""
    deg = np.diff(pos)
    w = deg[crd]
    out = np.zeros(len(pos) - 1, dtype=np.int64)
    nz = deg > 0
    out[nz] = np.add.reduceat(w, pos[:-1][nz])
    return out


def bench_tricount(rt, orc, gen, args):
    scale = args.scale or 20
    n = 1 << scale
    log(f"generating R-MAT scale {scale}")
    pos, crd, val = gen.rmat_symmetric_csr(scale=scale, edge_factor=16, seed=20, values="ones")
    lpos, lcrd, lval = gen.strictly_lower(pos, crd, val)
    del pos, crd, val
    nnzL = len(lcrd)
    deg = np.diff(lpos)
    nprod = int(deg[lcrd].sum())
    L = rt.CsrMatrix.from_arrays((n, n), lpos, lcrd, lval)
    out = {}
    step = lambda: out.__setitem__("count", rt.triangle_count(L))
    first_ms, kept_bytes = first_call(rt, step)
    wall_ms, dev_ms = timed_steps(rt, step, args.steps, args.warmup)
    kt = kernel_times(rt, step, args.steps)
    # rows with many products take a workgroup each, the others a wavefront each: two kernels that run side by side
    # on two streams, so their durations overlap and the span of both is what counts
    dom = "spgemm_masked_sum || spgemm_masked_sum_small"
    dom_ms = max(kt[k]["avg_ms"] for k in ("spgemm_masked_sum", "spgemm_masked_sum_small") if k in kt)
    flops = 2.0 * nprod
    ib = 4
    alg_bytes = nnzL * (ib + 8) + (n + 1) * ib + 8
    cpu = None
    parity = None
    if not args.no_cpu:
        log("CPU checker, full workload")
        t0 = time.perf_counter()
        want = orc.tricount_masked(lpos, lcrd, lval)
        t = time.perf_counter() - t0
        parity = bool(want == out["count"])
        cpu = {"value": flops / t / 1e9, "unit": "GFLOP/s", "cores": 1, "kind": "port",
               "sample": f"the full workload once, {t:.1f} s, single thread (the reference never parallelises "
                         f"sparse-output loops)", "count": want, "seconds": t}
        # a stronger baseline than the reference offers: the same nest row-parallel over the host's cores
        t0 = time.perf_counter()
        want_mt = orc.tricount_masked(lpos, lcrd, lval, threads=True)
        t_mt = time.perf_counter() - t0
        cpu["openmp"] = {"value": flops / t_mt / 1e9, "unit": "GFLOP/s", "cores": host_threads(), "seconds": t_mt,
                         "count_equal": bool(want_mt == want),
                         "speedup_of_gpu": t_mt / (dev_ms * 1e-3)}
    return {
        "metric": "masked SpGEMM triangle count GFLOP/s (2 flops per masked-candidate product) on 1 MI355X",
        "value": flops / (dev_ms * 1e-3) / 1e9, "unit": "GFLOP/s", "ms_per_step": dev_ms, "dtype": "f64",
        "config": {"workload": "tricount_rmat", "scale": scale, "edge_factor": 16, "nnz_L": int(nnzL),
                   "products": nprod, "triangles": out["count"], "seed": 20},
        "roofline": {"bound": "hbm", "achieved": alg_bytes / (dom_ms * 1e-3) / 1e9, "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": alg_bytes / (dom_ms * 1e-3) / 1e9 / HBM_PEAK_GBS,
                     "traffic": measured_traffic("tricount_rmat")[0] if scale == 20 else None, "kernel": dom,
                     "kernel_avg_ms": dom_ms, "algorithmic_bytes": int(alg_bytes)},
        "plan": {"first_call_ms": first_ms, "plan_ms": max(first_ms - dev_ms, 0.0), "kept_device_bytes": int(kept_bytes)},
        "cpu_baseline": cpu, "speedup_vs_cpu": (cpu["seconds"] / (dev_ms * 1e-3)) if cpu else None,
        "kernels": kt, "wall_ms_per_step": wall_ms, "parity_sample_ok": parity,
    }


def bench_spgemm(rt, orc, gen, args):
    """C = A*A on the symmetrised R-MAT graph.  The symbolic phase runs over all rows; the numeric
    phase runs in row blocks sized to a fixed output budget and each block is dropped (at scale 20 the
    whole of C is larger than HBM); one extra, untimed pass sums the values of every block for the check."""
    scale = args.scale or 20
    n = 1 << scale
    log(f"generating R-MAT scale {scale}")
    pos, crd, val = gen.rmat_symmetric_csr(scale=scale, edge_factor=16, seed=20)
    nnzA = len(crd)
    rowprod = _row_products(pos, crd)
    nprod = int(rowprod.sum())
    log(f"nnz(A) = {nnzA}, products = {nprod}; uploading")
    A = rt.CsrMatrix.from_arrays((n, n), pos, crd, val)
    budget = int(args.budget_gb * (1 << 30)) // 12          # entries per block
    state = {}

    mask = A if args.masked else None      # C<A> = A*A: the output holds the stored entries of A that receive a product
    semiring = tuple(args.semiring.split(",")) if args.semiring else None       # e.g. min,plus

    def step(check=False):
        # the whole product: symbolic over all rows, numeric block by block into the same buffers.  With `check`
        # every block is also summed before it is dropped; that pass is the bench's own and stays out of the
        # timed steps (it reads each block once more: 47 ms at scale 20).
        dpos, nnzC = rt.spgemm_symbolic(A, A, mask=mask)
        log(f"symbolic done: nnz(C) = {nnzC}")
        hpos = dpos.to_numpy()
        maxrow = int(np.diff(hpos).max()) if n else 0
        if maxrow > budget:
            raise RuntimeError("a single row exceeds the block budget; raise --budget-gb")
        cap = max(min(budget, int(nnzC)), 1)
        if state.get("cap") != cap:        # output block buffers are allocated once and reused
            state["dcrd"], state["dval"] = rt.DeviceArray(cap, np.int32), rt.DeviceArray(cap)
            state["cap"] = cap
        dcrd, dval = state["dcrd"], state["dval"]
        rb, blocks, vsum = 0, 0, 0.0
        while rb < n:
            re = int(np.searchsorted(hpos, hpos[rb] + cap, side="right")) - 1
            re = min(max(re, rb + 1), n)
            rt.spgemm_numeric(A, A, dpos, rb, re, dcrd, dval, mask=mask, semiring=semiring)
            if check:
                vsum += rt.reduce_sum(dval, int(hpos[re] - hpos[rb]))
            log(f"numeric rows [{rb},{re}): {int(hpos[re] - hpos[rb])} entries")
            rb = re
            blocks += 1
        state.update(nnzC=int(nnzC), blocks=blocks, hpos=hpos, dpos=dpos)
        if check:
            state["vsum"] = vsum

    # every step is seconds long: per-kernel event timing stays on during the timed steps
    first_ms, kept_bytes = first_call(rt, step)
    kept_bytes -= 12 * state["cap"]          # the output block buffers are the caller's, not the library's
    step(check=True)
    for _ in range(args.warmup):
        step()
    rt.profile_reset()
    rt.profile_enable(True)
    wall_ms, dev_ms = timed_steps(rt, step, args.steps, 0)
    rep = rt.profile_report()
    rt.profile_enable(False)
    kt = {k: {"launches": c, "avg_ms": ms / max(c, 1)} for k, (c, ms) in rep.items()}
    nnzC = state["nnzC"]
    flops = 2.0 * nprod
    one_call = None
    if args.masked and 12 * nnzC < 32 * (1 << 30):
        # what lowered code gets (comet_hip_spgemm_csr): both phases in one call, which for a masked product is one
        # walk - values and "met a product" flags of the mask's pairs, the row pointers from the flags
        def whole():
            rt.spgemm(A, A, mask, semiring=semiring).free()
        whole()
        rt.sync()
        t0 = time.perf_counter()
        for _ in range(3):
            whole()
        rt.sync()
        one_call = {"ms": (time.perf_counter() - t0) * 1e3 / 3,
                    "note": "comet_hip_spgemm_csr: the product in one call (wall time of 3 calls, each allocating and "
                            "freeing its result); the steps above time the symbolic and the numeric call of the "
                            "two-phase protocol"}
    ib = 4
    alg_bytes = nnzA * (8 + ib) + (n + 1) * ib + nnzC * (8 + ib) + 8 * (n + 1)
    sym_ms = sum(v["avg_ms"] * v["launches"] for k, v in kt.items() if k.startswith("spgemm_symbolic")) / args.steps
    num_ms = sum(v["avg_ms"] * v["launches"] for k, v in kt.items()
                 if k.startswith("spgemm_numeric") or k in ("spgemm_row_products", "radix_sort_pairs")) / args.steps
    # sum of all values is a size-independent invariant: sum(C) = sum_k colsum(A)[k] * rowsum(A)[k]
    rowsum = np.add.reduceat(val, pos[:-1][np.diff(pos) > 0])
    rs = np.zeros(n)
    rs[np.diff(pos) > 0] = rowsum
    cs = np.bincount(crd, weights=val, minlength=n)
    invariant = float(np.dot(cs, rs))
    cpu = None
    parity = {"sum_values_rel_err": abs(state["vsum"] - invariant) / invariant} if not (args.masked or semiring) else {}
    if not args.no_cpu:
        # CPU checker on a row sample holding about args.cpu_products products, both phases, single thread
        rng = np.random.default_rng(0)
        target = args.cpu_products
        picks, acc = [], 0
        order = rng.permutation(n // 256)
        for b in order:
            r0, r1 = b * 256, (b + 1) * 256
            p = int(rowprod[r0:r1].sum())
            if p == 0 or acc + p > 1.5 * target:
                continue
            picks.append((r0, r1))
            acc += p
            if acc >= target:
                break
        t = 0.0
        struct_ok = True
        hpos = state["hpos"]
        log(f"CPU checker on {len(picks)} row blocks ({acc} products)")
        for (r0, r1) in picks:
            t0 = time.perf_counter()
            cp, cc, cv = orc.spgemm(pos, crd, val, pos, crd, val, n, rows=(r0, r1),
                                    mask=(pos, crd) if args.masked else None, semiring=semiring)
            t += time.perf_counter() - t0
            struct_ok &= bool(np.array_equal(cp, hpos[r0:r1 + 1] - hpos[r0]))
            cnt = int(hpos[r1] - hpos[r0])
            if cnt <= state["cap"]:
                rt.spgemm_numeric(A, A, state["dpos"], r0, r1, state["dcrd"], state["dval"], mask=mask, semiring=semiring)
                gc, gv = state["dcrd"].to_numpy(cnt), state["dval"].to_numpy(cnt)
                struct_ok &= bool(np.array_equal(gc, cc)) and bool(np.all(np.abs(gv - cv) <= 1e-12 * np.abs(cv)))
            log(f"  rows [{r0},{r1}): {cnt} entries checked, CPU time so far {t:.1f} s, ok = {struct_ok}")
        parity["sampled_blocks_bit_exact_structure_and_1e-12_values"] = struct_ok
        cpu = {"value": 2.0 * acc / t / 1e9, "unit": "GFLOP/s", "cores": 1, "kind": "port",
               "sample": f"{len(picks)} blocks of 256 rows holding {acc} of {nprod} products, symbolic + numeric, "
                         f"{t:.1f} s, single thread; extrapolated whole-job time {t * nprod / acc:.0f} s",
               "extrapolated_seconds": t * nprod / acc}
        if semiring is None:
            # a stronger baseline than the reference offers: both phases row-parallel over the host's cores,
            # the sampled rows as one range each
            t_mt = 0.0
            for (r0, r1) in picks:
                t0 = time.perf_counter()
                orc.spgemm(pos, crd, val, pos, crd, val, n, rows=(r0, r1), mask=(pos, crd) if args.masked else None,
                           threads=True)
                t_mt += time.perf_counter() - t0
            cpu["openmp"] = {"value": 2.0 * acc / t_mt / 1e9, "unit": "GFLOP/s", "cores": host_threads(),
                             "extrapolated_seconds": t_mt * nprod / acc,
                             "speedup_of_gpu": (t_mt * nprod / acc) / (dev_ms * 1e-3)}
    return {
        "metric": "Gustavson SpGEMM GFLOP/s (2 flops per product, symbolic + numeric) on 1 MI355X",
        "value": flops / (dev_ms * 1e-3) / 1e9, "unit": "GFLOP/s", "ms_per_step": dev_ms, "dtype": "f64",
        "config": {"workload": ("spgemm_rmat_AxA_masked_by_A" if args.masked else "spgemm_rmat_AxA") +
                               ("_" + "_".join(semiring) if semiring else ""), "scale": scale, "edge_factor": 16, "nnz_A": int(nnzA),
                   "products": nprod, "nnz_C": nnzC, "row_blocks": state["blocks"], "block_budget_gb": args.budget_gb,
                   "seed": 20,
                   **({"note": "flops = 2 per product of the unmasked walk, the convention of the row-by-row form; the "
                               "dot-product form the library uses looks up min(|A_i|, |B^T_j|) entries per stored pair "
                               "of the mask"} if args.masked else {})},
        "roofline": {"bound": "hbm", "achieved": alg_bytes / ((sym_ms + num_ms) * 1e-3) / 1e9, "peak": HBM_PEAK_GBS,
                     "unit": "GB/s", "frac": alg_bytes / ((sym_ms + num_ms) * 1e-3) / 1e9 / HBM_PEAK_GBS,
                     "traffic": measured_traffic("spgemm_rmat_AxA_masked_by_A" if args.masked else "spgemm_rmat_AxA")[0]
                     if (scale, args.budget_gb) == (20, 48.0) else None,
                     "kernel": " + ".join(sorted(k for k in kt if k.startswith("spgemm_symbolic") or k.startswith("spgemm_numeric"))),
                     "kernel_avg_ms": sym_ms + num_ms,
                     "symbolic_ms": sym_ms, "numeric_ms": num_ms, "algorithmic_bytes": int(alg_bytes)},
        "plan": {"first_call_ms": first_ms, "plan_ms": max(first_ms - dev_ms, 0.0), "kept_device_bytes": int(kept_bytes),
                 "note": "first product minus a steady-state product; bytes = block pointers of the right operand, "
                         "row lists and the slabs and bitmaps the library caches"},
        "one_call": one_call,
        "cpu_baseline": cpu, "speedup_vs_cpu": (cpu["extrapolated_seconds"] / (dev_ms * 1e-3)) if cpu else None,
        "kernels": kt, "wall_ms_per_step": wall_ms, "parity_sample_ok": parity,
    }


def bench_copy(rt, orc, gen, args):
    """Streaming yardsticks of a known size: the plain 8-byte-per-lane copy that the FETCH_SIZE / WRITE_SIZE
    counters of the other kernels are scaled by, and three tuned ones (16 bytes per lane: copy with ordinary and
    with non-temporal accesses, read only, write only) that say what the memory system gives a kernel that does
    nothing but move bytes."""
    n = args.n or (1 << 27)            # 1 GiB read + 1 GiB written
    src = rt.DeviceArray(n, zero=True)
    dst = rt.DeviceArray(n)
    lib = rt.lib()
    plain = lambda: rt._check(lib.comet_hip_copy_f64(dst.ptr, src.ptr, n), "comet_hip_copy_f64")
    plain()
    wall_ms, dev_ms = timed_steps(rt, plain, args.steps, args.warmup)
    kt = kernel_times(rt, plain, args.steps)
    dom_ms = kt["copy_f64_kernel"]["avg_ms"]
    nbytes = 16.0 * n
    tuned = {}
    for name, mode, moved in (("copy16", 0, 16.0 * n), ("copy16_nontemporal", 1, 16.0 * n), ("read16", 2, 8.0 * n),
                              ("write16", 3, 8.0 * n)):
        best = None
        for wg in (4, 8, 16, 32):
            step = lambda: rt._check(lib.comet_hip_stream_bench(mode, dst.ptr, src.ptr, n, wg), "comet_hip_stream_bench")
            step()
            _, ms = timed_steps(rt, step, args.steps, args.warmup)
            if best is None or ms < best[0]:
                best = (ms, wg)
        tuned[name] = {"ms": best[0], "GB/s": moved / (best[0] * 1e-3) / 1e9,
                       "frac_of_peak": moved / (best[0] * 1e-3) / 1e9 / HBM_PEAK_GBS, "workgroups_per_cu": best[1],
                       "bytes": int(moved)}
    return {
        "metric": "device copy GB/s (counter calibration)", "value": nbytes / (dev_ms * 1e-3) / 1e9, "unit": "GB/s",
        "ms_per_step": dev_ms, "dtype": "f64", "config": {"workload": "copy_f64", "elements": n},
        "roofline": {"bound": "hbm", "achieved": nbytes / (dom_ms * 1e-3) / 1e9, "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": nbytes / (dom_ms * 1e-3) / 1e9 / HBM_PEAK_GBS, "traffic": None, "kernel": "copy_f64_kernel",
                     "kernel_avg_ms": dom_ms, "algorithmic_bytes": int(nbytes)},
        "tuned_yardsticks": tuned,
        "cpu_baseline": None, "kernels": kt, "wall_ms_per_step": wall_ms, "parity_sample_ok": None,
    }


def bench_coo2csr(rt, orc, gen, args):
    """The reader's ordering step: the tuples of the SpMM matrix in shuffled order -> device CSR."""
    n = args.n or 500_000
    pos, crd, val = gen.zipf_csr(n=n, mean=16.0, cap=4096, seed=2)
    nnz = len(crd)
    row = np.repeat(np.arange(n, dtype=np.int64), np.diff(pos))
    perm = np.random.Generator(np.random.PCG64(5)).permutation(nnz)
    row, col, v = row[perm], crd[perm], val[perm]
    drow = rt.DeviceArray.from_numpy(row.astype(np.int32))
    dcol = rt.DeviceArray.from_numpy(col.astype(np.int32))
    dval = rt.DeviceArray.from_numpy(v)
    out = {}

    def step():
        out["A"] = rt.CsrMatrix.from_coo_device((n, n), drow, dcol, dval)     # the previous result is freed here
    step()
    wall_ms, dev_ms = timed_steps(rt, step, args.steps, args.warmup)
    kt = kernel_times(rt, step, args.steps)
    p, c, vv = out["A"].to_arrays()
    parity_ok = bool(np.array_equal(p, pos) and np.array_equal(c, crd) and np.array_equal(vv, val))
    # tuples read once (4 + 4 + 8 B each), CSR written once (4 + 8 B each, 8 B per row pointer)
    alg_bytes = nnz * 16 + nnz * 12 + 8 * (n + 1)
    dom = "radix_sort_pairs"
    dom_ms = kt[dom]["avg_ms"]
    sort_bytes = nnz * 12 * 2     # one read and one write of (key, position) if the sort were a single pass
    cpu = None
    if not args.no_cpu:
        t, reps = cpu_time(lambda: orc.coo_to_csr(n, row, col, v), budget_s=20.0, min_reps=1)
        cpu = {"value": nnz / t / 1e6, "unit": "Mtuples/s", "cores": 1, "kind": "port",
               "sample": f"the full workload, best of {reps} runs, {t:.2f} s each (stable sort by (row, col), "
                         "filter, row pointers, single thread as in the reference's reader)"}
    return {
        "metric": "COO -> CSR ordering Mtuples/s on 1 MI355X", "value": nnz / (dev_ms * 1e-3) / 1e6,
        "unit": "Mtuples/s", "ms_per_step": dev_ms, "dtype": "u64 keys / f64 values",
        "config": {"workload": "coo_to_csr_zipf_shuffled", "rows": n, "cols": n, "tuples": int(nnz), "seed": 2},
        "roofline": {"bound": "hbm", "achieved": sort_bytes / (dom_ms * 1e-3) / 1e9, "peak": HBM_PEAK_GBS,
                     "unit": "GB/s", "frac": sort_bytes / (dom_ms * 1e-3) / 1e9 / HBM_PEAK_GBS, "traffic": None,
                     "kernel": dom + " (rocPRIM, all its passes)", "kernel_avg_ms": dom_ms,
                     "algorithmic_bytes": int(sort_bytes), "whole_conversion_algorithmic_bytes": int(alg_bytes)},
        "cpu_baseline": cpu, "kernels": kt, "wall_ms_per_step": wall_ms, "parity_sample_ok": parity_ok,
    }


def bench_gather(rt, orc, gen, args):
    """How fast the CUs take rows of 512 bytes out of the L2 when nothing else is done with them: the ceiling of
    the SpMM sweep, whose long rows need nnz x 512 bytes of such gathers.  Every workgroup (16 wavefronts, one per
    CU) draws its rows from the part of the table that belongs to its XCD (4 MiB or less: L2 hits)."""
    import ctypes as C
    rows_per_xcd = args.n or 4096
    wgs, per_wave = 256, 4096
    rng = np.random.Generator(np.random.PCG64(7))
    xcd = (np.arange(wgs * 16) // 16) % 8
    idx = (xcd[:, None] * rows_per_xcd + rng.integers(0, rows_per_xcd, (wgs * 16, per_wave))).astype(np.int32)
    d_idx = rt.DeviceArray.from_numpy(idx)
    table = rt.DeviceArray((8 * rows_per_xcd, 64), zero=True)
    out = rt.DeviceArray(wgs * 1024)
    step = lambda: rt._check(rt.lib().comet_hip_gather_rows_bench(wgs, per_wave, d_idx.ptr, table.ptr,
                                                                  8 * rows_per_xcd, out.ptr), "gather bench")
    step()
    wall_ms, dev_ms = timed_steps(rt, step, args.steps, args.warmup)
    kt = kernel_times(rt, step, args.steps)
    dom_ms = kt["gather_rows_bench"]["avg_ms"]
    nbytes = float(idx.size) * 512
    return {
        "metric": "rows of 512 B gathered from the L2, TB/s (ceiling of the SpMM sweep)", "value": nbytes / (dev_ms * 1e-3) / 1e12,
        "unit": "TB/s", "ms_per_step": dev_ms, "dtype": "f64",
        "config": {"workload": "gather_rows_l2", "table_rows_per_xcd": rows_per_xcd, "table_bytes_per_xcd": rows_per_xcd * 512,
                   "gathers": int(idx.size), "workgroups": wgs, "wavefronts_per_workgroup": 16, "loads_in_flight": 16},
        "roofline": {"bound": "l2 -> CU", "achieved": nbytes / (dom_ms * 1e-3) / 1e9, "peak": None, "unit": "GB/s",
                     "frac": None, "traffic": None, "kernel": "gather_rows_bench", "kernel_avg_ms": dom_ms,
                     "rows_per_second": idx.size / (dom_ms * 1e-3),
                     "bytes_per_clock_per_cu_at_2.4GHz": nbytes / (dom_ms * 1e-3) / 256 / 2.4e9},
        "cpu_baseline": None, "kernels": kt, "wall_ms_per_step": wall_ms, "parity_sample_ok": None,
    }


def bench_headline(rt, orc, gen, args):
    """The metric names SpMM and SpGEMM: the SpMM line carries, under "also", the SpGEMM, masked-SpGEMM (materialised,
    and summed: the triangle count) workloads at R-MAT scale 20 with their own roofline, CPU baseline and parity, plus SpMV and the
    TTGT contraction - each a short run of its own workload function."""
    import copy
    import gc
    res = bench_spmm(rt, orc, gen, args)
    also = {}
    for name, fn, steps, warmup in (("spgemm_rmat20", bench_spgemm, 2, 0), ("spgemm_masked_rmat20", bench_spgemm, 2, 0),
                                    ("tricount_rmat20", bench_tricount, 5, 1),
                                    ("spmv_poisson_1m", bench_spmv, 20, 3), ("ttgt_64x4", bench_ttgt, 5, 1)):
        gc.collect()
        sub_args = copy.copy(args)
        sub_args.steps, sub_args.warmup, sub_args.n = steps, warmup, 0
        sub_args.masked = name == "spgemm_masked_rmat20"
        if sub_args.masked:
            sub_args.cpu_products = args.cpu_products // 3      # a third of the CPU sample: the default run stays short
        log(f"also: {name}")
        try:
            sub = fn(rt, orc, gen, sub_args)
            sub["steps"], sub["warmup"] = steps, warmup
            sub.pop("kernels", None)
            also[name] = sub
        except Exception as exc:          # a failing side workload is reported, the headline line still prints
            also[name] = {"error": f"{type(exc).__name__}: {exc}"}
    res["also"] = also
    return res


WORKLOADS = {"headline": bench_headline, "gather": bench_gather, "copy": bench_copy, "spmm": bench_spmm, "spmv": bench_spmv, "sddmm": bench_sddmm, "ttgt": bench_ttgt, "tricount": bench_tricount,
             "spgemm": bench_spgemm, "coo2csr": bench_coo2csr}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=3)
    ap.add_argument("--workload", choices=sorted(WORKLOADS), default="headline",
                    help="headline (default): SpMM as the value, SpGEMM / triangle count / SpMV / TTGT under \"also\"")
    ap.add_argument("--n", type=int, default=0, help="override the problem size (rows, or extent for ttgt)")
    ap.add_argument("--scale", type=int, default=0, help="R-MAT scale for tricount / spgemm (default 20)")
    ap.add_argument("--candidate", type=int, default=-1, help="force a TTGT candidate (default: cost rule)")
    ap.add_argument("--budget-gb", type=float, default=48.0, help="spgemm: output bytes per numeric row block")
    ap.add_argument("--cpu-products", type=int, default=1_500_000_000, help="spgemm: products in the CPU sample")
    ap.add_argument("--masked", action="store_true", help="spgemm: the masked product C<A> = A*A, materialised")
    ap.add_argument("--semiring", default="", help="spgemm: reduce,mult of another semiring, e.g. min,plus")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--no-peak", action="store_true", help="ttgt: skip the MFMA peak yardstick kernel")
    ap.add_argument("--plan-at-once", action="store_true",
                    help="spmm, spmv: build the matrix's plan at its first product instead of its second, so that every "
                         "launch of a profiled run is a steady-state one")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py: this build runs on exactly one GPU (every kernel is single-device and no figure at "
                 "several GPUs is produced); rerun with --gpus 1")
    if args.plan_at_once:
        os.environ["COMET_HIP_PLAN_AT_ONCE"] = "1"        # read by the library at every product
    from comet_amd import gen, runtime as rt
    from oracle import oracle as orc
    rt.init(0)
    res = WORKLOADS[args.workload](rt, orc, gen, args)
    line = {"metric": res.pop("metric"), "value": res.pop("value"), "unit": res.pop("unit"), "n_gpus": 1,
            "steps": args.steps, "warmup": args.warmup, "ms_per_step": res.pop("ms_per_step"),
            "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": res.pop("dtype"),
            "data": "synthetic (seeded numpy PCG64, generated on the host, resident in HBM before timing)",
            "config": res.pop("config"), "roofline": res.pop("roofline"), "cpu_baseline": res.pop("cpu_baseline"),
            "device": rt.device_name()}
    line.update(res)
    print(json.dumps(line))


if __name__ == "__main__":
    main()
