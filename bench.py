#!/usr/bin/env python3
"""Benchmark of the CSR SpMV / SpMM hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload NAME] [--only]

A step is one SpMV (or SpMM) call through the C-ABI on a synthetic workload that is already
resident in HBM; analysis (split points, column slices) is done once, outside the timed region,
and reported separately.  Prints ONE JSON line.  `value` is effective GB/s = algorithmic bytes /
time, with
    SpMV bytes = nnz*(sv+4) + (m+1)*4 + n*sv   + m*sv  *(beta != 0 ? 2 : 1)
    SpMM bytes = nnz*(sv+4) + (m+1)*4 + k*N*sv + m*N*sv*(beta != 0 ? 2 : 1)
All five benchmark configurations are measured (unless --only); the one named by --workload
supplies the headline fields, the others are listed under "workloads".

Per workload, on the GPU:
  ms_per_step     K calls back to back between two synchronisations (the whole-job figure)
  event_ms_*      one HIP event pair per call on the launch stream; when beta != 0 the output is
                  restored from a pristine copy before every call, outside the event pair (the
                  reference's test loop does the same, hip/test/level2/spmv_csr_r_f64_test.hip:183-198)
  cold_ms         as event_ms, after a 1 GiB sweep that evicts the caches before every call
  noplan_ms       the call without kept analysis (split points recomputed inside every call, as
                  the reference does)
  unchanged_caller_ms   SpMV: what a caller that never calls the analysis gets by default through the
                  generic API: a plan made on first use that may hold a copy of the values, checked
                  against the caller's values by checksum in every call (unchanged_caller_kernel)
  changing_caller_ms    the same caller when the values do change in place before every call (the copy,
                  where the plan holds one, is brought up to date inside the call)
  update_values_ms      asx_plan_update_values on the plan of ms_per_step (0 where it holds no values)
and on the host (unless --no-cpu), the reference's own CPU kernels (oracle/_ref, kind
"reference") or their C restatement (kind "port") on the same inputs: all physical cores of the
box's share, and one thread.
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0  # MI355X published HBM3E peak
# the five BASELINE configurations, and config 2's matrix in fp64 (the "uniform fp64" case the target names)
ORDER = ["banded_f64", "uniform16_f32", "uniform16_f64", "powerlaw_f64", "stencil5_f64", "spmm_zipf_f32"]
# not BASELINE configurations: a dense-block matrix for the MFMA SpMM variant, a 7-point stencil on 256^3
EXTRA = ["spmm_banded_f32", "stencil7_f64"]
KERNEL_NAMES = {3: "k_spmv_stream", 6: "k_spmv_vector", 9: "k_spmv_merge", 15: "k_spmv_flat",
                101: "k_sliced_products+k_sliced_reduce", 102: "k_spmv_window", 5: "k_spmm_row", 7: "k_spmm_merge", 10: "k_spmm_blocked"}

# Traffic beyond the L2s per call measured with rocprofv3 --pmc (FETCH_SIZE, WRITE_SIZE in KiB per
# dispatch, summed over the kernels of one call with kept analysis; see profiles/), scaled by the
# same counters' reading for a plain copy of known size (FETCH_SIZE reads half the bytes,
# WRITE_SIZE all of them).  The Infinity Cache serves part of it: the counters read the same with
# warm and with cold caches.
MEASURED_TRAFFIC_BYTES = {
    "banded_f64": 458_624,  # profiles/spmv_vector_banded_f64.md
    "uniform16_f32": 256_483_686,  # profiles/spmv_sliced_uniform16_f32.md
    "uniform16_f64": 478_017_157,  # profiles/spmv_sliced_uniform16_f64.md
    "powerlaw_f64": 730_483_835,  # profiles/spmv_sliced_powerlaw_f64.md
    "stencil5_f64": 1_142_530_786,  # profiles/spmv_window_stencil5_f64.md
    "spmm_zipf_f32": 4_965_331_333,  # profiles/spmm_merge_spmm_zipf_f32.md
    "spmm_banded_f32": 1_870_263_890,  # profiles/spmm_blocked_spmm_banded_f32.md
    "stencil7_f64": 1_630_404_585,  # profiles/spmv_window_stencil7_256_f64.md
}


def parse():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=100)
    ap.add_argument("--warmup", type=int, default=10)
    ap.add_argument("--workload", default="powerlaw_f64", choices=ORDER + EXTRA)
    ap.add_argument("--only", action="store_true", help="measure only --workload")
    ap.add_argument("--alg", type=int, default=0, help="kernel id (0 = what the analysis picks)")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--cpu-seconds", type=float, default=60.0,
                    help="budget of the whole CPU baseline leg (split evenly over workloads and thread counts)")
    ap.add_argument("--calibrate-gather", action="store_true",
                    help="only run the random-line gather kernel (lines per second the memory system delivers "
                         "past the L2s: the bound of a gather without reuse)")
    ap.add_argument("--selection-audit", action="store_true",
                    help="only time, over families of matrices, the plan DEFAULT picks against every kernel that "
                         "accepts the matrix; prints a markdown table and one JSON line")
    ap.add_argument("--calibrate-copy", action="store_true",
                    help="only run the plain copy kernel on 1 GiB (known traffic, for scaling profiler counters)")
    return ap.parse_args()


def measure(w, steps, warmup, alg):
    """Returns a dict of measurements for workload w (arrays on host)."""
    import numpy as np
    import torch
    from library_amd import capi

    dev = lambda a: torch.from_numpy(a).cuda()
    d_rp, d_col, d_val, d_x = dev(w.row_ptr), dev(w.col), dev(w.val), dev(w.x)
    d_y0 = dev(w.y.copy())
    d_y = d_y0.clone()
    spmm = w.kind == "spmm"
    restore = w.beta != 0
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    plan = capi.Plan(spmm, alg, w.val.dtype, w.m, w.n, w.nnz, d_rp, ncols=w.ncols, col=d_col, val=d_val)
    torch.cuda.synchronize()
    analysis_ms = (time.perf_counter() - t0) * 1e3
    ws = torch.empty(max(plan.workspace_bytes, 256), dtype=torch.uint8, device="cuda")

    def step():
        if spmm:
            capi.spmm(d_rp, d_col, d_val, d_x, d_y, w.ncols, w.alpha, w.beta, plan=plan, workspace=ws, k=w.n)
        else:
            capi.spmv(d_rp, d_col, d_val, d_x, d_y, w.alpha, w.beta, plan=plan, workspace=ws)

    for _ in range(warmup):
        step()
    # (a) K steps back to back, bracketed by synchronisation: the whole-job figure.  (With
    #     beta != 0 the output feeds the next call; the values stay finite and the time per call
    #     does not depend on them.)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(steps):
        step()
    torch.cuda.synchronize()
    wall_ms = (time.perf_counter() - t0) * 1e3 / steps

    # (b) one HIP event pair per call on the launch stream, fresh output before every call
    def timed_calls(count, before=None):
        starts = [torch.cuda.Event(enable_timing=True) for _ in range(count)]
        ends = [torch.cuda.Event(enable_timing=True) for _ in range(count)]
        for i in range(count):
            if restore:
                d_y.copy_(d_y0)
            if before is not None:
                before()
            starts[i].record()
            step()
            ends[i].record()
        torch.cuda.synchronize()
        return np.array([s.elapsed_time(e) for s, e in zip(starts, ends)])

    per_call = timed_calls(steps)
    # (c) cold caches: a 1 GiB sweep between calls evicts the L2s and the Infinity Cache
    sweep = torch.empty(1 << 30, dtype=torch.uint8, device="cuda")
    cold = timed_calls(max(5, min(20, steps // 5)), before=lambda: sweep.fill_(1))
    del sweep
    # (d) the same call without kept analysis (split points recomputed inside every call, as the
    #     reference does): what a caller that never calls *_analysis / *_preprocess sees
    vt = capi.value_type(w.val.dtype)
    if spmm:
        need = capi.lib().asx_spmm_workspace_bytes(0, vt, w.m, w.nnz, w.ncols)
    else:
        need = capi.lib().asx_spmv_workspace_bytes(0, vt, w.m, w.nnz)
    ws2 = torch.empty(max(need, 256), dtype=torch.uint8, device="cuda")

    def step_noplan():
        if spmm:
            capi.spmm(d_rp, d_col, d_val, d_x, d_y, w.ncols, w.alpha, w.beta, alg=0, workspace=ws2, k=w.n)
        else:
            capi.spmv(d_rp, d_col, d_val, d_x, d_y, w.alpha, w.beta, alg=0, workspace=ws2)

    for _ in range(3):
        step_noplan()
    torch.cuda.synchronize()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    nrep = max(5, steps // 5)
    e0.record()
    for _ in range(nrep):
        step_noplan()
    e1.record()
    torch.cuda.synchronize()
    noplan_ms = e0.elapsed_time(e1) / nrep
    # (e) SpMV, what a caller written for the reference gets by default (no analysis call, values may
    #     change in place): analysis on first use that may keep a copy of the values, and in every
    #     call two checksums of the caller's values on the device with a refresh of the copy where
    #     they differ.  DEFAULT's choice counts that read, so the kernel may be another one.
    checked_ms, checked_kernel, changing_ms, update_ms = None, None, None, None
    if not spmm:
        cplan = capi.Plan(False, alg, w.val.dtype, w.m, w.n, w.nnz, d_rp, col=d_col, val=d_val, checked=True)
        checked_kernel = KERNEL_NAMES.get(cplan.alg, str(cplan.alg)) + (" + checksum" if cplan.checked else "")
        ws3 = torch.empty(max(cplan.workspace_bytes, 256), dtype=torch.uint8, device="cuda")

        def step_checked():
            cplan.refresh_if_changed(d_val)
            capi.spmv(d_rp, d_col, d_val, d_x, d_y, w.alpha, w.beta, plan=cplan, workspace=ws3)

        for _ in range(3):
            step_checked()
        torch.cuda.synchronize()
        e0.record()
        for _ in range(nrep):
            step_checked()
        e1.record()
        torch.cuda.synchronize()
        checked_ms = e0.elapsed_time(e1) / nrep
        # the same with values that differ from one call to the next (two arrays that differ in one
        # element, passed in turn: what the plan sees is its values changed in place)
        d_val2 = d_val.clone()
        d_val2[w.nnz // 2] += 1.0
        vals = (d_val2, d_val)

        def step_changing(i):
            cplan.refresh_if_changed(vals[i & 1])
            capi.spmv(d_rp, d_col, vals[i & 1], d_x, d_y, w.alpha, w.beta, plan=cplan, workspace=ws3)

        for i in range(4):
            step_changing(i)
        torch.cuda.synchronize()
        e0.record()
        for i in range(nrep):
            step_changing(i)
        e1.record()
        torch.cuda.synchronize()
        changing_ms = e0.elapsed_time(e1) / nrep
        cplan.refresh_if_changed(d_val)
        cplan.destroy()
        del d_val2
        # and what the caller of an explicit analysis pays to say that the values changed
        for _ in range(3):
            plan.update_values(d_val)
        torch.cuda.synchronize()
        e0.record()
        for _ in range(nrep):
            plan.update_values(d_val)
        e1.record()
        torch.cuda.synchronize()
        update_ms = e0.elapsed_time(e1) / nrep if plan.holds_values else 0.0
    nbytes = w.bytes_algorithmic()
    res = {
        "workload": w.name, "kind": w.kind, "dtype": "f64" if w.dtype.itemsize == 8 else "f32",
        "m": w.m, "n": w.n, "nnz": w.nnz, "ncols": w.ncols, "alpha": w.alpha, "beta": w.beta,
        "max_row": int(np.diff(w.row_ptr).max()) if w.m else 0,
        "kernel": KERNEL_NAMES.get(plan.alg, str(plan.alg)),
        "bytes": nbytes, "bytes_y_twice": w.bytes_algorithmic(y_twice=True), "flops": w.flops,
        "analysis_ms": round(analysis_ms, 3),
        "ms_per_step": wall_ms,
        "event_ms_mean": float(per_call.mean()), "event_ms_median": float(np.median(per_call)),
        "event_ms_min": float(per_call.min()),
        "cold_ms_median": float(np.median(cold)),
        "noplan_ms": float(noplan_ms),
        "unchanged_caller_ms": None if checked_ms is None else float(checked_ms), "unchanged_caller_kernel": checked_kernel,
        "changing_caller_ms": None if changing_ms is None else float(changing_ms),
        "update_values_ms": None if update_ms is None else float(update_ms),
    }
    res["gbs"] = nbytes / (wall_ms * 1e-3) / 1e9
    res["gflops"] = w.flops / (wall_ms * 1e-3) / 1e9
    res["gbs_event"] = nbytes / (res["event_ms_mean"] * 1e-3) / 1e9
    res["frac_hbm_peak"] = res["gbs_event"] / HBM_PEAK_GBS
    plan.destroy()
    del d_rp, d_col, d_val, d_x, d_y, d_y0, ws, ws2
    torch.cuda.empty_cache()
    return res


def copy_calibration(steps, nbytes=1 << 30):
    """Plain device copy of nbytes (reads nbytes, writes nbytes): the practical streaming
    ceiling of this chip, and a launch of known traffic for scaling FETCH_SIZE / WRITE_SIZE."""
    import torch
    from library_amd import capi
    src = torch.zeros(nbytes, dtype=torch.uint8, device="cuda")
    dst = torch.empty_like(src)
    stream = torch.cuda.current_stream().cuda_stream
    for _ in range(3):
        capi.lib().asx_copy_bytes(src.data_ptr(), dst.data_ptr(), nbytes, stream)
    torch.cuda.synchronize()
    s, e = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    s.record()
    for _ in range(steps):
        capi.lib().asx_copy_bytes(src.data_ptr(), dst.data_ptr(), nbytes, stream)
    e.record()
    torch.cuda.synchronize()
    ms = s.elapsed_time(e) / steps
    return {"copy_bytes_read": nbytes, "copy_bytes_written": nbytes, "ms": ms,
            "read_plus_write_gbs": 2 * nbytes / (ms * 1e-3) / 1e9}


def load_plan_kernels():
    """The first launch of a kernel in a process loads its code; for the kernels that build the
    sliced and window plans (sorts, scans, placement) that is about 20 ms, paid once per process.
    One small matrix through each builder, so that analysis_ms below is what every later matrix
    sees.  Returns the time these first builds took (ms)."""
    import numpy as np
    import torch
    from library_amd import capi
    rng = np.random.default_rng(0)
    m = n = 1 << 15
    lens = np.full(m, 8, dtype=np.int64)
    rp = np.zeros(m + 1, dtype=np.int32)
    rp[1:] = np.cumsum(lens)
    took = {}
    for name, alg, col in (("sliced", capi.SPMV_SLICED, np.sort(rng.integers(0, n, (m, 8)), axis=1)),
                           ("window", capi.SPMV_WINDOW, np.clip(np.arange(m)[:, None] + np.arange(-4, 4)[None, :], 0, n - 1))):
        col = np.ascontiguousarray(col.reshape(-1).astype(np.int32))
        val = rng.uniform(-1, 1, col.size)
        d = [torch.from_numpy(x).cuda() for x in (rp, col, val)]
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        plan = capi.Plan(False, alg, val.dtype, m, n, col.size, d[0], col=d[1], val=d[2])
        torch.cuda.synchronize()
        took[name] = round((time.perf_counter() - t0) * 1e3, 3)
        plan.destroy()
    return took


def gather_calibration(loads_per_lane=128):
    """Independent random reads that miss the L2s: one 128-byte line per lane, or one 256-byte row
    (two lines) per wave, from buffers that fit the 256 MB Infinity Cache (64 MiB), are as large as
    config 5's B (256 MiB) or exceed every cache (2 GiB).  Lines per second = the ceiling for a
    gather without reuse, whatever the kernel around it."""
    import torch
    from library_amd import capi
    import ctypes as C
    L = capi.lib()
    nthreads = C.c_int(0)
    L.asx_gather_lines(None, 0, 1, 8, None, C.byref(nthreads), None)
    out = torch.empty(nthreads.value, dtype=torch.int32, device="cuda")
    stream = torch.cuda.current_stream().cuda_stream
    rows = []
    for mib in (64, 256, 2048):
        buf = torch.zeros(mib << 20, dtype=torch.uint8, device="cuda")
        for group in (1, 64):
            per_lane = loads_per_lane * (16 if group == 64 else 1)  # a wave's load is 2 lines, not 64
            for _ in range(2):
                rc = L.asx_gather_lines(buf.data_ptr(), buf.numel(), group, per_lane, out.data_ptr(), None, stream)
                assert rc == 0, rc
            torch.cuda.synchronize()
            s, e = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            reps = 5
            s.record()
            for _ in range(reps):
                L.asx_gather_lines(buf.data_ptr(), buf.numel(), group, per_lane, out.data_ptr(), None, stream)
            e.record()
            torch.cuda.synchronize()
            ms = s.elapsed_time(e) / reps
            loads = nthreads.value * per_lane                  # lane loads
            lines = loads if group == 1 else loads // 64 * 2    # 128-byte lines fetched
            rows.append({"buffer_mib": mib, "group_lanes": group, "ms": ms, "lines": lines,
                         "g_lines_per_s": lines / (ms * 1e-3) / 1e9, "tb_per_s_of_lines": lines * 128 / (ms * 1e-3) / 1e12})
        del buf
    return {"gather": rows}


def host_cpus():
    """nproc, sockets and physical cores of this host, and the thread count the baseline uses:
    the physical cores, capped by the box's CPU share (OMP_NUM_THREADS, 16 on a one-GPU box)."""
    nproc = os.cpu_count() or 1
    sockets, cores = set(), set()
    try:
        phys = core = None
        for line in open("/proc/cpuinfo"):
            if line.startswith("physical id"):
                phys = line.split(":")[1].strip()
            elif line.startswith("core id"):
                core = line.split(":")[1].strip()
            elif not line.strip():
                if phys is not None and core is not None:
                    sockets.add(phys)
                    cores.add((phys, core))
                phys = core = None
    except OSError:
        pass
    physical = len(cores) or nproc
    share = int(os.environ.get("OMP_NUM_THREADS", "0") or 0) or nproc
    return {"nproc": nproc, "sockets": len(sockets) or 1, "physical_cores": physical, "cpu_share": share,
            "threads_used": max(1, min(physical, share, nproc))}


def _time_calls(call, budget_s, max_calls):
    """Warm-up call (first touch, thread pool), then as many timed calls as fit the budget."""
    import numpy as np
    t_start = time.perf_counter()
    call()
    warm = time.perf_counter() - t_start
    times = []
    while len(times) < max_calls and (time.perf_counter() - t_start) + warm < budget_s:
        t0 = time.perf_counter()
        call()
        times.append(time.perf_counter() - t0)
    warmed = bool(times)
    if not times:
        times = [warm]  # one call was all the budget allowed: it is the (cold) sample
    return float(np.median(times)), len(times), warmed


def cpu_baseline(w, threads, budget_s):
    """The reference's own CPU path (oracle/_ref, kind "reference") or, where that is not built,
    the C restatement (kind "port"), timed on this host for workload w with `threads` OpenMP
    threads.  SpMV runs at full size.  The reference's SpMM builds a rows x (k/256 + 1) table of
    ints in every call (hygon/util/partition.cpp:178-201; 17 GB and tens of seconds at this
    shape), so it is timed on the first 1/16 of the rows of A (B and C at full width), and the
    restatement (one K block, no table) at full size beside it."""
    import numpy as np
    from oracle.bindings import Oracle, Ref

    def rates(nbytes, flops, t):
        return {"gbs": nbytes / t / 1e9, "gflops": flops / t / 1e9, "ms_per_call": t * 1e3}

    out = {"threads": threads}
    have_ref = Ref.available()
    sv = w.dtype.itemsize
    if w.kind == "spmv":
        y = w.y.copy()
        if have_ref:
            ref = Ref()
            h = ref.create(w.row_ptr, w.col, w.val, w.n)
            call = lambda: ref.mv(h, w.x, w.alpha, w.beta, y, threads)
        else:
            orc = Oracle()
            call = lambda: orc.spmv(w.row_ptr, w.col, w.val, w.x, w.alpha, w.beta, w.y, threads)
        t, n, warmed = _time_calls(call, budget_s, 1000)
        if have_ref:
            ref.destroy(h)
        out.update(rates(w.bytes_algorithmic(), w.flops, t))
        out.update({"kind": "reference" if have_ref else "port", "calls_timed": n, "warmed_up": warmed,
                    "sample": f"{w.name} at full size"})
        return out
    # SpMM
    orc = Oracle()
    if have_ref:
        rows = max(1, w.m // 16)
        nz = int(w.row_ptr[rows])
        rp = np.ascontiguousarray(w.row_ptr[:rows + 1])
        ref = Ref()
        h = ref.create(rp, w.col[:nz], w.val[:nz], w.n)
        Cs = w.y[:rows * w.ncols].copy()
        call = lambda: ref.mm(h, w.x, w.ncols, w.alpha, w.beta, Cs, threads)
        t, n, warmed = _time_calls(call, budget_s * 0.6, 20)
        ref.destroy(h)
        ymul = 2 if w.beta != 0 else 1
        sbytes = nz * (sv + 4) + (rows + 1) * 4 + w.n * w.ncols * sv + rows * w.ncols * sv * ymul
        out.update(rates(sbytes, 2 * nz * w.ncols, t))
        out.update({"kind": "reference", "calls_timed": n, "warmed_up": warmed,
                    "sample": f"{w.name}: the first {rows} of {w.m} rows of A ({nz} stored elements), B and C {w.ncols} wide; "
                              f"the reference's per-call table of rows x (k/256 + 1) ints is {rows * (w.n // 256 + 1) * 4 / 1e9:.1f} GB "
                              f"for the sample, {w.m * (w.n // 256 + 1) * 4 / 1e9:.1f} GB at full size"})
        budget_s *= 0.4
    Cf = w.y.copy()
    call = lambda: orc.spmm(w.row_ptr, w.col, w.val, w.x, w.ncols, w.alpha, w.beta, Cf, threads)
    t, n, warmed = _time_calls(call, budget_s, 20)
    port = rates(w.bytes_algorithmic(), w.flops, t)
    port.update({"kind": "port", "calls_timed": n, "warmed_up": warmed,
                 "sample": f"{w.name} at full size, C restatement of the reference's row kernel with one K block (no table)"})
    if have_ref:
        out["restatement_full_size"] = port
    else:
        out.update(port)
    return out


def main():
    a = parse()
    if a.gpus != 1:
        print(f"bench.py measures one GPU; --gpus {a.gpus} is not supported "
              "(the path has no multi-GPU part: rows shard by nnz with an all-gather of x)",
              file=sys.stderr)
        sys.exit(2)
    import torch
    from library_amd import capi, workloads as W
    assert torch.cuda.is_available(), "bench.py needs the GPU"
    capi.lib()

    if a.calibrate_gather:
        print(json.dumps(gather_calibration()))
        return
    if a.calibrate_copy:
        print(json.dumps(copy_calibration(a.steps)))
        return
    if a.selection_audit:
        from library_amd import selection_audit
        load_plan_kernels()
        rows = selection_audit.run()
        print(selection_audit.markdown(rows))
        print(json.dumps({"selection_audit": rows, "worst_ratio": max(r["ratio"] for r in rows)}))
        return
    names = [a.workload] if (a.only or a.workload in EXTRA) else ORDER
    first_use_ms = load_plan_kernels()
    cpus = host_cpus()
    legs = [cpus["threads_used"]] + ([1] if cpus["threads_used"] > 1 else [])
    leg_budget = a.cpu_seconds / (len(names) * len(legs))
    results, cpu_by_workload = {}, {}
    for name in names:
        w = W.CONFIGS[name]()
        results[name] = measure(w, a.steps, a.warmup, a.alg if name == a.workload else 0)
        if not a.no_cpu:
            rows = []
            for threads in legs:
                try:
                    rows.append(cpu_baseline(w, threads, leg_budget))
                except Exception as e:  # the baseline is a reported extra; never lose the GPU line to it
                    rows.append({"threads": threads, "kind": "unavailable", "sample": repr(e)})
            cpu_by_workload[name] = rows
        del w
    head = results[a.workload]
    cpu = None
    if not a.no_cpu:
        c = cpu_by_workload[a.workload][0]
        cpu = {"value": c.get("gbs"), "unit": "GB/s", "cores": c["threads"], "kind": c.get("kind"),
               "sample": f"{c.get('sample')}; median of {c.get('calls_timed')} calls after "
                         f"{'one' if c.get('warmed_up') else 'no'} warm-up call, {c['threads']} OpenMP threads "
                         f"(host: nproc {cpus['nproc']}, {cpus['sockets']} socket(s), {cpus['physical_cores']} physical cores, "
                         f"CPU share {cpus['cpu_share']})",
               "ms_per_call": c.get("ms_per_call"), "gflops": c.get("gflops"),
               "one_thread": next(({"value": r.get("gbs"), "ms_per_call": r.get("ms_per_call"), "calls_timed": r.get("calls_timed")}
                                   for r in cpu_by_workload[a.workload] if r["threads"] == 1), None)}
    traffic = MEASURED_TRAFFIC_BYTES.get(a.workload)
    line = {
        "metric": "effective HBM GB/s, CSR " + ("SpMM N=64 fp32" if head["kind"] == "spmm" else f"SpMV {head['dtype']}")
                  + " (algorithmic bytes / time)",
        "value": head["gbs"], "unit": "GB/s", "n_gpus": 1, "steps": a.steps, "warmup": a.warmup,
        "ms_per_step": head["ms_per_step"], "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": head["dtype"], "data": "synthetic",
        "config": {"workload": a.workload, "m": head["m"], "n": head["n"], "nnz": head["nnz"], "ncols": head["ncols"],
                   "alpha": head["alpha"], "beta": head["beta"], "max_row": head["max_row"], "kernel": head["kernel"],
                   "analysis_ms": head["analysis_ms"], "first_plan_build_in_process_ms": first_use_ms},
        "gflops": head["gflops"], "pct_hbm_peak": 100.0 * head["gbs"] / HBM_PEAK_GBS,
        "roofline": {"bound": "hbm", "achieved": head["gbs_event"], "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": head["frac_hbm_peak"], "traffic": traffic, "kernel": head["kernel"],
                     "bytes_per_launch": head["bytes"], "launch_ms": head["event_ms_mean"]},
        "cpu_baseline": cpu,
        "host_cpus": cpus,
        "cpu_baseline_by_workload": cpu_by_workload,
        "roofline_by_workload": {n: {"kernel": results[n]["kernel"], "achieved": round(results[n]["gbs_event"], 1),
                                     "frac": round(results[n]["frac_hbm_peak"], 4),
                                     "traffic": MEASURED_TRAFFIC_BYTES.get(n)} for n in names},
        "workloads": [{k: (round(v, 4) if isinstance(v, float) else v) for k, v in results[n].items()} for n in names],
    }
    print(json.dumps(line))


if __name__ == "__main__":
    main()
