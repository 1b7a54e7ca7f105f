#!/usr/bin/env python3
"""Benchmark of the CSR SpMV / SpMM hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload NAME] [--only]

A step is one SpMV (or SpMM) call through the C-ABI on a synthetic workload that is already
resident in HBM; analysis (split points) is done once, outside the timed region, and reported
separately.  Prints ONE JSON line.  `value` is effective GB/s = algorithmic bytes / time, with
    SpMV bytes = nnz*(sv+4) + (m+1)*4 + n*sv   + m*sv  *(beta != 0 ? 2 : 1)
    SpMM bytes = nnz*(sv+4) + (m+1)*4 + k*N*sv + m*N*sv*(beta != 0 ? 2 : 1)
All five benchmark configurations are measured (unless --only); the one named by --workload
supplies the headline fields, the others are listed under "workloads".
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0  # MI355X published HBM3E peak
ORDER = ["banded_f64", "uniform16_f32", "powerlaw_f64", "stencil5_f64", "spmm_zipf_f32"]
EXTRA = ["spmm_banded_f32"]  # not a BASELINE configuration: dense-block matrix for the MFMA SpMM variant
KERNEL_NAMES = {3: "k_spmv_stream", 6: "k_spmv_vector", 9: "k_spmv_merge", 15: "k_spmv_flat", 100: "k_spmv_panel", 5: "k_spmm_row", 7: "k_spmm_merge",
                10: "k_spmm_blocked"}

# HBM traffic per call measured with rocprofv3 --pmc (FETCH_SIZE, WRITE_SIZE; see profiles/),
# scaled by the same counters' reading for a plain copy of known size.  None = not measured.
MEASURED_TRAFFIC_BYTES = {
    "powerlaw_f64": (305282.3 * 2 + 111347.2) * 1024,     # profiles/spmv_panel_powerlaw_f64.md
    "stencil5_f64": (679827.7 * 2 + 138992.2) * 1024,    # profiles/spmv_flat_stencil5_f64.md
    "uniform16_f32": (215067.3 * 2 + 4699.0) * 1024,     # profiles/spmv_flat_uniform16_f32.md
    "spmm_banded_f32": (741844.7 * 2 + 340585.3) * 1024,  # profiles/spmm_blocked_spmm_banded_f32.md
    "spmm_zipf_f32": (2284685.2 * 2 + 278616.5) * 1024,  # profiles/spmm_merge_spmm_zipf_f32.md
}


def parse():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=100)
    ap.add_argument("--warmup", type=int, default=10)
    ap.add_argument("--workload", default="powerlaw_f64", choices=ORDER + EXTRA)
    ap.add_argument("--only", action="store_true", help="measure only --workload")
    ap.add_argument("--alg", type=int, default=0, help="kernel id (0 = pick from the histogram)")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--cpu-seconds", type=float, default=12.0, help="budget of the CPU baseline leg")
    ap.add_argument("--probe", action="store_true",
                    help="only run the stream / stream+gather probes on --workload (what the chip sustains "
                         "for this matrix without reduction and write)")
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
    d_y = dev(w.y.copy())
    spmm = w.kind == "spmm"
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
    # (a) K steps back to back, bracketed by synchronisation: the whole-job figure
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(steps):
        step()
    torch.cuda.synchronize()
    wall_ms = (time.perf_counter() - t0) * 1e3 / steps
    # (b) one HIP event pair per call on the launch stream: per-call device time
    starts = [torch.cuda.Event(enable_timing=True) for _ in range(steps)]
    ends = [torch.cuda.Event(enable_timing=True) for _ in range(steps)]
    for i in range(steps):
        starts[i].record()
        step()
        ends[i].record()
    torch.cuda.synchronize()
    per_call = np.array([s.elapsed_time(e) for s, e in zip(starts, ends)])
    # (c) the same call without kept analysis (split points recomputed inside every call, as the
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
        "noplan_ms": float(noplan_ms),
    }
    res["gbs"] = nbytes / (wall_ms * 1e-3) / 1e9
    res["gflops"] = w.flops / (wall_ms * 1e-3) / 1e9
    res["gbs_event"] = nbytes / (res["event_ms_mean"] * 1e-3) / 1e9
    res["frac_hbm_peak"] = res["gbs_event"] / HBM_PEAK_GBS
    plan.destroy()
    del d_rp, d_col, d_val, d_x, d_y, ws, ws2
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


def probe(w, steps):
    """Stream-only and stream+gather rates for workload w (no reduction, no output)."""
    import torch
    from library_amd import capi
    dev = lambda a: torch.from_numpy(a).cuda()
    d_col, d_val, d_x = dev(w.col), dev(w.val), dev(w.x)
    sink = torch.zeros(16, dtype=d_val.dtype, device="cuda")
    vt = capi.value_type(w.val.dtype)
    stream = torch.cuda.current_stream().cuda_stream
    out = {"workload": w.name, "nnz": w.nnz, "stream_bytes": w.nnz * (w.dtype.itemsize + 4)}
    for mode, key in ((0, "stream"), (1, "stream_gather"), (10, "gather_slice_per_xcd"), (11, "gather_16_slices_2_phases"),
                      (12, "gather_slices_mixed_over_xcds")):
        if mode < 10:
            call = lambda: capi.lib().asx_probe_stream_gather(vt, mode, w.nnz, d_col.data_ptr(), d_val.data_ptr(),
                                                              d_x.data_ptr(), sink.data_ptr(), stream)
        else:
            call = lambda: capi.lib().asx_probe_sliced_gather(vt, mode - 10, w.nnz, w.n, d_col.data_ptr(),
                                                              d_val.data_ptr(), d_x.data_ptr(), sink.data_ptr(), stream)
        for _ in range(3):
            call()
        torch.cuda.synchronize()
        s, e = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        s.record()
        for _ in range(steps):
            call()
        e.record()
        torch.cuda.synchronize()
        ms = s.elapsed_time(e) / steps
        out[key + "_us"] = ms * 1e3
        out[key + "_gbs_of_col_val"] = out["stream_bytes"] / (ms * 1e-3) / 1e9
        out[key + "_gnnz_per_s"] = w.nnz / (ms * 1e-3) / 1e9
    return out


def cpu_baseline(w, budget_s):
    """The reference's own CPU path (oracle/_ref, kind "reference") or, where that is not
    built, the C restatement (kind "port"), timed on this host for the same workload."""
    import numpy as np
    from oracle.bindings import Oracle, Ref

    threads = min(os.cpu_count() or 1, int(os.environ.get("OMP_NUM_THREADS", "16") or 16), 16)
    nbytes = w.bytes_algorithmic()
    times = []
    if Ref.available():
        kind = "reference"
        ref = Ref()
        h = ref.create(w.row_ptr, w.col, w.val, w.n)
        y = w.y.copy()

        def call():
            if w.kind == "spmm":
                ref.mm(h, w.x, w.ncols, w.alpha, w.beta, y, threads)
            else:
                ref.mv(h, w.x, w.alpha, w.beta, y, threads)
    else:
        kind = "port"
        orc = Oracle()

        def call():
            if w.kind == "spmm":
                orc.spmm(w.row_ptr, w.col, w.val, w.x, w.ncols, w.alpha, w.beta, w.y, threads)
            else:
                orc.spmv(w.row_ptr, w.col, w.val, w.x, w.alpha, w.beta, w.y, threads)
    t_start = time.perf_counter()
    call()  # warm-up (first touch, thread pool)
    warm = time.perf_counter() - t_start
    reps = 0
    while reps < 1000 and (time.perf_counter() - t_start) < budget_s and (reps < 3 or warm * (reps + 2) < budget_s):
        t0 = time.perf_counter()
        call()
        times.append(time.perf_counter() - t0)
        reps += 1
    if not times:
        times = [warm]
    t = float(np.median(times))
    if kind == "reference":
        ref.destroy(h)
    return {"value": nbytes / t / 1e9, "unit": "GB/s", "cores": threads, "kind": kind,
            "sample": f"{w.name} at full size, median of {len(times)} calls after 1 warm-up, {threads} OpenMP threads",
            "ms_per_call": t * 1e3, "gflops": w.flops / t / 1e9}


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

    if a.calibrate_copy:
        print(json.dumps(copy_calibration(a.steps)))
        return
    if a.probe:
        print(json.dumps(probe(W.CONFIGS[a.workload](), a.steps)))
        return
    names = [a.workload] if (a.only or a.workload in EXTRA) else ORDER
    results = {}
    head_w = None
    for name in names:
        w = W.CONFIGS[name]()
        results[name] = measure(w, a.steps, a.warmup, a.alg if name == a.workload else 0)
        if name == a.workload:
            head_w = w
        else:
            del w
    head = results[a.workload]
    cpu = None
    if not a.no_cpu:
        try:
            cpu = cpu_baseline(head_w, a.cpu_seconds)
        except Exception as e:  # the baseline is a reported extra; never lose the GPU line to it
            cpu = {"value": None, "unit": "GB/s", "cores": 0, "kind": "unavailable", "sample": repr(e)}
    traffic = MEASURED_TRAFFIC_BYTES.get(a.workload)
    line = {
        "metric": "effective HBM GB/s, CSR " + ("SpMM N=64 fp32" if head["kind"] == "spmm" else f"SpMV {head['dtype']}")
                  + " (algorithmic bytes / time)",
        "value": head["gbs"], "unit": "GB/s", "n_gpus": 1, "steps": a.steps, "warmup": a.warmup,
        "ms_per_step": head["ms_per_step"], "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": head["dtype"], "data": "synthetic",
        "config": {"workload": a.workload, "m": head["m"], "n": head["n"], "nnz": head["nnz"], "ncols": head["ncols"],
                   "alpha": head["alpha"], "beta": head["beta"], "max_row": head["max_row"], "kernel": head["kernel"],
                   "analysis_ms": head["analysis_ms"]},
        "gflops": head["gflops"], "pct_hbm_peak": 100.0 * head["gbs"] / HBM_PEAK_GBS,
        "roofline": {"bound": "hbm", "achieved": head["gbs_event"], "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": head["frac_hbm_peak"], "traffic": traffic, "kernel": head["kernel"],
                     "bytes_per_launch": head["bytes"], "launch_ms": head["event_ms_mean"]},
        "cpu_baseline": cpu,
        "roofline_by_workload": {n: {"kernel": results[n]["kernel"], "achieved": round(results[n]["gbs_event"], 1),
                                     "frac": round(results[n]["frac_hbm_peak"], 4),
                                     "traffic": MEASURED_TRAFFIC_BYTES.get(n)} for n in names},
        "workloads": [{k: (round(v, 4) if isinstance(v, float) else v) for k, v in results[n].items()} for n in names],
    }
    print(json.dumps(line))


if __name__ == "__main__":
    main()
