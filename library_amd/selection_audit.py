"""What DEFAULT picks against every kernel that accepts the matrix, over families of matrices.

    python bench.py --selection-audit            # prints a markdown table and one JSON line

For every family the analysis is run with ASX_SPMV_DEFAULT and with every explicit kernel id; every
plan is timed (HIP events around back-to-back calls, y = 1.5 A x + 0.5 y; DEFAULT's plan twice, the
lower of the two counts) and the table lists
DEFAULT's time over the best one.  A rule-based choice (row-length histogram, sizes, a column
sample) cannot be the fastest everywhere; the audit shows how far off it gets.
"""
from __future__ import annotations

import numpy as np

from . import capi, workloads as W


def _csr_from_keys(keys, m, n):
    """Sorted unique (row * n + col) keys -> row_ptr, col."""
    keys = np.unique(keys)
    rows = keys // n
    rp = np.zeros(m + 1, np.int64)
    np.cumsum(np.bincount(rows, minlength=m), out=rp[1:])
    return rp.astype(np.int32), (keys % n).astype(np.int32)


def _stencil3d(nx, ny, nz, points):
    idx = np.arange(nx * ny * nz, dtype=np.int64)
    i, j, k = idx % nx, (idx // nx) % ny, idx // (nx * ny)
    keys = []
    for dk in (-1, 0, 1):
        for dj in (-1, 0, 1):
            for di in (-1, 0, 1):
                if points != 27 and abs(di) + abs(dj) + abs(dk) > 1:
                    continue
                ii, jj, kk = i + di, j + dj, k + dk
                ok = (ii >= 0) & (ii < nx) & (jj >= 0) & (jj < ny) & (kk >= 0) & (kk < nz)
                keys.append(idx[ok] * idx.size + (ii + nx * (jj + ny * kk))[ok])
    return _csr_from_keys(np.concatenate(keys), idx.size, idx.size)


def _near_diagonal(m, n, per_row, reach, rng, keep=1.0):
    """per_row columns per row, uniform within +-reach of the (scaled) diagonal; a fraction `keep` of the rows."""
    r = np.arange(m, dtype=np.int64)
    if keep < 1.0:
        r = r[rng.random(m) < keep]
    centre = r * n // m
    c = centre[:, None] + rng.integers(-reach, reach + 1, (r.size, per_row))
    c = np.clip(c, 0, n - 1)
    return _csr_from_keys((r[:, None] * n + c).reshape(-1), m, n)


def _block_clustered(m, n, clusters, width, rng):
    """Rows in groups of 64 share `clusters` runs of `width` consecutive columns at random places."""
    g = m // 64
    starts = rng.integers(0, n - width, (g, clusters))
    cols = (starts[:, :, None] + np.arange(width)[None, None, :]).reshape(g, -1)
    r = np.arange(g * 64, dtype=np.int64)
    return _csr_from_keys((r[:, None] * n + cols[r // 64]).reshape(-1), m, n)


def families():
    """name -> (dtype, row_ptr, col, n); generated lazily, one at a time."""
    rng = np.random.default_rng(2024)

    def fixed(m, n, k, dt):
        rp, col, _ = W.csr_fixed(m, n, k, dt, seed=1)
        return rp, col, n

    def zipf(alpha10, dt=np.float64):
        rp, col, _ = W.csr_zipf(1 << 21, 1 << 21, alpha10, 1.0, 100000, 0.01, dt, seed=2)
        return rp, col, 1 << 21

    def band(half):
        rp, col, _ = W.csr_banded(1 << 21, half, np.float64, seed=3)
        return rp, col, 1 << 21

    fams = []
    for k in (4, 16, 64):
        for dt in (np.float32, np.float64):
            n = (8 << 20) // np.dtype(dt).itemsize
            m = (1 << 24) // k
            fams.append((f"uniform {k}/row, x 8 MB, {np.dtype(dt).name}", dt, lambda m=m, n=n, k=k, dt=dt: fixed(m, n, k, dt)))
    for xmb in (2, 32):
        for dt in (np.float32, np.float64):
            n = (xmb << 20) // np.dtype(dt).itemsize
            fams.append((f"uniform 16/row, x {xmb} MB, {np.dtype(dt).name}", dt, lambda n=n, dt=dt: fixed(1 << 20, n, 16, dt)))
    for a in (16, 20, 24):
        fams.append((f"Zipf {a / 10:.1f} rows, 2M x 2M, float64", np.float64, lambda a=a: zipf(a)))
    for half, name in ((4, 9), (9, 19), (32, 65)):
        fams.append((f"band of {name}, 2M rows, float64", np.float64, lambda half=half: band(half)))
    fams.append(("5-point stencil 2048^2, float64", np.float64, lambda: W.csr_stencil5(2048, 2048)[:2] + (2048 * 2048,)))
    fams.append(("7-point stencil 160^3, float64", np.float64, lambda: _stencil3d(160, 160, 160, 7) + (160 ** 3,)))
    fams.append(("27-point stencil 96^3, float64", np.float64, lambda: _stencil3d(96, 96, 96, 27) + (96 ** 3,)))
    fams.append(("5-point stencil 2048^2, float32", np.float32, lambda: W.csr_stencil5(2048, 2048)[:2] + (2048 * 2048,)))
    fams.append(("7-point stencil 160^3, float32", np.float32, lambda: _stencil3d(160, 160, 160, 7) + (160 ** 3,)))
    fams.append(("64-row groups sharing 8 runs of 16 columns, float64", np.float64,
                 lambda: _block_clustered(1 << 18, 1 << 21, 8, 16, rng) + (1 << 21,)))
    fams.append(("12/row within +-50000 of the diagonal (wider than a window), float64", np.float64,
                 lambda: _near_diagonal(1 << 20, 1 << 20, 12, 50000, rng) + (1 << 20,)))
    fams.append(("12/row within +-4000 of the diagonal, float64", np.float64,
                 lambda: _near_diagonal(1 << 20, 1 << 20, 12, 4000, rng) + (1 << 20,)))
    fams.append(("hypersparse: 1 in 4 of 12M rows holds 1 element near the diagonal, float64", np.float64,
                 lambda: _near_diagonal(12 << 20, 12 << 20, 1, 100, rng, keep=0.25) + (12 << 20,)))
    fams.append(("2 scattered per row, 4M x 4M, float64", np.float64, lambda: fixed(1 << 22, 1 << 22, 2, np.float64)))
    # sizes that are no powers of two: slices that do not divide the workgroups, blocks that do not divide the rows
    fams.append(("uniform 16/row, 1048576 x 1300000 (80 slices), float64", np.float64, lambda: fixed(1 << 20, 1300000, 16, np.float64)))
    fams.append(("uniform 16/row, 1500000 x 700000 (22 slices), float32", np.float32, lambda: fixed(1500000, 700000, 16, np.float32)))
    fams.append(("uniform 16/row, 700001 x 2500000 (153 slices), float64", np.float64, lambda: fixed(700001, 2500000, 16, np.float64)))
    fams.append(("5-point stencil 3000 x 1500, float64", np.float64, lambda: W.csr_stencil5(3000, 1500)[:2] + (3000 * 1500,)))
    fams.append(("7-point stencil 200 x 150 x 100, float64", np.float64, lambda: _stencil3d(200, 150, 100, 7) + (200 * 150 * 100,)))
    fams.append(("band of 9, 3000001 rows, float64", np.float64, lambda: W.csr_banded(3000001, 4, np.float64, seed=3)[:2] + (3000001,)))
    return fams


KERNELS = [("vector", capi.SPMV_VECTOR), ("stream", capi.SPMV_STREAM), ("merge", capi.SPMV_MERGE), ("flat", capi.SPMV_FLAT),
           ("sliced", capi.SPMV_SLICED), ("window", capi.SPMV_WINDOW)]
NAMES = {v: k for k, v in KERNELS}


def _time_plan(torch, d, x, y, plan, alg, calls):
    ws = torch.empty(max(plan.workspace_bytes, 256), dtype=torch.uint8, device="cuda")
    for _ in range(3):
        capi.spmv(d[0], d[1], d[2], x, y, 1.5, 0.5, alg=alg, plan=plan, workspace=ws)
    torch.cuda.synchronize()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record()
    for _ in range(calls):
        capi.spmv(d[0], d[1], d[2], x, y, 1.5, 0.5, alg=alg, plan=plan, workspace=ws)
    e1.record()
    torch.cuda.synchronize()
    return e0.elapsed_time(e1) / calls * 1e3  # us


def run(calls=20, slow_us=20000.0):
    import torch
    rows = []
    for name, dt, make in families():
        rp, col, n = make()
        m, nnz = rp.size - 1, col.size
        rng = np.random.default_rng(7)
        val = rng.uniform(-1, 1, nnz).astype(dt)
        d = [torch.from_numpy(a).cuda() for a in (rp, col, val)]
        x = torch.from_numpy(rng.uniform(-1, 1, n).astype(dt)).cuda()
        y = torch.from_numpy(rng.uniform(-1, 1, m).astype(dt)).cuda()
        times = {}
        plan = capi.Plan(False, capi.SPMV_DEFAULT, np.dtype(dt), m, n, nnz, d[0], col=d[1], val=d[2])
        chosen = NAMES.get(plan.alg, str(plan.alg))
        t_default = _time_plan(torch, d, x, y, plan, capi.SPMV_DEFAULT, calls)
        default_plan = plan
        for kname, alg in KERNELS:
            try:
                plan = capi.Plan(False, alg, np.dtype(dt), m, n, nnz, d[0], col=d[1], val=d[2])
            except capi.AsxError:
                continue  # the kernel does not take this matrix
            # one call first: a kernel that is hopeless here (one lane group per 100000-element row) is
            # not timed twenty times over
            t1 = _time_plan(torch, d, x, y, plan, alg, 1)
            times[kname] = t1 if t1 > slow_us else _time_plan(torch, d, x, y, plan, alg, calls)
            plan.destroy()
        # DEFAULT's plan once more, behind the others: the first timing on fresh allocations has read
        # up to 15 % high for the very kernel that reads the same when forced
        t_default = min(t_default, _time_plan(torch, d, x, y, default_plan, capi.SPMV_DEFAULT, calls))
        default_plan.destroy()
        best = min(times, key=times.get)
        sv = np.dtype(dt).itemsize
        nbytes = nnz * (sv + 4) + (m + 1) * 4 + n * sv + 2 * m * sv
        rows.append({"family": name, "m": m, "n": n, "nnz": nnz, "default": chosen, "default_us": round(t_default, 1),
                     "best": best, "best_us": round(times[best], 1), "ratio": round(t_default / times[best], 3),
                     "frac_hbm_peak": round(nbytes / (t_default * 1e-6) / 8e12, 3),
                     "all_us": {k: round(v, 1) for k, v in times.items()}})
        print(f"  {name}: DEFAULT -> {chosen} {t_default:.1f} us, best {best} {times[best]:.1f} us", flush=True)
        del d, x, y
        torch.cuda.empty_cache()
    return rows


def markdown(rows):
    out = ["| matrix | stored elements | DEFAULT picks | time | % of 8 TB/s | best kernel | its time | DEFAULT / best | the others |",
           "|---|---|---|---|---|---|---|---|---|"]
    for r in rows:
        others = ", ".join(f"{k} {v:.0f}" for k, v in sorted(r["all_us"].items(), key=lambda kv: kv[1]) if k not in (r["best"],))
        out.append(f"| {r['family']} | {r['nnz'] / 1e6:.1f} M | {r['default']} | {r['default_us']:.1f} us | {100 * r['frac_hbm_peak']:.1f} | "
                   f"{r['best']} | {r['best_us']:.1f} us | {r['ratio']:.2f} | {others} |")
    return "\n".join(out)
