"""GPU parity: the HIP path, called through the C-ABI, against the CPU oracle on the same
inputs.  Integer analysis outputs must be bit-identical; values must satisfy, per element,
    |y_gpu - y_ref| <= tol * (|alpha| * sum_j |a_ij x_j| + |beta * y0_i|)
with tol = 1e-12 (fp64) / 1e-5 (fp32): the bound for a pure reordering of the row's sum."""
import numpy as np
import pytest

import plan_check

from conftest import analysis_shapes, csr_from_lengths, row_ptr_from_lengths

pytestmark = pytest.mark.gpu

TOL = {np.dtype(np.float64): 1e-12, np.dtype(np.float32): 1e-5}


@pytest.fixture(scope="module")
def torch():
    import torch
    assert torch.cuda.is_available(), "these tests need the GPU"
    return torch


@pytest.fixture(scope="module")
def capi(torch):
    from library_amd import capi
    capi.lib()  # raises if the HIP library is not built: there is no fallback
    return capi


def dev(torch, a):
    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


def spmv_scale(rp, col, val, x, alpha, beta, y0):
    import scipy.sparse as sp
    A = sp.csr_matrix((np.abs(val.astype(np.float64)), col, rp), shape=(rp.size - 1, x.size))
    return abs(alpha) * (A @ np.abs(x.astype(np.float64))) + abs(beta) * np.abs(y0.astype(np.float64))


def assert_close(got, ref, scale, dtype, what=""):
    err = np.abs(got.astype(np.float64) - ref.astype(np.float64))
    bound = TOL[np.dtype(dtype)] * scale
    bad = np.flatnonzero(~(err <= bound))
    assert bad.size == 0, f"{what}: {bad.size} elements out of tolerance, first {bad[:5]}, err {err[bad[:5]]}, bound {bound[bad[:5]]}"


# ------------------------------------------------------------------ analysis, bit exact
def test_analysis_bit_exact(torch, capi, oracle):
    for name, lens in analysis_shapes().items():
        rp = row_ptr_from_lengths(lens)
        m, nnz = rp.size - 1, int(rp[-1])
        d_rp = dev(torch, rp)
        for t in (1, 2, 3, 8, 25, 64, 1000):
            assert np.array_equal(capi.partition_rows_by_nnz(d_rp, t).cpu().numpy(), oracle.partition_rows_by_nnz(rp, t)), (name, t)
        for items in (1, 7, 64, 1024, 2048):
            assert np.array_equal(capi.nnz_split_rows(d_rp, nnz, items).cpu().numpy(), oracle.nnz_split_rows(rp, items)), (name, items)
        for items in (1, 5, 128, 2048, 4096):
            xs, ys = capi.merge_path_search(d_rp, nnz, items)
            oxs, oys = oracle.merge_path_search(rp, items)
            assert np.array_equal(xs.cpu().numpy(), oxs) and np.array_equal(ys.cpu().numpy(), oys), (name, items)
        for ws, base in ((32, 2), (64, 1), (32, 160)):
            nw = capi.loadbalance_nwarps(nnz, ws, base)
            assert nw == oracle.loadbalance_nwarps(nnz, ws, base)
            if nw > 0:
                assert np.array_equal(capi.loadbalance_partition(d_rp, nnz, ws, nw).cpu().numpy(),
                                      oracle.loadbalance_partition(rp, ws, nw)), (name, ws)
        hist, stats = capi.row_length_histogram(d_rp)
        lens_a = np.asarray(lens)
        bins = np.where(lens_a == 0, 0, np.floor(np.log2(np.maximum(lens_a, 1))).astype(int) + 1)
        assert np.array_equal(hist.cpu().numpy(), np.bincount(bins, minlength=33))
        counts, _ = oracle.find_rows_counts(rp, 2, 1024)
        assert stats.cpu().numpy().tolist() == [int(lens_a.max()), *[int(c) for c in counts]], name


def test_analysis_on_benchmark_shapes(torch, capi, oracle):
    from library_amd import workloads as W
    for rp in (W.csr_zipf(1 << 18, 1 << 18, 20, 1.0, 200000, 0.01, np.float64)[0], W.csr_stencil5(512, 512)[0]):
        nnz = int(rp[-1])
        d_rp = dev(torch, rp)
        xs, ys = capi.merge_path_search(d_rp, nnz, 4096)  # the reference's SpMV tile
        oxs, oys = oracle.merge_path_search(rp, 4096)
        assert np.array_equal(xs.cpu().numpy(), oxs) and np.array_equal(ys.cpu().numpy(), oys)
        assert np.array_equal(capi.nnz_split_rows(d_rp, nnz, 64).cpu().numpy(), oracle.nnz_split_rows(rp, 64))
        assert np.array_equal(capi.nnz_split_rows(d_rp, nnz, 1024).cpu().numpy(), oracle.nnz_split_rows(rp, 1024))
        assert np.array_equal(capi.partition_rows_by_nnz(d_rp, 16).cpu().numpy(), oracle.partition_rows_by_nnz(rp, 16))


# ------------------------------------------------------------------ SpMV
ALGS = ["vector", "stream", "merge", "flat"]


def alg_id(capi, name):
    return {"vector": capi.SPMV_VECTOR, "stream": capi.SPMV_STREAM, "merge": capi.SPMV_MERGE, "flat": capi.SPMV_FLAT}[name]


def run_spmv(torch, capi, rp, col, val, x, y0, alpha, beta, alg, use_plan, n=None):
    d = [dev(torch, a) for a in (rp, col, val, x)]
    y = dev(torch, y0)
    plan = None
    if use_plan:
        plan = capi.Plan(False, alg, val.dtype, rp.size - 1, x.size, col.size, d[0])
    capi.spmv(d[0], d[1], d[2], d[3], y, alpha, beta, alg=alg, plan=plan, n=n)
    torch.cuda.synchronize()
    out = y.cpu().numpy()
    if plan is not None:
        plan.destroy()
    return out


@pytest.mark.parametrize("dtype", [np.float64, np.float32])
@pytest.mark.parametrize("alg", ALGS)
def test_spmv_shapes(torch, capi, oracle, dtype, alg):
    rng = np.random.default_rng(17)
    for name, lens in analysis_shapes().items():
        ncols = int(max(np.max(lens), 64)) + 13
        rp, col, val = csr_from_lengths(lens, ncols, 5, dtype)
        x = rng.uniform(-1, 1, ncols).astype(dtype)
        y0 = rng.uniform(-1, 1, rp.size - 1).astype(dtype)
        for alpha, beta in ((1.0, 0.0), (1.5, 0.5)):
            ref = oracle.spmv(rp, col, val, x, alpha, beta, y0, 2)
            scale = spmv_scale(rp, col, val, x, alpha, beta, y0)
            for use_plan in (False, True):
                got = run_spmv(torch, capi, rp, col, val, x, y0, alpha, beta, alg_id(capi, alg), use_plan)
                assert_close(got, ref, scale, dtype, f"{name} {alg} plan={use_plan} a={alpha} b={beta}")


@pytest.mark.parametrize("alg", ALGS)
def test_spmv_golden_vectors(torch, capi, golden, alg):
    from library_amd import workloads as W
    w = W.banded_f64()
    g = golden("banded_f64.npz")
    scale = spmv_scale(w.row_ptr, w.col, w.val, w.x, 1.0, 0.0, w.y)
    got = run_spmv(torch, capi, w.row_ptr, w.col, w.val, w.x, w.y, 1.0, 0.0, alg_id(capi, alg), True)
    assert_close(got, g["y_a1_b0"], scale, np.float64, "banded a=1 b=0")
    scale = spmv_scale(w.row_ptr, w.col, w.val, w.x, 2.0, 3.0, w.y)
    got = run_spmv(torch, capi, w.row_ptr, w.col, w.val, w.x, w.y, 2.0, 3.0, alg_id(capi, alg), False)
    assert_close(got, g["y_a2_b3"], scale, np.float64, "banded a=2 b=3")
    for tag, dtype in (("f64", np.float64), ("f32", np.float32)):
        g = golden(f"rows_{tag}.npz")
        a, b = float(g["alpha"]), float(g["beta"])
        scale = spmv_scale(g["row_ptr"], g["col"], g["val"], g["x"], a, b, g["y0"])
        got = run_spmv(torch, capi, g["row_ptr"], g["col"], g["val"], g["x"], g["y0"], a, b, alg_id(capi, alg), True)
        assert_close(got, g["y"], scale, dtype, f"rows_{tag}")


@pytest.mark.parametrize("alg", ALGS)
def test_spmv_integer_inputs_bit_exact(torch, capi, oracle, alg):
    # every partial sum is exactly representable: any summation order gives the same bits
    rng = np.random.default_rng(2)
    lens = np.r_[rng.integers(0, 70, 3000), 30000, rng.integers(0, 9, 500)]
    for dtype in (np.float64, np.float32):
        rp, col, _ = csr_from_lengths(lens, 40000, 3, dtype)
        val = rng.integers(-8, 9, col.size).astype(dtype)
        x = rng.integers(-8, 9, 40000).astype(dtype)
        y0 = rng.integers(-8, 9, lens.size).astype(dtype)
        ref = oracle.spmv(rp, col, val, x, 2.0, 3.0, y0, 2)
        got = run_spmv(torch, capi, rp, col, val, x, y0, 2.0, 3.0, alg_id(capi, alg), True)
        assert np.array_equal(got, ref)


@pytest.mark.parametrize("alg", ALGS)
def test_spmv_beta_zero_does_not_read_y_and_is_reproducible(torch, capi, oracle, alg):
    # beta == 0: y is write-only (BLAS convention; the reference's CPU kernel multiplies and so
    # would propagate NaN, its GPU kernels memset y first).  Runs are bit-reproducible.
    rng = np.random.default_rng(8)
    lens = np.minimum(rng.zipf(1.6, 20000), 9000)
    rp, col, val = csr_from_lengths(lens, 30000, 9, np.float64)
    x = rng.uniform(-1, 1, 30000)
    ynan = np.full(lens.size, np.nan)
    a = run_spmv(torch, capi, rp, col, val, x, ynan, 1.0, 0.0, alg_id(capi, alg), True)
    b = run_spmv(torch, capi, rp, col, val, x, ynan, 1.0, 0.0, alg_id(capi, alg), False)
    assert not np.isnan(a).any()
    assert np.array_equal(a, b)
    ref = oracle.spmv(rp, col, val, x, 1.0, 0.0, np.zeros(lens.size), 2)
    assert_close(a, ref, spmv_scale(rp, col, val, x, 1.0, 0.0, np.zeros(lens.size)), np.float64, "nan-y")


def test_spmv_closed_forms(torch, capi):
    from library_amd import workloads as W
    rp, col, val = W.csr_stencil5(300, 200)
    m = 300 * 200
    for alg in (capi.SPMV_VECTOR, capi.SPMV_STREAM, capi.SPMV_MERGE, capi.SPMV_FLAT, capi.SPMV_DEFAULT):
        y = run_spmv(torch, capi, rp, col, val, np.ones(m), np.zeros(m), 1.0, 0.0, alg, True)
        assert np.array_equal(y, 4.0 - (np.diff(rp) - 1))  # 0 interior, 1 edge, 2 corner
    # diagonal matrix: y_i = alpha a_i x_i + beta y_i, one product per row
    n = 5000
    rng = np.random.default_rng(0)
    a, x, y0 = rng.uniform(-1, 1, n), rng.uniform(-1, 1, n), rng.uniform(-1, 1, n)
    rpd, cold = np.arange(n + 1, dtype=np.int32), np.arange(n, dtype=np.int32)
    for alg in (capi.SPMV_VECTOR, capi.SPMV_STREAM, capi.SPMV_MERGE, capi.SPMV_FLAT):
        y = run_spmv(torch, capi, rpd, cold, a, x, y0, 1.5, 0.5, alg, False)
        assert np.all(np.abs(y - (1.5 * a * x + 0.5 * y0)) <= 1e-15 * (np.abs(1.5 * a * x) + np.abs(0.5 * y0)))


def test_spmv_errors_and_empty(torch, capi):
    L = capi.lib()
    rp = dev(torch, np.array([0, 1, 2], dtype=np.int32))
    col = dev(torch, np.array([0, 1], dtype=np.int32))
    val = dev(torch, np.array([1.0, 2.0]))
    x = dev(torch, np.array([1.0, 1.0]))
    y = dev(torch, np.array([5.0, 5.0]))
    # unsupported algorithm id (COO), missing workspace, plan of the wrong kind
    with pytest.raises(capi.AsxError) as e:
        capi.spmv(rp, col, val, x, y, 1.0, 0.0, alg=1)
    assert e.value.code == 6
    assert L.asx_spmv_csr_f64(None, capi.SPMV_MERGE, 2, 2, 2, 1.0, rp.data_ptr(), col.data_ptr(), val.data_ptr(),
                              x.data_ptr(), 0.0, y.data_ptr(), None, 0, None) == 7
    ws = torch.empty(16, dtype=torch.uint8, device="cuda")
    assert L.asx_spmv_csr_f64(None, capi.SPMV_MERGE, 2, 2, 2, 1.0, rp.data_ptr(), col.data_ptr(), val.data_ptr(),
                              x.data_ptr(), 0.0, y.data_ptr(), ws.data_ptr(), 16, None) == 10
    plan = capi.Plan(True, capi.SPMM_MERGE, np.dtype(np.float64), 2, 2, 2, rp, ncols=4)
    with pytest.raises(capi.AsxError) as e:
        capi.spmv(rp, col, val, x, y, 1.0, 0.0, plan=plan)
    assert e.value.code == 3
    plan.destroy()
    # m == 0 is a no-op (also through a plan built without a row_ptr); a matrix with no stored elements scales y
    assert L.asx_spmv_csr_f64(None, 0, 0, 0, 0, 1.0, None, None, None, None, 0.0, None, None, 0, None) == 0
    for alg in (capi.SPMV_DEFAULT, capi.SPMV_STREAM, capi.SPMV_MERGE, capi.SPMV_VECTOR, capi.SPMV_FLAT):
        h = capi.C.c_void_p()
        assert L.asx_plan_create(capi.C.byref(h), 0, alg, capi.R_64F, 0, 0, 0, None, 1, None) == 0
        assert L.asx_spmv_csr_f64(h, alg, 0, 0, 0, 1.0, None, None, None, None, 0.0, None, None, 0, None) == 0
        assert L.asx_plan_destroy(h) == 0
    h = capi.C.c_void_p()
    assert L.asx_plan_create(capi.C.byref(h), 1, capi.SPMM_MERGE, capi.R_32F, 0, 0, 0, None, 64, None) == 0
    assert L.asx_plan_destroy(h) == 0
    rp0 = dev(torch, np.zeros(4, dtype=np.int32))
    e0 = torch.empty(0, dtype=torch.int32, device="cuda")
    v0 = torch.empty(0, dtype=torch.float64, device="cuda")
    for alg in (capi.SPMV_VECTOR, capi.SPMV_STREAM, capi.SPMV_MERGE, capi.SPMV_FLAT):
        y3 = dev(torch, np.array([1.0, 2.0, 3.0]))
        capi.spmv(rp0, e0, v0, x, y3, 2.0, 0.5, alg=alg, n=2)
        torch.cuda.synchronize()
        assert y3.cpu().numpy().tolist() == [0.5, 1.0, 1.5]


def test_default_plan_and_histogram(torch, capi):
    from library_amd import workloads as W
    rp, col, val = W.csr_stencil5(128, 128)  # launch-bound size: the single-launch kernel
    p = capi.Plan(False, capi.SPMV_DEFAULT, np.dtype(np.float64), rp.size - 1, rp.size - 1, col.size, dev(torch, rp))
    assert p.alg == capi.SPMV_VECTOR
    hist, stats = p.histogram()
    assert stats[0] == 5 and hist.sum() == rp.size - 1
    p.destroy()
    rp, col, val = W.csr_stencil5(512, 512)
    p = capi.Plan(False, capi.SPMV_DEFAULT, np.dtype(np.float64), rp.size - 1, rp.size - 1, col.size, dev(torch, rp))
    assert p.alg == capi.SPMV_FLAT
    p.destroy()
    rp = row_ptr_from_lengths(np.r_[np.full(1000, 3), 50000])
    p = capi.Plan(False, capi.SPMV_DEFAULT, np.dtype(np.float64), rp.size - 1, 60000, int(rp[-1]), dev(torch, rp))
    assert p.alg == capi.SPMV_MERGE
    p.destroy()
    lens = np.zeros(600000, dtype=np.int64)  # mostly empty rows: row ends must count as work
    lens[::7] = 5
    rp = row_ptr_from_lengths(lens)
    p = capi.Plan(False, capi.SPMV_DEFAULT, np.dtype(np.float64), rp.size - 1, 1000, int(rp[-1]), dev(torch, rp))
    assert p.alg == capi.SPMV_MERGE
    p.destroy()


# ------------------------------------------------------------------ SpMM
def spmm_scale(rp, col, val, B, n, alpha, beta, C0):
    import scipy.sparse as sp
    k = B.size // n
    A = sp.csr_matrix((np.abs(val.astype(np.float64)), col, rp), shape=(rp.size - 1, k))
    return (abs(alpha) * (A @ np.abs(B.reshape(k, n).astype(np.float64))) + abs(beta) * np.abs(C0.reshape(-1, n).astype(np.float64))).ravel()


def run_spmm(torch, capi, rp, col, val, B, C0, n, alpha, beta, alg, use_plan):
    d = [dev(torch, a) for a in (rp, col, val, B)]
    Cm = dev(torch, C0)
    k = B.size // n
    plan = capi.Plan(True, alg, val.dtype, rp.size - 1, k, col.size, d[0], ncols=n) if use_plan else None
    capi.spmm(d[0], d[1], d[2], d[3], Cm, n, alpha, beta, alg=alg, plan=plan, k=k)
    torch.cuda.synchronize()
    out = Cm.cpu().numpy()
    if plan is not None:
        plan.destroy()
    return out


@pytest.mark.parametrize("dtype", [np.float32, np.float64])
@pytest.mark.parametrize("alg", ["row", "merge"])
def test_spmm_shapes(torch, capi, oracle, dtype, alg):
    algid = capi.SPMM_ROW if alg == "row" else capi.SPMM_MERGE
    rng = np.random.default_rng(23)
    shapes = analysis_shapes()
    for name in ("uniform7", "giant_mid", "empties", "leading_empty", "all_empty", "one_row", "zipf"):
        lens = shapes[name]
        k = int(max(np.max(lens), 64)) + 5
        rp, col, val = csr_from_lengths(lens, k, 6, dtype)
        for n in (1, 7, 64, 65, 130):
            if name not in ("zipf", "uniform7") and n not in (7, 64):
                continue
            B = rng.uniform(-1, 1, k * n).astype(dtype)
            C0 = rng.uniform(-1, 1, (rp.size - 1) * n).astype(dtype)
            for alpha, beta in ((1.0, 1.0), (2.0, 0.0)):
                ref = oracle.spmm(rp, col, val, B, n, alpha, beta, C0, 4)
                scale = spmm_scale(rp, col, val, B, n, alpha, beta, C0)
                got = run_spmm(torch, capi, rp, col, val, B, C0, n, alpha, beta, algid, use_plan=(n == 64))
                assert_close(got, ref, scale, dtype, f"{name} n={n} {alg} a={alpha} b={beta}")


def test_spmm_golden_vectors(torch, capi, golden):
    g = golden("spmm_f32.npz")
    a, b = float(g["alpha"]), float(g["beta"])
    for n in (1, 7, 8, 64, 65):
        scale = spmm_scale(g["row_ptr"], g["col"], g["val"], g[f"B{n}"], n, a, b, g[f"C0_{n}"])
        for alg in (capi.SPMM_ROW, capi.SPMM_MERGE):
            got = run_spmm(torch, capi, g["row_ptr"], g["col"], g["val"], g[f"B{n}"], g[f"C0_{n}"], n, a, b, alg, False)
            assert_close(got, g[f"C{n}"], scale, np.float32, f"spmm golden n={n}")
    g = golden("spmm_f64.npz")
    for n in (1, 8, 13):
        scale = spmm_scale(g["row_ptr"], g["col"], g["val"], g[f"B{n}"], n, a, b, g[f"C0_{n}"])
        got = run_spmm(torch, capi, g["row_ptr"], g["col"], g["val"], g[f"B{n}"], g[f"C0_{n}"], n, a, b, capi.SPMM_MERGE, True)
        assert_close(got, g[f"C{n}"], scale, np.float64, f"spmm f64 golden n={n}")


def test_spmm_padded_leading_dimensions_and_integers(torch, capi, oracle):
    rng = np.random.default_rng(31)
    lens = np.r_[rng.integers(0, 20, 400), 3000, rng.integers(0, 5, 100)]
    rp, col, _ = csr_from_lengths(lens, 3500, 7, np.float32)
    val = rng.integers(-4, 5, col.size).astype(np.float32)
    n, ldb, ldc = 64, 72, 80
    B = rng.integers(-4, 5, 3500 * ldb).astype(np.float32)
    C0 = rng.integers(-4, 5, lens.size * ldc).astype(np.float32)
    ref = oracle.spmm(rp, col, val, B, n, 2.0, 3.0, C0, 4, ldb=ldb, ldc=ldc)
    for alg in (capi.SPMM_ROW, capi.SPMM_MERGE):
        d = [dev(torch, a) for a in (rp, col, val, B)]
        Cm = dev(torch, C0)
        capi.spmm(d[0], d[1], d[2], d[3], Cm, n, 2.0, 3.0, alg=alg, ldb=ldb, ldc=ldc, k=3500)
        torch.cuda.synchronize()
        assert np.array_equal(Cm.cpu().numpy(), ref)  # integers: exact, and padding columns untouched


# ------------------------------------------------------------------ benchmark configurations at full size
def test_benchmark_configs_full_size(torch, capi, oracle):
    from library_amd import workloads as W
    # the BASELINE configurations 2-4, config 2's matrix in fp64, and a 7-point stencil on 160^3 (the
    # bench extra at a size whose oracle run stays short: stacked planes, y read ahead for beta != 0)
    for name in ("uniform16_f32", "uniform16_f64", "powerlaw_f64", "stencil5_f64", "stencil7_f64"):
        w = W.CONFIGS[name](160, 160, 160) if name == "stencil7_f64" else W.CONFIGS[name]()
        ref = oracle.spmv(w.row_ptr, w.col, w.val, w.x, w.alpha, w.beta, w.y, 16)
        scale = spmv_scale(w.row_ptr, w.col, w.val, w.x, w.alpha, w.beta, w.y)
        d = [dev(torch, a) for a in (w.row_ptr, w.col, w.val, w.x)]
        for alg in (capi.SPMV_DEFAULT, capi.SPMV_VECTOR, capi.SPMV_STREAM, capi.SPMV_MERGE, capi.SPMV_FLAT):
            if name == "powerlaw_f64" and alg == capi.SPMV_STREAM:
                pass  # still correct, only slow on the longest rows; keep it covered
            y = dev(torch, w.y)
            plan = capi.Plan(False, alg, w.val.dtype, w.m, w.n, w.nnz, d[0])
            capi.spmv(d[0], d[1], d[2], d[3], y, w.alpha, w.beta, alg=alg, plan=plan)
            torch.cuda.synchronize()
            assert_close(y.cpu().numpy(), ref, scale, w.dtype, f"{name} alg={alg}")
            plan.destroy()
        if name in ("powerlaw_f64", "uniform16_f32", "uniform16_f64"):
            # plans that may look at columns and values: the column-sliced kernel, forced and as
            # DEFAULT's choice on these matrices (scattered columns; the choice is rule-based, so two
            # plan builds agree)
            across_plans = []
            for alg in (capi.SPMV_SLICED, capi.SPMV_DEFAULT, capi.SPMV_DEFAULT):
                plan = capi.Plan(False, alg, w.val.dtype, w.m, w.n, w.nnz, d[0], col=d[1], val=d[2])
                assert plan.alg == capi.SPMV_SLICED and plan.holds_values
                # the partial sums of a call: a workspace of this size, or the plan's own buffer
                assert plan.workspace_bytes == (plan.info("partial_sums") + 256) * w.val.dtype.itemsize
                outs = []
                for rep in range(2):
                    y = dev(torch, w.y)
                    capi.spmv(d[0], d[1], d[2], d[3], y, w.alpha, w.beta, alg=alg, plan=plan,
                              workspace=None if rep == 0 else False)
                    torch.cuda.synchronize()
                    outs.append(y.cpu().numpy())
                    assert_close(outs[-1], ref, scale, w.dtype, f"{name} sliced alg={alg} rep={rep}")
                assert np.array_equal(outs[0], outs[1]), "two calls through one plan must agree bit for bit"
                across_plans.append(outs[0])
                plan.destroy()
            assert all(np.array_equal(across_plans[0], o) for o in across_plans[1:]), \
                "plans built again from the same matrix must give the same bits"
        else:
            # rows that reach only nearby columns: the row-block kernel with its window of x in LDS,
            # forced and as DEFAULT's choice; without columns and values DEFAULT stays row-ordered
            across_plans = []
            for alg in (capi.SPMV_WINDOW, capi.SPMV_DEFAULT):
                plan = capi.Plan(False, alg, w.val.dtype, w.m, w.n, w.nnz, d[0], col=d[1], val=d[2])
                assert plan.alg == capi.SPMV_WINDOW and plan.workspace_bytes == 0  # no row is cut
                # every row holds two elements or more: fp32 values are read where the caller keeps them
                assert plan.info("by_reference") == int(w.val.dtype == np.float32) and plan.holds_values == (w.val.dtype != np.float32)
                outs = []
                for rep in range(2):
                    y = dev(torch, w.y)
                    capi.spmv(d[0], d[1], d[2], d[3], y, w.alpha, w.beta, alg=alg, plan=plan)
                    torch.cuda.synchronize()
                    outs.append(y.cpu().numpy())
                    assert_close(outs[-1], ref, scale, w.dtype, f"{name} window alg={alg} rep={rep}")
                assert np.array_equal(outs[0], outs[1])
                across_plans.append(outs[0])
                plan.destroy()
            assert np.array_equal(across_plans[0], across_plans[1]), "plans built again must give the same bits"
            plan = capi.Plan(False, capi.SPMV_DEFAULT, w.val.dtype, w.m, w.n, w.nnz, d[0])
            assert plan.alg == capi.SPMV_FLAT and not plan.holds_values
            plan.destroy()
        del d
    w = W.spmm_zipf_f32()
    ref = oracle.spmm(w.row_ptr, w.col, w.val, w.x, w.ncols, w.alpha, w.beta, w.y, 16)
    scale = spmm_scale(w.row_ptr, w.col, w.val, w.x, w.ncols, w.alpha, w.beta, w.y)
    got = run_spmm(torch, capi, w.row_ptr, w.col, w.val, w.x, w.y, w.ncols, w.alpha, w.beta, capi.SPMM_DEFAULT, True)
    assert_close(got, ref, scale, np.float32, "spmm_zipf_f32")


# ------------------------------------------------------------------ blocked (MFMA) SpMM
def _block_structured(rng, m, k, dtype, density=0.7):
    """Rows in groups of 16 share column quads: most 16x4 blocks are well filled."""
    rows, cols = [], []
    for br in range((m + 15) // 16):
        nq = (k + 3) // 4
        quads = rng.choice(nq, size=min(nq, int(rng.integers(1, 6))), replace=False)
        for r in range(br * 16, min(br * 16 + 16, m)):
            for q in quads:
                for c in range(q * 4, min(q * 4 + 4, k)):
                    if rng.random() < density:
                        rows.append(r)
                        cols.append(c)
    import scipy.sparse as sp
    A = sp.csr_matrix((rng.uniform(-1, 1, len(rows)).astype(dtype), (rows, cols)), shape=(m, k))
    A.sort_indices()
    return A.indptr.astype(np.int32), A.indices.astype(np.int32), A.data.astype(dtype)


@pytest.mark.parametrize("dtype", [np.float32, np.float64])
def test_spmm_blocked_mfma(torch, capi, oracle, dtype):
    rng = np.random.default_rng(61)
    for m, k in ((1000, 1003), (16, 4), (37, 9), (4096, 2048)):
        rp, col, val = _block_structured(rng, m, k, dtype)
        d = [dev(torch, a) for a in (rp, col, val)]
        for n in (64, 16, 7, 130):
            B = rng.uniform(-1, 1, k * n).astype(dtype)
            C0 = rng.uniform(-1, 1, m * n).astype(dtype)
            plan = capi.Plan(True, capi.SPMM_BLOCKED, np.dtype(dtype), m, k, col.size, d[0], ncols=n, col=d[1], val=d[2])
            assert plan.alg == capi.SPMM_BLOCKED
            nblocks, fill = plan.block_stats()
            keys = np.unique((np.repeat(np.arange(m), np.diff(rp)) // 16).astype(np.int64) * (1 << 31) + col // 4)
            assert nblocks == keys.size and abs(fill - col.size / (64.0 * keys.size)) < 1e-12
            for alpha, beta in ((1.0, 1.0), (2.0, 0.0)):
                ref = oracle.spmm(rp, col, val, B, n, alpha, beta, C0, 4)
                scale = spmm_scale(rp, col, val, B, n, alpha, beta, C0)
                Cm = dev(torch, C0)
                capi.spmm(d[0], d[1], d[2], dev(torch, B), Cm, n, alpha, beta, alg=capi.SPMM_BLOCKED, plan=plan, k=k)
                torch.cuda.synchronize()
                assert_close(Cm.cpu().numpy(), ref, scale, dtype, f"blocked m={m} k={k} n={n} a={alpha} b={beta}")
            plan.destroy()


@pytest.mark.parametrize("dtype", [np.float32, np.float64])
def test_spmm_blocked_repeated_entries_and_value_update(torch, capi, oracle, dtype):
    """CSR may repeat a (row, column): the blocked copy sums the repeats, as the row-wise kernels
    and the reference do.  After the values change, one asx_plan_update_values brings the plan's
    copy up to date."""
    rng = np.random.default_rng(63)
    m, k, n = 300, 260, 64
    rp, col, val = _block_structured(rng, m, k, dtype)
    # repeat about a fifth of the stored elements once or twice, next to the original
    reps = rng.choice([1, 1, 1, 1, 2, 3], size=col.size)
    rows = np.repeat(np.arange(m), np.diff(rp))
    rows2, col2 = np.repeat(rows, reps), np.repeat(col, reps)
    val2 = rng.uniform(-1, 1, col2.size).astype(dtype)
    rp2 = np.zeros(m + 1, np.int32)
    np.cumsum(np.bincount(rows2, minlength=m), out=rp2[1:])
    col2 = col2.astype(np.int32)
    B = rng.uniform(-1, 1, k * n).astype(dtype)
    C0 = rng.uniform(-1, 1, m * n).astype(dtype)
    d = [dev(torch, a) for a in (rp2, col2, val2)]
    for alg in (capi.SPMM_BLOCKED, capi.SPMM_DEFAULT):
        plan = capi.Plan(True, alg, np.dtype(dtype), m, k, col2.size, d[0], ncols=n, col=d[1], val=d[2])
        assert plan.alg == capi.SPMM_BLOCKED and plan.holds_values
        ref = oracle.spmm(rp2, col2, val2, B, n, 1.5, 0.5, C0, 4)
        Cm = dev(torch, C0)
        capi.spmm(d[0], d[1], d[2], dev(torch, B), Cm, n, 1.5, 0.5, alg=alg, plan=plan, k=k)
        torch.cuda.synchronize()
        assert_close(Cm.cpu().numpy(), ref, spmm_scale(rp2, col2, val2, B, n, 1.5, 0.5, C0), dtype, f"repeats alg={alg}")
        val3 = rng.uniform(-1, 1, col2.size).astype(dtype)
        d3 = dev(torch, val3)
        plan.update_values(d3)
        ref = oracle.spmm(rp2, col2, val3, B, n, 1.5, 0.5, C0, 4)
        Cm = dev(torch, C0)
        capi.spmm(d[0], d[1], d3, dev(torch, B), Cm, n, 1.5, 0.5, alg=alg, plan=plan, k=k)
        torch.cuda.synchronize()
        assert_close(Cm.cpu().numpy(), ref, spmm_scale(rp2, col2, val3, B, n, 1.5, 0.5, C0), dtype, f"updated alg={alg}")
        plan.destroy()


def test_spmm_default_picks_blocked_only_for_dense_blocks(torch, capi, oracle):
    rng = np.random.default_rng(62)
    # dense blocks: DEFAULT -> MFMA kernel
    rp, col, val = _block_structured(rng, 2048, 2048, np.float32, density=0.9)
    d = [dev(torch, a) for a in (rp, col, val)]
    plan = capi.Plan(True, capi.SPMM_DEFAULT, np.dtype(np.float32), 2048, 2048, col.size, d[0], ncols=64, col=d[1], val=d[2])
    assert plan.alg == capi.SPMM_BLOCKED and plan.block_stats()[1] > 0.5
    plan.destroy()
    # uniform random columns: blocks hold ~1 element, DEFAULT -> merge kernel
    lens = rng.integers(1, 20, 3000)
    rp, col, val = csr_from_lengths(lens, 100000, 9, np.float32)
    d = [dev(torch, a) for a in (rp, col, val)]
    plan = capi.Plan(True, capi.SPMM_DEFAULT, np.dtype(np.float32), 3000, 100000, col.size, d[0], ncols=64, col=d[1], val=d[2])
    assert plan.alg == capi.SPMM_MERGE
    plan.destroy()
    # asking for the blocked kernel without its plan is an error, not a silent fallback
    B = dev(torch, np.zeros(100000 * 64, dtype=np.float32))
    Cm = dev(torch, np.zeros(3000 * 64, dtype=np.float32))
    with pytest.raises(capi.AsxError) as e:
        capi.spmm(d[0], d[1], d[2], B, Cm, 64, 1.0, 0.0, alg=capi.SPMM_BLOCKED, k=100000)
    assert e.value.code == 1


# ------------------------------------------------------------------ COO -> CSR
def test_coo_sort_and_coo2csr(torch, capi, oracle):
    rng = np.random.default_rng(71)
    for name, lens in analysis_shapes().items():
        ncols = int(max(np.max(lens), 64)) + 3
        rp, col, val = csr_from_lengths(lens, ncols, 11, np.float64)
        m = rp.size - 1
        row_ind = np.repeat(np.arange(m, dtype=np.int32), np.diff(rp))
        assert np.array_equal(capi.coo2csr(dev(torch, row_ind), m).cpu().numpy(), oracle.coo2csr(row_ind, m)), name
        if col.size == 0:
            continue
        perm = rng.permutation(col.size)
        for dtype in (np.float64, np.float32):
            r, c, v = dev(torch, row_ind[perm]), dev(torch, col[perm]), dev(torch, val[perm].astype(dtype))
            capi.coo_sort(r, c, v)
            torch.cuda.synchronize()
            assert np.array_equal(r.cpu().numpy(), row_ind) and np.array_equal(c.cpu().numpy(), col)
            assert np.array_equal(v.cpu().numpy(), val.astype(dtype))


# ------------------------------------------------------------------ operand conversions, bit exact
def test_csr_transpose_rebase_dense_transpose(torch, capi):
    """The transposed copy must equal a stable counting transpose (each row of A^T in ascending row
    of A, duplicate entries in stored order): checked against numpy's stable argsort, with the
    transpose of the transpose giving A back, for both index bases."""
    rng = np.random.default_rng(81)
    for name, lens in analysis_shapes().items():
        n = int(max(np.max(lens), 64)) + 5
        rp, col, val = csr_from_lengths(lens, n, 12, np.float64)
        if col.size:  # duplicate entries: repeat some columns inside their rows
            dup = rng.integers(0, col.size, max(col.size // 20, 1))
            dup = dup[dup + 1 < col.size]
            rows = np.repeat(np.arange(rp.size - 1), np.diff(rp))
            keep = rows[dup] == rows[dup + 1]
            col[dup[keep] + 1] = col[dup[keep]]
        m = rp.size - 1
        rows = np.repeat(np.arange(m, dtype=np.int32), np.diff(rp))
        order = np.argsort(col, kind="stable")
        rp_t = np.zeros(n + 1, dtype=np.int32)
        np.cumsum(np.bincount(col, minlength=n), out=rp_t[1:])
        for dtype in (np.float64, np.float32):
            v = val.astype(dtype)
            for base in (0, 1):
                got = capi.csr_transpose(dev(torch, rp + base), dev(torch, col + base), dev(torch, v), n, idx_base=base)
                torch.cuda.synchronize()
                assert np.array_equal(got[0].cpu().numpy(), rp_t), (name, base)
                assert np.array_equal(got[1].cpu().numpy(), rows[order]), (name, base)
                assert np.array_equal(got[2].cpu().numpy(), v[order]), (name, base)
            back = capi.csr_transpose(got[0], got[1], got[2], m)
            torch.cuda.synchronize()
            assert np.array_equal(back[0].cpu().numpy(), rp)
            assert np.array_equal(back[1].cpu().numpy(), col) and np.array_equal(back[2].cpu().numpy(), v)
        r0, c0 = capi.csr_rebase(dev(torch, rp + 1), dev(torch, col + 1), 1)
        torch.cuda.synchronize()
        assert np.array_equal(r0.cpu().numpy(), rp) and np.array_equal(c0.cpu().numpy(), col)
    for dtype in (np.float32, np.float64):
        for rows_, cols_, ld_in, ld_out in ((1, 1, 1, 1), (64, 64, 64, 64), (65, 63, 70, 67), (300, 7, 7, 300), (3, 1000, 1001, 5)):
            a = rng.uniform(-1, 1, rows_ * ld_in).astype(dtype)
            out = np.full(cols_ * ld_out, 7.0, dtype=dtype)
            d_out = dev(torch, out)
            capi.dense_transpose(dev(torch, a), rows_, cols_, ld_in, d_out, ld_out)
            torch.cuda.synchronize()
            want = out.reshape(cols_, ld_out).copy()
            want[:, :rows_] = a.reshape(rows_, ld_in)[:, :cols_].T
            assert np.array_equal(d_out.cpu().numpy().reshape(cols_, ld_out), want), (rows_, cols_)


# ------------------------------------------------------------------ column-sliced SpMV
@pytest.mark.parametrize("dtype", [np.float64, np.float32])
def test_spmv_sliced_kernel_shapes(torch, capi, oracle, dtype):
    """The sliced kernel forced on small matrices of every awkward shape: slices without elements,
    runs longer than a tile (cut into several partial sums of one row), runs of empty rows, a
    single slice in use, a last slice narrower than the others, more than 64 slices (several
    groups of ranges per row block), beta = 0 over NaN, two calls through one plan, and a value
    update through the kept permutation."""
    rng = np.random.default_rng(91)
    width = 131072 // np.dtype(dtype).itemsize
    cases = []
    for name, lens in analysis_shapes().items():
        if np.sum(lens) == 0:
            continue
        n = int(max(np.max(lens), 64)) + 29
        cases.append((name, csr_from_lengths(lens, n, 6, dtype), n))
    # a few columns in the first slice only; in the last (narrow) slice only; spread over 3 slices
    n3 = 2 * width + 777
    lens = np.r_[rng.integers(0, 9, 3000), 20000]
    rp, col, val = csr_from_lengths(lens, n3, 8, dtype)
    cases.append(("first_slice", (rp, (col % 100).astype(np.int32), val), n3))
    cases.append(("last_slice", (rp, (n3 - 1 - col % 50).astype(np.int32), val), n3))
    cases.append(("spread3", (rp, col, val), n3))
    # 70 slices: row blocks walk two groups of ranges; rows of 300 reach most slices
    n70 = 69 * width + 5
    lens = np.r_[rng.integers(0, 4, 500), np.full(40, 300), 0, 0, 9000]
    cases.append(("slices70", csr_from_lengths(lens, n70, 9, dtype), n70))
    # 300 slices: the builder's and the value update's tables for more than 256 slices
    n300 = 299 * width + 77
    cases.append(("slices300", csr_from_lengths(np.r_[rng.integers(0, 30, 3000), np.full(20, 700)], n300, 13, dtype), n300))
    for name, (rp, col, val), n in cases:
        m = rp.size - 1
        x = rng.uniform(-1, 1, n).astype(dtype)
        y0 = rng.uniform(-1, 1, m).astype(dtype)
        d = [dev(torch, a) for a in (rp, col, val, x)]
        plan = capi.Plan(False, capi.SPMV_SLICED, np.dtype(dtype), m, n, col.size, d[0], col=d[1], val=d[2])
        assert plan.alg == capi.SPMV_SLICED and plan.holds_values
        plan_check.check_plan(plan, capi, rp, col, n, np.dtype(dtype).itemsize)
        for alpha, beta in ((1.5, 0.5), (1.0, 0.0), (-2.0, 1.0)):
            ref = oracle.spmv(rp, col, val, x, dtype(alpha), dtype(beta), y0 if beta else np.zeros_like(y0), 2)
            scale = spmv_scale(rp, col, val, x, alpha, beta, y0)
            for rep in range(2):
                y = dev(torch, y0 if beta else np.full(m, np.nan, dtype=dtype))
                capi.spmv(d[0], d[1], d[2], d[3], y, alpha, beta, alg=capi.SPMV_SLICED, plan=plan)
                torch.cuda.synchronize()
                assert_close(y.cpu().numpy(), ref, scale, dtype, f"{name} a={alpha} b={beta} rep={rep}")
        # new values, same pattern: stale until the plan is told, the oracle's answer afterwards
        val2 = rng.uniform(-1, 1, val.size).astype(dtype)
        d2 = dev(torch, val2)
        plan.update_values(d2)
        ref = oracle.spmv(rp, col, val2, x, dtype(1.5), dtype(0.5), y0, 2)
        y = dev(torch, y0)
        capi.spmv(d[0], d[1], d2, d[3], y, 1.5, 0.5, alg=capi.SPMV_SLICED, plan=plan)
        torch.cuda.synchronize()
        assert_close(y.cpu().numpy(), ref, spmv_scale(rp, col, val2, x, 1.5, 0.5, y0), dtype, f"{name} updated values")
        plan.destroy()
    # the sliced kernel needs its plan; a plan without columns and values cannot be a sliced plan
    L = capi.lib()
    h = capi.C.c_void_p()
    assert L.asx_plan_create(capi.C.byref(h), 0, capi.SPMV_SLICED, capi.R_64F, 10, 10, 10, capi._ptr(d[0]), 1, None) == 6
    assert L.asx_spmv_csr_f64(None, capi.SPMV_SLICED, 1, 1, 0, 1.0, capi._ptr(d[0]), None, None, None, 0.0,
                              capi._ptr(d[3]), None, 0, None) == 6
    # argument errors of the plan constructor that takes columns and values
    for args, want in (((None, capi.SPMV_SLICED, capi.R_64F, 10, 10, 10, capi._ptr(d[0]), capi._ptr(d[1]), capi._ptr(d[2]), None), 7),
                       ((capi.C.byref(h), capi.SPMV_SLICED, capi.R_64F, 10, 10, 10, capi._ptr(d[0]), None, capi._ptr(d[2]), None), 7),
                       ((capi.C.byref(h), capi.SPMV_SLICED, capi.R_64F, -1, 10, 10, capi._ptr(d[0]), capi._ptr(d[1]), capi._ptr(d[2]), None), 10),
                       ((capi.C.byref(h), capi.SPMV_SLICED, capi.R_64F, 10, 10, 0, capi._ptr(d[0]), capi._ptr(d[1]), capi._ptr(d[2]), None), 10),
                       ((capi.C.byref(h), capi.SPMV_SLICED, 7, 10, 10, 10, capi._ptr(d[0]), capi._ptr(d[1]), capi._ptr(d[2]), None), 6),
                       ((capi.C.byref(h), 1, capi.R_64F, 10, 10, 10, capi._ptr(d[0]), capi._ptr(d[1]), capi._ptr(d[2]), None), 6)):
        assert L.asx_spmv_plan_create(*args) == want, args
    assert L.asx_plan_update_values(None, None, None) == 7
    assert L.asx_plan_holds_values(None) == 0


def _banded_random(rng, m, n, half, dens, dtype, empty=0.1, longrow=None):
    """Rows around the (scaled) diagonal: columns within +-half of it, a fraction `dens` of them
    stored, some rows empty, optionally one row that takes every column in reach."""
    rp = np.zeros(m + 1, np.int32)
    cl = []
    for r in range(m):
        c = int(r * (n - 1) / max(m - 1, 1))
        lo, hi = max(0, c - half), min(n, c + half + 1)
        k = 0 if rng.random() < empty else max(1, int(rng.binomial(hi - lo, dens)))
        if longrow is not None and r == longrow:
            k = hi - lo
        cs = np.sort(rng.choice(np.arange(lo, hi), size=min(k, hi - lo), replace=False))
        cl.append(cs)
        rp[r + 1] = rp[r] + cs.size
    col = np.concatenate(cl).astype(np.int32)
    return rp, col, rng.uniform(-1, 1, col.size).astype(dtype)


@pytest.mark.parametrize("dtype", [np.float64, np.float32])
def test_spmv_window_kernel_shapes(torch, capi, oracle, dtype):
    """The row-block kernel forced on banded matrices: empty rows (a slot of their own), rows cut by
    tile starts (carry pass), a row of 1401 spanning six tiles and one of 13001 spanning 51, a block whose last tile is mostly
    padding, a rectangular matrix, the 5-point stencil, beta = 0 over NaN, two calls through one
    plan, a value update; and NOT_SUPPORTED for rows that reach further than a window."""
    rng = np.random.default_rng(93)
    from library_amd import workloads as W
    cases = []
    for (m, n, half, dens, lr) in ((3000, 3000, 40, 0.3, None), (5000, 9000, 700, 0.02, 2500), (700, 700, 300, 0.9, 10),
                                   (20000, 20000, 3, 1.0, None), (257, 300, 100, 0.2, None), (1, 5, 2, 1.0, None)):
        cases.append((f"band {m}x{n} +-{half}", _banded_random(rng, m, n, half, dens, dtype, longrow=lr), n))
    # without empty rows (and no row of one element): plans that read A's values in place
    for (m, n, half, dens, lr) in ((3000, 3000, 40, 0.3, None), (5000, 9000, 700, 0.02, 2500), (2000, 2000, 2, 1.0, None)):
        cases.append((f"full rows {m}x{n} +-{half}", _banded_random(rng, m, n, half, dens, dtype, empty=0.0, longrow=lr), n))
    # a row of 13001 stored elements: 51 tiles whose carries the lanes of a wave add up together
    cases.append(("band 9000x14000 +-6500", _banded_random(rng, 9000, 14000, 6500, 0.02, dtype, longrow=4000), 14000))
    st = W.stencil5_f64(300, 200)
    cases.append(("stencil 300x200", (st.row_ptr, st.col, st.val.astype(dtype)), st.n))
    # windows that move backwards from one block of rows to the next, inside what a ring could still
    # hold: the columns below the chain's first window were never fetched.  Large enough (2^20 rows)
    # for chains of several blocks.
    zig = [(1000, 1400), (200, 600), (5000, 5300), (4000, 4200), (4100, 4900), (0, 50), (9000, 9900), (8990, 9100)]
    groups = 4096
    lens = rng.integers(0, 9, 256 * groups)
    rp = np.zeros(lens.size + 1, np.int32)
    rp[1:] = np.cumsum(lens)
    g = (np.repeat(np.arange(lens.size), lens) // 256) % len(zig)
    zlo = np.array([z[0] for z in zig])[g]
    zw = np.array([z[1] - z[0] for z in zig])[g]
    # distinct ascending columns inside a row: a random start and a stride that keeps 8 of them in range
    within = np.arange(rp[-1]) - np.repeat(rp[:-1], lens)
    col = (zlo + (rng.integers(0, 5, rp[-1])[np.repeat(rp[:-1], lens)] + within * (zw // 9))).astype(np.int32)
    cases.append(("windows moving backwards", (rp, col, rng.uniform(-1, 1, col.size).astype(dtype)), 10000))
    for name, (rp, col, val), n in cases:
        m = rp.size - 1
        x = rng.uniform(-1, 1, n).astype(dtype)
        y0 = rng.uniform(-1, 1, m).astype(dtype)
        d = [dev(torch, a) for a in (rp, col, val, x)]
        full_rows = bool(np.diff(rp).min() >= 2)  # rows that fill their two slots: the values can be read in place
        assert full_rows == name.startswith(("full rows", "stencil", "band 1x5")), name  # the one-row matrix: 3 elements
        # fp32 plans read the values in place wherever they can; fp64 ones when the plan is to follow
        # values changed in place (a checked plan), and then check nothing
        for checked in ((False, True) if full_rows else (False,)):
            plan = capi.Plan(False, capi.SPMV_WINDOW, np.dtype(dtype), m, n, col.size, d[0], col=d[1], val=d[2], checked=checked)
            assert plan.alg == capi.SPMV_WINDOW
            in_place = int(full_rows and (checked or dtype == np.float32))
            assert plan.info("by_reference") == in_place and plan.holds_values == (not in_place) and not plan.checked, name
            plan_check.check_plan(plan, capi, rp, col, n, np.dtype(dtype).itemsize)
            assert plan.workspace_bytes == plan.info("carry_pass") * plan.info("tiles") * np.dtype(dtype).itemsize
            assert plan.info("bands") == 1 and plan.info("rows_per_block") % 256 == 0 and plan.info("tiles") > 0
            if name == "windows moving backwards":
                assert plan.info("chains") < -(-m // plan.info("rows_per_block")), "chains of several blocks expected"
            for alpha, beta in ((1.5, 0.5), (1.0, 0.0), (-2.0, 1.0)):
                ref = oracle.spmv(rp, col, val, x, dtype(alpha), dtype(beta), y0 if beta else np.zeros_like(y0), 2)
                scale = spmv_scale(rp, col, val, x, alpha, beta, y0)
                for rep in range(2):
                    y = dev(torch, y0 if beta else np.full(m, np.nan, dtype=dtype))
                    capi.spmv(d[0], d[1], d[2], d[3], y, alpha, beta, alg=capi.SPMV_WINDOW, plan=plan)
                    torch.cuda.synchronize()
                    assert_close(y.cpu().numpy(), ref, scale, dtype, f"{name} a={alpha} b={beta} rep={rep} checked={checked}")
            val2 = rng.uniform(-1, 1, val.size).astype(dtype)
            d2 = dev(torch, val2)
            plan.update_values(d2)  # nothing to do for a plan that reads the values in place
            y = dev(torch, y0)
            capi.spmv(d[0], d[1], d2, d[3], y, 1.5, 0.5, alg=capi.SPMV_WINDOW, plan=plan)
            torch.cuda.synchronize()
            assert_close(y.cpu().numpy(), oracle.spmv(rp, col, val2, x, dtype(1.5), dtype(0.5), y0, 2),
                         spmv_scale(rp, col, val2, x, 1.5, 0.5, y0), dtype, f"{name} updated values")
            plan.destroy()
    # rows that reach far (uniform random columns over 200 000) are not this kernel's matrix; a row
    # that alone reaches over more columns than the ring holds is not either
    L = capi.lib()
    for lens, ncols in ((rng.integers(1, 9, 2000), 200000), (np.r_[np.full(50, 3), 17000, np.full(50, 3)], 20000)):
        rp, col, val = csr_from_lengths(lens, ncols, 5, dtype)
        d = [dev(torch, a) for a in (rp, col, val)]
        h = capi.C.c_void_p()
        assert L.asx_spmv_plan_create(capi.C.byref(h), capi.SPMV_WINDOW, capi.value_type(np.dtype(dtype)), rp.size - 1,
                                      ncols, col.size, capi._ptr(d[0]), capi._ptr(d[1]), capi._ptr(d[2]), None) == 6
        assert not h.value


def test_spmv_sliced_wide_steps(torch, capi, oracle):
    """Pass 2 of the sliced kernel reads a row block's partial sums inside a slice 64 at a time, or,
    when those ranges are long, 128 (fp64) or 256 (fp32) at a time, several consecutive ones per
    lane from unaligned addresses.  Matrices whose mean range is beyond the thresholds."""
    W = pytest.importorskip("library_amd.workloads")
    rng = np.random.default_rng(171)
    for dtype, m, n, k, want in ((np.float32, 120000, 40000, 48, 160.0), (np.float64, 200000, 180000, 16, 80.0)):
        rp, col, val = W.csr_fixed(m, n, k, dtype, seed=3)
        x = rng.uniform(-1, 1, n).astype(dtype)
        y0 = rng.uniform(-1, 1, m).astype(dtype)
        d = [dev(torch, a) for a in (rp, col, val, x)]
        plan = capi.Plan(False, capi.SPMV_SLICED, np.dtype(dtype), m, n, col.size, d[0], col=d[1], val=d[2])
        plan_check.check_plan(plan, capi, rp, col, n, np.dtype(dtype).itemsize)
        nrb = -(-m // plan.info("rows_per_wave"))
        mean_range = plan.info("partial_sums") / (nrb * plan.info("slices"))
        assert mean_range >= want, (mean_range, plan.info("rows_per_wave"), plan.info("slices"))
        for alpha, beta in ((1.5, 0.5), (1.0, 0.0)):
            ref = oracle.spmv(rp, col, val, x, dtype(alpha), dtype(beta), y0 if beta else np.zeros_like(y0), 4)
            scale = spmv_scale(rp, col, val, x, alpha, beta, y0)
            outs = []
            for rep in range(2):
                y = dev(torch, y0 if beta else np.full(m, np.nan, dtype=dtype))
                capi.spmv(d[0], d[1], d[2], d[3], y, alpha, beta, alg=capi.SPMV_SLICED, plan=plan)
                torch.cuda.synchronize()
                outs.append(y.cpu().numpy())
                assert_close(outs[-1], ref, scale, dtype, f"{np.dtype(dtype).name} a={alpha} b={beta} rep={rep}")
            assert np.array_equal(outs[0], outs[1]), "two calls through one plan must agree bit for bit"
        plan.destroy()


def test_spmv_sliced_workgroups_that_reach_over_the_end_of_a_slice(torch, capi, oracle):
    """Pass 1 hands its workgroups equal shares of all tiles; a share that reaches over the start
    of a slice (further than 32 tiles on either side) is worked off as two pieces with two slices of x,
    one after the other.  Three slices and about a hundred tiles per share: workgroups of two pieces,
    and every workgroup's share within a tile or so of the others'."""
    W = pytest.importorskip("library_amd.workloads")
    rng = np.random.default_rng(181)
    for dtype, m, n, k in ((np.float64, 400000, 40000, 16), (np.float32, 400000, 90000, 16)):
        rp, col, val = W.csr_fixed(m, n, k, dtype, seed=5)
        x = rng.uniform(-1, 1, n).astype(dtype)
        y0 = rng.uniform(-1, 1, m).astype(dtype)
        d = [dev(torch, a) for a in (rp, col, val, x)]
        plan = capi.Plan(False, capi.SPMV_SLICED, np.dtype(dtype), m, n, col.size, d[0], col=d[1], val=d[2])
        plan_check.check_plan(plan, capi, rp, col, n, np.dtype(dtype).itemsize)
        assert plan.info("slices") == 3
        pieces = plan.export("workgroups").reshape(-1, 4)
        wgs = plan.export("wg_pieces").reshape(-1, 8)
        assert wgs.shape[0] == plan.info("workgroups") and (wgs[:, 1] - wgs[:, 0]).max() == 2, "a workgroup of two pieces expected"
        share = np.array([(pieces[a:b, 2] - pieces[a:b, 1]).sum() for a, b in wgs[:, :2]])
        assert share.max() - share.min() <= 64 and share.sum() == plan.info("tiles"), (share.min(), share.max())
        # the same pieces as the rule restated on the host gives for one share per compute unit
        cus = capi.C.c_int(0)
        assert capi.lib().asx_device_info(capi.C.byref(cus), None) == 0
        width = 131072 // np.dtype(dtype).itemsize
        tile_off = np.r_[0, np.cumsum(-(-np.bincount(col // width, minlength=3) // 256))]
        want_pieces, want_wgs = plan_check.split_tiles(tile_off, cus.value)
        assert np.array_equal(pieces.reshape(-1), want_pieces)
        assert sorted(map(tuple, wgs.tolist())) == sorted(map(tuple, want_wgs.reshape(-1, 8).tolist()))
        for alpha, beta in ((1.5, 0.5), (1.0, 0.0)):
            ref = oracle.spmv(rp, col, val, x, dtype(alpha), dtype(beta), y0 if beta else np.zeros_like(y0), 4)
            y = dev(torch, y0 if beta else np.full(m, np.nan, dtype=dtype))
            capi.spmv(d[0], d[1], d[2], d[3], y, alpha, beta, alg=capi.SPMV_SLICED, plan=plan)
            torch.cuda.synchronize()
            assert_close(y.cpu().numpy(), ref, spmv_scale(rp, col, val, x, alpha, beta, y0), dtype, f"{np.dtype(dtype).name} a={alpha} b={beta}")
        plan.destroy()


def _diagonal_bands(rng, m, n, bands, dens, dtype, empty=0.05):
    """Rows whose columns lie on bands of diagonals: for every (lo, hi) in `bands` the columns
    centre + lo .. centre + hi (centre = r n // m) that fall inside the matrix, a fraction `dens`
    of them stored; some rows empty."""
    r = np.arange(m, dtype=np.int64)
    centre = r * n // m
    keys = []
    for lo, hi in bands:
        for off in range(lo, hi + 1):
            c = centre + off
            keep = (c >= 0) & (c < n) & (rng.random(m) < dens)
            keys.append(r[keep] * n + c[keep])
    key = np.unique(np.concatenate(keys))
    rows = key // n
    rows_empty = rng.random(m) < empty
    key = key[~rows_empty[rows]]
    rows = key // n
    rp = np.zeros(m + 1, np.int64)
    np.add.at(rp, rows + 1, 1)
    rp = np.cumsum(rp).astype(np.int32)
    col = (key % n).astype(np.int32)
    return rp, col, rng.uniform(-1, 1, col.size).astype(dtype)


@pytest.mark.parametrize("dtype", [np.float64, np.float32])
def test_spmv_window_kernel_bands_of_diagonals(torch, capi, oracle, dtype):
    """Matrices no single window holds but a few bands of diagonals do (the planes of a stencil on
    a three-dimensional grid): a 7-point and a 27-point stencil on 96 x 96 x 12 and a 7-point one on
    95 x 95 x 14 (stacked planes), three bands that are no planes, random bands on a
    rectangular matrix with an odd number of columns, five bands (the two closest are joined), long
    rows that tiles cut (carry pass); and NOT_SUPPORTED where the bands are too wide for the LDS."""
    rng = np.random.default_rng(131)
    nx, ny, nz = 96, 96, 12
    plane = nx * ny
    cases = []

    def stencil3d(points, nx=nx, ny=ny, nz=nz):
        plane = nx * ny
        idx = np.arange(nx * ny * nz, dtype=np.int64)
        i, j, k = idx % nx, (idx // nx) % ny, idx // plane
        rng3 = (-1, 0, 1)
        offs = [(di, dj, dk) for dk in rng3 for dj in rng3 for di in rng3
                if points == 27 or abs(di) + abs(dj) + abs(dk) <= 1]
        keys = []
        for di, dj, dk in offs:
            ii, jj, kk = i + di, j + dj, k + dk
            ok = (ii >= 0) & (ii < nx) & (jj >= 0) & (jj < ny) & (kk >= 0) & (kk < nz)
            keys.append(idx[ok] * idx.size + (ii + nx * (jj + ny * kk))[ok])
        key = np.sort(np.concatenate(keys))
        rp = np.zeros(idx.size + 1, np.int64)
        np.add.at(rp, key // idx.size + 1, 1)
        return np.cumsum(rp).astype(np.int32), (key % idx.size).astype(np.int32), rng.uniform(-1, 1, key.size).astype(dtype)

    for pts in (7, 27):
        cases.append((f"stencil {pts} points", stencil3d(pts), nx * ny * nz))
    # planes of 9025 points (no multiple of 64, nor of the 16-byte units x is fetched in), blocks of 361 rows
    cases.append(("stencil 7 points, planes of 9025", stencil3d(7, 95, 95, 14), 9025 * 14))
    # three bands whose distance does not divide the rows: a ring per band
    cases.append(("three bands", _diagonal_bands(rng, 50000, 50000, [(-9501, -9499), (-2, 2), (9499, 9501)], 0.9, dtype), 50000))
    cases.append(("two far bands, rectangular", _diagonal_bands(rng, 50000, 70001, [(-30000, -29990), (-5, 40)], 0.5, dtype), 70001))
    cases.append(("five bands", _diagonal_bands(rng, 40000, 40000, [(-20000, -20000), (-9000, -8990), (0, 0), (300, 310), (15000, 15001)],
                                                0.9, dtype), 40000))
    cases.append(("long rows", _diagonal_bands(rng, 9000, 60000, [(-25000, -24400), (0, 500)], 0.8, dtype), 60000))
    L = capi.lib()
    for name, (rp, col, val), n in cases:
        m = rp.size - 1
        x = rng.uniform(-1, 1, n).astype(dtype)
        y0 = rng.uniform(-1, 1, m).astype(dtype)
        d = [dev(torch, a) for a in (rp, col, val, x)]
        # the grids without dropped elements have no row of fewer than two elements: fp32 plans read
        # their values in place, fp64 plans when they are to follow values changed in place
        full_rows = bool(np.diff(rp).min() >= 2)
        for checked in ((False, True) if full_rows else (False,)):
            plan = capi.Plan(False, capi.SPMV_WINDOW, np.dtype(dtype), m, n, col.size, d[0], col=d[1], val=d[2], checked=checked)
            assert plan.alg == capi.SPMV_WINDOW
            in_place = int(full_rows and (checked or dtype == np.float32))
            assert plan.info("by_reference") == in_place and plan.holds_values == (not in_place) and not plan.checked, name
            plan_check.check_plan(plan, capi, rp, col, n, np.dtype(dtype).itemsize)
            assert plan.workspace_bytes == plan.info("carry_pass") * plan.info("tiles") * np.dtype(dtype).itemsize
            assert 2 <= plan.info("bands") <= 4 and plan.info("slices") == -1, (name, plan.info("bands"))
            # the stencils' three bands lie whole planes apart: their blocks are stored plane above plane
            # and x is fetched about once (a ring per band: three times)
            want_planes = {"stencil 7 points": plane, "stencil 27 points": plane, "stencil 7 points, planes of 9025": 9025}.get(name, 0)
            assert plan.info("stacked_rows") == want_planes, (name, plan.info("stacked_rows"))
            if want_planes:  # past the first block of a chain a block fetches the plane above it only
                pcs = plan.export("pieces").reshape(-1, 3, 4)
                fetches = (pcs[:, :, 1] > pcs[:, :, 0]).sum(axis=1)
                first = np.zeros(fetches.size, bool)
                first[plan.export("workgroups").reshape(-1, 2)[:, 0]] = True
                assert np.all(fetches[~first] <= 1) and np.all(fetches[first] >= 2), name
            if name in ("stencil 7 points", "long rows"):  # rows of at most 16 are never cut by tiles
                assert plan.info("carry_pass") == (1 if name == "long rows" else 0), name
            for alpha, beta in ((1.5, 0.5), (1.0, 0.0)):
                ref = oracle.spmv(rp, col, val, x, dtype(alpha), dtype(beta), y0 if beta else np.zeros_like(y0), 2)
                scale = spmv_scale(rp, col, val, x, alpha, beta, y0)
                for rep in range(2):
                    y = dev(torch, y0 if beta else np.full(m, np.nan, dtype=dtype))
                    capi.spmv(d[0], d[1], d[2], d[3], y, alpha, beta, alg=capi.SPMV_WINDOW, plan=plan)
                    torch.cuda.synchronize()
                    assert_close(y.cpu().numpy(), ref, scale, dtype, f"{name} a={alpha} b={beta} rep={rep} checked={checked}")
            plan.destroy()
    # three bands of 9000 diagonals each: 27000 columns a block, more than the LDS holds
    rp, col, val = _diagonal_bands(rng, 30000, 90000, [(-40000, -31000), (0, 9000), (30000, 39000)], 0.002, dtype)
    d = [dev(torch, a) for a in (rp, col, val)]
    h = capi.C.c_void_p()
    assert L.asx_spmv_plan_create(capi.C.byref(h), capi.SPMV_WINDOW, capi.value_type(np.dtype(dtype)), rp.size - 1, 90000,
                                  col.size, capi._ptr(d[0]), capi._ptr(d[1]), capi._ptr(d[2]), None) == 6
    assert not h.value


@pytest.mark.parametrize("dtype", [np.float64, np.float32])
def test_regrouped_kernels_with_x_off_a_16_byte_boundary(torch, capi, oracle, dtype):
    """x passed as a view that starts one element into an allocation (a sub-vector behind
    vecX->values): its address is no multiple of 16, so the kernels that copy x into LDS take their
    element-by-element fetch; and matrices with 1 to 3 columns, shorter than one 16-byte unit.
    Window plans with one band and with bands of diagonals, and a sliced plan."""
    rng = np.random.default_rng(211)
    cases = [("band", capi.SPMV_WINDOW, _banded_random(rng, 9000, 9000, 300, 0.05, dtype, longrow=700), 9000),
             ("two bands", capi.SPMV_WINDOW, _diagonal_bands(rng, 50000, 70001, [(-30000, -29990), (-5, 40)], 0.5, dtype), 70001),
             ("scattered", capi.SPMV_SLICED, csr_from_lengths(np.minimum(rng.zipf(1.6, 30000), 2000), 70001, 3, dtype), 70001)]
    for n in (1, 2, 3):
        lens = rng.integers(0, n + 1, 5000)
        cases.append((f"{n} columns", capi.SPMV_WINDOW, csr_from_lengths(lens, n, 5, dtype), n))
        cases.append((f"{n} columns", capi.SPMV_SLICED, csr_from_lengths(lens, n, 5, dtype), n))
    for name, alg, (rp, col, val), n in cases:
        m = rp.size - 1
        x = rng.uniform(-1, 1, n).astype(dtype)
        y0 = rng.uniform(-1, 1, m).astype(dtype)
        d = [dev(torch, a) for a in (rp, col, val)]
        xbuf = dev(torch, np.r_[dtype(7.0), x, dtype(9.0)])
        xv = xbuf[1:1 + n]
        assert xv.data_ptr() % 16 != 0 and xv.data_ptr() == xbuf.data_ptr() + np.dtype(dtype).itemsize
        plan = capi.Plan(False, alg, np.dtype(dtype), m, n, col.size, d[0], col=d[1], val=d[2])
        plan_check.check_plan(plan, capi, rp, col, n, np.dtype(dtype).itemsize)
        ref = oracle.spmv(rp, col, val, x, dtype(1.5), dtype(0.5), y0, 2)
        for xin, tag in ((xv, "offset x"), (dev(torch, x), "aligned x")):
            y = dev(torch, y0)
            capi.spmv(d[0], d[1], d[2], xin, y, 1.5, 0.5, alg=alg, plan=plan, n=n)
            torch.cuda.synchronize()
            assert_close(y.cpu().numpy(), ref, spmv_scale(rp, col, val, x, 1.5, 0.5, y0), dtype, f"{name} alg {alg} {tag}")
        plan.destroy()


def test_sliced_and_window_calls_replay_in_a_hip_graph(torch, capi, oracle):
    """A call with a sliced or window plan is kernels only (no allocation, copy, memset or
    synchronisation): captured once in a HIP graph it must give the eager result on every replay,
    with eager work and synchronisations of the program between the replays."""
    rng = np.random.default_rng(151)
    lens = np.minimum(rng.zipf(1.6, 20000), 3000)
    cases = [(capi.SPMV_SLICED, csr_from_lengths(lens, 90000, 7, np.float64), 90000),
             (capi.SPMV_WINDOW, _banded_random(rng, 20000, 20000, 300, 0.05, np.float64, longrow=700), 20000)]
    for alg, (rp, col, val), n in cases:
        m = rp.size - 1
        x = rng.uniform(-1, 1, n)
        y0 = rng.uniform(-1, 1, m)
        d = [dev(torch, a) for a in (rp, col, val, x)]
        plan = capi.Plan(False, alg, val.dtype, m, n, col.size, d[0], col=d[1], val=d[2])
        ws = torch.empty(max(plan.workspace_bytes, 256), dtype=torch.uint8, device="cuda")  # no allocation while capturing
        y_eager = dev(torch, y0)
        capi.spmv(d[0], d[1], d[2], d[3], y_eager, 1.5, 0.5, alg=alg, plan=plan, workspace=ws)
        torch.cuda.synchronize()
        eager = y_eager.cpu().numpy()
        assert_close(eager, oracle.spmv(rp, col, val, x, 1.5, 0.5, y0, 2), spmv_scale(rp, col, val, x, 1.5, 0.5, y0),
                     np.float64, f"eager alg {alg}")
        y = dev(torch, y0)
        side = torch.cuda.Stream()
        graph = torch.cuda.CUDAGraph()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            with torch.cuda.graph(graph, stream=side):
                capi.spmv(d[0], d[1], d[2], d[3], y, 1.5, 0.5, alg=alg, plan=plan, workspace=ws)
        torch.cuda.synchronize()
        for rep in range(3):
            y.copy_(dev(torch, y0))                      # eager work between the replays
            scratch = (d[3] * 2.0).sum().item()          # and a synchronisation
            assert np.isfinite(scratch)
            graph.replay()
            torch.cuda.synchronize()
            assert np.array_equal(y.cpu().numpy(), eager), f"alg {alg} replay {rep}"
        del graph
        plan.destroy()
    # checked plans: the check of the values, the update of the copy and the multiply are kernels
    # only as well; captured together they follow values changed in place between two replays.
    # A sliced plan (checksums, copy brought up to date) and a window plan over full rows (values
    # read in place: nothing but the multiply)
    cases = [(capi.SPMV_SLICED, csr_from_lengths(lens, 90000, 7, np.float64), 90000),
             (capi.SPMV_WINDOW, _banded_random(rng, 20000, 20000, 300, 0.05, np.float64, empty=0.0, longrow=700), 20000)]
    for alg, (rp, col, val), n in cases:
        m = rp.size - 1
        x = rng.uniform(-1, 1, n)
        y0 = rng.uniform(-1, 1, m)
        d = [dev(torch, a) for a in (rp, col, val, x)]
        plan = capi.Plan(False, alg, val.dtype, m, n, col.size, d[0], col=d[1], val=d[2], checked=True)
        assert plan.checked == (alg == capi.SPMV_SLICED) and plan.holds_values == (alg == capi.SPMV_SLICED)
        ws = torch.empty(max(plan.workspace_bytes, 256), dtype=torch.uint8, device="cuda")
        y = dev(torch, y0)
        plan.refresh_if_changed(d[2])  # once outside: whatever the first call sets up is set up
        capi.spmv(d[0], d[1], d[2], d[3], y, 1.5, 0.5, alg=alg, plan=plan, workspace=ws)
        torch.cuda.synchronize()
        side = torch.cuda.Stream()
        graph = torch.cuda.CUDAGraph()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            with torch.cuda.graph(graph, stream=side):
                plan.refresh_if_changed(d[2])
                capi.spmv(d[0], d[1], d[2], d[3], y, 1.5, 0.5, alg=alg, plan=plan, workspace=ws)
        torch.cuda.synchronize()
        cur = val.copy()
        for rep in range(4):
            if rep:  # the caller overwrites values in place: one, then many, then the first ones again
                cur = val.copy() if rep == 3 else cur
                if rep == 1:
                    cur[col.size // 3] += 0.5
                elif rep == 2:
                    cur = rng.uniform(-1, 1, col.size)
                d[2].copy_(torch.from_numpy(cur))
            y.copy_(dev(torch, y0))
            graph.replay()
            torch.cuda.synchronize()
            assert_close(y.cpu().numpy(), oracle.spmv(rp, col, cur, x, 1.5, 0.5, y0, 2), spmv_scale(rp, col, cur, x, 1.5, 0.5, y0),
                         np.float64, f"checked alg {alg} replay {rep}")
        del graph
        plan.destroy()


def test_one_plan_two_streams_two_workspaces(torch, capi, oracle):
    """Calls through one sliced (window) plan that each bring a workspace of plan.workspace_bytes keep
    their partial sums (carries) apart: two streams run them at the same time on different x, and
    both results are the oracle's.  After asx_plan_release_scratch a call without a workspace is
    refused and one with a workspace still works."""
    rng = np.random.default_rng(163)
    lens = np.minimum(rng.zipf(1.5, 60000), 4000)
    cases = [(capi.SPMV_SLICED, csr_from_lengths(lens, 120000, 11, np.float64), 120000),
             (capi.SPMV_WINDOW, _banded_random(rng, 20000, 20000, 300, 0.05, np.float64, longrow=700), 20000)]
    for alg, (rp, col, val), n in cases:
        m = rp.size - 1
        xs = [rng.uniform(-1, 1, n) for _ in range(2)]
        y0 = rng.uniform(-1, 1, m)
        refs = [oracle.spmv(rp, col, val, x, 1.5, 0.5, y0, 2) for x in xs]
        scales = [spmv_scale(rp, col, val, x, 1.5, 0.5, y0) for x in xs]
        d = [dev(torch, a) for a in (rp, col, val)]
        dx = [dev(torch, x) for x in xs]
        plan = capi.Plan(False, alg, val.dtype, m, n, col.size, d[0], col=d[1], val=d[2])
        need = plan.workspace_bytes
        assert need > 0 and capi.lib().asx_plan_own_scratch_bytes(plan.h) == need, alg
        ws = [torch.empty(need, dtype=torch.uint8, device="cuda") for _ in range(2)]
        streams = [torch.cuda.Stream() for _ in range(2)]
        torch.cuda.synchronize()
        for rep in range(5):
            ys = [dev(torch, y0) for _ in range(2)]
            torch.cuda.synchronize()
            for k in range(2):
                with torch.cuda.stream(streams[k]):
                    capi.spmv(d[0], d[1], d[2], dx[k], ys[k], 1.5, 0.5, alg=alg, plan=plan, workspace=ws[k])
            torch.cuda.synchronize()
            for k in range(2):
                assert_close(ys[k].cpu().numpy(), refs[k], scales[k], np.float64, f"alg {alg} rep {rep} stream {k}")
        plan.release_scratch()
        assert capi.lib().asx_plan_own_scratch_bytes(plan.h) == 0
        y = dev(torch, y0)
        with pytest.raises(capi.AsxError):
            capi.spmv(d[0], d[1], d[2], dx[0], y, 1.5, 0.5, alg=alg, plan=plan, workspace=False)
        capi.spmv(d[0], d[1], d[2], dx[0], y, 1.5, 0.5, alg=alg, plan=plan, workspace=ws[0])
        torch.cuda.synchronize()
        assert_close(y.cpu().numpy(), refs[0], scales[0], np.float64, f"alg {alg} after release")
        plan.destroy()


def test_default_keeps_the_row_block_copy_off_matrices_of_mostly_empty_rows(torch, capi, oracle):
    """The window format gives every empty row a slot of its own (value, column word, source index,
    read in every call): for a matrix with far more rows than stored elements that is more traffic
    than the row offsets the other kernels stream.  Three quarters of 9 M rows empty, the rest
    with one element next to the diagonal (columns as local as they get): DEFAULT must not pick the
    window kernel, the forced window plan still works, and both give the oracle's result."""
    rng = np.random.default_rng(171)
    m = n = 9 << 20
    rows = np.nonzero(rng.random(m) < 0.25)[0]
    col = np.clip(rows + rng.integers(-100, 101, rows.size), 0, n - 1).astype(np.int32)
    rp = np.zeros(m + 1, np.int32)
    np.cumsum(np.bincount(rows, minlength=m), out=rp[1:])
    assert col.size >= 1 << 21
    val = rng.uniform(-1, 1, col.size)
    x = rng.uniform(-1, 1, n)
    y0 = rng.uniform(-1, 1, m)
    ref = oracle.spmv(rp, col, val, x, 1.5, 0.5, y0, 8)
    scale = spmv_scale(rp, col, val, x, 1.5, 0.5, y0)
    d = [dev(torch, a) for a in (rp, col, val, x)]
    plan = capi.Plan(False, capi.SPMV_DEFAULT, val.dtype, m, n, col.size, d[0], col=d[1], val=d[2])
    assert plan.alg != capi.SPMV_WINDOW, plan.alg
    forced = capi.Plan(False, capi.SPMV_WINDOW, val.dtype, m, n, col.size, d[0], col=d[1], val=d[2])
    assert forced.info("tiles") * 256 >= m, "a slot per row, empty or not"
    for p in (plan, forced):
        y = dev(torch, y0)
        capi.spmv(d[0], d[1], d[2], d[3], y, 1.5, 0.5, plan=p)
        torch.cuda.synchronize()
        assert_close(y.cpu().numpy(), ref, scale, np.float64, f"kernel {p.alg}")
        p.destroy()


def test_default_workspace_covers_every_choice(torch, capi, oracle):
    """alphasparseSpMV_bufferSize(DEFAULT) is asx_spmv_workspace_bytes(DEFAULT): whatever kernel a
    DEFAULT plan settles on must fit in it.  Hypersparse (the plan takes the merge-path kernel,
    whose carry array follows m + nnz) and very long rows, with an exactly sized workspace."""
    rng = np.random.default_rng(77)
    L = capi.lib()
    shapes = {
        "hypersparse": np.where(rng.random(2_000_000) < 0.05, 1, 0),
        "long_rows": np.r_[np.full(20, 9000), rng.integers(0, 3, 300000)],
    }
    for name, lens in shapes.items():
        m = lens.size
        n = 50000
        rp = np.zeros(m + 1, np.int32)
        rp[1:] = np.cumsum(lens)
        nnz = int(rp[-1])
        col = np.sort(rng.integers(0, n, nnz).astype(np.int32))  # order inside rows does not matter here
        rows = np.repeat(np.arange(m), lens)
        order = np.lexsort((col, rows))
        col = col[order]
        val = rng.uniform(-1, 1, nnz)
        x = rng.uniform(-1, 1, n)
        y0 = rng.uniform(-1, 1, m)
        d = [dev(torch, a) for a in (rp, col, val, x)]
        plan = capi.Plan(False, capi.SPMV_DEFAULT, val.dtype, m, n, nnz, d[0], col=d[1], val=d[2])
        budget = L.asx_spmv_workspace_bytes(capi.SPMV_DEFAULT, capi.R_64F, m, nnz)
        assert plan.alg == capi.SPMV_MERGE, name
        assert plan.workspace_bytes <= budget, (name, plan.workspace_bytes, budget)
        ws = torch.empty(budget, dtype=torch.uint8, device="cuda")
        y = dev(torch, y0)
        capi.spmv(d[0], d[1], d[2], d[3], y, 1.5, 0.5, plan=plan, workspace=ws)
        torch.cuda.synchronize()
        ref = oracle.spmv(rp, col, val, x, 1.5, 0.5, y0, 4)
        assert_close(y.cpu().numpy(), ref, spmv_scale(rp, col, val, x, 1.5, 0.5, y0), np.float64, name)
        plan.destroy()


# ------------------------------------------------------------------ randomised shapes, every SpMV kernel
def test_spmv_random_shapes_all_kernels(torch, capi, oracle):
    rng = np.random.default_rng(2024)
    for case in range(90):
        kind = case % 6
        m = int(rng.integers(1, 4000))
        if kind == 0:
            lens = rng.integers(0, 12, m)
        elif kind == 1:
            lens = np.minimum(rng.zipf(1.5, m), 6000)
        elif kind == 2:  # runs of empty rows between long rows
            lens = np.where(rng.random(m) < 0.02, rng.integers(500, 5000, m), 0)
        elif kind == 3:  # rows that end exactly on 4-, 1024- and 2048-element boundaries
            lens = rng.choice([4, 8, 1020, 1024, 1028, 2044, 2048, 2052, 0, 1], m if m < 40 else 40)
        elif kind == 4:
            lens = np.r_[rng.integers(0, 3, m), int(rng.integers(3000, 30000)), rng.integers(0, 3, 5)]
        else:
            lens = rng.integers(30, 36, m)  # around the row-mode / walk-mode threshold of the flat kernel
        ncols = int(max(np.max(lens), 8)) + int(rng.integers(1, 50))
        dtype = np.float64 if case % 2 == 0 else np.float32
        rp, col, val = csr_from_lengths(lens, ncols, 1000 + case, dtype)
        x = rng.uniform(-1, 1, ncols).astype(dtype)
        y0 = rng.uniform(-1, 1, rp.size - 1).astype(dtype)
        alpha, beta = ((1.0, 0.0), (1.5, 0.5), (-2.0, 1.0))[case % 3]
        ref = oracle.spmv(rp, col, val, x, alpha, beta, y0, 2)
        scale = spmv_scale(rp, col, val, x, alpha, beta, y0)
        for alg in ALGS:
            got = run_spmv(torch, capi, rp, col, val, x, y0, alpha, beta, alg_id(capi, alg), use_plan=(case % 4 < 2))
            assert_close(got, ref, scale, dtype, f"case {case} kind {kind} {alg}")
        if col.size:  # the sliced kernel needs its plan
            d = [dev(torch, a) for a in (rp, col, val, x)]
            y = dev(torch, y0)
            plan = capi.Plan(False, capi.SPMV_SLICED, np.dtype(dtype), rp.size - 1, ncols, col.size, d[0], col=d[1], val=d[2])
            plan_check.check_plan(plan, capi, rp, col, ncols, np.dtype(dtype).itemsize)
            capi.spmv(d[0], d[1], d[2], d[3], y, alpha, beta, alg=capi.SPMV_SLICED, plan=plan)
            torch.cuda.synchronize()
            assert_close(y.cpu().numpy(), ref, scale, dtype, f"case {case} kind {kind} sliced")
            plan.destroy()
            # the row-block kernel where it applies (columns within reach, no row longer than 2048)
            h = capi.C.c_void_p()
            rc = capi.lib().asx_spmv_plan_create(capi.C.byref(h), capi.SPMV_WINDOW, capi.value_type(np.dtype(dtype)),
                                                 rp.size - 1, ncols, col.size, capi._ptr(d[0]), capi._ptr(d[1]),
                                                 capi._ptr(d[2]), None)
            assert rc in (0, 6), rc
            if rc == 0:
                plan_check.check_plan(capi.Plan.adopt(h), capi, rp, col, ncols, np.dtype(dtype).itemsize)
                y = dev(torch, y0)
                fn = capi.lib().asx_spmv_csr_f64 if dtype == np.float64 else capi.lib().asx_spmv_csr_f32
                assert fn(h, capi.SPMV_WINDOW, rp.size - 1, ncols, col.size, alpha, capi._ptr(d[0]), capi._ptr(d[1]),
                          capi._ptr(d[2]), capi._ptr(d[3]), beta, capi._ptr(y), None, 0, capi._stream()) == 0
                torch.cuda.synchronize()
                assert_close(y.cpu().numpy(), ref, scale, dtype, f"case {case} kind {kind} window")
                capi.lib().asx_plan_destroy(h)


# ------------------------------------------------------------------ measurement helper
def test_calibration_copy_runs(torch, capi):
    """The benchmark's copy kernel copies, and rejects sizes that are no multiple of 16."""
    L = capi.lib()
    rng = np.random.default_rng(5)
    stream = capi._stream()
    src = dev(torch, rng.integers(0, 255, 1 << 20).astype(np.uint8))
    dst = torch.zeros_like(src)
    assert L.asx_copy_bytes(capi._ptr(src), capi._ptr(dst), src.numel(), stream) == 0
    torch.cuda.synchronize()
    assert torch.equal(src, dst)
    assert L.asx_copy_bytes(capi._ptr(src), capi._ptr(dst), 17, stream) == 10
    # the random-line gather of the benchmark: runs for both group sizes, refuses others
    import ctypes as C
    nthreads = C.c_int(0)
    assert L.asx_gather_lines(None, 0, 1, 8, None, C.byref(nthreads), None) == 0 and nthreads.value > 0
    out = torch.zeros(nthreads.value, dtype=torch.int32, device="cuda")
    buf = torch.ones(1 << 22, dtype=torch.int32, device="cuda")
    for group in (1, 64):
        assert L.asx_gather_lines(capi._ptr(buf), buf.numel() * 4, group, 16, capi._ptr(out), None, stream) == 0
        torch.cuda.synchronize()
        assert int(out.min()) == 16 and int(out.max()) == 16  # 16 loads of the value 1 per lane
    assert L.asx_gather_lines(capi._ptr(buf), buf.numel() * 4, 3, 16, capi._ptr(out), None, stream) == 3
    assert L.asx_gather_lines(capi._ptr(buf), buf.numel() * 4, 1, 12, capi._ptr(out), None, stream) == 3


# ------------------------------------------------------------------ checked plans (values changed in place)
@pytest.mark.parametrize("dtype", [np.float64, np.float32])
def test_checked_plans_follow_values_changed_in_place(torch, capi, oracle, dtype):
    """asx_spmv_plan_create_checked + asx_plan_refresh_if_changed: a plan that holds a copy of A's
    values notices, by two checksums taken on the device before every call, that the caller changed
    values in place, and refreshes its copy; with unchanged values the call gives the same bits as
    before.  Sliced plan (scattered columns) and window plans (a band whose values are read in
    place: nothing kept, nothing checked; a band with empty rows: a checked copy), DEFAULT's choice; a single
    changed value, two swapped values (same multiset: only position-dependent sums see it), a flipped
    sign, all values; a small matrix stays row-ordered and unchecked."""
    from library_amd import workloads as W
    rng = np.random.default_rng(77)
    cases = []
    rp, col, val = W.csr_fixed(1 << 18, 1 << 20, 12, dtype, 3)
    cases.append(("scattered", rp, col, val, 1 << 20, capi.SPMV_SLICED))
    rp, col, val = W.csr_banded(1 << 19, 4, dtype, 5)
    cases.append(("band of 9", rp, col, val, 1 << 19, capi.SPMV_WINDOW))
    rp, col, val = _banded_random(rng, 60000, 60000, 30, 0.3, dtype)  # one row in ten is empty
    cases.append(("band with empty rows", rp, col, val, 60000, capi.SPMV_WINDOW))
    for name, rp, col, val, n, want_alg in cases:
        m, nnz = rp.size - 1, col.size
        x = rng.uniform(-1, 1, n).astype(dtype)
        y0 = rng.uniform(-1, 1, m).astype(dtype)
        d_rp, d_col, d_val, d_x = (dev(torch, a) for a in (rp, col, val, x))
        for alg in (want_alg, capi.SPMV_DEFAULT):
            d_val.copy_(torch.from_numpy(val))
            plan = capi.Plan(False, alg, np.dtype(dtype), m, n, nnz, d_rp, col=d_col, val=d_val, checked=True)
            if alg == capi.SPMV_DEFAULT and plan.alg != want_alg:
                # DEFAULT counted the price of checking and stayed with a kernel that reads the caller's values
                assert not plan.checked and not plan.holds_values, (name, plan.alg)
                plan.destroy()
                continue
            # a window plan over rows of two elements or more keeps no copy: nothing to check or refresh,
            # and the same sequence of in-place changes must come out right all the same
            by_ref = plan.alg == capi.SPMV_WINDOW and plan.info("by_reference") == 1
            assert plan.alg == want_alg and by_ref == (name == "band of 9"), (name, plan.alg)
            assert plan.checked == (not by_ref) and plan.holds_values == (not by_ref), name

            def product(values):
                ref = oracle.spmv(rp, col, values, x, dtype(1.5), dtype(0.5), y0, 4)
                y = dev(torch, y0)
                plan.refresh_if_changed(d_val)
                capi.spmv(d_rp, d_col, d_val, d_x, y, 1.5, 0.5, alg=alg, plan=plan)
                torch.cuda.synchronize()
                got = y.cpu().numpy()
                assert_close(got, ref, spmv_scale(rp, col, values, x, 1.5, 0.5, y0), dtype, f"{name} alg={alg}")
                return got
            first = product(val)
            assert np.array_equal(first, product(val)), "unchanged values: the same bits"
            cur = val.copy()
            cur[nnz // 3] += dtype(0.25)  # one value
            d_val.copy_(torch.from_numpy(cur))
            one = product(cur)
            assert not np.array_equal(one, first)
            i, j = 17, nnz - 5            # two values swapped
            cur[i], cur[j] = cur[j], cur[i]
            d_val.copy_(torch.from_numpy(cur))
            swapped = product(cur)
            assert not np.array_equal(swapped, one)
            cur[nnz // 2] = -cur[nnz // 2]  # one sign
            d_val.copy_(torch.from_numpy(cur))
            assert not np.array_equal(product(cur), swapped)
            cur = rng.uniform(-1, 1, nnz).astype(dtype)  # all of them
            d_val.copy_(torch.from_numpy(cur))
            product(cur)
            d_val.copy_(torch.from_numpy(val))  # and back: the first product again, bit for bit
            assert np.array_equal(product(val), first)
            # the explicit refresh keeps the checksums in step: nothing to do in the next check
            cur = rng.uniform(-1, 1, nnz).astype(dtype)
            d_val.copy_(torch.from_numpy(cur))
            plan.update_values(d_val)
            product(cur)
            plan.destroy()
    # a matrix too small to regroup: row-ordered, reads the caller's values, nothing to check
    rp, col, val = csr_from_lengths(rng.integers(0, 9, 3000), 5000, 7, dtype)
    d = [dev(torch, a) for a in (rp, col, val)]
    plan = capi.Plan(False, capi.SPMV_DEFAULT, np.dtype(dtype), rp.size - 1, 5000, col.size, d[0], col=d[1], val=d[2], checked=True)
    assert not plan.checked and not plan.holds_values
    plan.refresh_if_changed(d[2])
    plan.destroy()
    L = capi.lib()
    assert L.asx_plan_refresh_if_changed(None, None, None) == 7 and L.asx_plan_is_checked(None) == 0
    # values off a 16-byte boundary (a view one element into an allocation): no checksums can be
    # taken, so a kernel asked for by name that would copy them is refused (INVALID_VALUE) ...
    rp, col, val = csr_from_lengths(rng.integers(0, 9, 3000), 5000, 7, dtype)
    d_rp, d_col = dev(torch, rp), dev(torch, col)
    room = torch.zeros(col.size + 1, dtype=torch.float64 if dtype == np.float64 else torch.float32, device="cuda")
    room[1:] = torch.from_numpy(val)
    h = capi.C.c_void_p()
    for alg in (capi.SPMV_SLICED, capi.SPMV_WINDOW):
        assert L.asx_spmv_plan_create_checked(capi.C.byref(h), alg, capi.value_type(np.dtype(dtype)), rp.size - 1, 5000, col.size,
                                              capi._ptr(d_rp), capi._ptr(d_col), capi._ptr(room[1:]), None) == 3
        assert not h.value
    # ... while a window plan that reads them in place takes them as they are
    rp, col, val = W.csr_banded(20000, 4, dtype, 5)
    room = torch.zeros(col.size + 1, dtype=room.dtype, device="cuda")
    room[1:] = torch.from_numpy(val)
    d_rp, d_col = dev(torch, rp), dev(torch, col)
    x = rng.uniform(-1, 1, 20000).astype(dtype)
    plan = capi.Plan(False, capi.SPMV_WINDOW, np.dtype(dtype), 20000, 20000, col.size, d_rp, col=d_col, val=room[1:], checked=True)
    assert plan.info("by_reference") == 1 and not plan.checked
    y = torch.zeros(20000, dtype=room.dtype, device="cuda")
    capi.spmv(d_rp, d_col, room[1:], dev(torch, x), y, 1.0, 0.0, alg=capi.SPMV_WINDOW, plan=plan)
    torch.cuda.synchronize()
    assert_close(y.cpu().numpy(), oracle.spmv(rp, col, val, x, dtype(1.0), dtype(0.0), np.zeros(20000, dtype), 4),
                 spmv_scale(rp, col, val, x, 1.0, 0.0, np.zeros(20000, dtype)), dtype, "values in place off a 16-byte boundary")
    plan.destroy()
