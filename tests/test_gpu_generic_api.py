"""The generic C++ API (alphasparseSpMV / alphasparseSpMM with the reference's signatures),
exercised by a C++ caller written like the reference's own GPU tests, checked against the CPU
oracle.  The caller is built by the repository's build step (tests/cxx/generic_api_caller)."""
import os
import subprocess

import numpy as np
import pytest

from conftest import ROOT, csr_from_lengths
from test_gpu_parity import assert_close, spmm_scale, spmv_scale

pytestmark = pytest.mark.gpu
EXE = os.path.join(ROOT, "tests", "cxx", "generic_api_caller")


def _run_case(tmp_path, op, dtype, rp, col, val, x, y, ncols, alg, alpha, beta, analysis, variant=(0, 0, 0, 0, 0),
              n=None, val2=None, env=None, x2=None, tag="", said=None):
    """variant = (trans_a, idx_base, col_major_b, col_major_c, trans_b); n = columns of A."""
    d = tmp_path / f"{op}_{np.dtype(dtype).name}_{alg}_{analysis}_{''.join(map(str, variant))}{'_env' if env else ''}{tag}"
    d.mkdir()
    for name, a in (("row_ptr", rp), ("col", col), ("val", val), ("x", x), ("y", y)):
        np.ascontiguousarray(a).tofile(d / f"{name}.bin")
    if val2 is not None:  # analysis == 2: values written over A's after the first products; 3: a second descriptor's
        np.ascontiguousarray(val2).tofile(d / "val2.bin")
    if x2 is not None:  # analysis == 4: the second stream's input vector
        np.ascontiguousarray(x2).tofile(d / "x2.bin")
    tag = "f64" if np.dtype(dtype) == np.float64 else "f32"
    if n is None:
        n = x.size // ncols
    (d / "meta.txt").write_text(f"{op} {tag} {rp.size - 1} {n} {col.size} {ncols} {alg} {alpha!r} {beta!r} {analysis}\n"
                                + " ".join(map(str, variant)) + "\n")
    r = subprocess.run([EXE, str(d)], capture_output=True, text=True, timeout=120,
                       env=dict(os.environ, **env) if env else None)
    assert r.returncode == 0, (r.returncode, r.stdout, r.stderr)
    if said is not None:
        said.append(r.stdout)
    return np.fromfile(d / "out.bin", dtype=dtype)


def test_selftest():
    assert os.path.exists(EXE), "build step did not produce the C++ caller"
    r = subprocess.run([EXE, "--selftest"], capture_output=True, text=True, timeout=120)
    assert r.returncode == 0 and "selftest ok" in r.stdout, (r.returncode, r.stdout, r.stderr)


@pytest.mark.parametrize("dtype", [np.float64, np.float32])
def test_spmv_through_generic_api(tmp_path, oracle, dtype):
    rng = np.random.default_rng(41)
    lens = np.r_[np.minimum(rng.zipf(1.8, 20000), 4000), 30000, np.zeros(40, int)]
    rp, col, val = csr_from_lengths(lens, 40000, 42, dtype)
    x = rng.uniform(-1, 1, 40000).astype(dtype)
    y0 = rng.uniform(-1, 1, lens.size).astype(dtype)
    alpha, beta = 2.1, 3.2  # the reference's GPU test scalars (hip/test/level2/spmv_csr_r_f64_test.hip:49)
    ref = oracle.spmv(rp, col, val, x, dtype(alpha), dtype(beta), y0, 4)
    scale = spmv_scale(rp, col, val, x, alpha, beta, y0)
    # the algorithm ids the reference's test loops over, plus DEFAULT
    for alg, analysis in ((0, 0), (0, 1), (6, 0), (7, 0), (9, 1), (11, 0), (12, 1), (13, 0), (16, 0), (2, 0), (17, 0)):
        got = _run_case(tmp_path, "spmv", dtype, rp, col, val, x, y0, 1, alg, alpha, beta, analysis)
        assert_close(got, ref, scale, dtype, f"alg {alg} analysis {analysis}")


def test_spmm_through_generic_api(tmp_path, oracle):
    rng = np.random.default_rng(43)
    lens = np.r_[np.minimum(rng.zipf(2.0, 5000) * 3, 2000), 6000]
    rp, col, val = csr_from_lengths(lens, 7000, 44, np.float32)
    n = 64
    B = rng.uniform(-1, 1, 7000 * n).astype(np.float32)
    C0 = rng.uniform(-1, 1, lens.size * n).astype(np.float32)
    alpha, beta = 2.0, 3.0  # hip/test/level3/spmm_csr_row_r_f32_test.hip:45-46
    ref = oracle.spmm(rp, col, val, B, n, alpha, beta, C0, 4)
    scale = spmm_scale(rp, col, val, B, n, alpha, beta, C0)
    for alg, analysis in ((0, 0), (0, 1), (5, 0), (6, 0), (7, 1), (8, 0), (9, 0), (10, 1)):
        got = _run_case(tmp_path, "spmm", np.float32, rp, col, val, B, C0, n, alg, alpha, beta, analysis)
        assert_close(got, ref, scale, np.float32, f"spmm alg {alg} analysis {analysis}")


def _transpose_csr(rp, col, val, n):
    """A^T with the stored elements of each row in ascending row of A, duplicates in stored order."""
    rows = np.repeat(np.arange(rp.size - 1, dtype=np.int32), np.diff(rp))
    order = np.argsort(col, kind="stable")
    rp_t = np.zeros(n + 1, dtype=np.int32)
    np.cumsum(np.bincount(col, minlength=n), out=rp_t[1:])
    return rp_t, rows[order].astype(np.int32), val[order]


@pytest.mark.parametrize("dtype", [np.float64, np.float32])
def test_spmv_transpose_and_one_based(tmp_path, oracle, dtype):
    """opA = TRANSPOSE and idx_base = ONE against the oracle run on the explicitly transposed /
    rebased matrix (a rectangular one, so a mix-up of rows and columns cannot pass)."""
    rng = np.random.default_rng(51)
    lens = np.r_[np.minimum(rng.zipf(1.7, 9000), 3000), 12000, np.zeros(25, int)]
    m, n = lens.size, 15000
    rp, col, val = csr_from_lengths(lens, n, 52, dtype)
    alpha, beta = 2.1, 3.2
    x_n = rng.uniform(-1, 1, n).astype(dtype)
    y_m = rng.uniform(-1, 1, m).astype(dtype)
    x_m = rng.uniform(-1, 1, m).astype(dtype)
    y_n = rng.uniform(-1, 1, n).astype(dtype)
    ref_n = oracle.spmv(rp, col, val, x_n, dtype(alpha), dtype(beta), y_m, 4)
    rp_t, col_t, val_t = _transpose_csr(rp, col, val, n)
    ref_t = oracle.spmv(rp_t, col_t, val_t, x_m, dtype(alpha), dtype(beta), y_n, 4)
    scale_n = spmv_scale(rp, col, val, x_n, alpha, beta, y_m)
    scale_t = spmv_scale(rp_t, col_t, val_t, x_m, alpha, beta, y_n)
    for alg, analysis in ((0, 0), (0, 1), (9, 1), (6, 0), (3, 1)):
        for base in (0, 1):
            if base:
                got = _run_case(tmp_path, "spmv", dtype, rp + 1, col + 1, val, x_n, y_m, 1, alg, alpha, beta, analysis,
                                (0, 1, 0, 0, 0), n=n)
                assert_close(got, ref_n, scale_n, dtype, f"one-based alg {alg} analysis {analysis}")
            got = _run_case(tmp_path, "spmv", dtype, rp + base, col + base, val, x_m, y_n, 1, alg, alpha, beta, analysis,
                            (1, base, 0, 0, 0), n=n)
            assert_close(got, ref_t, scale_t, dtype, f"transpose base {base} alg {alg} analysis {analysis}")


@pytest.mark.parametrize("dtype", [np.float32, np.float64])
def test_spmm_layouts_and_ops(tmp_path, oracle, dtype):
    """Column-major B / C, opB = TRANSPOSE, opA = TRANSPOSE and one-based A: every variant must give
    the row-major, non-transposed result of the same product."""
    rng = np.random.default_rng(53)
    lens = np.r_[np.minimum(rng.zipf(2.0, 1500) * 2, 700), 2000, np.zeros(9, int)]
    m, k, ncols = lens.size, 2100, 40
    rp, col, val = csr_from_lengths(lens, k, 54, dtype)
    alpha, beta = 2.0, 3.0
    B = rng.uniform(-1, 1, (k, ncols)).astype(dtype)
    C0 = rng.uniform(-1, 1, (m, ncols)).astype(dtype)
    ref = oracle.spmm(rp, col, val, B.ravel(), ncols, alpha, beta, C0.ravel(), 4).reshape(m, ncols)
    scale = spmm_scale(rp, col, val, B.ravel(), ncols, alpha, beta, C0.ravel()).reshape(m, ncols)
    for alg, analysis, (cb, cc, tb) in ((0, 0, (1, 0, 0)), (0, 1, (0, 1, 0)), (7, 0, (1, 1, 0)), (5, 0, (0, 0, 1)),
                                        (0, 1, (1, 1, 1)), (10, 1, (1, 1, 0))):
        # memory of B: op(B) = B.  Row-major without opB and column-major with opB hold B itself
        b_mem = B if cb == tb else B.T
        c_mem = C0.T if cc else C0
        got = _run_case(tmp_path, "spmm", dtype, rp, col, val, np.ascontiguousarray(b_mem).ravel(),
                        np.ascontiguousarray(c_mem).ravel(), ncols, alg, alpha, beta, analysis, (0, 0, cb, cc, tb), n=k)
        got = got.reshape(ncols, m).T if cc else got.reshape(m, ncols)
        assert_close(got.ravel(), ref.ravel(), scale.ravel(), dtype, f"alg {alg} analysis {analysis} cb{cb} cc{cc} tb{tb}")
    # beta = 0 with a column-major C full of NaN: C must not be read
    nanC = np.full((ncols, m), np.nan, dtype=dtype)
    ref0 = oracle.spmm(rp, col, val, B.ravel(), ncols, alpha, 0.0, np.zeros(m * ncols, dtype), 4)
    got = _run_case(tmp_path, "spmm", dtype, rp, col, val, B.ravel(), nanC.ravel(), ncols, 0, alpha, 0.0, 0,
                    (0, 0, 0, 1, 0), n=k)
    assert_close(got.reshape(ncols, m).T.ravel(), ref0, scale.ravel(), dtype, "beta 0, column-major C")
    # opA = TRANSPOSE (one-based): C (k x ncols) = alpha * A^T * Bm (m x ncols) + beta * C
    rp_t, col_t, val_t = _transpose_csr(rp, col, val, k)
    Bm = rng.uniform(-1, 1, (m, ncols)).astype(dtype)
    Ck = rng.uniform(-1, 1, (k, ncols)).astype(dtype)
    ref_t = oracle.spmm(rp_t, col_t, val_t, Bm.ravel(), ncols, alpha, beta, Ck.ravel(), 4)
    scale_t = spmm_scale(rp_t, col_t, val_t, Bm.ravel(), ncols, alpha, beta, Ck.ravel())
    for alg, analysis, cc in ((0, 0, 0), (0, 1, 1), (5, 1, 0)):
        c_mem = Ck.T if cc else Ck
        got = _run_case(tmp_path, "spmm", dtype, rp + 1, col + 1, val, Bm.ravel(), np.ascontiguousarray(c_mem).ravel(),
                        ncols, alg, alpha, beta, analysis, (1, 1, 0, cc, 0), n=k)
        got = got.reshape(ncols, k).T if cc else got.reshape(k, ncols)
        assert_close(got.ravel(), ref_t, scale_t, dtype, f"opA=T alg {alg} analysis {analysis} cc{cc}")


CLI = os.path.join(ROOT, "library_amd", "bin", "alphasparse_amd_cli")


def test_cli_on_matrixmarket_files(tmp_path):
    """The command-line driver end to end: MatrixMarket file -> device sort -> CSR -> generic API,
    with its own --check (double-precision host loop) for SpMV and SpMM variants."""
    import scipy.io
    import scipy.sparse as sp
    assert os.path.exists(CLI), "build step did not produce the command-line driver"
    A = sp.random(3000, 2500, density=0.004, random_state=3, format="coo", dtype=np.float64)
    gen = tmp_path / "general.mtx"
    scipy.io.mmwrite(str(gen), A, precision=17)
    S = sp.random(1500, 1500, density=0.01, random_state=4, format="coo", dtype=np.float64)
    sym = tmp_path / "sym.mtx"
    scipy.io.mmwrite(str(sym), sp.tril(S) + sp.tril(S, -1).T, symmetry="symmetric", precision=17)
    metrics = tmp_path / "metrics.csv"
    runs = [
        [f"--data-file={gen}", "--data-type=D", "--check", "--iter=3", "--warmup=1", f"--metrics-file={metrics}"],
        [f"--data-file={gen}", "--data-type=S", "--check", "--iter=2", "--warmup=1", "--alg_num=9", "--analysis"],
        [f"--data-file={gen}", "--data-type=D", "--check", "--iter=2", "--warmup=1", "--transA=T", "--alg_num=0"],
        [f"--data-file={sym}", "--op=spmm", "--data-type=S", "--check", "--iter=2", "--warmup=1", "--cols=40"],
        [f"--data-file={gen}", "--op=spmm", "--data-type=D", "--check", "--iter=2", "--warmup=1", "--cols=9",
         "--layout=C", "--transA=T", "--alg_num=0", "--analysis"],
    ]
    for args in runs:
        r = subprocess.run([CLI, *args], capture_output=True, text=True, timeout=120)
        assert r.returncode == 0, (args, r.returncode, r.stdout[-2000:], r.stderr[-2000:])
        assert "correct: require" in r.stdout and "error: require" not in r.stdout, r.stdout
        assert "alphasparse alg" in r.stdout
    lines = metrics.read_text().strip().splitlines()
    assert len(lines) == 8 and all(len(l.split(",")) == 11 for l in lines)  # DEFAULT + the reference's 7 ids
    r = subprocess.run([CLI, f"--data-file={tmp_path / 'none.mtx'}"], capture_output=True, text=True, timeout=60)
    assert r.returncode == 4


def test_spmv_analysis_on_a_scattered_matrix(tmp_path, oracle):
    """A matrix DEFAULT's analysis takes the column-sliced kernel for (4 M scattered stored elements,
    x of 8 MiB): the buffer alphasparseSpMV_bufferSize reported must do, the result must match, also
    for opA = TRANSPOSE, and after the caller overwrites A's values and calls the analysis again the
    product must be the one of the new values."""
    from library_amd import workloads as W
    rp, col, val = W.csr_zipf(1 << 20, 1 << 20, 20, 1.0, 5000, 0.01, np.float64, 3)
    n = 1 << 20
    assert col.size >= 1 << 22
    rng = np.random.default_rng(61)
    x = rng.uniform(-1, 1, n)
    y0 = rng.uniform(-1, 1, rp.size - 1)
    alpha, beta = 2.1, 3.2
    ref = oracle.spmv(rp, col, val, x, alpha, beta, y0, 8)
    scale = spmv_scale(rp, col, val, x, alpha, beta, y0)
    got = _run_case(tmp_path, "spmv", np.float64, rp, col, val, x, y0, 1, 0, alpha, beta, 1)
    assert_close(got, ref, scale, np.float64, "DEFAULT with analysis")
    val2 = rng.uniform(-1, 1, val.size)
    got = _run_case(tmp_path, "spmv", np.float64, rp, col, val, x, y0, 1, 0, alpha, beta, 2, val2=val2)
    assert_close(got, oracle.spmv(rp, col, val2, x, alpha, beta, y0, 8), spmv_scale(rp, col, val2, x, alpha, beta, y0),
                 np.float64, "DEFAULT, values changed, analysis called again")
    # two descriptors that share row offsets and columns, each with its own values (analysis = 3):
    # out2.bin is the second descriptor's product, out.bin the first one's, computed after it
    got = _run_case(tmp_path, "spmv", np.float64, rp, col, val, x, y0, 1, 0, alpha, beta, 3, val2=val2)
    assert_close(got, ref, scale, np.float64, "DEFAULT, first of two descriptors sharing row_ptr")
    got2 = np.fromfile(next(tmp_path.glob("spmv_float64_0_3_*")) / "out2.bin", dtype=np.float64)
    assert_close(got2, oracle.spmv(rp, col, val2, x, alpha, beta, y0, 8), spmv_scale(rp, col, val2, x, alpha, beta, y0),
                 np.float64, "DEFAULT, second of two descriptors sharing row_ptr")
    rp_t, col_t, val_t = _transpose_csr(rp, col, val, n)
    ref_t = oracle.spmv(rp_t, col_t, val_t, y0, alpha, beta, x, 8)
    got = _run_case(tmp_path, "spmv", np.float64, rp, col, val, y0, x, 1, 0, alpha, beta, 1, (1, 0, 0, 0, 0), n=n)
    assert_close(got, ref_t, spmv_scale(rp_t, col_t, val_t, y0, alpha, beta, x), np.float64, "transpose, DEFAULT with analysis")


def test_two_streams_share_one_analysed_descriptor(tmp_path, oracle):
    """Two handles, each on a stream of its own, call alphasparseSpMV on one analysed descriptor at
    the same time, each with a buffer of its own sized by alphasparseSpMV_bufferSize after the
    analysis (analysis = 4 in the caller program): both products must be the oracle's.  On the
    scattered matrix the analysis keeps column slices, whose per-call partial sums then live in the
    callers' buffers; on the band matrix with long rows it keeps row blocks with a carry pass."""
    from library_amd import workloads as W
    rng = np.random.default_rng(67)
    rp, col, val = W.csr_zipf(1 << 20, 1 << 20, 20, 1.0, 5000, 0.01, np.float64, 9)
    cases = [("scattered", rp, col, val, 1 << 20)]
    m, offs = 100000, np.arange(-60, 61)  # a band of 121 diagonals, a fifth of it stored: rows of about 24
    cols = np.arange(m)[:, None] + offs[None, :]
    mask = (rng.random(cols.shape) < 0.2) & (cols >= 0) & (cols < m)
    rp = np.zeros(m + 1, np.int32)
    np.cumsum(mask.sum(1), out=rp[1:])
    col = cols[mask].astype(np.int32)
    cases.append(("band", rp, col, rng.uniform(-1, 1, col.size), m))
    for name, rp, col, val, n in cases:
        assert col.size >= 1 << 21, name
        x = rng.uniform(-1, 1, n)
        x2 = rng.uniform(-1, 1, n)
        y0 = rng.uniform(-1, 1, rp.size - 1)
        alpha, beta = 2.1, 3.2
        got = _run_case(tmp_path, "spmv", np.float64, rp, col, val, x, y0, 1, 0, alpha, beta, 4, x2=x2, tag=name)
        assert_close(got, oracle.spmv(rp, col, val, x, alpha, beta, y0, 8), spmv_scale(rp, col, val, x, alpha, beta, y0),
                     np.float64, f"{name}: first stream")
        got2 = np.fromfile(next(tmp_path.glob(f"spmv_float64_0_4_*{name}")) / "out2.bin", dtype=np.float64)
        assert_close(got2, oracle.spmv(rp, col, val, x2, alpha, beta, y0, 8), spmv_scale(rp, col, val, x2, alpha, beta, y0),
                     np.float64, f"{name}: second stream")


def test_analysis_on_first_use(tmp_path, oracle):
    """A caller that never calls alphasparseSpMV_analysis / alphasparseSpMM_preprocess (the reference's
    own test loops do not) gets kept analysis from its first call on.  SpMV by default: the full
    analysis (column slices on this matrix) with a copy of the values that every call checks against
    the caller's values by checksum, so that values changed in place between two calls are picked up
    without a word from the caller; ALPHASPARSE_AMD_AUTO_ANALYSIS=structure: only analysis that reads
    the caller's values in every call (a row-ordered kernel's split points); =1: the full one,
    unchecked; =0: none.  The caller program prints the kept kernel and checks that the descriptor
    ends up analysed or not."""
    from library_amd import workloads as W
    rp, col, val = W.csr_zipf(1 << 20, 1 << 20, 20, 1.0, 5000, 0.01, np.float64, 5)
    n = 1 << 20
    rng = np.random.default_rng(71)
    x = rng.uniform(-1, 1, n)
    y0 = rng.uniform(-1, 1, rp.size - 1)
    ref, scale = oracle.spmv(rp, col, val, x, 2.1, 3.2, y0, 8), spmv_scale(rp, col, val, x, 2.1, 3.2, y0)
    for env, kernels in ((None, ("kernel sliced",)), ({"ALPHASPARSE_AMD_AUTO_ANALYSIS": "structure"}, ("kernel flat", "kernel merge")),
                         ({"ALPHASPARSE_AMD_AUTO_ANALYSIS": "1"}, ("kernel sliced",)),
                         ({"ALPHASPARSE_AMD_AUTO_ANALYSIS": "0"}, ("kernel none",))):
        said = []
        if env is None and "ALPHASPARSE_AMD_AUTO_ANALYSIS" in os.environ:
            env = {"ALPHASPARSE_AMD_AUTO_ANALYSIS": "checked"}
        got = _run_case(tmp_path, "spmv", np.float64, rp, col, val, x, y0, 1, 0, 2.1, 3.2, 0, env=env, said=said,
                        tag="" if env is None else "_" + list(env.values())[0])
        assert_close(got, ref, scale, np.float64, f"SpMV, analysis on first use, {env}")
        assert any(k in said[0] for k in kernels), (env, said[0])
    # values changed in place between calls, no analysis call: a few of them, all of them, two of
    # them swapped, one sign flipped
    few = val.copy()
    few[rng.integers(0, val.size, 5)] *= 3.0
    swapped = val.copy()
    i, j = 12345, val.size - 7
    swapped[i], swapped[j] = val[j], val[i]
    sign = val.copy()
    sign[val.size // 2] = -sign[val.size // 2]
    for name, val2 in (("few", few), ("all", rng.uniform(-1, 1, val.size)), ("swapped", swapped), ("sign", sign)):
        for env in (None, {"ALPHASPARSE_AMD_AUTO_ANALYSIS": "structure"}):
            if env is None and "ALPHASPARSE_AMD_AUTO_ANALYSIS" in os.environ:
                env = {"ALPHASPARSE_AMD_AUTO_ANALYSIS": "checked"}
            said = []
            got = _run_case(tmp_path, "spmv", np.float64, rp, col, val, x, y0, 1, 0, 2.1, 3.2, 5, env=env, said=said, val2=val2,
                            tag=f"_{name}" + ("" if env is None else "_" + list(env.values())[0]))
            ref2, scale2 = oracle.spmv(rp, col, val2, x, 2.1, 3.2, y0, 8), spmv_scale(rp, col, val2, x, 2.1, 3.2, y0)
            assert_close(got, ref2, scale2, np.float64, f"values changed in place ({name}), no analysis call, {env}")
            if name in ("swapped", "sign"):  # the change is one the tolerance alone would not show
                assert not np.array_equal(got, _run_case(tmp_path, "spmv", np.float64, rp, col, val, x, y0, 1, 0, 2.1, 3.2, 0, env=env,
                                                         tag=f"_{name}_before" + ("" if env is None else "_s")))
            assert ("kernel sliced" in said[0]) == (env is None or env["ALPHASPARSE_AMD_AUTO_ANALYSIS"] == "checked"), said[0]
    from test_gpu_parity import _block_structured
    m, k, nc = 700, 640, 64
    rp, col, val = _block_structured(rng, m, k, np.float32)
    B = rng.uniform(-1, 1, k * nc).astype(np.float32)
    C0 = rng.uniform(-1, 1, m * nc).astype(np.float32)
    ref, scale = oracle.spmm(rp, col, val, B, nc, 2.0, 3.0, C0, 4), spmm_scale(rp, col, val, B, nc, 2.0, 3.0, C0)
    for env, kernel in ((None, "kernel merge"), ({"ALPHASPARSE_AMD_AUTO_ANALYSIS": "1"}, "kernel blocked")):
        said = []
        got = _run_case(tmp_path, "spmm", np.float32, rp, col, val, B, C0, nc, 0, 2.0, 3.0, 0, env=env, said=said,
                        tag="" if env is None else "_full")
        assert_close(got, ref, scale, np.float32, f"SpMM, analysis on first use, {env}")
        assert kernel in said[0], (env, said[0])


def test_spmm_blocked_values_changed_after_preprocess(tmp_path, oracle):
    """ALPHASPARSE_SPMM_CSR_ALG6 keeps a blocked copy of A's values: after the caller overwrites the
    values and calls alphasparseSpMM_preprocess again, the product is the one of the new values."""
    from test_gpu_parity import _block_structured
    rng = np.random.default_rng(67)
    m, k, n = 700, 640, 64
    rp, col, val = _block_structured(rng, m, k, np.float32)
    B = rng.uniform(-1, 1, k * n).astype(np.float32)
    C0 = rng.uniform(-1, 1, m * n).astype(np.float32)
    val2 = rng.uniform(-1, 1, val.size).astype(np.float32)
    got = _run_case(tmp_path, "spmm", np.float32, rp, col, val, B, C0, n, 10, 2.0, 3.0, 2, val2=val2)
    assert_close(got, oracle.spmm(rp, col, val2, B, n, 2.0, 3.0, C0, 4), spmm_scale(rp, col, val2, B, n, 2.0, 3.0, C0),
                 np.float32, "ALG6, values changed, preprocess called again")


def test_cli_on_the_reference_matrix():
    """matrix_test/mhd1280b.mtx of the reference (kept as tests/golden/mhd1280b.mtx), run the way the
    reference's drivers are run: every listed algorithm, with --check, in both precisions."""
    mtx = os.path.join(ROOT, "tests", "golden", "mhd1280b.mtx")
    for args in (["--data-type=D", "--check", "--iter=5", "--warmup=2"],
                 ["--data-type=S", "--check", "--iter=5", "--warmup=2", "--analysis"],
                 ["--op=spmm", "--data-type=S", "--check", "--iter=3", "--warmup=1", "--cols=64"],
                 ["--op=spmm", "--data-type=D", "--check", "--iter=3", "--warmup=1", "--cols=17", "--layout=C"]):
        r = subprocess.run([CLI, f"--data-file={mtx}", *args], capture_output=True, text=True, timeout=120)
        assert r.returncode == 0, (args, r.returncode, r.stdout[-2000:], r.stderr[-2000:])
        assert "Dimensions: 1280 x 1280, NNZ: 22778" in r.stdout
        assert "correct: require" in r.stdout and "error: require" not in r.stdout, r.stdout
