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


def _run_case(tmp_path, op, dtype, rp, col, val, x, y, ncols, alg, alpha, beta, analysis):
    d = tmp_path / f"{op}_{np.dtype(dtype).name}_{alg}_{analysis}"
    d.mkdir()
    for name, a in (("row_ptr", rp), ("col", col), ("val", val), ("x", x), ("y", y)):
        np.ascontiguousarray(a).tofile(d / f"{name}.bin")
    tag = "f64" if np.dtype(dtype) == np.float64 else "f32"
    n = x.size // ncols
    (d / "meta.txt").write_text(f"{op} {tag} {rp.size - 1} {n} {col.size} {ncols} {alg} {alpha!r} {beta!r} {analysis}\n")
    r = subprocess.run([EXE, str(d)], capture_output=True, text=True, timeout=120)
    assert r.returncode == 0, (r.returncode, r.stdout, r.stderr)
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
