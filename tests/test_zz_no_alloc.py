"""asx_spmv_csr_f64_noalloc: the plan-less fp64 SpMV whose workspace is an array inside the
library.  Through the C-ABI, against asx_spmv_csr_f64 with a caller's workspace (same kernels:
the results must agree bit for bit), on two calls in a row, the second with a smaller input."""
import ctypes as C

import numpy as np
import pytest

from conftest import csr_from_lengths

pytestmark = pytest.mark.gpu


def test_no_alloc_entry_point_matches_the_workspace_one():
    import torch
    from library_amd import capi
    L = capi.lib()
    rng = np.random.default_rng(404)
    dev = lambda a: torch.from_numpy(np.ascontiguousarray(a)).cuda()
    stream = capi._stream()
    cap = L.asx_spmv_noalloc_max_workspace()
    assert cap == 4 << 20
    # first a larger matrix with long rows, rows cut by tile boundaries and empty rows, then a smaller one
    shapes = [np.r_[np.minimum(rng.zipf(1.7, 60000), 3000), 25000, np.zeros(50, int), rng.integers(0, 6, 4000)],
              np.r_[rng.integers(0, 9, 700), 5000]]
    for alg in (capi.SPMV_DEFAULT, capi.SPMV_MERGE, capi.SPMV_STREAM, capi.SPMV_VECTOR):
        for lens in shapes:
            n = 40000
            rp, col, val = csr_from_lengths(lens, n, 7, np.float64)
            m, nnz = rp.size - 1, col.size
            x = rng.uniform(-1, 1, n)
            y0 = rng.uniform(-1, 1, m)
            d_rp, d_col, d_val, d_x = dev(rp), dev(col), dev(val), dev(x)
            for alpha, beta in ((1.5, 0.5), (1.0, 0.0)):
                want = dev(y0)
                capi.spmv(d_rp, d_col, d_val, d_x, want, alpha, beta, alg=alg)
                got = dev(y0)
                rc = L.asx_spmv_csr_f64_noalloc(alg, m, n, nnz, alpha, capi._ptr(d_rp), capi._ptr(d_col), capi._ptr(d_val),
                                                capi._ptr(d_x), beta, capi._ptr(got), stream)
                assert rc == 0, (alg, rc)
                torch.cuda.synchronize()
                assert torch.equal(got, want), (alg, m, alpha, beta)
    # captured into a HIP graph (the array's address is known by now: asx_device_info and the eager
    # calls above looked it up) and replayed with eager work and synchronisations in between
    assert L.asx_device_info(None, None) == 0
    alg, alpha, beta, n = capi.SPMV_DEFAULT, 1.5, 0.5, 40000  # the flat kernel: split points and carries in the array
    rp, col, val = csr_from_lengths(shapes[0], n, 7, np.float64)
    m, nnz = rp.size - 1, col.size
    x, y0 = rng.uniform(-1, 1, n), rng.uniform(-1, 1, m)
    d_rp, d_col, d_val, d_x = dev(rp), dev(col), dev(val), dev(x)
    want = dev(y0)
    capi.spmv(d_rp, d_col, d_val, d_x, want, alpha, beta, alg=alg)
    torch.cuda.synchronize()
    eager = want.cpu().numpy()
    y = dev(y0)
    side = torch.cuda.Stream()
    graph = torch.cuda.CUDAGraph()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        with torch.cuda.graph(graph, stream=side):
            rc = L.asx_spmv_csr_f64_noalloc(alg, m, n, nnz, alpha, capi._ptr(d_rp), capi._ptr(d_col), capi._ptr(d_val),
                                            capi._ptr(d_x), beta, capi._ptr(y), capi._stream())
            assert rc == 0
    torch.cuda.synchronize()
    for rep in range(3):
        y.copy_(dev(y0))
        assert np.isfinite((d_x * 2.0).sum().item())
        graph.replay()
        torch.cuda.synchronize()
        assert np.array_equal(y.cpu().numpy(), eager), f"replay {rep}"
    del graph
    # too large for the array: refused before anything is launched or read
    y = dev(np.zeros(4))
    rc = L.asx_spmv_csr_f64_noalloc(capi.SPMV_DEFAULT, 4, 4, 2**31 - 1, 1.0, capi._ptr(y), capi._ptr(y), capi._ptr(y),
                                    capi._ptr(y), 0.0, capi._ptr(y), stream)
    assert rc == 10
    assert L.asx_spmv_workspace_bytes(capi.SPMV_DEFAULT, capi.R_64F, 4, 2**31 - 1) > cap
    assert L.asx_spmv_csr_f64_noalloc(1, 4, 4, 4, 1.0, None, None, None, None, 0.0, None, stream) == 6  # COO id
    assert L.asx_spmv_csr_f64_noalloc(0, -1, 4, 4, 1.0, None, None, None, None, 0.0, None, stream) == 10
