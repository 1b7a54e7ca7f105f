"""Deterministic synthetic workloads for the CSR SpMV / SpMM benchmark configurations.

Thin ctypes view over ``csrc/workload_gen.c`` (C + OpenMP).  Arrays are numpy, host side;
callers move them to the device.  ``CONFIGS`` names the five benchmark shapes.
"""
from __future__ import annotations

import ctypes as C
import os
from dataclasses import dataclass, field

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "libasx_workloads.so")
_lib = None

# stream ids: one per generated array, so arrays are independent of each other
S_VAL, S_COL, S_LEN, S_EMPTY, S_X, S_Y, S_B, S_C = range(1, 9)


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(_LIB_PATH):
            raise RuntimeError(
                f"{_LIB_PATH} is not built; run `python -c 'import __graft_entry__ as g; g.build()'`")
        L = C.CDLL(_LIB_PATH)
        i32p, f32p, f64p = (C.POINTER(C.c_int32), C.POINTER(C.c_float), C.POINTER(C.c_double))
        u64 = C.c_uint64
        L.wl_fill_uniform_f64.argtypes = [f64p, C.c_int64, C.c_double, C.c_double, u64, u64]
        L.wl_fill_uniform_f32.argtypes = [f32p, C.c_int64, C.c_float, C.c_float, u64, u64]
        L.wl_banded_row_ptr.argtypes = [C.c_int32, C.c_int32, i32p]
        L.wl_banded_row_ptr.restype = C.c_int64
        L.wl_banded_cols.argtypes = [C.c_int32, C.c_int32, i32p, i32p]
        L.wl_fixed_row_ptr.argtypes = [C.c_int32, C.c_int32, i32p]
        L.wl_fixed_row_ptr.restype = C.c_int64
        L.wl_random_cols.argtypes = [C.c_int32, C.c_int32, i32p, i32p, u64, u64]
        L.wl_zipf_row_ptr.argtypes = [C.c_int32, C.c_int32, C.c_double, C.c_int32, C.c_double, i32p,
                                      u64, u64, u64]
        L.wl_zipf_row_ptr.restype = C.c_int64
        L.wl_stencil5_row_ptr.argtypes = [C.c_int32, C.c_int32, i32p]
        L.wl_stencil5_row_ptr.restype = C.c_int64
        L.wl_stencil5_fill_f64.argtypes = [C.c_int32, C.c_int32, i32p, i32p, f64p]
        L.wl_stencil7_row_ptr.argtypes = [C.c_int32, C.c_int32, C.c_int32, i32p]
        L.wl_stencil7_row_ptr.restype = C.c_int64
        L.wl_stencil7_fill_f64.argtypes = [C.c_int32, C.c_int32, C.c_int32, i32p, i32p, f64p]
        for f in (L.wl_fill_uniform_f64, L.wl_fill_uniform_f32, L.wl_banded_cols, L.wl_random_cols,
                  L.wl_stencil5_fill_f64, L.wl_stencil7_fill_f64):
            f.restype = None
        _lib = L
    return _lib


def _p(a, ct):
    return a.ctypes.data_as(C.POINTER(ct))


def uniform(n, dtype, lo, hi, seed, stream):
    out = np.empty(int(n), dtype=dtype)
    if out.dtype == np.float64:
        lib().wl_fill_uniform_f64(_p(out, C.c_double), out.size, lo, hi, seed, stream)
    elif out.dtype == np.float32:
        lib().wl_fill_uniform_f32(_p(out, C.c_float), out.size, lo, hi, seed, stream)
    else:
        raise TypeError(dtype)
    return out


@dataclass
class Workload:
    name: str
    kind: str              # "spmv" | "spmm"
    dtype: np.dtype
    m: int
    n: int                 # columns of A
    nnz: int
    row_ptr: np.ndarray
    col: np.ndarray
    val: np.ndarray
    alpha: float
    beta: float
    x: np.ndarray = None   # spmv: length n ; spmm: B, n x ncols row-major
    y: np.ndarray = None   # spmv: length m ; spmm: C, m x ncols row-major
    ncols: int = 1
    meta: dict = field(default_factory=dict)

    @property
    def flops(self):
        return 2 * self.nnz * self.ncols

    def bytes_algorithmic(self, y_twice=None):
        """vals + col_idx + row_ptr + x/B read + y/C write (+ read when beta != 0)."""
        sv = self.dtype.itemsize
        ymul = 2 if (self.beta != 0 if y_twice is None else y_twice) else 1
        return (self.nnz * (sv + 4) + (self.m + 1) * 4 + self.n * self.ncols * sv
                + self.m * self.ncols * sv * ymul)


def csr_banded(m, half_bw, dtype, seed=0):
    row_ptr = np.empty(m + 1, dtype=np.int32)
    nnz = lib().wl_banded_row_ptr(m, half_bw, _p(row_ptr, C.c_int32))
    col = np.empty(nnz, dtype=np.int32)
    lib().wl_banded_cols(m, half_bw, _p(row_ptr, C.c_int32), _p(col, C.c_int32))
    val = uniform(nnz, dtype, -1.0, 1.0, seed, S_VAL)
    return row_ptr, col, val


def csr_fixed(m, n, k, dtype, seed=0):
    row_ptr = np.empty(m + 1, dtype=np.int32)
    nnz = lib().wl_fixed_row_ptr(m, k, _p(row_ptr, C.c_int32))
    if nnz < 0:
        raise ValueError("nnz does not fit int32")
    col = np.empty(nnz, dtype=np.int32)
    lib().wl_random_cols(m, n, _p(row_ptr, C.c_int32), _p(col, C.c_int32), seed, S_COL)
    val = uniform(nnz, dtype, -1.0, 1.0, seed, S_VAL)
    return row_ptr, col, val


def csr_zipf(m, n, alpha10, scale, max_len, empty_frac, dtype, seed=0):
    row_ptr = np.empty(m + 1, dtype=np.int32)
    nnz = lib().wl_zipf_row_ptr(m, alpha10, scale, max_len, empty_frac, _p(row_ptr, C.c_int32), seed,
                                S_LEN, S_EMPTY)
    if nnz < 0:
        raise ValueError("nnz does not fit int32")
    col = np.empty(nnz, dtype=np.int32)
    lib().wl_random_cols(m, n, _p(row_ptr, C.c_int32), _p(col, C.c_int32), seed, S_COL)
    val = uniform(nnz, dtype, -1.0, 1.0, seed, S_VAL)
    return row_ptr, col, val


def csr_stencil5(nx, ny):
    m = nx * ny
    row_ptr = np.empty(m + 1, dtype=np.int32)
    nnz = lib().wl_stencil5_row_ptr(nx, ny, _p(row_ptr, C.c_int32))
    col = np.empty(nnz, dtype=np.int32)
    val = np.empty(nnz, dtype=np.float64)
    lib().wl_stencil5_fill_f64(nx, ny, _p(row_ptr, C.c_int32), _p(col, C.c_int32), _p(val, C.c_double))
    return row_ptr, col, val


def csr_stencil7(nx, ny, nz):
    m = nx * ny * nz
    row_ptr = np.empty(m + 1, dtype=np.int32)
    nnz = lib().wl_stencil7_row_ptr(nx, ny, nz, _p(row_ptr, C.c_int32))
    col = np.empty(nnz, dtype=np.int32)
    val = np.empty(nnz, dtype=np.float64)
    lib().wl_stencil7_fill_f64(nx, ny, nz, _p(row_ptr, C.c_int32), _p(col, C.c_int32), _p(val, C.c_double))
    return row_ptr, col, val


# Scale applied to Zipf(2.2) draws so that the realised mean row length of the SpMM
# configuration is 16.0 +- 0.1 after rounding and clipping to [1, 50000].
SPMM_ZIPF_SCALE = 4.76


def _spmv(name, dtype, rp, col, val, n, alpha, beta, seed, xlo=-1.0, **meta):
    m = rp.size - 1
    x = uniform(n, dtype, xlo, 1.0, seed, S_X)
    y = uniform(m, dtype, -1.0, 1.0, seed, S_Y)
    return Workload(name, "spmv", np.dtype(dtype), m, n, int(rp[-1]), rp, col, val, alpha, beta, x, y,
                    1, meta)


def banded_f64(m=1280, half_bw=9, seed=0):
    """Config 1: 1280x1280 banded +-9, fp64, y = 1.0*A*x + 0.0*y."""
    rp, col, val = csr_banded(m, half_bw, np.float64, seed)
    return _spmv("banded_f64", np.float64, rp, col, val, m, 1.0, 0.0, seed)


def uniform16_f32(m=1 << 20, k=16, seed=0):
    """Config 2: m x m, exactly k uniform sorted distinct columns per row, fp32, alpha=1.5 beta=0.5."""
    rp, col, val = csr_fixed(m, m, k, np.float32, seed)
    return _spmv("uniform16_f32", np.float32, rp, col, val, m, 1.5, 0.5, seed)


def uniform16_f64(m=1 << 20, k=16, seed=0):
    """Not a BASELINE configuration: config 2's matrix in fp64 (y = 1.5*A*x + 0.5*y)."""
    rp, col, val = csr_fixed(m, m, k, np.float64, seed)
    return _spmv("uniform16_f64", np.float64, rp, col, val, m, 1.5, 0.5, seed)


def powerlaw_f64(m=1 << 22, max_len=200000, empty_frac=0.01, seed=0, alpha=1.0, beta=0.0):
    """Config 3: Zipf(2.0) row lengths clipped to [1, max_len], 1% empty rows, fp64."""
    rp, col, val = csr_zipf(m, m, 20, 1.0, min(max_len, m), empty_frac, np.float64, seed)
    return _spmv("powerlaw_f64", np.float64, rp, col, val, m, alpha, beta, seed)


def stencil5_f64(nx=4096, ny=4096, seed=0):
    """Config 4: 2D 5-point Laplacian, fp64, x ~ U(0,1), y = 1.0*A*x + 0.0*y."""
    rp, col, val = csr_stencil5(nx, ny)
    return _spmv("stencil5_f64", np.float64, rp, col, val, nx * ny, 1.0, 0.0, seed, xlo=0.0)


def stencil7_f64(nx=256, ny=256, nz=256, seed=0):
    """Not a BASELINE configuration: 3D 7-point Laplacian in natural order (planes of nx * ny points),
    fp64, x ~ U(0,1), y = 1.5*A*x + 0.5*y."""
    rp, col, val = csr_stencil7(nx, ny, nz)
    return _spmv("stencil7_f64", np.float64, rp, col, val, nx * ny * nz, 1.5, 0.5, seed, xlo=0.0)


def spmm_zipf_f32(m=1 << 20, ncols=64, max_len=50000, seed=0, scale=SPMM_ZIPF_SCALE):
    """Config 5: C = 1.0*A*B + 1.0*C, A m x m Zipf(2.2)-shaped rows (mean 16), B, C m x ncols fp32."""
    rp, col, val = csr_zipf(m, m, 22, scale, min(max_len, m), 0.0, np.float32, seed)
    B = uniform(m * ncols, np.float32, -1.0, 1.0, seed, S_B)
    Cm = uniform(m * ncols, np.float32, -1.0, 1.0, seed, S_C)
    return Workload("spmm_zipf_f32", "spmm", np.dtype(np.float32), m, m, int(rp[-1]), rp, col, val, 1.0,
                    1.0, B, Cm, ncols, {"scale": scale})


def spmm_banded_f32(m=1 << 20, half_bw=32, ncols=64, seed=0):
    """Not a BASELINE configuration: a banded A (dense 16x4 blocks) for the blocked MFMA SpMM."""
    rp, col, val = csr_banded(m, half_bw, np.float32, seed)
    B = uniform(m * ncols, np.float32, -1.0, 1.0, seed, S_B)
    Cm = uniform(m * ncols, np.float32, -1.0, 1.0, seed, S_C)
    return Workload("spmm_banded_f32", "spmm", np.dtype(np.float32), m, m, int(rp[-1]), rp, col, val, 1.0,
                    1.0, B, Cm, ncols, {"half_bw": half_bw})


CONFIGS = {
    "banded_f64": banded_f64,
    "uniform16_f32": uniform16_f32,
    "powerlaw_f64": powerlaw_f64,
    "stencil5_f64": stencil5_f64,
    "spmm_zipf_f32": spmm_zipf_f32,
    "spmm_banded_f32": spmm_banded_f32,
    "uniform16_f64": uniform16_f64,
    "stencil7_f64": stencil7_f64,
}
