"""ctypes view of the CPU oracle.  TEST INFRASTRUCTURE ONLY.

``Oracle``  -> oracle/liboracle.so, the C restatement (always available once built).
``Ref``     -> oracle/_ref/*.so, the reference's own CPU path compiled from its sources
               (present only where oracle/Makefile's `ref` target has been run; the
               prebuilt files travel with the tree, the sources do not).
Only tests, the smoke check and the benchmark's CPU-baseline leg may import this module.
"""
from __future__ import annotations

import ctypes as C
import os

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
ORACLE_SO = os.path.join(_HERE, "liboracle.so")
REF_SO = os.path.join(_HERE, "_ref", "libalphasparse_ref.so")
REF_HIPHOST_SO = os.path.join(_HERE, "_ref", "libalphasparse_ref_hiphost.so")

i32p, u64p = C.POINTER(C.c_int32), C.POINTER(C.c_uint64)
f32p, f64p = C.POINTER(C.c_float), C.POINTER(C.c_double)


def _p(a, ct):
    return a.ctypes.data_as(C.POINTER(ct))


def _i32(a):
    a = np.ascontiguousarray(a, dtype=np.int32)
    return a


class Oracle:
    def __init__(self, path=ORACLE_SO):
        if not os.path.exists(path):
            raise RuntimeError(f"{path} missing: run `make -C oracle oracle`")
        L = self.L = C.CDLL(path)
        L.orc_partition_rows_by_nnz.argtypes = [i32p, C.c_int32, C.c_int32, i32p]
        L.orc_spmv_csr_f64.argtypes = [C.c_int32, i32p, i32p, f64p, f64p, C.c_double, C.c_double, f64p, C.c_int]
        L.orc_spmv_csr_f32.argtypes = [C.c_int32, i32p, i32p, f32p, f32p, C.c_float, C.c_float, f32p, C.c_int]
        L.orc_spmm_csr_row_f32.argtypes = [C.c_int32, i32p, i32p, f32p, f32p, C.c_int32, C.c_int32,
                                           C.c_float, C.c_float, f32p, C.c_int32, C.c_int]
        L.orc_spmm_csr_row_f64.argtypes = [C.c_int32, i32p, i32p, f64p, f64p, C.c_int32, C.c_int32,
                                           C.c_double, C.c_double, f64p, C.c_int32, C.c_int]
        L.orc_nnz_split_rows.argtypes = [i32p, C.c_int32, C.c_int32, C.c_int32, i32p]
        L.orc_merge_path_search.argtypes = [i32p, C.c_int32, C.c_int32, C.c_int32, i32p, i32p]
        L.orc_loadbalance_nwarps.argtypes = [C.c_int64, C.c_int64, C.c_int64]
        L.orc_loadbalance_nwarps.restype = C.c_int64
        L.orc_loadbalance_partition.argtypes = [i32p, C.c_int32, C.c_int32, C.c_int32, C.c_int32, i32p]
        L.orc_find_rows_counts.argtypes = [i32p, C.c_int32, C.c_int32, C.c_int32, i32p, C.POINTER(C.c_int64)]
        L.orc_csr_adaptive_row_blocks.argtypes = [i32p, C.c_int32, u64p, C.c_size_t]
        L.orc_csr_adaptive_row_blocks.restype = C.c_size_t
        L.orc_coo2csr.argtypes = [i32p, C.c_int32, C.c_int32, i32p]
        L.orc_coo2csr.restype = None
        for name in ("orc_partition_rows_by_nnz", "orc_spmv_csr_f64", "orc_spmv_csr_f32",
                     "orc_spmm_csr_row_f32", "orc_spmm_csr_row_f64", "orc_nnz_split_rows",
                     "orc_merge_path_search", "orc_loadbalance_partition", "orc_find_rows_counts"):
            getattr(L, name).restype = None

    # ---- integer analysis ----
    def partition_rows_by_nnz(self, row_ptr, nthreads):
        row_ptr = _i32(row_ptr)
        m = row_ptr.size - 1
        out = np.empty(nthreads + 1, dtype=np.int32)
        row_end = np.ascontiguousarray(row_ptr[1:])
        self.L.orc_partition_rows_by_nnz(_p(row_end, C.c_int32), m, nthreads, _p(out, C.c_int32))
        return out

    def nnz_split_rows(self, row_ptr, items):
        row_ptr = _i32(row_ptr)
        m, nnz = row_ptr.size - 1, int(row_ptr[-1])
        nseg = (nnz + items - 1) // items
        out = np.empty(nseg + 1, dtype=np.int32)
        self.L.orc_nnz_split_rows(_p(row_ptr, C.c_int32), m, nnz, items, _p(out, C.c_int32))
        return out

    def merge_path_search(self, row_ptr, items):
        row_ptr = _i32(row_ptr)
        m, nnz = row_ptr.size - 1, int(row_ptr[-1])
        nblk = (m + nnz + items - 1) // items
        xs = np.empty(nblk + 1, dtype=np.int32)
        ys = np.empty(nblk + 1, dtype=np.int32)
        self.L.orc_merge_path_search(_p(row_ptr, C.c_int32), m, nnz, items, _p(xs, C.c_int32), _p(ys, C.c_int32))
        return xs, ys

    def loadbalance_nwarps(self, nnz, warp_size, nwarps_base):
        return int(self.L.orc_loadbalance_nwarps(nnz, warp_size, nwarps_base))

    def loadbalance_partition(self, row_ptr, warp_size, nwarps):
        row_ptr = _i32(row_ptr)
        m, nnz = row_ptr.size - 1, int(row_ptr[-1])
        out = np.empty(max(nwarps, 0), dtype=np.int32)
        self.L.orc_loadbalance_partition(_p(row_ptr, C.c_int32), m, nnz, warp_size, nwarps, _p(out, C.c_int32))
        return out

    def find_rows_counts(self, row_ptr, thr1=2, thr2=1024):
        row_ptr = _i32(row_ptr)
        counts = np.zeros(3, dtype=np.int32)
        mid = C.c_int64(0)
        self.L.orc_find_rows_counts(_p(row_ptr, C.c_int32), row_ptr.size - 1, thr1, thr2,
                                    _p(counts, C.c_int32), C.byref(mid))
        return counts, int(mid.value)

    def csr_adaptive_row_blocks(self, row_ptr):
        row_ptr = _i32(row_ptr)
        m = row_ptr.size - 1
        cap = 2 * m + int(row_ptr[-1]) // 1024 + 16
        out = np.zeros(cap, dtype=np.uint64)
        n = self.L.orc_csr_adaptive_row_blocks(_p(row_ptr, C.c_int32), m, _p(out, C.c_uint64), cap)
        assert n <= cap
        return out[:n].copy()

    def coo2csr(self, row_ind, m):
        row_ind = _i32(row_ind)
        out = np.empty(m + 1, dtype=np.int32)
        self.L.orc_coo2csr(_p(row_ind, C.c_int32), row_ind.size, m, _p(out, C.c_int32))
        return out

    # ---- values ----
    def spmv(self, row_ptr, col, val, x, alpha, beta, y, nthreads=1):
        """Returns alpha*A*x + beta*y computed with the reference's rounding sequence."""
        row_ptr, col = _i32(row_ptr), _i32(col)
        m = row_ptr.size - 1
        out = np.array(y, copy=True)
        if val.dtype == np.float64:
            self.L.orc_spmv_csr_f64(m, _p(row_ptr, C.c_int32), _p(col, C.c_int32), _p(val, C.c_double),
                                    _p(x, C.c_double), alpha, beta, _p(out, C.c_double), nthreads)
        elif val.dtype == np.float32:
            self.L.orc_spmv_csr_f32(m, _p(row_ptr, C.c_int32), _p(col, C.c_int32), _p(val, C.c_float),
                                    _p(x, C.c_float), alpha, beta, _p(out, C.c_float), nthreads)
        else:
            raise TypeError(val.dtype)
        return out

    def spmm(self, row_ptr, col, val, B, ncols, alpha, beta, Cm, nthreads=1, ldb=None, ldc=None):
        row_ptr, col = _i32(row_ptr), _i32(col)
        m = row_ptr.size - 1
        ldb = ncols if ldb is None else ldb
        ldc = ncols if ldc is None else ldc
        out = np.array(Cm, copy=True)
        if val.dtype == np.float32:
            self.L.orc_spmm_csr_row_f32(m, _p(row_ptr, C.c_int32), _p(col, C.c_int32), _p(val, C.c_float),
                                        _p(B, C.c_float), ncols, ldb, alpha, beta, _p(out, C.c_float), ldc, nthreads)
        elif val.dtype == np.float64:
            self.L.orc_spmm_csr_row_f64(m, _p(row_ptr, C.c_int32), _p(col, C.c_int32), _p(val, C.c_double),
                                        _p(B, C.c_double), ncols, ldb, alpha, beta, _p(out, C.c_double), ldc, nthreads)
        else:
            raise TypeError(val.dtype)
        return out


class Ref:
    """The reference's own CPU path (compiled from its sources) — present only if built."""

    @staticmethod
    def available():
        return os.path.exists(REF_SO)

    def __init__(self):
        if not os.path.exists(REF_SO):
            raise RuntimeError(f"{REF_SO} missing: run `make -C oracle ref` where the reference is mounted")
        L = self.L = C.CDLL(REF_SO)
        L.ref_partition_rows_by_nnz.argtypes = [i32p, C.c_int32, C.c_int32, i32p]
        L.ref_partition_rows_by_nnz.restype = None
        L.ref_create_csr_f64.argtypes = [C.c_int32, C.c_int32, i32p, i32p, f64p]
        L.ref_create_csr_f64.restype = C.c_void_p
        L.ref_create_csr_f32.argtypes = [C.c_int32, C.c_int32, i32p, i32p, f32p]
        L.ref_create_csr_f32.restype = C.c_void_p
        L.ref_destroy.argtypes = [C.c_void_p]
        L.ref_destroy.restype = None
        L.ref_mv_f64.argtypes = [C.c_void_p, f64p, C.c_double, C.c_double, f64p, C.c_int]
        L.ref_mv_f32.argtypes = [C.c_void_p, f32p, C.c_float, C.c_float, f32p, C.c_int]
        L.ref_mm_row_f32.argtypes = [C.c_void_p, f32p, C.c_int32, C.c_int32, C.c_float, C.c_float, f32p,
                                     C.c_int32, C.c_int]
        L.ref_mm_row_f64.argtypes = [C.c_void_p, f64p, C.c_int32, C.c_int32, C.c_double, C.c_double, f64p,
                                     C.c_int32, C.c_int]
        self.H = None
        if os.path.exists(REF_HIPHOST_SO):
            try:
                H = C.CDLL(REF_HIPHOST_SO)
                H.ref_csr_adaptive_row_blocks.argtypes = [i32p, C.c_int32, u64p, C.c_size_t]
                H.ref_csr_adaptive_row_blocks.restype = C.c_size_t
                self.H = H
            except OSError:
                self.H = None

    def partition_rows_by_nnz(self, row_ptr, nthreads):
        row_ptr = _i32(row_ptr)
        out = np.empty(nthreads + 1, dtype=np.int32)
        row_end = np.ascontiguousarray(row_ptr[1:])
        self.L.ref_partition_rows_by_nnz(_p(row_end, C.c_int32), row_ptr.size - 1, nthreads, _p(out, C.c_int32))
        return out

    def create(self, row_ptr, col, val, n):
        row_ptr, col = _i32(row_ptr), _i32(col)
        m = row_ptr.size - 1
        if val.dtype == np.float64:
            h = self.L.ref_create_csr_f64(m, n, _p(row_ptr, C.c_int32), _p(col, C.c_int32), _p(val, C.c_double))
        else:
            h = self.L.ref_create_csr_f32(m, n, _p(row_ptr, C.c_int32), _p(col, C.c_int32), _p(val, C.c_float))
        if not h:
            raise RuntimeError("reference create_csr failed")
        return h

    def destroy(self, h):
        self.L.ref_destroy(h)

    def mv(self, h, x, alpha, beta, y_inout, nthreads=1):
        if x.dtype == np.float64:
            st = self.L.ref_mv_f64(h, _p(x, C.c_double), alpha, beta, _p(y_inout, C.c_double), nthreads)
        else:
            st = self.L.ref_mv_f32(h, _p(x, C.c_float), alpha, beta, _p(y_inout, C.c_float), nthreads)
        if st != 0:
            raise RuntimeError(f"reference mv status {st}")

    def mm(self, h, B, ncols, alpha, beta, C_inout, nthreads=1, ldb=None, ldc=None):
        ldb = ncols if ldb is None else ldb
        ldc = ncols if ldc is None else ldc
        if B.dtype == np.float32:
            st = self.L.ref_mm_row_f32(h, _p(B, C.c_float), ncols, ldb, alpha, beta, _p(C_inout, C.c_float), ldc, nthreads)
        else:
            st = self.L.ref_mm_row_f64(h, _p(B, C.c_double), ncols, ldb, alpha, beta, _p(C_inout, C.c_double), ldc, nthreads)
        if st != 0:
            raise RuntimeError(f"reference mm status {st}")

    def spmv(self, row_ptr, col, val, x, alpha, beta, y, nthreads=1):
        h = self.create(row_ptr, col, val, x.size)
        out = np.array(y, copy=True)
        self.mv(h, x, alpha, beta, out, nthreads)
        self.destroy(h)
        return out

    def spmm(self, row_ptr, col, val, B, ncols, alpha, beta, Cm, nthreads=1):
        h = self.create(row_ptr, col, val, B.size // ncols)
        out = np.array(Cm, copy=True)
        self.mm(h, B, ncols, alpha, beta, out, nthreads)
        self.destroy(h)
        return out

    def csr_adaptive_row_blocks(self, row_ptr):
        if self.H is None:
            raise RuntimeError("hip-host reference library not loadable")
        row_ptr = _i32(row_ptr)
        m = row_ptr.size - 1
        cap = 2 * m + int(row_ptr[-1]) // 1024 + 16
        out = np.zeros(cap, dtype=np.uint64)
        n = self.H.ref_csr_adaptive_row_blocks(_p(row_ptr, C.c_int32), m, _p(out, C.c_uint64), cap)
        return out[:n].copy()
