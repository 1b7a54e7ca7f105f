"""ctypes view of the C-ABI in include/alphasparse_amd.h (used by tests and the benchmark).

Device buffers are torch tensors; only their ``data_ptr()`` crosses into the library.  There
is no fallback: if the shared library is missing, loading raises.
"""
from __future__ import annotations

import ctypes as C
import os

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libalphasparse_amd.so")

R_32F, R_64F = 0, 1
SPMV_DEFAULT, SPMV_STREAM, SPMV_VECTOR, SPMV_MERGE, SPMV_FLAT, SPMV_SLICED, SPMV_WINDOW = 0, 3, 6, 9, 15, 101, 102
SPMM_DEFAULT, SPMM_ROW, SPMM_MERGE, SPMM_BLOCKED = 0, 5, 7, 10

STATUS = {0: "SUCCESS", 1: "NOT_INITIALIZED", 2: "ALLOC_FAILED", 3: "INVALID_VALUE",
          4: "EXECUTION_FAILED", 5: "INTERNAL_ERROR", 6: "NOT_SUPPORTED", 7: "INVALID_POINTER",
          8: "INVALID_HANDLE", 9: "INVALID_KERNEL_PARAM", 10: "INVALID_SIZE"}

# every symbol include/alphasparse_amd.h (and, last, include/alphasparse_amd_bench.h) declares
EXPORTS = [
    "asx_version", "asx_device_info", "asx_row_length_histogram", "asx_partition_rows_by_nnz",
    "asx_nnz_split_rows", "asx_merge_path_search", "asx_loadbalance_nwarps",
    "asx_loadbalance_partition", "asx_csr_adaptive_row_blocks", "asx_coo2csr", "asx_coo_sort", "asx_csr_transpose", "asx_csr_rebase",
    "asx_dense_transpose", "asx_mtx_read", "asx_host_free", "asx_spmv_plan_create",
    "asx_plan_update_values", "asx_plan_holds_values", "asx_spmv_plan_create_checked", "asx_plan_refresh_if_changed",
    "asx_plan_is_checked", "asx_plan_info", "asx_plan_create",
    "asx_spmm_plan_create", "asx_plan_block_stats", "asx_plan_destroy", "asx_plan_alg", "asx_kernel_name", "asx_plan_workspace_bytes", "asx_plan_histogram",
    "asx_plan_release_scratch", "asx_plan_own_scratch_bytes", "asx_plan_export",
    "asx_spmv_resolve_alg", "asx_spmv_workspace_bytes", "asx_spmv_csr_f64", "asx_spmv_csr_f32",
    "asx_spmv_csr_f64_noalloc", "asx_spmv_noalloc_max_workspace",
    "asx_spmm_resolve_alg", "asx_spmm_workspace_bytes", "asx_spmm_csr_f32", "asx_spmm_csr_f64",
    "asx_copy_bytes", "asx_gather_lines",
]


class AsxError(RuntimeError):
    def __init__(self, code, where):
        super().__init__(f"{where}: status {code} ({STATUS.get(code, '?')})")
        self.code = code


_lib = None


def lib():
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise RuntimeError(f"{LIB_PATH} is not built (python -m library_amd.build); there is no fallback path")
    L = C.CDLL(LIB_PATH)
    vp, i32, i64, sz = C.c_void_p, C.c_int32, C.c_int64, C.c_size_t
    L.asx_version.restype = C.c_char_p
    L.asx_device_info.argtypes = [C.POINTER(C.c_int), C.POINTER(C.c_int)]
    L.asx_row_length_histogram.argtypes = [vp, i32, vp, vp, vp]
    L.asx_partition_rows_by_nnz.argtypes = [vp, i32, i32, vp, vp]
    L.asx_nnz_split_rows.argtypes = [vp, i32, i32, i32, vp, vp]
    L.asx_merge_path_search.argtypes = [vp, i32, i32, i32, vp, vp, vp]
    L.asx_loadbalance_nwarps.argtypes = [i64, i64, i64]
    L.asx_loadbalance_nwarps.restype = i64
    L.asx_loadbalance_partition.argtypes = [vp, i32, i32, i32, i32, vp, vp]
    L.asx_csr_adaptive_row_blocks.argtypes = [vp, i32, vp, sz, C.POINTER(sz)]
    L.asx_coo2csr.argtypes = [vp, i32, i32, vp, vp]
    L.asx_coo_sort.argtypes = [C.c_int, vp, vp, vp, i32, vp]
    L.asx_csr_transpose.argtypes = [C.c_int, i32, i32, i32, i32, vp, vp, vp, vp, vp, vp, vp]
    L.asx_csr_rebase.argtypes = [i32, i32, i32, vp, vp, vp, vp, vp]
    L.asx_dense_transpose.argtypes = [C.c_int, C.c_int64, C.c_int64, vp, C.c_int64, vp, C.c_int64, vp]
    L.asx_mtx_read.argtypes = [C.c_char_p, C.c_int] + [C.POINTER(i32)] * 3 + [C.POINTER(vp)] * 3
    L.asx_host_free.argtypes = [vp]
    L.asx_host_free.restype = None
    L.asx_plan_create.argtypes = [C.POINTER(vp), C.c_int, C.c_int, C.c_int, i32, i32, i32, vp, i32, vp]
    L.asx_spmm_plan_create.argtypes = [C.POINTER(vp), C.c_int, C.c_int, i32, i32, i32, vp, vp, vp, i32, vp]
    L.asx_spmv_plan_create.argtypes = [C.POINTER(vp), C.c_int, C.c_int, i32, i32, i32, vp, vp, vp, vp]
    L.asx_spmv_plan_create_checked.argtypes = [C.POINTER(vp), C.c_int, C.c_int, i32, i32, i32, vp, vp, vp, vp]
    L.asx_plan_refresh_if_changed.argtypes = [vp, vp, vp]
    L.asx_plan_is_checked.argtypes = [vp]
    L.asx_plan_update_values.argtypes = [vp, vp, vp]
    L.asx_plan_holds_values.argtypes = [vp]
    L.asx_plan_block_stats.argtypes = [vp, C.POINTER(i64), C.POINTER(C.c_double)]
    L.asx_plan_destroy.argtypes = [vp]
    L.asx_plan_alg.argtypes = [vp]
    L.asx_kernel_name.argtypes = [C.c_int, C.c_int]
    L.asx_kernel_name.restype = C.c_char_p
    L.asx_plan_workspace_bytes.argtypes = [vp]
    L.asx_plan_workspace_bytes.restype = sz
    L.asx_plan_histogram.argtypes = [vp, vp, vp]
    L.asx_plan_release_scratch.argtypes = [vp]
    L.asx_plan_own_scratch_bytes.argtypes = [vp]
    L.asx_plan_own_scratch_bytes.restype = sz
    L.asx_plan_export.argtypes = [vp, C.c_int, vp, sz, C.POINTER(sz), vp]
    L.asx_spmv_resolve_alg.argtypes = [C.c_int, i32, i32]
    L.asx_spmv_workspace_bytes.argtypes = [C.c_int, C.c_int, i32, i32]
    L.asx_spmv_workspace_bytes.restype = sz
    L.asx_spmv_csr_f64.argtypes = [vp, C.c_int, i32, i32, i32, C.c_double, vp, vp, vp, vp, C.c_double, vp, vp, sz, vp]
    L.asx_spmv_csr_f32.argtypes = [vp, C.c_int, i32, i32, i32, C.c_float, vp, vp, vp, vp, C.c_float, vp, vp, sz, vp]
    L.asx_spmv_csr_f64_noalloc.argtypes = [C.c_int, i32, i32, i32, C.c_double, vp, vp, vp, vp, C.c_double, vp, vp]
    L.asx_spmv_noalloc_max_workspace.argtypes = []
    L.asx_spmv_noalloc_max_workspace.restype = sz
    L.asx_spmm_resolve_alg.argtypes = [C.c_int, i32, i32, i32]
    L.asx_spmm_workspace_bytes.argtypes = [C.c_int, C.c_int, i32, i32, i32]
    L.asx_spmm_workspace_bytes.restype = sz
    L.asx_spmm_csr_f32.argtypes = [vp, C.c_int, i32, i32, i32, i32, C.c_float, vp, vp, vp, vp, i64, C.c_float, vp, i64, vp, sz, vp]
    L.asx_spmm_csr_f64.argtypes = [vp, C.c_int, i32, i32, i32, i32, C.c_double, vp, vp, vp, vp, i64, C.c_double, vp, i64, vp, sz, vp]
    L.asx_copy_bytes.argtypes = [vp, vp, sz, vp]
    L.asx_plan_info.argtypes = [vp, C.c_int]
    L.asx_plan_info.restype = i64
    L.asx_gather_lines.argtypes = [vp, sz, C.c_int, C.c_int, vp, C.POINTER(C.c_int), vp]
    _lib = L
    return L


def _check(code, where):
    if code != 0:
        raise AsxError(code, where)


def _ptr(t):
    return None if t is None else C.c_void_p(t.data_ptr())


def _stream():
    import torch
    return C.c_void_p(torch.cuda.current_stream().cuda_stream)


def value_type(dtype):
    import torch
    return {torch.float32: R_32F, torch.float64: R_64F, np.dtype(np.float32): R_32F,
            np.dtype(np.float64): R_64F}[dtype]


# ------------------------------------------------------------------------------ analysis
def row_length_histogram(row_ptr):
    import torch
    m = row_ptr.numel() - 1
    hist = torch.empty(33, dtype=torch.int64, device=row_ptr.device)
    stats = torch.empty(4, dtype=torch.int64, device=row_ptr.device)
    _check(lib().asx_row_length_histogram(_ptr(row_ptr), m, _ptr(hist), _ptr(stats), _stream()), "asx_row_length_histogram")
    return hist, stats


def partition_rows_by_nnz(row_ptr, nparts):
    import torch
    m = row_ptr.numel() - 1
    out = torch.empty(nparts + 1, dtype=torch.int32, device=row_ptr.device)
    _check(lib().asx_partition_rows_by_nnz(_ptr(row_ptr), m, nparts, _ptr(out), _stream()), "asx_partition_rows_by_nnz")
    return out


def nnz_split_rows(row_ptr, nnz, items):
    import torch
    m = row_ptr.numel() - 1
    nseg = (nnz + items - 1) // items
    out = torch.empty(nseg + 1, dtype=torch.int32, device=row_ptr.device)
    _check(lib().asx_nnz_split_rows(_ptr(row_ptr), m, nnz, items, _ptr(out), _stream()), "asx_nnz_split_rows")
    return out


def merge_path_search(row_ptr, nnz, items):
    import torch
    m = row_ptr.numel() - 1
    nblk = (m + nnz + items - 1) // items
    xs = torch.empty(nblk + 1, dtype=torch.int32, device=row_ptr.device)
    ys = torch.empty(nblk + 1, dtype=torch.int32, device=row_ptr.device)
    _check(lib().asx_merge_path_search(_ptr(row_ptr), m, nnz, items, _ptr(xs), _ptr(ys), _stream()), "asx_merge_path_search")
    return xs, ys


def loadbalance_nwarps(nnz, warp_size, nwarps_base):
    return int(lib().asx_loadbalance_nwarps(nnz, warp_size, nwarps_base))


def loadbalance_partition(row_ptr, nnz, warp_size, nwarps):
    import torch
    m = row_ptr.numel() - 1
    out = torch.empty(max(nwarps, 1), dtype=torch.int32, device=row_ptr.device)
    _check(lib().asx_loadbalance_partition(_ptr(row_ptr), m, nnz, warp_size, nwarps, _ptr(out), _stream()), "asx_loadbalance_partition")
    return out[:nwarps]


def coo2csr(row_ind, m):
    import torch
    out = torch.empty(m + 1, dtype=torch.int32, device=row_ind.device)
    _check(lib().asx_coo2csr(_ptr(row_ind), row_ind.numel(), m, _ptr(out), _stream()), "asx_coo2csr")
    return out


def coo_sort(row_ind, col_ind, val):
    _check(lib().asx_coo_sort(value_type(val.dtype), _ptr(row_ind), _ptr(col_ind), _ptr(val), row_ind.numel(), _stream()),
           "asx_coo_sort")


def csr_transpose(row_ptr, col, val, n, idx_base=0):
    """A (m x n CSR, device tensors) -> (row_ptr_t, col_t, val_t) of A^T, zero-based."""
    import torch
    m = row_ptr.numel() - 1
    nnz = col.numel()
    rp = torch.empty(n + 1, dtype=torch.int32, device=row_ptr.device)
    ct = torch.empty(nnz, dtype=torch.int32, device=row_ptr.device)
    vt = torch.empty(nnz, dtype=val.dtype, device=row_ptr.device)
    _check(lib().asx_csr_transpose(value_type(val.dtype), m, n, nnz, idx_base, _ptr(row_ptr), _ptr(col), _ptr(val),
                                   _ptr(rp), _ptr(ct), _ptr(vt), _stream()), "asx_csr_transpose")
    return rp, ct, vt


def csr_rebase(row_ptr, col, idx_base):
    import torch
    rp = torch.empty_like(row_ptr)
    c = torch.empty_like(col)
    _check(lib().asx_csr_rebase(row_ptr.numel() - 1, col.numel(), idx_base, _ptr(row_ptr), _ptr(col), _ptr(rp), _ptr(c),
                                _stream()), "asx_csr_rebase")
    return rp, c


def dense_transpose(a, rows, cols, ld_in, out, ld_out):
    """out[c*ld_out + r] = a[r*ld_in + c] on flat device tensors."""
    _check(lib().asx_dense_transpose(value_type(a.dtype), rows, cols, _ptr(a), ld_in, _ptr(out), ld_out, _stream()),
           "asx_dense_transpose")


def mtx_read(path, dtype):
    """MatrixMarket coordinate file -> (m, n, row, col, val) as numpy arrays (host; no GPU needed)."""
    import numpy as np
    dtype = np.dtype(dtype)
    m, n, nnz = C.c_int32(), C.c_int32(), C.c_int32()
    row, col, val = C.c_void_p(), C.c_void_p(), C.c_void_p()
    _check(lib().asx_mtx_read(str(path).encode(), R_64F if dtype == np.float64 else R_32F, C.byref(m), C.byref(n),
                              C.byref(nnz), C.byref(row), C.byref(col), C.byref(val)), "asx_mtx_read")
    try:
        k = nnz.value
        r = np.ctypeslib.as_array(C.cast(row, C.POINTER(C.c_int32)), (k,)).copy() if k else np.empty(0, np.int32)
        c = np.ctypeslib.as_array(C.cast(col, C.POINTER(C.c_int32)), (k,)).copy() if k else np.empty(0, np.int32)
        ct = C.c_double if dtype == np.float64 else C.c_float
        v = np.ctypeslib.as_array(C.cast(val, C.POINTER(ct)), (k,)).copy() if k else np.empty(0, dtype)
    finally:
        for p in (row, col, val):
            lib().asx_host_free(p)
    return m.value, n.value, r, c, v


def csr_adaptive_row_blocks(row_ptr_host):
    """Host routine on a host (numpy int32) row_ptr."""
    rp = np.ascontiguousarray(row_ptr_host, dtype=np.int32)
    m = rp.size - 1
    n = C.c_size_t(0)
    _check(lib().asx_csr_adaptive_row_blocks(rp.ctypes.data_as(C.c_void_p), m, None, 0, C.byref(n)), "asx_csr_adaptive_row_blocks")
    out = np.zeros(n.value, dtype=np.uint64)
    n2 = C.c_size_t(0)
    _check(lib().asx_csr_adaptive_row_blocks(rp.ctypes.data_as(C.c_void_p), m, out.ctypes.data_as(C.c_void_p), out.size, C.byref(n2)), "asx_csr_adaptive_row_blocks")
    assert n2.value == n.value
    return out


# ------------------------------------------------------------------------------ plans
class Plan:
    def __init__(self, is_spmm, alg, dtype, m, n, nnz, row_ptr, ncols=1, col=None, val=None, checked=False):
        h = C.c_void_p()
        if checked:
            _check(lib().asx_spmv_plan_create_checked(C.byref(h), alg, value_type(dtype), m, n, nnz, _ptr(row_ptr), _ptr(col),
                                                      _ptr(val), _stream()), "asx_spmv_plan_create_checked")
        elif is_spmm and col is not None and val is not None:
            _check(lib().asx_spmm_plan_create(C.byref(h), alg, value_type(dtype), m, n, nnz, _ptr(row_ptr), _ptr(col),
                                              _ptr(val), ncols, _stream()), "asx_spmm_plan_create")
        elif not is_spmm and col is not None and val is not None:
            _check(lib().asx_spmv_plan_create(C.byref(h), alg, value_type(dtype), m, n, nnz, _ptr(row_ptr), _ptr(col),
                                              _ptr(val), _stream()), "asx_spmv_plan_create")
        else:
            _check(lib().asx_plan_create(C.byref(h), int(is_spmm), alg, value_type(dtype), m, n, nnz, _ptr(row_ptr),
                                         ncols, _stream()), "asx_plan_create")
        self.h = h
        self._keep = (row_ptr, col, val)  # keep alive

    @classmethod
    def adopt(cls, handle):
        """A view of a plan made through the C-ABI directly; destroying it stays with the caller."""
        p = cls.__new__(cls)
        p.h = handle
        p._keep = ()
        p._owned = False
        return p

    def block_stats(self):
        n, f = C.c_int64(0), C.c_double(0.0)
        _check(lib().asx_plan_block_stats(self.h, C.byref(n), C.byref(f)), "asx_plan_block_stats")
        return n.value, f.value

    @property
    def alg(self):
        return lib().asx_plan_alg(self.h)

    @property
    def workspace_bytes(self):
        return lib().asx_plan_workspace_bytes(self.h)

    def histogram(self):
        hist = np.zeros(33, dtype=np.int64)
        stats = np.zeros(4, dtype=np.int64)
        _check(lib().asx_plan_histogram(self.h, hist.ctypes.data_as(C.c_void_p), stats.ctypes.data_as(C.c_void_p)), "asx_plan_histogram")
        return hist, stats

    @property
    def checked(self):
        return bool(lib().asx_plan_is_checked(self.h))

    def refresh_if_changed(self, val):
        """asx_plan_refresh_if_changed: checksums of val, and the plan's copy refreshed on the device where they differ."""
        _check(lib().asx_plan_refresh_if_changed(self.h, _ptr(val), _stream()), "asx_plan_refresh_if_changed")

    def update_values(self, val):
        _check(lib().asx_plan_update_values(self.h, _ptr(val), _stream()), "asx_plan_update_values")
        self._keep = (self._keep[0], self._keep[1], val)

    INFO = {"tiles": 0, "slices": 1, "partial_sums": 2, "rows_per_wave": 3, "rows_per_block": 4, "bands": 5,
            "chains": 6, "carry_pass": 7, "row_blocks": 8, "steps": 9, "width": 10, "workgroups": 11, "pieces": 12,
            "stacked_rows": 13, "by_reference": 14}
    # asx_plan_export: name -> (id, element type; "value" = the plan's value type)
    ARRAYS = {"val": (0, "value"), "cf": (1, np.uint16), "perm": (2, np.int32), "tile_words": (3, np.int32),
              "workgroups": (4, np.int32), "partial_rows": (5, np.uint16), "ranges": (6, np.int32),
              "step_ptr": (7, np.int32), "steps": (8, np.int32), "blocks": (9, np.int32), "pieces": (10, np.int32),
              "wg_pieces": (11, np.int32)}

    def export(self, name, value_dtype=None):
        """One array of a sliced or window plan as a flat numpy array (asx_plan_export)."""
        what, dt = self.ARRAYS[name]
        dt = np.dtype(value_dtype if dt == "value" else dt)
        nbytes = C.c_size_t(0)
        _check(lib().asx_plan_export(self.h, what, None, 0, C.byref(nbytes), _stream()), "asx_plan_export")
        out = np.empty(nbytes.value // dt.itemsize, dtype=dt)
        if nbytes.value:
            _check(lib().asx_plan_export(self.h, what, out.ctypes.data_as(C.c_void_p), out.nbytes, C.byref(nbytes),
                                         _stream()), "asx_plan_export")
        return out

    def release_scratch(self):
        _check(lib().asx_plan_release_scratch(self.h), "asx_plan_release_scratch")

    def info(self, what):
        """A figure of a sliced or window plan (asx_plan_info); -1 where it does not apply."""
        return int(lib().asx_plan_info(self.h, self.INFO[what]))

    @property
    def holds_values(self):
        return bool(lib().asx_plan_holds_values(self.h))

    def destroy(self):
        if self.h and getattr(self, "_owned", True):
            lib().asx_plan_destroy(self.h)
        self.h = None

    def __del__(self):
        try:
            self.destroy()
        except Exception:
            pass


def _workspace(nbytes, device):
    import torch
    return torch.empty(max(int(nbytes), 256), dtype=torch.uint8, device=device)


# ------------------------------------------------------------------------------ SpMV / SpMM
def spmv(row_ptr, col, val, x, y, alpha, beta, alg=SPMV_DEFAULT, plan=None, workspace=None, n=None):
    """y <- alpha*A*x + beta*y in place (torch CUDA tensors).  Returns y.  workspace=None allocates
    what the call needs; workspace=False passes none (a sliced or window plan then uses its own buffer)."""
    m = row_ptr.numel() - 1
    n = x.numel() if n is None else n
    nnz = col.numel()
    vt = value_type(val.dtype)
    need = plan.workspace_bytes if plan is not None else lib().asx_spmv_workspace_bytes(alg, vt, m, nnz)
    if workspace is None:
        workspace = _workspace(need, val.device)
    ws_ptr, ws_bytes = (None, 0) if workspace is False else (_ptr(workspace), workspace.numel() * workspace.element_size())
    fn = lib().asx_spmv_csr_f64 if vt == R_64F else lib().asx_spmv_csr_f32
    _check(fn(plan.h if plan is not None else None, alg, m, n, nnz, alpha, _ptr(row_ptr), _ptr(col), _ptr(val),
              _ptr(x), beta, _ptr(y), ws_ptr, ws_bytes, _stream()), "asx_spmv_csr")
    return y


def spmm(row_ptr, col, val, B, Cm, ncols, alpha, beta, alg=SPMM_DEFAULT, plan=None, workspace=None,
         ldb=None, ldc=None, k=None):
    """C <- alpha*A*B + beta*C in place; B (k x ncols), C (m x ncols) row-major torch CUDA tensors."""
    m = row_ptr.numel() - 1
    nnz = col.numel()
    ldb = ncols if ldb is None else ldb
    ldc = ncols if ldc is None else ldc
    k = B.numel() // ldb if k is None else k
    vt = value_type(val.dtype)
    need = plan.workspace_bytes if plan is not None else lib().asx_spmm_workspace_bytes(alg, vt, m, nnz, ncols)
    if workspace is None:
        workspace = _workspace(need, val.device)
    fn = lib().asx_spmm_csr_f64 if vt == R_64F else lib().asx_spmm_csr_f32
    _check(fn(plan.h if plan is not None else None, alg, m, k, nnz, ncols, alpha, _ptr(row_ptr), _ptr(col), _ptr(val),
              _ptr(B), ldb, beta, _ptr(Cm), ldc, _ptr(workspace), workspace.numel(), _stream()), "asx_spmm_csr")
    return Cm
