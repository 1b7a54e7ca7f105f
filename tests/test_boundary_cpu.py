"""Host-side checks that need no GPU: the shared library loads, exports every C-ABI symbol
the header declares and the C++ entry points of the generic API under the reference's mangled
names; host-only logic (algorithm mapping, workspace sizes, descriptor checks, the host row-block
routine) behaves as documented."""
import ctypes as C
import os
import re
import subprocess

import numpy as np
import pytest

from conftest import ROOT, analysis_shapes, row_ptr_from_lengths
from library_amd import capi

# C++-mangled names a caller compiled against the reference headers links to (Itanium ABI)
MANGLED = [
    "_Z10initHandlePP20alphasparse_handle_s",
    "_Z20alphasparseGetHandlePP20alphasparse_handle_s",
    "_Z26alphasparse_destory_handleP20alphasparse_handle_s",
    "_Z22alphasparseCreateDnVecPP24_alphasparse_dnvec_descrlPv19alphasparseDataType",
    "_Z22alphasparseCreateDnMatPP24_alphasparse_dnmat_descrlllPv19alphasparseDataType18alphasparseOrder_t",
    "_Z26alphasparseSpMV_bufferSizeP20alphasparse_handle_s22alphasparseOperation_tPKvP22_alphasparseSpMatDescrP24_alphasparse_dnvec_descrS3_S7_19alphasparseDataType20alphasparseSpMVAlg_tPm",
    "_Z24alphasparseSpMV_analysisP20alphasparse_handle_s22alphasparseOperation_tP22_alphasparseSpMatDescr20alphasparseSpMVAlg_t",
    "_Z15alphasparseSpMVP20alphasparse_handle_s22alphasparseOperation_tPKvP22_alphasparseSpMatDescrP24_alphasparse_dnvec_descrS3_S7_19alphasparseDataType20alphasparseSpMVAlg_tPv",
    "_Z21alphasparseSpMV_clearP20alphasparse_handle_s20alphasparseSpMVAlg_t",
    "_Z26alphasparseSpMM_bufferSizeP20alphasparse_handle_s22alphasparseOperation_tS1_PKvP22_alphasparseSpMatDescrP24_alphasparse_dnmat_descrS3_S7_19alphasparseDataType20alphasparseSpMMAlg_tPm",
    "_Z26alphasparseSpMM_preprocessP20alphasparse_handle_s22alphasparseOperation_tS1_PKvP22_alphasparseSpMatDescrP24_alphasparse_dnmat_descrS3_S7_19alphasparseDataType20alphasparseSpMMAlg_tPm",
    "_Z16alphasparse_spmvP20alphasparse_handle_s22alphasparseOperation_tPKvP22_alphasparseSpMatDescrP24_alphasparse_dnvec_descrS3_S7_22alphasparse_datatype_t26alphasparse_dcu_spmv_alg_tPmPv",
    "_Z15alphasparseSpMMP20alphasparse_handle_s22alphasparseOperation_tS1_PKvP22_alphasparseSpMatDescrP24_alphasparse_dnmat_descrS3_S7_19alphasparseDataType20alphasparseSpMMAlg_tPv",
]


@pytest.fixture(scope="module")
def lib():
    if not os.path.exists(capi.LIB_PATH):
        from library_amd import build
        build.build_library()
    return capi.lib()


def test_header_symbols_are_exported(lib):
    header = open(os.path.join(ROOT, "include", "alphasparse_amd.h")).read()
    header += open(os.path.join(ROOT, "include", "alphasparse_amd_bench.h")).read()
    declared = sorted(set(re.findall(r"\b(asx_[a-z0-9_]+)\s*\(", header)))
    assert declared, "no declarations found"
    assert sorted(capi.EXPORTS) == declared  # the ctypes view covers the whole header
    for name in declared:
        assert hasattr(lib, name), name


def test_generic_api_mangled_names(lib):
    out = subprocess.run(["nm", "-D", "--defined-only", capi.LIB_PATH], check=True, capture_output=True, text=True).stdout
    exported = {line.split()[-1] for line in out.splitlines() if line.strip()}
    for name in MANGLED:
        assert name in exported, name


def test_nothing_else_is_exported(lib):
    """The drop-in library exports the C-ABI, the generic API's C++ names (those a caller compiled
    against the reference's headers links to, plus what the alphasparseCreateCsr<T> template and
    the descriptor destructors resolve to) and nothing else: no launcher, no helper, no kernel stub."""
    out = subprocess.run(["nm", "-D", "--defined-only", capi.LIB_PATH], check=True, capture_output=True, text=True).stdout
    exported = {line.split()[-1] for line in out.splitlines() if line.strip()}
    also = {
        "_Z27alphasparseCreateCsrUntypedPP22_alphasparseSpMatDescrlllPiS2_Pv22alphasparseIndexType_tS4_22alphasparseIndexBase_t19alphasparseDataType",
        "_Z23alphasparseDestroySpMatP22_alphasparseSpMatDescr",
        "_Z23alphasparseDestroyDnVecP24_alphasparse_dnvec_descr",
        "_Z23alphasparseDestroyDnMatP24_alphasparse_dnmat_descr",
        "_Z24alphasparseAmdKeptKernelP22_alphasparseSpMatDescr22alphasparseOperation_tiii",  # alphasparseAmdKeptKernel (no counterpart in the reference)
    }
    extra = exported - set(capi.EXPORTS) - set(MANGLED) - also
    assert not extra, sorted(extra)


def test_struct_layouts_match_the_reference_fixture(tmp_path):
    """tests/golden/layout.json holds sizeof / offsetof of the boundary structs as the reference's
    own headers give them (written by tests/golden/make_layout.py in the build container).  The
    same probe compiled against this repository's include/ must print the same numbers."""
    import json
    want = json.load(open(os.path.join(ROOT, "tests", "golden", "layout.json")))
    exe = str(tmp_path / "layout_probe")
    subprocess.run(["g++", "-std=c++17", "-w", "-D__HIP_PLATFORM_AMD__", "-I/opt/rocm/include",
                    "-I" + os.path.join(ROOT, "include"), os.path.join(ROOT, "tests", "golden", "layout_probe.cpp"),
                    "-o", exe], check=True)
    got = json.loads(subprocess.run([exe], check=True, capture_output=True, text=True).stdout)
    got.pop("end", None)
    assert got == want, {k: (got.get(k), want.get(k)) for k in set(got) | set(want) if got.get(k) != want.get(k)}
    assert want["sizeof(alphasparse_handle_s)"] == 1608 and want["sizeof(_alphasparse_mat_descr)"] == 144


def test_default_workspace_covers_merge_and_flat(lib):
    """alphasparseSpMV_bufferSize(DEFAULT) reports asx_spmv_workspace_bytes(DEFAULT); a DEFAULT
    analysis may settle on the flat or the merge-path kernel, so it must cover both, also for
    hypersparse matrices where the merge-path carry array (one value per 2048 rows + stored
    elements) is the larger."""
    for vt in (capi.R_32F, capi.R_64F):
        for m, nnz in ((2_000_000, 100_000), (1 << 22, 34_000_000), (10, 10), (1 << 24, 1 << 20), (300_000, 200_000),
                       (1, 0), (5_000_000, 1)):
            d = lib.asx_spmv_workspace_bytes(capi.SPMV_DEFAULT, vt, m, nnz)
            assert d >= lib.asx_spmv_workspace_bytes(capi.SPMV_MERGE, vt, m, nnz), (vt, m, nnz)
            assert d >= lib.asx_spmv_workspace_bytes(capi.SPMV_FLAT, vt, m, nnz), (vt, m, nnz)


def test_alg_mapping_and_workspace(lib):
    # reference algorithm ids -> kernels (spdef.h:345-365)
    for alg in (5, 6, 10, 16):
        assert lib.asx_spmv_resolve_alg(alg, 100, 1000) == capi.SPMV_VECTOR
    for alg in (2, 3, 8):
        assert lib.asx_spmv_resolve_alg(alg, 100, 1000) == capi.SPMV_STREAM
    for alg in (0, 11, 12, 13, 14, 15, 18):
        assert lib.asx_spmv_resolve_alg(alg, 100, 1000) == capi.SPMV_FLAT
    for alg in (7, 9, 17):
        assert lib.asx_spmv_resolve_alg(alg, 100, 1000) == capi.SPMV_MERGE
    for alg in (1, 4, 19, -1):
        assert lib.asx_spmv_resolve_alg(alg, 100, 1000) < 0
    assert lib.asx_spmv_workspace_bytes(capi.SPMV_VECTOR, capi.R_64F, 1000, 5000) == 0
    m, nnz = 4194304, 34106138
    tiles = (m + nnz + 2047) // 2048
    need = lib.asx_spmv_workspace_bytes(capi.SPMV_MERGE, capi.R_64F, m, nnz)
    assert need >= 2 * (tiles + 1) * 4 + tiles * 8 and need % 256 == 0
    assert lib.asx_spmv_workspace_bytes(capi.SPMV_MERGE, capi.R_32F, m, nnz) < need
    assert lib.asx_spmm_resolve_alg(0, 10, 10, 64) == capi.SPMM_MERGE
    assert lib.asx_spmm_resolve_alg(5, 10, 10, 64) == capi.SPMM_ROW
    assert lib.asx_spmm_resolve_alg(1, 10, 10, 64) < 0
    assert lib.asx_spmm_workspace_bytes(capi.SPMM_ROW, capi.R_32F, 10, 10, 64) == 0


def test_argument_errors_need_no_gpu(lib):
    # size / pointer checks come before any device work
    assert lib.asx_spmv_csr_f64(None, 0, -1, 1, 0, 1.0, None, None, None, None, 0.0, None, None, 0, None) == 10
    assert lib.asx_spmv_csr_f64(None, 0, 5, 5, 0, 1.0, None, None, None, None, 0.0, None, None, 0, None) == 7
    assert lib.asx_spmv_csr_f32(None, 0, 0, 0, 0, 1.0, None, None, None, None, 0.0, None, None, 0, None) == 0
    assert lib.asx_spmm_csr_f32(None, 0, 5, 5, 0, -2, 1.0, None, None, None, None, 1, 0.0, None, 1, None, 0, None) == 10
    assert lib.asx_partition_rows_by_nnz(None, 0, 4, None, None) == 10
    assert lib.asx_nnz_split_rows(None, 5, 5, 0, None, None) == 10
    assert lib.asx_copy_bytes(None, None, 16, None) == 7


def test_descriptor_checks(lib):
    # alphasparseCreateDnVec / DnMat argument checking (hip/util/handle.hip:648-744)
    dnvec = getattr(lib, MANGLED[3])
    dnvec.argtypes = [C.POINTER(C.c_void_p), C.c_int64, C.c_void_p, C.c_int]
    d = C.c_void_p()
    buf = (C.c_double * 4)()
    assert dnvec(None, 4, buf, 1) == 7      # INVALID_POINTER
    assert dnvec(C.byref(d), -1, buf, 1) == 10  # INVALID_SIZE
    assert dnvec(C.byref(d), 4, None, 1) == 7
    assert dnvec(C.byref(d), 4, buf, 1) == 0 and d.value
    size = C.c_int64.from_address(d.value + 8).value  # {init, size, values, data_type}
    assert size == 4
    dnmat = getattr(lib, MANGLED[4])
    dnmat.argtypes = [C.POINTER(C.c_void_p), C.c_int64, C.c_int64, C.c_int64, C.c_void_p, C.c_int, C.c_int]
    assert dnmat(None, 2, 2, 2, buf, 1, 0) == 7
    assert dnmat(C.byref(d), -2, 2, 2, buf, 1, 0) == 10
    assert dnmat(C.byref(d), 2, 2, 2, None, 1, 0) == 7
    assert dnmat(C.byref(d), 2, 2, 2, buf, 1, 0) == 0


def test_host_row_blocks(lib, oracle, golden):
    g = golden("row_blocks.npz")
    for name in sorted({k.split("__")[0] for k in g.files}):
        assert np.array_equal(capi.csr_adaptive_row_blocks(g[f"{name}__row_ptr"]), g[f"{name}__blocks"]), name
    for name, lens in analysis_shapes().items():
        rp = row_ptr_from_lengths(lens)
        assert np.array_equal(capi.csr_adaptive_row_blocks(rp), oracle.csr_adaptive_row_blocks(rp)), name


def test_loadbalance_nwarps_host(lib, oracle):
    for nnz in (0, 1, 199999, 200000, 1999999, 2000000, 19999999, 20000000, 199999999, 200000000, 2**31 - 1):
        for ws, base in ((32, 160), (64, 520)):
            assert capi.loadbalance_nwarps(nnz, ws, base) == oracle.loadbalance_nwarps(nnz, ws, base)


def test_workload_generator_is_deterministic():
    from library_amd import workloads as W
    import xxhash
    w = W.uniform16_f32(m=4096)
    assert w.nnz == 4096 * 16 and np.all(np.diff(w.row_ptr) == 16)
    cols = w.col.reshape(4096, 16)
    assert np.all(np.diff(cols, axis=1) > 0) and cols.min() >= 0 and cols.max() < 4096
    w2 = W.uniform16_f32(m=4096)
    assert xxhash.xxh64(w.col.tobytes()).hexdigest() == xxhash.xxh64(w2.col.tobytes()).hexdigest()
    p = W.powerlaw_f64(m=1 << 14)
    lens = np.diff(p.row_ptr)
    assert lens.max() <= 1 << 14 and 0.003 < (lens == 0).mean() < 0.03
    for r in np.flatnonzero(lens > 1)[:200]:
        c = p.col[p.row_ptr[r]:p.row_ptr[r + 1]]
        assert np.all(np.diff(c) > 0)
    s = W.spmm_zipf_f32(m=1 << 12, ncols=8)
    assert s.x.size == (1 << 12) * 8 and s.y.size == (1 << 12) * 8


def test_build_reads_the_compilers_kernel_resources():
    """library_amd.build turns the compiler's kernel-resource-usage remarks into a table and refuses
    kernels that spill registers to scratch memory; the table of the library that is built here
    lists the hot kernels without scratch."""
    from library_amd import build
    text = """
/x/asx_spmm.hip:133:1: remark: Function Name: _ZN3asx18k_spmm_snap_splitsEiiPKiS1_S1_PiS2_ [-Rpass-analysis=kernel-resource-usage]
  133 | {
      | ^
/x/asx_spmm.hip:133:1: remark:     TotalSGPRs: 20 [-Rpass-analysis=kernel-resource-usage]
/x/asx_spmm.hip:133:1: remark:     VGPRs: 11 [-Rpass-analysis=kernel-resource-usage]
/x/asx_spmm.hip:133:1: remark:     ScratchSize [bytes/lane]: 60 [-Rpass-analysis=kernel-resource-usage]
/x/asx_spmm.hip:133:1: remark:     Occupancy [waves/SIMD]: 8 [-Rpass-analysis=kernel-resource-usage]
/x/asx_spmm.hip:133:1: remark:     LDS Size [bytes/block]: 4112 [-Rpass-analysis=kernel-resource-usage]
/x/other.hip:1:1: remark: Function Name: _ZN7rocprim6kernelEv [-Rpass-analysis=kernel-resource-usage]
/x/other.hip:1:1: remark:     VGPRs: 99 [-Rpass-analysis=kernel-resource-usage]
"""
    table = build.kernel_resources(text)
    assert list(table) == ["_ZN3asx18k_spmm_snap_splitsEiiPKiS1_S1_PiS2_"]  # only this library's kernels
    r = table["_ZN3asx18k_spmm_snap_splitsEiiPKiS1_S1_PiS2_"]
    assert (r["TotalSGPRs"], r["VGPRs"], r["ScratchSize"], r["Occupancy"], r["LDS Size"]) == (20, 11, 60, 8, 4112)
    path = os.path.join(ROOT, "library_amd", "build", "kernel_resources.txt")
    if os.path.exists(path):
        lines = open(path).read().splitlines()
        assert lines and all(" scratch=0 " in l for l in lines)
        assert any("k_spmv_window" in l for l in lines) and any("k_sliced_products" in l for l in lines)
