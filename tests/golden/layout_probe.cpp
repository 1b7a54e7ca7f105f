// Prints sizeof / offsetof of the structs that cross the generic-API boundary, as JSON.
// Compiled twice: against the reference's include/ (tests/golden/make_layout.py, writes
// layout.json in the build container) and against this repository's include/
// (tests/test_boundary_cpu.py, compares with layout.json).
#include <cstddef>
#include <cstdio>
#include <hip/hip_runtime.h>
#include "alphasparse.h"
#define SZ(T) printf("  \"sizeof(" #T ")\": %zu,\n", sizeof(T))
#define OFF(T, f) printf("  \"offsetof(" #T "," #f ")\": %zu,\n", offsetof(T, f))
int main() {
  printf("{\n");
  SZ(alphasparse_handle_s);
  OFF(alphasparse_handle_s, device); OFF(alphasparse_handle_s, wavefront_size); OFF(alphasparse_handle_s, properties);
  OFF(alphasparse_handle_s, stream); OFF(alphasparse_handle_s, streams); OFF(alphasparse_handle_s, pointer_mode);
  OFF(alphasparse_handle_s, layer_mode); OFF(alphasparse_handle_s, buffer_size); OFF(alphasparse_handle_s, buffer);
  OFF(alphasparse_handle_s, sone); OFF(alphasparse_handle_s, done); OFF(alphasparse_handle_s, check_flag);
  OFF(alphasparse_handle_s, process); OFF(alphasparse_handle_s, pflat_analysis_data);
  SZ(_alphasparseSpMatDescr);
  OFF(_alphasparseSpMatDescr, init); OFF(_alphasparseSpMatDescr, analysed); OFF(_alphasparseSpMatDescr, rows);
  OFF(_alphasparseSpMatDescr, cols); OFF(_alphasparseSpMatDescr, nnz); OFF(_alphasparseSpMatDescr, row_data);
  OFF(_alphasparseSpMatDescr, col_data); OFF(_alphasparseSpMatDescr, val_data); OFF(_alphasparseSpMatDescr, const_row_data);
  OFF(_alphasparseSpMatDescr, row_type); OFF(_alphasparseSpMatDescr, col_type); OFF(_alphasparseSpMatDescr, data_type);
  OFF(_alphasparseSpMatDescr, idx_base); OFF(_alphasparseSpMatDescr, format); OFF(_alphasparseSpMatDescr, descr);
  OFF(_alphasparseSpMatDescr, info); OFF(_alphasparseSpMatDescr, block_dir); OFF(_alphasparseSpMatDescr, batch_count);
  OFF(_alphasparseSpMatDescr, columns_values_batch_stride);
  SZ(_alphasparse_mat_descr);
  OFF(_alphasparse_mat_descr, type); OFF(_alphasparse_mat_descr, base); OFF(_alphasparse_mat_descr, max_nnz_per_row);
  OFF(_alphasparse_mat_descr, spgemm_reuse_flag); OFF(_alphasparse_mat_descr, row_map); OFF(_alphasparse_mat_descr, h_level_size);
  OFF(_alphasparse_mat_descr, h_chain_size); OFF(_alphasparse_mat_descr, in_degree); OFF(_alphasparse_mat_descr, csr_row_idx);
  OFF(_alphasparse_mat_descr, csr_rdiag); OFF(_alphasparse_mat_descr, rcsr_rdiag);
  SZ(_alphasparse_dnvec_descr);
  OFF(_alphasparse_dnvec_descr, size); OFF(_alphasparse_dnvec_descr, values); OFF(_alphasparse_dnvec_descr, data_type);
  SZ(_alphasparse_dnmat_descr);
  OFF(_alphasparse_dnmat_descr, rows); OFF(_alphasparse_dnmat_descr, cols); OFF(_alphasparse_dnmat_descr, ld);
  OFF(_alphasparse_dnmat_descr, values); OFF(_alphasparse_dnmat_descr, data_type); OFF(_alphasparse_dnmat_descr, order);
  SZ(_alphasparse_csrmv_info);
  OFF(_alphasparse_csrmv_info, algo); OFF(_alphasparse_csrmv_info, size); OFF(_alphasparse_csrmv_info, row_blocks);
  OFF(_alphasparse_csrmv_info, partition); OFF(_alphasparse_csrmv_info, coordinate); OFF(_alphasparse_csrmv_info, num_merge_tiles);
  OFF(_alphasparse_csrmv_info, r_csr_row_ptr); OFF(_alphasparse_csrmv_info, trans); OFF(_alphasparse_csrmv_info, m);
  OFF(_alphasparse_csrmv_info, nnz); OFF(_alphasparse_csrmv_info, descr); OFF(_alphasparse_csrmv_info, csr_row_ptr);
  OFF(_alphasparse_csrmv_info, csr_col_ind);
  SZ(_alphasparse_mat_info);
  OFF(_alphasparse_mat_info, csrmv_info); OFF(_alphasparse_mat_info, csrgemm_info); OFF(_alphasparse_mat_info, zero_pivot);
  OFF(_alphasparse_mat_info, boost_enable); OFF(_alphasparse_mat_info, boost_val);
  printf("  \"end\": 0\n}\n");
}
