// TEST INFRASTRUCTURE ONLY.  extern "C" door onto a *host* routine that lives in one of the
// reference's HIP headers: ComputeRowBlocks (hip/kernel/level2/alphasparse_spmv_csr_adaptive.h:
// 354-568).  No arithmetic here; the header is compiled where it lies by oracle/Makefile.  The
// device kernels that header also defines are compiled but never launched (no GPU is needed).
// (clac_size in alphasparse_spmv_csr_row_partition_ginkgo.h is not reachable this way: that
// header does not compile on its own, WARP_SIZE is undefined in the hip/ tree.)
#include <cstdint>
#include <vector>

#include "hip/kernel/level2/alphasparse_spmv_csr_adaptive.h"

extern "C" {

// Returns the entry count the reference writes (its reported size is twice that).
size_t ref_csr_adaptive_row_blocks(const int32_t *row_ptr, int32_t m, uint64_t *out, size_t cap)
{
    size_t size = 0;
    ComputeRowBlocks<int32_t>((unsigned long long *)nullptr, size, row_ptr, m, false);
    std::vector<unsigned long long> blocks(size, 0ULL);
    ComputeRowBlocks<int32_t>(blocks.data(), size, row_ptr, m, true);
    size_t n = size / 2;
    for (size_t i = 0; i < n && i < cap; ++i) out[i] = (uint64_t)blocks[i];
    return n;
}

}  // extern "C"
