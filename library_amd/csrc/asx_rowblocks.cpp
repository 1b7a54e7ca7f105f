// Host construction of CSR-Adaptive row blocks with the packing and cut rules of the
// reference's ComputeRowBlocks (hip/kernel/level2/alphasparse_spmv_csr_adaptive.h:354-568;
// constants at :6-11; helper include/alphasparse/common.h:12-20,192-200).  The reference runs
// this on the host on a host copy of row_ptr inside every adaptive SpMV call; here it is an
// analysis entry point of its own.  Output entries: (first_row << 32) | low bits, where the
// low bits are the workgroup index inside a long row, or the number of lanes per row for a
// block of several rows.
#include <cmath>
#include <cstddef>
#include <cstdint>

#include "../../include/alphasparse_amd.h"

namespace {

constexpr uint64_t kBlockNnz = 1024;     // stored elements per row block
constexpr uint64_t kLongRowFactor = 3;   // a long row gets one workgroup per 3*1024 elements
constexpr uint32_t kWorkgroup = 256;
constexpr int32_t kLongRow = 128;        // rows longer than this start a "long" run
constexpr int32_t kShortRow = 32;        // a row shorter than this ends it

uint32_t largest_pow2_not_above(uint32_t v)
{
    v |= v >> 1;
    v |= v >> 2;
    v |= v >> 4;
    v |= v >> 8;
    v |= v >> 16;
    return v - (v >> 1);
}

class Emitter {
public:
    Emitter(uint64_t *out, size_t cap) : out_(out), cap_(cap) {}
    void put(uint64_t v)
    {
        if (n_ < cap_) out_[n_] = v;
        ++n_;
    }
    // ORs the lanes-per-row count into the entry that opened the block just closed
    void tag_opening(uint64_t rows_in_block)
    {
        if (rows_in_block > 1 && n_ >= 2 && n_ - 2 < cap_)
            out_[n_ - 2] |= largest_pow2_not_above((uint32_t)(kWorkgroup / rows_in_block));
    }
    size_t count() const { return n_; }

private:
    uint64_t *out_;
    size_t cap_;
    size_t n_ = 0;
};

}  // namespace

extern "C" int asx_csr_adaptive_row_blocks(const int32_t *h_row_ptr, int32_t m, uint64_t *h_out,
                                           size_t cap, size_t *count)
{
    if (m < 0) return ASX_STATUS_INVALID_SIZE;
    if (!h_row_ptr || !count || (cap > 0 && !h_out)) return ASX_STATUS_INVALID_POINTER;

    // A sizing call (cap too small to hold everything) still has to know the row stored in the
    // last entry; track it separately so the result does not depend on cap.
    Emitter em(h_out, cap);
    uint64_t last_entry_row = 0;
    auto put = [&](uint64_t v) {
        em.put(v);
        last_entry_row = v >> 32;
    };

    put(0);
    uint64_t filled = 0;      // stored elements in the open block
    uint64_t open_at = 0;     // first row of the open block
    int32_t long_run = 0;     // >0 inside a run of long rows, -1 on the first short row after one
    const uint64_t rows = (uint64_t)m;
    uint64_t i = 1;
    for (; i <= rows; ++i) {
        const int32_t len = h_row_ptr[i] - h_row_ptr[i - 1];
        filled += (uint64_t)len;

        if (len > kLongRow)
            ++long_run;
        else if (long_run > 0)
            long_run = len < kShortRow ? -1 : long_run + 1;

        const bool close_before_row = (long_run == 1 && i - open_at > 1) || long_run == -1;
        if (close_before_row) {
            // short rows before a long one, or long rows before a short one, get their own block
            put((i - 1) << 32);
            em.tag_opening((i - 1) - open_at);
            open_at = i - 1;
            filled = (uint64_t)len;
            if (long_run == -1) long_run = 0;
        }

        const uint64_t rows_open = i - open_at;
        if (rows_open == 1 && filled > kBlockNnz) {
            // a single row larger than a block: split across workgroups
            int32_t groups = (int32_t)std::ceil((double)len / (double)(kLongRowFactor * kBlockNnz));
            if (groups > (1 << 24)) groups = 1 << 24;
            for (int32_t w = 1; w < groups; ++w) put(((i - 1) << 32) | (uint64_t)w);
            put(i << 32);
            open_at = i;
            filled = 0;
            long_run = 0;
        } else if (rows_open > 1 && filled > kBlockNnz) {
            // this row overflows the block: close in front of it and look at it again
            --i;
            put(i << 32);
            em.tag_opening(i - open_at);
            open_at = i;
            filled = 0;
            long_run = 0;
        } else if (filled == kBlockNnz) {
            put(i << 32);
            em.tag_opening(i - open_at);
            open_at = i;
            filled = 0;
            long_run = 0;
        }
    }
    if (last_entry_row != rows) {
        put(rows << 32);
        // lanes per row of the trailing block are derived from the loop index after the loop
        // (rows + 1), as in the reference
        if (rows - open_at > 1 && em.count() >= 2 && em.count() - 2 < cap)
            h_out[em.count() - 2] |= largest_pow2_not_above((uint32_t)(kWorkgroup / (i - open_at)));
    }
    *count = em.count();
    return ASX_STATUS_SUCCESS;
}
