/*
 * Measurement helper of the benchmark; not part of the drop-in interface (nothing in the
 * reference corresponds to it, and callers of the library do not need it).
 */
#ifndef ALPHASPARSE_AMD_BENCH_H
#define ALPHASPARSE_AMD_BENCH_H

#include <stddef.h>

#ifdef __cplusplus
extern "C" {
#endif

/* A coalesced copy kernel of `bytes` bytes (multiple of 16) on `stream` (a hipStream_t passed as
 * void*): a launch of known traffic, for scaling the profiler's FETCH_SIZE / WRITE_SIZE readings. */
int asx_copy_bytes(const void *d_src, void *d_dst, size_t bytes, void *stream);

/* Pseudo-random reads of a buffer of `bytes` bytes, 8 in flight per lane: group_lanes = 1, every
 * lane reads one 32-bit word of a 128-byte line of its own; group_lanes = 64, every wave reads
 * 256 consecutive bytes (the row of B an N = 64 fp32 SpMM fetches per stored element).  Every
 * lane issues loads_per_lane loads (a multiple of 8) and writes one word to d_out, which holds
 * *nthreads words (call with d_out = NULL to learn *nthreads).  Measures the rate at which the
 * memory system delivers independent lines past the L2s: the bound of a gather without reuse. */
int asx_gather_lines(const void *d_buf, size_t bytes, int group_lanes, int loads_per_lane, void *d_out, int *nthreads,
                     void *stream);

#ifdef __cplusplus
}
#endif
#endif
