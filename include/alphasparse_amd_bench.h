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

#ifdef __cplusplus
}
#endif
#endif
