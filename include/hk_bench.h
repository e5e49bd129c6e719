/* hk_bench.h -- the streaming yardstick bench.py measures the operator kernels against.
 *
 * A library of its own (libhk_bench.so): a measurement tool with no counterpart in the reference, kept out of
 * libhk_rowwise.so so that the operator library exports operators and the device layer only.  Types and return
 * codes are those of hk_rowwise.h. */
#ifndef HK_BENCH_H_
#define HK_BENCH_H_

#include "hk_rowwise.h"

#ifdef __cplusplus
extern "C" {
#endif

/* Moves `bytes` per array, `reads` arrays in (0..2) and `writes` arrays out (0..2), with workgroups of
 * `block_threads` (64, 128, 256, 512, 1024), `vectors_per_thread` 16-byte vectors in flight per thread (1, 2, 4), the
 * non-temporal hint on loads / stores, and either a one-shot grid (`workgroups_per_cu` 0) or that many workgroups
 * per compute unit walking the arrays.  The best shape of a read : write mix is the roof the operator kernels with
 * that mix are measured against (bench.py --all).  Arguments are checked before anything is computed from them. */
HK_API int hk_bench_stream_probe(void* dst0, void* dst1, const void* src0, const void* src1, int reads, int writes,
                                 size_t bytes, int block_threads, int vectors_per_thread, int nt_loads,
                                 int nt_stores, int workgroups_per_cu, hkStream_t stream);

/* The persistent two-in / one-out walk of hk_bench_stream_probe, software-pipelined the way the backward norm kernels
 * are: `workgroups_per_cu` (1..8) workgroups of `block_threads` (256, 512, 1024) per compute unit each own every n-th
 * tile of block_threads vectors and keep a ring of `depth` (1..4) tiles of both inputs in flight per thread; with
 * `barrier` != 0 every tile also goes through one workgroup barrier and a small LDS exchange (the cost of a row
 * reduction across wavefronts).  `bytes` per array, a whole number of tiles.  The best depth is the ceiling of that
 * kernel design whatever arithmetic is put into it. */
HK_API int hk_bench_ring_probe(void* dst, const void* src0, const void* src1, size_t bytes, int block_threads,
                               int depth, int barrier, int workgroups_per_cu, hkStream_t stream);

/* Text of the last error this library returned on the calling thread. */
HK_API const char* hk_bench_last_error(void);

#ifdef __cplusplus
}
#endif

#endif /* HK_BENCH_H_ */
