/*
 * mcclx_bench.h -- what the MEASUREMENT build of the library (libmcclx_bench.so,
 * `python -m mccl_amd.build --bench`) exports on top of mcclx.h.  None of it is
 * part of the drop-in boundary and none of it has a counterpart in the
 * reference; the shipped libmcclx.so has none of these symbols.
 *
 * The measurement build is the same source compiled with
 * -DMCCLX_TUNE_TIMELINE=1: every block of a by-value fold launch can record
 * when it started, when it had its data and when it had issued its last store.
 */
#ifndef MCCLX_BENCH_H
#define MCCLX_BENCH_H

#include "mcclx.h"

#ifdef __cplusplus
extern "C" {
#endif

/* One launch on `hip_stream` (a hipStream_t) that only reads (write = 0) or only
 * writes (write = 1) nbytes of `buf` (4-byte aligned; its contents are unspecified
 * afterwards) with the copy kernel's access shape: the one-directional ceilings a
 * fold launch of the same footprint is compared with. */
MCCLX_API int mcclx_bench_probe(void* hip_stream, void* buf, uint64_t nbytes, int write);

/* Where the next by-value fold launches of this library put their per-block
 * records: a device buffer cut into `slots` regions of `records_per_slot` records
 * of 32 bytes (start, data, end in ticks of the 100 MHz wall clock; HW_ID and
 * XCC_ID registers), used round robin, one region per launch.  NULL stops it. */
MCCLX_API void mcclx_tune_timeline(void* device_buf, uint64_t slots, uint64_t records_per_slot);

#ifdef __cplusplus
}
#endif
#endif /* MCCLX_BENCH_H */
