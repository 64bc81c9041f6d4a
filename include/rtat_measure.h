/*
 * rtat_measure.h - measurement aids of librtat_native, kept apart from the BLAS boundary in
 * rtat_native.h: nothing here replaces a call the reference makes (src/gpu-api/gpu-api.h:87-113
 * has no counterpart), and a binding of the boundary does not need this header.  bench.py
 * uses it to measure, in the same run, what the memory system delivers to a plain streaming
 * kernel - the yardstick the bandwidth-bound entry points are reported against.
 */
#ifndef RTAT_MEASURE_H
#define RTAT_MEASURE_H

#include "rtat_native.h"

#ifdef __cplusplus
extern "C" {
#endif

/* A plain streaming kernel over the caller's device buffers, enqueued on the handle's
 * stream: the yardstick for the bandwidth-bound entry points (what the memory system
 * delivers to a kernel that only reads, only writes, or copies, with 16-byte accesses).
 * RTAT_PROBE_READ reads `bytes` from src (dst: at least 2 KiB, left untouched for finite
 * data), RTAT_PROBE_WRITE writes `bytes` of a constant pattern to dst (src ignored),
 * RTAT_PROBE_COPY copies src to dst.  bytes must be a multiple of 32 KiB, pointers 16-byte
 * aligned.  No counterpart in the reference (measurement aid, like rtat_device_peaks). */
typedef enum { RTAT_PROBE_READ = 0, RTAT_PROBE_WRITE = 1, RTAT_PROBE_COPY = 2 } rtat_probe_kind_t;
rtat_status_t rtat_hbm_probe(rtat_handle_t handle, int kind, const void* src, void* dst,
                             size_t bytes);

#ifdef __cplusplus
}
#endif
#endif /* RTAT_MEASURE_H */
