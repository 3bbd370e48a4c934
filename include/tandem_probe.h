/* libtandem_probe.so: a measurement kernel, built beside libtandem_hip.so from the same device
 * headers and NOT part of the plug-in. bench.py and the GPU tests load it; nothing in the library
 * or the package does. Plain C, like tandem_hip.h. */
#ifndef TANDEM_PROBE_H
#define TANDEM_PROBE_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* Measurement only; the reference has no counterpart. Reads `bytes` (a multiple of 16) from each of
 * `nreads` device buffers and writes as many to each of `nwrites` others (0..8 each), in the launch
 * geometry of the streaming kernels of libtandem_hip.so (workgroups of 128 lanes, `vectors_per_lane`
 * = 1 or 2 16-byte vectors per lane and stream, one tile per workgroup, tile order
 * tdm_tile_of(.., xcd_shift), `occupancy_pad` bytes of unused LDS per workgroup, non-temporal
 * accesses), without a table and without arithmetic: what the memory system gives a kernel with that
 * mix of streams. The written values are meaningless. `stream` is a hipStream_t. Returns 0, or 1
 * (bad argument) / 2 (runtime failure) with the message in tdm_probe_last_error(). */
int tdm_probe_stream_mix(const void* const* reads, int nreads, void* const* writes, int nwrites, int64_t bytes,
                         int vectors_per_lane, int xcd_shift, int occupancy_pad, void* stream);

/* The message of this thread's last failed call (empty before any). */
const char* tdm_probe_last_error(void);

#ifdef __cplusplus
}
#endif

#endif
