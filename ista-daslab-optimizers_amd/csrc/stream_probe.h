/*
 * Measurement tooling, not part of the optimizer's boundary: libmicroadam_probe.so holds
 * streaming kernels of known size that bench.py uses to calibrate the HBM counters and to find
 * the rate this device sustains for the step's access shape.  No counterpart in the reference.
 */
#ifndef MICROADAM_STREAM_PROBE_H
#define MICROADAM_STREAM_PROBE_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* Streams `bytes` (a multiple of 40960) of each array it
 * touches with the fused step's own access shape: 512-thread workgroups that each own one
 * contiguous 40 KiB stretch and move it as 16-byte accesses, a contiguous KiB per wave.
 * mode 0: reads a.  1: writes c.  2: c = a.  3: b = a + b (two reads, one write).
 * 4: reads a, b and e, writes b and e, with e a quarter as long as a (the step's gradient,
 *    parameter and 4-bit error-feedback streams: 7 bytes per bf16 element).
 * 5: writes c and reads the same stretch back once the stores have completed (does the L2 serve
 *    lines that were just written?).
 * nontemporal != 0 uses the cache-bypassing loads and stores the step uses.  workgroups > 0
 * caps the grid (each workgroup then takes several stretches in turn), 0 launches one per
 * stretch.  sink: 4 bytes of device memory (keeps the read-only mode's loads alive).  Used by
 * bench.py --calibration: the HBM counters are scaled by what they read for these kernels, and
 * the rates they reach are this device's ceiling for the step's traffic. */
int ma_stream_probe(int mode, int nontemporal, int64_t bytes, int64_t workgroups, const void *a,
                    void *b, void *c, void *e, void *sink, void *stream);

#ifdef __cplusplus
}
#endif
#endif
