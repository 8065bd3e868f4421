/*
 * ts2_probe.h - machine probes of the benchmark (libts2probe.so).  Not part of the product ABI: nothing in libts2amd.so depends on them.
 */
#ifndef TS2_PROBE_H
#define TS2_PROBE_H
#include <stdint.h>
#include "ts2_abi.h"

#ifdef __cplusplus
extern "C" {
#endif

/* Machine probes (no counterpart in the reference; they exist so that the benchmark can price kernels against what the device
 * sustains, beside the published peaks).
 * ts2_probe_mfma_rate: runs nothing but MFMAs of the given operand type (TS2_I8 / TS2_E4M3 / TS2_BF16) on every CU, iters x 4 per wave,
 *   with constant operands (randomData = 0) or per-lane hashed bit patterns (1), and returns the sustained rate in T(FL)OP/s.
 *   scratch: device buffer of at least 256 ints per CU.
 * ts2_probe_copy_rate: streaming copy, four 16-byte loads in flight per lane, of `bytes` bytes (a multiple of 16); returns read+write GB/s.
 * ts2_probe_clock_monitor: launches ONE wave on `stream` that, `samples` times, waits `periodTicks` ticks of the constant 100 MHz
 *   counter and records (ticks waited, shader-clock cycles elapsed) as two uint64 into out[2 * i], out[2 * i + 1]: cycles / ticks x 100
 *   is the shader clock in MHz while kernels launched on OTHER streams run.  It ends by itself after samples x periodTicks. */
int ts2_probe_mfma_rate(int32_t abType, int32_t randomData, int32_t iters, int32_t *scratch, int64_t scratchInts, double *topsOut, void *stream);
int ts2_probe_copy_rate(const void *src, void *dst, int64_t bytes, double *gbPerSecOut, void *stream);
int ts2_probe_clock_monitor(uint64_t *out, int32_t samples, int32_t periodTicks, void *stream);

#ifdef __cplusplus
}
#endif
#endif
