/*
 * dsx_probe — streaming probe of the benchmark harness (libdsx_probe.so).  Measurement tooling,
 * kept out of libdsx.so: it calibrates the HBM roofline and the HBM byte counters, nothing in
 * the rasterizer calls it.  No counterpart in the reference.
 */
#ifndef DSX_PROBE_H_
#define DSX_PROBE_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* One launch ("stream_probe_kernel" / "stream_probe_mixed_kernel") that streams `bytes` (a multiple
 * of 16) with one 16-byte element per thread, the access shape of the per-Gaussian kernels.
 * mode 0 reads src, 1 writes dst, 2 copies src to dst (src and dst hold `bytes` each); modes 3 and
 * 4 move `bytes` in all as 10 arrays read and 18 written per thread (src holds 10/28 of `bytes`,
 * dst 18/28), respectively 5 and 9: write-heavy mixes of many streams like the per-Gaussian
 * backward's.  milliseconds (host, may be NULL): the launch's duration from an event pair on
 * `stream`; the call then waits for the launch.  Returns 0, or a negative number: -1 bad
 * argument, -2 launch failed, -3 event call failed, -4 too large. */
int dsxp_stream_probe(const void* src, void* dst, size_t bytes, int mode, void* stream, float* milliseconds);

#ifdef __cplusplus
}
#endif
#endif
