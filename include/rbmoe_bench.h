/* Measurement helpers of the benchmark (librbmoe_bench.so).  Not part of the layer's boundary: nothing here has a
 * counterpart in the reference, nothing in librbmoe.so depends on it, and a host that only runs the layer never
 * loads it.  The reference measures with wall-clock phases around `synchronize`
 * (examples/profile_step.rs:74-151, src/transformer.rs:1323-1334); these are the pieces a roofline figure needs on
 * top of that: a stream and an event timer for hosts without a HIP binding, a cache flush that leaves no dirty
 * lines, and two calibration kernels.  Every function returns 0 or a HIP error code (-1: bad argument). */
#ifndef RBMOE_BENCH_H
#define RBMOE_BENCH_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* A non-blocking HIP stream of default priority (hand it to rbmoe_ctx_set_stream so that the layer's kernels, the
 * flush and the timer share it). */
int rbbench_stream_create(void** stream);
int rbbench_stream_destroy(void* stream);

/* Two HIP events: `start` records the first on the stream, `stop` records the second, waits for it and returns the
 * interval in milliseconds.  An interval carries a few microseconds of its own. */
int rbbench_timer_create(void** timer);
int rbbench_timer_start(void* timer, void* stream);
int rbbench_timer_stop(void* timer, void* stream, float* ms);
void rbbench_timer_destroy(void* timer);

/* Cache flush: a buffer of `bytes` (at least twice the 256 MiB Infinity Cache to be effective) that rbbench_flush
 * sweeps with loads only, so that what the next kernel reads comes from HBM and no dirty line drains while it
 * runs. */
int rbbench_flush_create(size_t bytes, void** flush);
int rbbench_flush(void* flush, void* stream);
void rbbench_flush_destroy(void* flush);

/* A kernel of nothing but 32x32x16 bf16 matrix-core multiplies, two waves on every SIMD, about 0.25 ms a launch:
 * the multiply rate the matrix cores sustain at the clock they settle at.  `launches` launches between one pair
 * of events. */
int rbbench_mfma_only(void* stream, int32_t launches, double* tflops, double* avg_launch_ms);

/* A plain read of `bytes` (16-byte loads; split over 512, 1024 and 2048 workgroups, the fastest split is
 * reported).  flush == NULL: `launches` launches back to back between one pair of events (the buffer stays in the
 * caches if it fits).  Otherwise the flush buffer is swept before every launch and each launch is timed by an
 * event pair of its own; the raw interval is reported, nothing is subtracted. */
int rbbench_read(void* stream, size_t bytes, int32_t launches, void* flush, double* gbs, double* avg_launch_ms);

#ifdef __cplusplus
}
#endif
#endif
