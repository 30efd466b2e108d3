/*
 * swc_hip_bench.h — measurement helpers of libswc_hip_bench.so, for benchmark
 * harnesses only.  Nothing here is an op of the reference or part of the
 * drop-in C ABI (include/swc_hip.h); generated programs never link it.
 */
#ifndef SWC_HIP_BENCH_H_
#define SWC_HIP_BENCH_H_

#include <stddef.h>

#ifdef __cplusplus
extern "C" {
#endif

/* Runs `iters` rounds of 16 independent v_mfma_f32_32x32x2_f32 per wavefront on
 * two workgroups per CU, on `hip_stream` (e.g. swc_hip_stream()), and returns the
 * elapsed milliseconds and the flop executed, so a harness can print the fp32
 * matrix rate the device sustains beside the datasheet figure.
 * scratch_dev: device buffer of at least 512 * cus floats.  Returns 0, or a
 * non-zero hipError_t. */
int swc_hip_bench_probe_mfma_f32(void *hip_stream, int cus, float *scratch_dev, size_t scratch_floats, int iters,
                                 float *ms_out, double *flop_out);

/* The shader clock while other work runs.  _start launches, on a stream of the bench library's own (default
 * priority), ONE wavefront that writes n pairs (100 MHz wall-clock ticks, shader-clock counter) into samples_dev
 * (2 n 64-bit words of device memory), sleeping sleeps x 8128 shader cycles (about 3.5 us each) between pairs,
 * and returns at once; the watcher ends by itself after its n pairs.  The harness then enqueues the work it
 * wants watched on its own stream, calls _wait, and reads the clock off consecutive pairs:
 * GHz = 0.1 x (shader difference) / (wall difference).  One wavefront on one CU does not disturb a kernel that
 * fills the chip.  1 < n <= 65536, 1 <= sleeps <= 64, n x sleeps <= 262144 (the watcher then ends within a second).
 * Return 0, or a non-zero hipError_t. */
int swc_hip_bench_clock_watch_start(unsigned long long *samples_dev, int n, int sleeps);
int swc_hip_bench_clock_watch_wait(void);

#ifdef __cplusplus
}
#endif
#endif /* SWC_HIP_BENCH_H_ */
