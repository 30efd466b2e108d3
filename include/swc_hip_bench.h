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

#ifdef __cplusplus
}
#endif
#endif /* SWC_HIP_BENCH_H_ */
