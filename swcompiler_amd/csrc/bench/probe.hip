// libswc_hip_bench.so — measurement helper for benchmark harnesses: the fp32
// MFMA rate this device sustains, so a harness can print the measured ceiling
// next to the datasheet one.  Not an op of the reference and not part of
// libswc_hip's C ABI; it shares no state with that library (the caller passes
// the stream to run on).
#include <hip/hip_runtime.h>

#include "swc_hip_bench.h"

namespace {

typedef float v16f __attribute__((ext_vector_type(16)));
constexpr int kProbeAcc = 4;     // independent accumulators per wavefront (hides the MFMA latency)
constexpr int kProbeUnroll = 4;

__global__ __launch_bounds__(256) void mfma_rate_probe(float *out, int iters, float a, float b) {
#if __HIP_DEVICE_COMPILE__
    v16f acc[kProbeAcc];
    for (int i = 0; i < kProbeAcc; ++i)
        for (int v = 0; v < 16; ++v) acc[i][v] = 0.f;
    for (int it = 0; it < iters; ++it) {
#pragma unroll
        for (int u = 0; u < kProbeUnroll; ++u)
#pragma unroll
            for (int i = 0; i < kProbeAcc; ++i) acc[i] = __builtin_amdgcn_mfma_f32_32x32x2f32(a, b, acc[i], 0, 0, 0);
    }
    float s = 0.f;
    for (int i = 0; i < kProbeAcc; ++i)
        for (int v = 0; v < 16; ++v) s += acc[i][v];
    out[blockIdx.x * 256 + threadIdx.x] = s;
#endif
}

// One wavefront that notes the 100 MHz wall clock and the shader clock counter side by side, `n` times, sleeping
// `sleeps` x 8128 shader cycles in between, and ends by itself.
__global__ __launch_bounds__(64) void clock_watch(unsigned long long *samples, int n, int sleeps) {
#if __HIP_DEVICE_COMPILE__
    for (int i = 0; i < n; ++i) {
        const unsigned long long wall = wall_clock64(), shader = clock64();
        if (threadIdx.x == 0) {
            samples[2 * i] = wall;
            samples[2 * i + 1] = shader;
        }
        for (int s = 0; s < sleeps; ++s) __builtin_amdgcn_s_sleep(127);
    }
#endif
}

hipStream_t g_watch_stream = nullptr;

} // namespace

#define PROBE_TRY(expr)                  \
    do {                                 \
        hipError_t e__ = (expr);         \
        if (e__ != hipSuccess) return (int)e__; \
    } while (0)

extern "C" int swc_hip_bench_probe_mfma_f32(void *hip_stream, int cus, float *scratch_dev, size_t scratch_floats,
                                            int iters, float *ms_out, double *flop_out) {
    if (!scratch_dev || !ms_out || !flop_out || iters <= 0 || cus <= 0) return (int)hipErrorInvalidValue;
    const int blocks = 2 * cus;   // two workgroups (8 wavefronts) per CU: every SIMD has two waves
    if (scratch_floats < (size_t)blocks * 256) return (int)hipErrorInvalidValue;
    hipStream_t s = (hipStream_t)hip_stream;
    hipEvent_t e0, e1;
    PROBE_TRY(hipEventCreate(&e0));
    PROBE_TRY(hipEventCreate(&e1));
    mfma_rate_probe<<<blocks, 256, 0, s>>>(scratch_dev, 16, 1.f, 1.f);   // code load, clocks
    PROBE_TRY(hipGetLastError());
    PROBE_TRY(hipEventRecord(e0, s));
    mfma_rate_probe<<<blocks, 256, 0, s>>>(scratch_dev, iters, 1.f, 1.f);
    PROBE_TRY(hipGetLastError());
    PROBE_TRY(hipEventRecord(e1, s));
    PROBE_TRY(hipEventSynchronize(e1));
    PROBE_TRY(hipEventElapsedTime(ms_out, e0, e1));
    (void)hipEventDestroy(e0);
    (void)hipEventDestroy(e1);
    // 32x32x2 MFMA = 2*32*32*2 = 4096 flop per wavefront instruction
    *flop_out = (double)blocks * 4 * (double)iters * kProbeUnroll * kProbeAcc * 4096.0;
    return 0;
}

extern "C" int swc_hip_bench_clock_watch_start(unsigned long long *samples_dev, int n, int sleeps) {
    if (!samples_dev || n <= 1 || n > (1 << 16) || sleeps < 1 || sleeps > 64 || (long)n * sleeps > (1L << 18))   // under a second
        return (int)hipErrorInvalidValue;
    if (!g_watch_stream) PROBE_TRY(hipStreamCreateWithFlags(&g_watch_stream, hipStreamNonBlocking));
    clock_watch<<<1, 64, 0, g_watch_stream>>>(samples_dev, n, sleeps);
    PROBE_TRY(hipGetLastError());
    return 0;
}

extern "C" int swc_hip_bench_clock_watch_wait(void) {
    if (!g_watch_stream) return (int)hipErrorInvalidValue;
    PROBE_TRY(hipStreamSynchronize(g_watch_stream));
    return 0;
}
