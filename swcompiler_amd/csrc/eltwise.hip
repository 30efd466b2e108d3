// Bandwidth-bound flat kernels: relu_f, vecAdd_f, their fusion, batchedadd_f,
// matrixTanh_f.  One pass over HBM with 128-bit accesses, one float4 per
// operand per thread and as many 256-thread workgroups as that takes (the
// measured optimum on MI355X: deeper per-thread unrolling lowered bandwidth);
// large tensors use non-temporal accesses.
#include "common.hpp"

using namespace swc_hip;

namespace {

constexpr int kThreads = 256;
constexpr int kUnroll = 1;                            // float4 per thread per operand

// (x > 0) ? x : 0 of kernels.h:578, kept as a compare+select: a max() would
// keep -0.0 and is not what the reference computes.
__device__ __forceinline__ float relu1(float x) { return (x > 0.f) ? x : 0.f; }

struct OpRelu {
    static constexpr int kInputs = 1;
    __device__ __forceinline__ static float apply(float a, float) { return relu1(a); }
};
struct OpAdd {
    static constexpr int kInputs = 2;
    __device__ __forceinline__ static float apply(float a, float b) { return a + b; }
};
struct OpAddRelu {
    static constexpr int kInputs = 2;
    __device__ __forceinline__ static float apply(float a, float b) { return relu1(a + b); }
};
struct OpTanh {  // kernels.h:62, all fp32
    static constexpr int kInputs = 1;
    __device__ __forceinline__ static float apply(float a, float) {
        return 1.f - 2.f / (expf(a * 2.f) + 1.f);
    }
};

template <class Op>
__device__ __forceinline__ float4 apply4(float4 a, float4 b) {
    return make_float4(Op::apply(a.x, b.x), Op::apply(a.y, b.y), Op::apply(a.z, b.z), Op::apply(a.w, b.w));
}

// n4 = number of whole float4; elements [4*n4, n) are the scalar tail, done by block 0.
template <class Op, bool NT>
__global__ __launch_bounds__(kThreads) void flat_vec4(const float *a, const float *b,
                                                      float *out, size_t n4, size_t n) {
    const float4 *a4 = reinterpret_cast<const float4 *>(a);
    const float4 *b4 = reinterpret_cast<const float4 *>(b);
    float4 *o4 = reinterpret_cast<float4 *>(out);
    const size_t base = (size_t)blockIdx.x * (kThreads * kUnroll) + threadIdx.x;
    float4 va[kUnroll], vb[kUnroll];
#pragma unroll
    for (int u = 0; u < kUnroll; ++u) {
        const size_t i = base + (size_t)u * kThreads;
        if (i < n4) {
            va[u] = ld4<NT>(a4 + i);
            if (Op::kInputs == 2) vb[u] = ld4<NT>(b4 + i);
        }
    }
#pragma unroll
    for (int u = 0; u < kUnroll; ++u) {
        const size_t i = base + (size_t)u * kThreads;
        if (i < n4) st4<NT>(o4 + i, apply4<Op>(va[u], Op::kInputs == 2 ? vb[u] : va[u]));
    }
    if (blockIdx.x == 0) {
        const size_t i = n4 * 4 + threadIdx.x;
        if (i < n) out[i] = Op::apply(a[i], Op::kInputs == 2 ? b[i] : 0.f);
    }
}

// any alignment
template <class Op>
__global__ __launch_bounds__(kThreads) void flat_scalar(const float *a, const float *b,
                                                        float *out, size_t n) {
    size_t i = (size_t)blockIdx.x * kThreads + threadIdx.x;
    const size_t step = (size_t)gridDim.x * kThreads;
    for (; i < n; i += step) out[i] = Op::apply(a[i], Op::kInputs == 2 ? b[i] : 0.f);
}

template <class Op>
int launch_flat(const char *who, const float *a, const float *b, float *out, size_t n) {
    if (n == 0) return SWC_HIP_OK;
    if (!a || !out || (Op::kInputs == 2 && !b)) return fail(SWC_HIP_EINVAL, "%s: null pointer", who);
    if (!b) b = a;
    if (aligned16(a) && aligned16(b) && aligned16(out) && n >= 4) {
        const size_t n4 = n / 4;
        const size_t blocks = (n4 + (size_t)kThreads * kUnroll - 1) / ((size_t)kThreads * kUnroll);
        if (blocks > 0x7fffffffu) return fail(SWC_HIP_EINVAL, "%s: size %zu too large", who, n);
        if (n * sizeof(float) >= kStreamingBytes)
            flat_vec4<Op, true><<<(unsigned)blocks, kThreads, 0, stream()>>>(a, b, out, n4, n);
        else
            flat_vec4<Op, false><<<(unsigned)blocks, kThreads, 0, stream()>>>(a, b, out, n4, n);
    } else {
        size_t blocks = (n + kThreads - 1) / kThreads;
        if (blocks > 65536) blocks = 65536;
        flat_scalar<Op><<<(unsigned)blocks, kThreads, 0, stream()>>>(a, b, out, n);
    }
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) return fail(SWC_HIP_ERUNTIME, "%s: launch failed: %s", who, hipGetErrorString(e));
    return SWC_HIP_OK;
}

// dest[r, j] = batch[r, j] + slice[j].  cols % 4 == 0 and 16-byte aligned:
// thread t of a block owns column quad (t % quads) and walks rows.
__global__ __launch_bounds__(kThreads) void batchedadd_vec4(float *dest, const float *batch,
                                                            const float *__restrict__ slice, size_t total4,
                                                            unsigned quads) {
    const float4 *b4 = reinterpret_cast<const float4 *>(batch);
    const float4 *s4 = reinterpret_cast<const float4 *>(slice);
    float4 *d4 = reinterpret_cast<float4 *>(dest);
    size_t i = (size_t)blockIdx.x * kThreads + threadIdx.x;
    const size_t step = (size_t)gridDim.x * kThreads;
    for (; i < total4; i += step) {
        const float4 s = s4[i % quads];
        const float4 v = b4[i];
        d4[i] = make_float4(v.x + s.x, v.y + s.y, v.z + s.z, v.w + s.w);
    }
}

__global__ __launch_bounds__(kThreads) void batchedadd_scalar(float *dest, const float *batch,
                                                              const float *__restrict__ slice, size_t total,
                                                              size_t cols) {
    size_t i = (size_t)blockIdx.x * kThreads + threadIdx.x;
    const size_t step = (size_t)gridDim.x * kThreads;
    for (; i < total; i += step) dest[i] = batch[i] + slice[i % cols];
}

} // namespace

extern "C" {

int swc_hip_relu_f(const float *src, float *dest, size_t size) {
    SWC_REQUIRE_INIT();
    return launch_flat<OpRelu>("swc_hip_relu_f", src, nullptr, dest, size);
}

int swc_hip_vecAdd_f(int size, const float *a, const float *b, float *c) {
    SWC_REQUIRE_INIT();
    SWC_ARG(size >= 0);
    return launch_flat<OpAdd>("swc_hip_vecAdd_f", a, b, c, (size_t)size);
}

int swc_hip_vecAddRelu_f(int size, const float *a, const float *b, float *c) {
    SWC_REQUIRE_INIT();
    SWC_ARG(size >= 0);
    return launch_flat<OpAddRelu>("swc_hip_vecAddRelu_f", a, b, c, (size_t)size);
}

int swc_hip_matrixTanh_f(int m, int n, const float *a, int lda, float *b, int ldb) {
    SWC_REQUIRE_INIT();
    SWC_ARG(m >= 0 && n >= 0 && lda >= n && ldb >= n);
    if (lda != n || ldb != n)
        return fail(SWC_HIP_EUNSUPPORTED, "swc_hip_matrixTanh_f: only dense rows (lda == ldb == n) are supported");
    return launch_flat<OpTanh>("swc_hip_matrixTanh_f", a, nullptr, b, (size_t)m * n);
}

int swc_hip_batchedadd_f(float *dest, const float *batch, const float *slice, size_t numSlice, size_t sliceSize) {
    SWC_REQUIRE_INIT();
    const size_t total = numSlice * sliceSize;
    if (total == 0) return SWC_HIP_OK;
    SWC_ARG(dest && batch && slice);
    if (sliceSize % 4 == 0 && aligned16(dest) && aligned16(batch) && aligned16(slice)) {
        const size_t total4 = total / 4;
        size_t blocks = (total4 + kThreads - 1) / kThreads;
        if (blocks > 16384) blocks = 16384;
        batchedadd_vec4<<<(unsigned)blocks, kThreads, 0, stream()>>>(dest, batch, slice, total4, (unsigned)(sliceSize / 4));
    } else {
        size_t blocks = (total + kThreads - 1) / kThreads;
        if (blocks > 16384) blocks = 16384;
        batchedadd_scalar<<<(unsigned)blocks, kThreads, 0, stream()>>>(dest, batch, slice, total, sliceSize);
    }
    SWC_LAUNCH_CHECK();
    return SWC_HIP_OK;
}

} // extern "C"
