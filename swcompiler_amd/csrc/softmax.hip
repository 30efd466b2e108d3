// matrixSoftmax_f (kernels.h:88-103), argMax_i (kernels.h:601-613) and accuracy_i (kernels.h:615-627).
//
// Softmax is one read and one write of the matrix (8 B/element): a 64-lane
// wavefront owns a row, keeps it in registers as float4s, and reduces the row
// maximum and the row sum with cross-lane shuffles; no LDS, no second read.
// Rows that do not fit that scheme (n not a multiple of 4, unaligned, or more
// than 64*4*kMaxVec columns) take the strided three-pass kernel, whose re-reads
// hit cache because one row is a few KB.
#include "common.hpp"

using namespace swc_hip;

namespace {

constexpr int kWave = 64;
constexpr int kRowsPerBlock = 4;  // wavefronts per block

__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) v = fmaxf(v, __shfl_xor(v, off, kWave));
    return v;
}
__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) v += __shfl_xor(v, off, kWave);
    return v;
}

// VEC = float4s per lane; row length n = 4*n4 with n4 <= 64*VEC.
template <int VEC, bool NT>
__global__ __launch_bounds__(kWave *kRowsPerBlock) void softmax_rows_reg(const float *a, float *b, int m, int n4,
                                                                         size_t lda, size_t ldb) {
    const int lane = threadIdx.x & (kWave - 1);
    const int row = blockIdx.x * kRowsPerBlock + (threadIdx.x >> 6);
    if (row >= m) return;
    const float4 *src = reinterpret_cast<const float4 *>(a + (size_t)row * lda);
    float4 *dst = reinterpret_cast<float4 *>(b + (size_t)row * ldb);
    float4 v[VEC];
    const float ninf = -__builtin_inff();
#pragma unroll
    for (int u = 0; u < VEC; ++u) {
        const int i = lane + u * kWave;
        v[u] = (i < n4) ? ld4<NT>(src + i) : make_float4(ninf, ninf, ninf, ninf);
    }
    float mx = ninf;
#pragma unroll
    for (int u = 0; u < VEC; ++u) mx = fmaxf(fmaxf(fmaxf(v[u].x, v[u].y), fmaxf(v[u].z, v[u].w)), mx);
    mx = wave_max(mx);
    float s = 0.f;
#pragma unroll
    for (int u = 0; u < VEC; ++u) {
        v[u].x = fast_exp(v[u].x - mx);
        v[u].y = fast_exp(v[u].y - mx);
        v[u].z = fast_exp(v[u].z - mx);
        v[u].w = fast_exp(v[u].w - mx);
        s += (v[u].x + v[u].y) + (v[u].z + v[u].w);   // padding lanes hold exp(-inf) = 0
    }
    s = wave_sum(s);
    const float inv = 1.f / s;
#pragma unroll
    for (int u = 0; u < VEC; ++u) {
        const int i = lane + u * kWave;
        if (i < n4) st4<NT>(dst + i, make_float4(v[u].x * inv, v[u].y * inv, v[u].z * inv, v[u].w * inv));
    }
}

// any n, any alignment: wave per row, strided scalar accesses, three passes.
__global__ __launch_bounds__(kWave *kRowsPerBlock) void softmax_rows_strided(const float *a, float *b, int m, int n,
                                                                             size_t lda, size_t ldb) {
    const int lane = threadIdx.x & (kWave - 1);
    const int row = blockIdx.x * kRowsPerBlock + (threadIdx.x >> 6);
    if (row >= m) return;
    const float *src = a + (size_t)row * lda;
    float *dst = b + (size_t)row * ldb;
    float mx = -__builtin_inff();
    for (int j = lane; j < n; j += kWave) mx = fmaxf(mx, src[j]);
    mx = wave_max(mx);
    float s = 0.f;
    for (int j = lane; j < n; j += kWave) s += fast_exp(src[j] - mx);
    s = wave_sum(s);
    const float inv = 1.f / s;
    for (int j = lane; j < n; j += kWave) dst[j] = fast_exp(src[j] - mx) * inv;
}

// Small n (the classifier heads, n = 10): one lane per row would waste the
// wave on strided loads; here a block stages 256 rows through registers with
// each lane owning one row, which is fine because the whole matrix is tiny.
__global__ __launch_bounds__(256) void softmax_rows_small(const float *a, float *b, int m, int n, size_t lda,
                                                          size_t ldb) {
    const int row = blockIdx.x * 256 + threadIdx.x;
    if (row >= m) return;
    const float *src = a + (size_t)row * lda;
    float *dst = b + (size_t)row * ldb;
    float mx = src[0];
    for (int j = 1; j < n; ++j) mx = fmaxf(mx, src[j]);
    float s = 0.f;
    for (int j = 0; j < n; ++j) s += fast_exp(src[j] - mx);
    const float inv = 1.f / s;
    for (int j = 0; j < n; ++j) dst[j] = fast_exp(src[j] - mx) * inv;
}

// argMax_i: one lane per row; top_k <= 8 kept sorted in registers.  Order is
// descending (value, column): a later column with an equal value goes first.
constexpr int kMaxTopK = 8;
__global__ __launch_bounds__(256) void argmax_rows(const float *in, int *idx, int m, int n, int top_k) {
    const int row = blockIdx.x * 256 + threadIdx.x;
    if (row >= m) return;
    const float *src = in + (size_t)row * n;
    float bv[kMaxTopK];
    int bi[kMaxTopK];
    int have = 0;
    for (int j = 0; j < n; ++j) {
        const float v = src[j];
        // position of (v, j) among the kept ones
        int pos = have;
        for (int t = have - 1; t >= 0; --t) {
            // (v,j) precedes (bv[t],bi[t]) when v > bv[t], or equal (j is always the larger column)
            if (v > bv[t] || v == bv[t]) pos = t;
            else break;
        }
        if (pos >= top_k) continue;
        const int last = (have < top_k) ? have : top_k - 1;
        for (int t = last; t > pos; --t) {
            bv[t] = bv[t - 1];
            bi[t] = bi[t - 1];
        }
        bv[pos] = v;
        bi[pos] = j;
        if (have < top_k) ++have;
    }
    for (int t = 0; t < top_k; ++t) idx[(size_t)row * top_k + t] = (t < have) ? bi[t] : 0;
}

// The same for long rows (a thousand classes): a wavefront per row.  Lane l keeps the top_k of columns l, l+64,
// ... as above; then top_k rounds pick the best head among the 64 lanes (descending (value, column)) and the
// lane that held it moves on to its next entry.
__device__ __forceinline__ bool goes_first(float v, int j, bool valid, float w, int i, bool wvalid) {
    if (!wvalid) return valid;
    if (!valid) return false;
    return v > w || (v == w && j > i);
}

__global__ __launch_bounds__(256) void argmax_rows_wave(const float *in, int *idx, int m, int n, int top_k) {
    const int lane = threadIdx.x & 63;
    const int row = blockIdx.x * 4 + (threadIdx.x >> 6);
    if (row >= m) return;   // whole wavefronts leave together
    const float *src = in + (size_t)row * n;
    float bv[kMaxTopK];
    int bi[kMaxTopK];
#pragma unroll
    for (int t = 0; t < kMaxTopK; ++t) bv[t] = 0.f, bi[t] = 0;
    int have = 0;
    for (int j = lane; j < n; j += 64) {
        const float v = src[j];
        // position among the kept ones; (v, j) precedes an equal value (j is the larger column)
        int pos = 0;
#pragma unroll
        for (int t = 0; t < kMaxTopK; ++t) pos += (t < have && !(v > bv[t] || v == bv[t])) ? 1 : 0;
        if (pos >= top_k) continue;
#pragma unroll
        for (int t = kMaxTopK - 1; t > 0; --t)
            if (t > pos) bv[t] = bv[t - 1], bi[t] = bi[t - 1];
#pragma unroll
        for (int t = 0; t < kMaxTopK; ++t)
            if (t == pos) bv[t] = v, bi[t] = j;
        if (have < top_k) ++have;
    }
    for (int t = 0; t < top_k; ++t) {
        float v = bv[0];
        int j = bi[0];
        bool valid = have > 0;
#pragma unroll
        for (int off = 32; off > 0; off >>= 1) {
            const float w = __shfl_xor(v, off);
            const int i = __shfl_xor(j, off);
            const bool wvalid = __shfl_xor((int)valid, off) != 0;
            if (goes_first(w, i, wvalid, v, j, valid)) v = w, j = i, valid = wvalid;
        }
        if (lane == 0) idx[(size_t)row * top_k + t] = valid ? j : 0;
        if (have > 0 && bi[0] == j) {   // this lane held the winner (columns are distinct across lanes): next entry
#pragma unroll
            for (int u = 0; u < kMaxTopK - 1; ++u) bv[u] = bv[u + 1], bi[u] = bi[u + 1];
            --have;
        }
    }
}

// accuracy_i: one lane per row looks for its label among the row's n predictions; the workgroup's count of
// hits and its row count go to the two counters with one integer atomic each, so repeated calls accumulate
// exactly as the host loop does, in any order.
__global__ __launch_bounds__(256) void accuracy_rows(const int *pred, const int *label, int *accum, int m, int n) {
    const int row = blockIdx.x * 256 + threadIdx.x;
    int hit = 0;
    if (row < m) {
        const int want = label[row];
        for (int j = 0; j < n; ++j) hit |= pred[(size_t)row * n + j] == want;
    }
    const int hits = __syncthreads_count(hit);
    if (threadIdx.x == 0) {
        const int rows = min(256, m - (int)blockIdx.x * 256);
        if (hits) atomicAdd(accum, hits);
        atomicAdd(accum + 1, rows);
    }
}

} // namespace

extern "C" {

int swc_hip_matrixSoftmax_f(int m, int n, const float *a, int lda, float *b, int ldb) {
    SWC_REQUIRE_INIT();
    SWC_ARG(m >= 0 && n >= 0);
    if (m == 0 || n == 0) return SWC_HIP_OK;
    SWC_ARG(a && b && lda >= n && ldb >= n);
    hipStream_t s = stream();
    const bool vec_ok = (n % 4 == 0) && (lda % 4 == 0) && (ldb % 4 == 0) && aligned16(a) && aligned16(b);
    const int n4 = n / 4;
    if (n <= 32) {
        softmax_rows_small<<<ceil_div(m, 256), 256, 0, s>>>(a, b, m, n, lda, ldb);
    } else if (vec_ok && n4 <= kWave * 8) {
        const unsigned blocks = ceil_div(m, kRowsPerBlock);
        const dim3 block(kWave * kRowsPerBlock);
        const bool nt = (size_t)m * n * sizeof(float) >= kStreamingBytes;
#define SWC_SOFTMAX_LAUNCH(V)                                                                       \
    do {                                                                                            \
        if (nt) softmax_rows_reg<V, true><<<blocks, block, 0, s>>>(a, b, m, n4, lda, ldb);          \
        else softmax_rows_reg<V, false><<<blocks, block, 0, s>>>(a, b, m, n4, lda, ldb);            \
    } while (0)
        if (n4 <= kWave * 1) SWC_SOFTMAX_LAUNCH(1);
        else if (n4 <= kWave * 2) SWC_SOFTMAX_LAUNCH(2);
        else if (n4 <= kWave * 4) SWC_SOFTMAX_LAUNCH(4);
        else SWC_SOFTMAX_LAUNCH(8);
#undef SWC_SOFTMAX_LAUNCH
    } else {
        softmax_rows_strided<<<ceil_div(m, kRowsPerBlock), kWave * kRowsPerBlock, 0, s>>>(a, b, m, n, lda, ldb);
    }
    SWC_LAUNCH_CHECK();
    return SWC_HIP_OK;
}

int swc_hip_argMax_i(const float *input, int *idx, int m, int n, int top_k) {
    SWC_REQUIRE_INIT();
    SWC_ARG(m >= 0 && n >= 0 && top_k >= 0);
    if (m == 0 || top_k == 0) return SWC_HIP_OK;
    SWC_ARG(input && idx && top_k <= n);
    if (top_k > kMaxTopK)
        return fail(SWC_HIP_EUNSUPPORTED, "swc_hip_argMax_i: top_k %d exceeds %d", top_k, kMaxTopK);
    if (n >= 128) argmax_rows_wave<<<ceil_div(m, 4), 256, 0, stream()>>>(input, idx, m, n, top_k);
    else argmax_rows<<<ceil_div(m, 256), 256, 0, stream()>>>(input, idx, m, n, top_k);
    SWC_LAUNCH_CHECK();
    return SWC_HIP_OK;
}

int swc_hip_accuracy_i(const int *pred, const int *label, int *accum_cnt, int m, int n) {
    SWC_REQUIRE_INIT();
    SWC_ARG(m >= 0 && n >= 0);
    if (m == 0) return SWC_HIP_OK;
    SWC_ARG(label && accum_cnt && (n == 0 || pred));
    accuracy_rows<<<ceil_div(m, 256), 256, 0, stream()>>>(pred, label, accum_cnt, m, n);
    SWC_LAUNCH_CHECK();
    return SWC_HIP_OK;
}

} // extern "C"
