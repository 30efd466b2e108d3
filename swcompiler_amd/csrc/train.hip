// The kernels a generated TRAINING program calls next to the inference ones,
// except the convolution gradient (conv.hip): matrixTrans_f,
// matrixTanhGrad_f, matrixSoftmaxWithLoss_f, matrixSoftmax[WithLoss]Grad_f,
// maxpoolGrad_f, batchedreduceadd_f, sgd_f, reluGrad_f
// (src/codegen/utils/kernels.h:68-86, 105-151, 380-442, 554-573, 586-590).
//
// All but the loss are bit-exact with the reference: element-wise kernels use
// the reference's operation sequence with contraction into FMA switched off
// (the reference is built for x86-64 without FMA), and the two kernels that
// accumulate (row sums, pooling gradient) add in the reference's order.
#include "common.hpp"

using namespace swc_hip;

namespace {

constexpr int kThreads = 256;

inline unsigned grid_for(size_t n, size_t per_block, unsigned cap = 65536) {
    const size_t b = (n + per_block - 1) / per_block;
    return (unsigned)(b > cap ? cap : (b ? b : 1));
}

// ------------------------------------------------------------- element-wise
// kernels.h:586-590
__global__ __launch_bounds__(kThreads) void relu_grad(float *sg, const float *src, const float *dg, size_t n) {
    size_t i = (size_t)blockIdx.x * kThreads + threadIdx.x;
    const size_t step = (size_t)gridDim.x * kThreads;
    for (; i < n; i += step) sg[i] = (src[i] > 0.f) ? dg[i] : 0.f;
}
template <bool NT>
__global__ __launch_bounds__(kThreads) void relu_grad4(float4 *sg, const float4 *src, const float4 *dg, size_t n4) {
    const size_t i = (size_t)blockIdx.x * kThreads + threadIdx.x;
    if (i >= n4) return;
    const float4 s = ld4<NT>(src + i), d = ld4<NT>(dg + i);
    st4<NT>(sg + i, make_float4(s.x > 0.f ? d.x : 0.f, s.y > 0.f ? d.y : 0.f, s.z > 0.f ? d.z : 0.f,
                                s.w > 0.f ? d.w : 0.f));
}

// kernels.h:79-86: fl(fl(1 - fl(b*b)) * c)
__global__ __launch_bounds__(kThreads) void tanh_grad(int m, int n, float *a, size_t lda, const float *b, size_t ldb,
                                                      const float *c, size_t ldc) {
#pragma clang fp contract(off)
    const size_t total = (size_t)m * n;
    size_t i = (size_t)blockIdx.x * kThreads + threadIdx.x;
    const size_t step = (size_t)gridDim.x * kThreads;
    for (; i < total; i += step) {
        const size_t r = i / n, j = i - r * n;
        const float bb = b[r * ldb + j];
        const float sq = bb * bb;
        const float one_minus = 1.f - sq;
        a[r * lda + j] = one_minus * c[r * ldc + j];
    }
}

// kernels.h:133-151: a = b - (selected[row] == col)
__global__ __launch_bounds__(kThreads) void softmax_grad(int m, int n, float *a, size_t lda, const float *b, size_t ldb,
                                                         const int *__restrict__ selected) {
    const size_t total = (size_t)m * n;
    size_t i = (size_t)blockIdx.x * kThreads + threadIdx.x;
    const size_t step = (size_t)gridDim.x * kThreads;
    for (; i < total; i += step) {
        const size_t r = i / n, j = i - r * n;
        const float delta = (selected[r] == (int)j) ? 1.f : 0.f;
        a[r * lda + j] = b[r * ldb + j] - delta;
    }
}

// kernels.h:565-573.  out may be w (the generated call passes the same tensor).
__global__ __launch_bounds__(kThreads) void sgd_step(size_t n, float *out, const float *w, const float *dw, float *mom,
                                                     float neglr, float decay, float momentum) {
#pragma clang fp contract(off)
    size_t i = (size_t)blockIdx.x * kThreads + threadIdx.x;
    const size_t step = (size_t)gridDim.x * kThreads;
    for (; i < n; i += step) {
        const float wd = w[i] * decay;
        const float g = wd + dw[i];
        const float t0 = g * neglr;
        const float t1 = mom[i] * momentum;
        const float neg_delta = t0 + t1;
        mom[i] = neg_delta;
        out[i] = out[i] + neg_delta;
    }
}

// The same four elements at a time; out == w (the generated call) is read once.
template <bool NT, bool IN_PLACE>
__global__ __launch_bounds__(kThreads) void sgd_step4(size_t n4, float4 *out, const float4 *w, const float4 *dw,
                                                      float4 *mom, float neglr, float decay, float momentum) {
#pragma clang fp contract(off)
    const size_t i = (size_t)blockIdx.x * kThreads + threadIdx.x;
    if (i >= n4) return;
    const float4 wv = ld4<NT>(w + i), gv = ld4<NT>(dw + i), mv = ld4<NT>(mom + i);
    const float4 ov = IN_PLACE ? wv : ld4<NT>(out + i);
    const float wa[4] = {wv.x, wv.y, wv.z, wv.w}, ga[4] = {gv.x, gv.y, gv.z, gv.w}, ma[4] = {mv.x, mv.y, mv.z, mv.w};
    const float oa[4] = {ov.x, ov.y, ov.z, ov.w};
    float nm[4], no[4];
#pragma unroll
    for (int e = 0; e < 4; ++e) {
        const float wd = wa[e] * decay;
        const float g = wd + ga[e];
        const float t0 = g * neglr;
        const float t1 = ma[e] * momentum;
        nm[e] = t0 + t1;
        no[e] = oa[e] + nm[e];
    }
    st4<NT>(mom + i, make_float4(nm[0], nm[1], nm[2], nm[3]));
    st4<NT>(out + i, make_float4(no[0], no[1], no[2], no[3]));
}

// kernels.h:68-76: B[n,m] = A[m,n]^T through a 32x33 LDS tile (coalesced on both sides)
__global__ __launch_bounds__(256) void matrix_trans(int m, int n, const float *__restrict__ a, size_t lda,
                                                    float *__restrict__ b, size_t ldb) {
    __shared__ float tile[32][33];
    const int tx = threadIdx.x & 31, ty = threadIdx.x >> 5;   // 32 x 8
    const int r0 = blockIdx.y * 32, c0 = blockIdx.x * 32;
#pragma unroll
    for (int k = 0; k < 4; ++k) {
        const int r = r0 + ty + 8 * k, c = c0 + tx;
        if (r < m && c < n) tile[ty + 8 * k][tx] = a[(size_t)r * lda + c];
    }
    __syncthreads();
#pragma unroll
    for (int k = 0; k < 4; ++k) {
        const int c = c0 + ty + 8 * k, r = r0 + tx;   // output row c, column r
        if (c < n && r < m) b[(size_t)c * ldb + r] = tile[tx][ty + 8 * k];
    }
}

// --------------------------------------------------------------- row sums
// kernels.h:554-563: dest[row] = sum of the row's sliceSize floats IN ORDER.
// A workgroup owns 64 rows; 64x64 tiles are staged through LDS with coalesced
// loads, then thread r adds the 64 values of row r one after the other — the
// reference's order, hence the reference's bits.
__global__ __launch_bounds__(kThreads) void row_sums(float *__restrict__ dest, const float *__restrict__ batch,
                                                     size_t rows, size_t cols) {
#pragma clang fp contract(off)
    __shared__ float tile[64][65];
    const size_t r0 = (size_t)blockIdx.x * 64;
    const int tx = threadIdx.x & 63, ty = threadIdx.x >> 6;   // 64 x 4
    float sum = 0.f;
    for (size_t c0 = 0; c0 < cols; c0 += 64) {
#pragma unroll
        for (int k = 0; k < 16; ++k) {
            const size_t r = r0 + ty + 4 * k, c = c0 + tx;
            tile[ty + 4 * k][tx] = (r < rows && c < cols) ? batch[r * cols + c] : 0.f;
        }
        __syncthreads();
        if (threadIdx.x < 64) {
            if (cols - c0 >= 64) {
                float v[64];
#pragma unroll
                for (int j = 0; j < 64; ++j) v[j] = tile[threadIdx.x][j];   // independent reads first ...
#pragma unroll
                for (int j = 0; j < 64; ++j) sum = sum + v[j];              // ... then the adds, in order
            } else {
                const int lim = (int)(cols - c0);
                for (int j = 0; j < lim; ++j) sum = sum + tile[threadIdx.x][j];
            }
        }
        __syncthreads();
    }
    if (threadIdx.x < 64 && r0 + threadIdx.x < rows) dest[r0 + threadIdx.x] = sum;
}

// ----------------------------------------------------- softmax with loss
// Per row: max, sum of expf(a - max) (wavefront reduction), and the row's loss
// term logf(sum * expf(max)) - a[selected] exactly as kernels.h:123 writes it.
__global__ __launch_bounds__(kThreads) void softmax_loss_terms(int m, int n, const float *__restrict__ a, size_t lda,
                                                               const int *__restrict__ selected,
                                                               float *__restrict__ terms) {
    const int lane = threadIdx.x & 63;
    const int row = blockIdx.x * (kThreads / 64) + (threadIdx.x >> 6);
    if (row >= m) return;
    const float *ar = a + (size_t)row * lda;
    float mx = ar[0];
    for (int j = lane; j < n; j += 64) mx = fmaxf(mx, ar[j]);
    for (int off = 32; off; off >>= 1) mx = fmaxf(mx, __shfl_xor(mx, off));
    float sum = 0.f;
    for (int j = lane; j < n; j += 64) sum += expf(ar[j] - mx);
    for (int off = 32; off; off >>= 1) sum += __shfl_xor(sum, off);
    if (lane == 0) terms[row] = logf(sum * expf(mx)) - ar[selected[row]];
}

// loss = (sum of the terms) / m in fp32 — one workgroup, a fixed order: thread t adds terms t, t+1024, ...,
// then the 1024 partial sums are halved ten times.  (The reference adds row after row; the terms already
// differ from its in the last bits through expf/logf, so the loss is held to a relative tolerance.)
__global__ __launch_bounds__(1024) void loss_mean(int m, const float *__restrict__ terms, float *__restrict__ loss) {
    __shared__ float red[1024];
    float sum = 0.f;
    for (int i = threadIdx.x; i < m; i += 1024) sum += terms[i];
    red[threadIdx.x] = sum;
    __syncthreads();
    for (int s = 512; s > 0; s >>= 1) {
        if ((int)threadIdx.x < s) red[threadIdx.x] += red[threadIdx.x + s];
        __syncthreads();
    }
    if (threadIdx.x == 0) *loss = red[0] / (float)m;
}

// ------------------------------------------------------ pooling gradient
struct PoolGeom {
    int N, H, W, C, OH, OW, kh, kw, sh, sw, pt, pl;
};

// One thread per INPUT element (VEC = 1) or per four consecutive channels of an
// input pixel (VEC = 4, 128-bit accesses): it visits, in the reference's
// (oy, ox) order, the windows that can select it and adds their gradients — a
// gather, so the sum is formed in the same order as the reference's scatter and
// needs no atomics.  Element (0,0) of every image also collects the windows that
// have no in-bounds tap when the geometry allows such windows (empty_windows).
template <int VEC>
__global__ __launch_bounds__(kThreads) void maxpool_grad(float *__restrict__ ig, const float *__restrict__ og,
                                                         const float *__restrict__ in, PoolGeom g, int empty_windows,
                                                         int row_base) {
#pragma clang fp contract(off)
    // row_base + blockIdx.y = image row (n*H + iy); blockIdx.x, threadIdx.x walk the row's W * C/VEC items: 32-bit index arithmetic
    const int cq = g.C / VEC;
    const int row_items = g.W * cq;
    const int image_row = row_base + blockIdx.y;
    const int iy = image_row % g.H, n = image_row / g.H;
    for (int item = blockIdx.x * kThreads + threadIdx.x; item < row_items; item += gridDim.x * kThreads) {
        const int ix = item / cq;
        const int c = (item - ix * cq) * VEC;
        float sum[VEC];
#pragma unroll
        for (int v = 0; v < VEC; ++v) sum[v] = 0.f;
        int oy_lo, oy_hi, ox_lo, ox_hi;
        if (empty_windows && iy == 0 && ix == 0) {
            oy_lo = 0, oy_hi = g.OH - 1, ox_lo = 0, ox_hi = g.OW - 1;
        } else {
            // windows with oy*sh - pt <= iy <= oy*sh - pt + kh - 1
            const int ay = iy + g.pt, ax = ix + g.pl;
            oy_lo = ay - g.kh + 1 <= 0 ? 0 : (ay - g.kh + 1 + g.sh - 1) / g.sh;
            oy_hi = ay / g.sh < g.OH - 1 ? ay / g.sh : g.OH - 1;
            ox_lo = ax - g.kw + 1 <= 0 ? 0 : (ax - g.kw + 1 + g.sw - 1) / g.sw;
            ox_hi = ax / g.sw < g.OW - 1 ? ax / g.sw : g.OW - 1;
        }
        for (int oy = oy_lo; oy <= oy_hi; ++oy)
            for (int ox = ox_lo; ox <= ox_hi; ++ox) {
                // the window's choice per channel: first maximum in (ky, kx) scan order among the in-bounds
                // taps; (0, 0) when no tap is in bounds, as the reference's initial max_ix = max_iy = 0
                bool uninit = true;
                float mx[VEC];
                int cy[VEC], cx[VEC];
#pragma unroll
                for (int v = 0; v < VEC; ++v) mx[v] = 0.f, cy[v] = 0, cx[v] = 0;
                for (int ky = 0; ky < g.kh; ++ky) {
                    const int wy = oy * g.sh - g.pt + ky;
                    if ((unsigned)wy >= (unsigned)g.H) continue;
                    for (int kx = 0; kx < g.kw; ++kx) {
                        const int wx = ox * g.sw - g.pl + kx;
                        if ((unsigned)wx >= (unsigned)g.W) continue;
                        const float *p = in + (((size_t)n * g.H + wy) * g.W + wx) * g.C + c;
                        float val[VEC];
                        if (VEC == 4) {
                            const float4 q = *reinterpret_cast<const float4 *>(p);
                            val[0] = q.x, val[VEC > 1 ? 1 : 0] = q.y, val[VEC > 2 ? 2 : 0] = q.z, val[VEC > 3 ? 3 : 0] = q.w;
                        } else {
                            val[0] = *p;
                        }
#pragma unroll
                        for (int v = 0; v < VEC; ++v)
                            if (uninit || val[v] > mx[v]) mx[v] = val[v], cy[v] = wy, cx[v] = wx;
                        uninit = false;
                    }
                }
                const float *gp = og + (((size_t)n * g.OH + oy) * g.OW + ox) * g.C + c;
                float gv[VEC];
                if (VEC == 4) {
                    const float4 q = *reinterpret_cast<const float4 *>(gp);
                    gv[0] = q.x, gv[VEC > 1 ? 1 : 0] = q.y, gv[VEC > 2 ? 2 : 0] = q.z, gv[VEC > 3 ? 3 : 0] = q.w;
                } else {
                    gv[0] = *gp;
                }
#pragma unroll
                for (int v = 0; v < VEC; ++v)
                    if (cy[v] == iy && cx[v] == ix) sum[v] = sum[v] + gv[v];
            }
        float *op = ig + (((size_t)n * g.H + iy) * g.W + ix) * g.C + c;
        if (VEC == 4) *reinterpret_cast<float4 *>(op) = make_float4(sum[0], sum[VEC > 1 ? 1 : 0], sum[VEC > 2 ? 2 : 0], sum[VEC > 3 ? 3 : 0]);
        else *op = sum[0];
    }
}

// Windows that tile the image exactly (stride = kernel, no padding, H = OH*kh, W = OW*kw): every input
// element lies in exactly one window, so one thread per window and channel quad reads its taps once, finds
// the first maximum in the reference's scan order and writes the whole window of the gradient — outputG at
// the chosen tap, zeros at the others.  item = (image row of windows, ox, channel quad).
// KH, KW > 0: the window size as a constant (all taps are loaded before the first comparison); 0: g.kh, g.kw.
template <bool NT, int KH, int KW>
__global__ __launch_bounds__(kThreads) void maxpool_grad_tiled(float *__restrict__ ig, const float *__restrict__ og,
                                                               const float *__restrict__ in, PoolGeom g, int row_base) {
    const int cq = g.C / 4;
    const int row_items = g.OW * cq;
    const int item = blockIdx.x * kThreads + threadIdx.x;
    if (item >= row_items) return;
    const int window_row = row_base + blockIdx.y;   // n*OH + oy
    const int oy = window_row % g.OH, n = window_row / g.OH;
    const int ox = item / cq;
    const int c = (item - ox * cq) * 4;
    const size_t first = (((size_t)n * g.H + (size_t)oy * g.kh) * g.W + (size_t)ox * g.kw) * g.C + c;   // tap (0,0)
    const size_t row_pitch = (size_t)g.W * g.C;
    const int kh = KH ? KH : g.kh, kw = KW ? KW : g.kw;
    const float4 gq = ld4<NT>(reinterpret_cast<const float4 *>(og + ((size_t)window_row * g.OW + ox) * g.C + c));
    float mx[4];
    int chosen[4] = {0, 0, 0, 0};
    if (KH) {
        float4 q[KH ? KH * KW : 1];
#pragma unroll
        for (int tap = 0; tap < KH * KW; ++tap)
            q[tap] = ld4<NT>(reinterpret_cast<const float4 *>(in + first + (tap / (KW ? KW : 1)) * row_pitch +
                                                              (size_t)(tap % (KW ? KW : 1)) * g.C));
#pragma unroll
        for (int tap = 0; tap < KH * KW; ++tap) {
            const float val[4] = {q[tap].x, q[tap].y, q[tap].z, q[tap].w};
#pragma unroll
            for (int v = 0; v < 4; ++v)
                if (tap == 0 || val[v] > mx[v]) mx[v] = val[v], chosen[v] = tap;
        }
    } else {
        for (int ky = 0; ky < kh; ++ky)
            for (int kx = 0; kx < kw; ++kx) {
                const float4 q = ld4<NT>(reinterpret_cast<const float4 *>(in + first + ky * row_pitch + (size_t)kx * g.C));
                const float val[4] = {q.x, q.y, q.z, q.w};
                const int tap = ky * kw + kx;
#pragma unroll
                for (int v = 0; v < 4; ++v)
                    if (tap == 0 || val[v] > mx[v]) mx[v] = val[v], chosen[v] = tap;
            }
    }
    const float gv[4] = {gq.x, gq.y, gq.z, gq.w};
    for (int ky = 0; ky < kh; ++ky)
        for (int kx = 0; kx < kw; ++kx) {
            const int tap = ky * kw + kx;
            // 0.f + outputG as the reference's "+=" into a zeroed gradient forms it (a -0 becomes +0)
            st4<NT>(reinterpret_cast<float4 *>(ig + first + ky * row_pitch + (size_t)kx * g.C),
                    make_float4(chosen[0] == tap ? 0.f + gv[0] : 0.f, chosen[1] == tap ? 0.f + gv[1] : 0.f,
                                chosen[2] == tap ? 0.f + gv[2] : 0.f, chosen[3] == tap ? 0.f + gv[3] : 0.f));
        }
}

} // namespace

extern "C" {

int swc_hip_reluGrad_f(float *srcGrad, const float *src, const float *destGrad, size_t size) {
    SWC_REQUIRE_INIT();
    if (size == 0) return SWC_HIP_OK;
    SWC_ARG(srcGrad && src && destGrad);
    if (size % 4 == 0 && aligned16(srcGrad) && aligned16(src) && aligned16(destGrad) && size / 4 / kThreads < 0x7fffffffu) {
        const size_t n4 = size / 4;
        const unsigned blocks = (unsigned)((n4 + kThreads - 1) / kThreads);
        if (size * sizeof(float) >= kStreamingBytes)
            relu_grad4<true><<<blocks, kThreads, 0, stream()>>>((float4 *)srcGrad, (const float4 *)src,
                                                                 (const float4 *)destGrad, n4);
        else
            relu_grad4<false><<<blocks, kThreads, 0, stream()>>>((float4 *)srcGrad, (const float4 *)src,
                                                                  (const float4 *)destGrad, n4);
    } else {
        relu_grad<<<grid_for(size, kThreads), kThreads, 0, stream()>>>(srcGrad, src, destGrad, size);
    }
    SWC_LAUNCH_CHECK();
    return SWC_HIP_OK;
}

int swc_hip_matrixTanhGrad_f(int m, int n, float *a, int lda, const float *b, int ldb, const float *c, int ldc) {
    SWC_REQUIRE_INIT();
    SWC_ARG(m >= 0 && n >= 0 && lda >= n && ldb >= n && ldc >= n);
    if (m == 0 || n == 0) return SWC_HIP_OK;
    SWC_ARG(a && b && c);
    tanh_grad<<<grid_for((size_t)m * n, kThreads), kThreads, 0, stream()>>>(m, n, a, lda, b, ldb, c, ldc);
    SWC_LAUNCH_CHECK();
    return SWC_HIP_OK;
}

int swc_hip_matrixSoftmaxGrad_f(int m, int n, float *a, int lda, const float *b, int ldb, const int *selected) {
    SWC_REQUIRE_INIT();
    SWC_ARG(m >= 0 && n >= 0 && lda >= n && ldb >= n);
    if (m == 0 || n == 0) return SWC_HIP_OK;
    SWC_ARG(a && b && selected);
    softmax_grad<<<grid_for((size_t)m * n, kThreads), kThreads, 0, stream()>>>(m, n, a, lda, b, ldb, selected);
    SWC_LAUNCH_CHECK();
    return SWC_HIP_OK;
}

int swc_hip_matrixSoftmaxWithLossGrad_f(int m, int n, float *a, int lda, const float *b, int ldb,
                                        const int *selected) {
    return swc_hip_matrixSoftmaxGrad_f(m, n, a, lda, b, ldb, selected);
}

int swc_hip_matrixSoftmaxWithLoss_f(int m, int n, const float *a, int lda, float *b, int ldb, const int *selected,
                                    float *loss) {
    SWC_REQUIRE_INIT();
    SWC_ARG(m >= 0 && n >= 0 && lda >= n && ldb >= n);
    SWC_ARG(loss != nullptr);
    if (m == 0 || n == 0) return swc_hip_fill_f(loss, 0.f, 1);   // the reference would divide 0 by m
    SWC_ARG(a && b && selected);
    float *terms = static_cast<float *>(workspace((size_t)m * sizeof(float), "swc_hip_matrixSoftmaxWithLoss_f"));
    if (!terms) return fail_code();
    // the loss terms read a before the softmax may overwrite it (b may alias a)
    softmax_loss_terms<<<ceil_div(m, kThreads / 64), kThreads, 0, stream()>>>(m, n, a, lda, selected, terms);
    SWC_LAUNCH_CHECK();
    loss_mean<<<1, 1024, 0, stream()>>>(m, terms, loss);
    SWC_LAUNCH_CHECK();
    return swc_hip_matrixSoftmax_f(m, n, a, lda, b, ldb);
}

size_t swc_hip_matrixSoftmaxWithLoss_workspace_bytes(int m, int n) {
    return (m > 0 && n > 0) ? (size_t)m * sizeof(float) : 0;
}

int swc_hip_matrixTrans_f(int m, int n, const float *a, int lda, float *b, int ldb) {
    SWC_REQUIRE_INIT();
    SWC_ARG(m >= 0 && n >= 0 && lda >= n && ldb >= m);
    if (m == 0 || n == 0) return SWC_HIP_OK;
    SWC_ARG(a && b && a != b);
    const dim3 grid(ceil_div(n, 32), ceil_div(m, 32));
    SWC_ARG(grid.y <= 65535);
    matrix_trans<<<grid, 256, 0, stream()>>>(m, n, a, lda, b, ldb);
    SWC_LAUNCH_CHECK();
    return SWC_HIP_OK;
}

int swc_hip_batchedreduceadd_f(float *dest, const float *batch, size_t numSlice, size_t sliceSize) {
    SWC_REQUIRE_INIT();
    if (numSlice == 0) return SWC_HIP_OK;
    SWC_ARG(dest && (batch || sliceSize == 0));
    SWC_ARG(numSlice / 64 < 0x7fffffffu);
    row_sums<<<ceil_div(numSlice, 64), kThreads, 0, stream()>>>(dest, batch, numSlice, sliceSize);
    SWC_LAUNCH_CHECK();
    return SWC_HIP_OK;
}

int swc_hip_sgd_f(size_t size, float *out, float *w, float *dw, float *dw_mom, float lr, float decay, float momentum,
                  size_t batch) {
    SWC_REQUIRE_INIT();
    if (size == 0) return SWC_HIP_OK;
    SWC_ARG(out && w && dw && dw_mom);
    const float neglr = -lr / (float)batch;   // float / size_t in the reference: the divisor converts to float
    const size_t n4 = size / 4;
    if (n4 && aligned16(out) && aligned16(w) && aligned16(dw) && aligned16(dw_mom) && n4 / kThreads < 0x7fffffffu) {
        const unsigned blocks = (unsigned)((n4 + kThreads - 1) / kThreads);
        const bool nt = size * sizeof(float) >= kStreamingBytes, in_place = out == w;
        auto kern = nt ? (in_place ? sgd_step4<true, true> : sgd_step4<true, false>)
                       : (in_place ? sgd_step4<false, true> : sgd_step4<false, false>);
        kern<<<blocks, kThreads, 0, stream()>>>(n4, (float4 *)out, (const float4 *)w, (const float4 *)dw, (float4 *)dw_mom,
                                               neglr, decay, momentum);
        SWC_LAUNCH_CHECK();
        const size_t done = n4 * 4;
        if (done == size) return SWC_HIP_OK;
        sgd_step<<<1, kThreads, 0, stream()>>>(size - done, out + done, w + done, dw + done, dw_mom + done, neglr, decay,
                                               momentum);
    } else {
        sgd_step<<<grid_for(size, kThreads), kThreads, 0, stream()>>>(size, out, w, dw, dw_mom, neglr, decay, momentum);
    }
    SWC_LAUNCH_CHECK();
    return SWC_HIP_OK;
}

int swc_hip_maxpoolGrad_f(float *inputG, const float *outputG, const float *input, const size_t *idims,
                          const size_t *odims, const size_t *kernels, const size_t *strides, const size_t *pads) {
    SWC_REQUIRE_INIT();
    SWC_ARG(idims && odims && kernels && strides && pads);
    for (int i = 0; i < 4; ++i) SWC_ARG(idims[i] < 0x7fffffffu && odims[i] < 0x7fffffffu);
    SWC_ARG(idims[0] == odims[0] && idims[3] == odims[3]);
    SWC_ARG(kernels[0] > 0 && kernels[1] > 0 && strides[0] > 0 && strides[1] > 0);
    SWC_ARG(kernels[0] < 65536 && kernels[1] < 65536 && strides[0] < 65536 && strides[1] < 65536 && pads[0] < 65536 &&
            pads[1] < 65536);
    const size_t total = idims[0] * idims[1] * idims[2] * idims[3];
    if (total == 0) return SWC_HIP_OK;
    SWC_ARG(inputG && input && (outputG || odims[1] * odims[2] == 0));
    PoolGeom g{(int)idims[0], (int)idims[1], (int)idims[2], (int)idims[3], (int)odims[1], (int)odims[2],
               (int)kernels[0], (int)kernels[1], (int)strides[0], (int)strides[1], (int)pads[0], (int)pads[1]};
    // can a window lie wholly in the padding?  (its rows or its columns all out of bounds)
    int empty = 0;
    if (g.OH > 0 && g.OW > 0) {
        const long last_y = (long)(g.OH - 1) * g.sh - g.pt, last_x = (long)(g.OW - 1) * g.sw - g.pl;
        empty = (g.kh - 1 - g.pt < 0) || (g.kw - 1 - g.pl < 0) || last_y >= g.H || last_x >= g.W;
    }
    const size_t image_rows = idims[0] * idims[1];
    SWC_ARG(image_rows <= 0x7fffffffu);
    const bool vec = g.C % 4 == 0 && aligned16(inputG) && aligned16(outputG) && aligned16(input);
    if (vec && g.sh == g.kh && g.sw == g.kw && g.pt == 0 && g.pl == 0 && (long)g.OH * g.kh == g.H &&
        (long)g.OW * g.kw == g.W && g.kh * g.kw <= 64) {
        const size_t window_rows = idims[0] * (size_t)g.OH;
        const unsigned blocks = ceil_div((size_t)g.OW * (g.C / 4), kThreads);
        const bool nt = total * sizeof(float) >= kStreamingBytes;
        auto kern = g.kh == 2 && g.kw == 2   ? (nt ? maxpool_grad_tiled<true, 2, 2> : maxpool_grad_tiled<false, 2, 2>)
                    : g.kh == 3 && g.kw == 3 ? (nt ? maxpool_grad_tiled<true, 3, 3> : maxpool_grad_tiled<false, 3, 3>)
                                             : (nt ? maxpool_grad_tiled<true, 0, 0> : maxpool_grad_tiled<false, 0, 0>);
        for (size_t r0 = 0; r0 < window_rows; r0 += 65535) {
            const unsigned rows = (unsigned)(window_rows - r0 < 65535 ? window_rows - r0 : 65535);
            kern<<<dim3(blocks, rows), kThreads, 0, stream()>>>(inputG, outputG, input, g, (int)r0);
            SWC_LAUNCH_CHECK();
        }
        return SWC_HIP_OK;
    }
    const size_t row_items = (size_t)g.W * (vec ? g.C / 4 : g.C);
    // grid.y is limited to 65535: rows beyond that are covered by launching in slabs of rows
    for (size_t r0 = 0; r0 < image_rows; r0 += 65535) {
        const unsigned rows = (unsigned)(image_rows - r0 < 65535 ? image_rows - r0 : 65535);
        const dim3 grid(grid_for(row_items, kThreads, 1024), rows);
        if (vec) maxpool_grad<4><<<grid, kThreads, 0, stream()>>>(inputG, outputG, input, g, empty, (int)r0);
        else maxpool_grad<1><<<grid, kThreads, 0, stream()>>>(inputG, outputG, input, g, empty, (int)r0);
        SWC_LAUNCH_CHECK();
    }
    SWC_LAUNCH_CHECK();
    return SWC_HIP_OK;
}

} // extern "C"
