// batchnormalization_f (kernels.h:496-517), maxpool_f (kernels.h:323-377) and
// their fusions, NHWC.  All are one pass over HBM; channels are the contiguous
// axis, so a thread owns four consecutive channels (one 128-bit access) and
// keeps their normalisation constants in registers while it walks rows.
//
// Arithmetic follows the reference exactly: var+eps is an fp32 add, everything
// after it is double ((x-mean) widened, times (var+eps)^-1/2, times scale, plus
// bias) with a single rounding to fp32 on the store.
#include "common.hpp"

using namespace swc_hip;

namespace {

constexpr int kThreads = 256;

struct BnQuad {
    float mean[4];
    double rs[4];     // (var+eps)^-1/2
    double scale[4];
    double bias[4];
};

__device__ __forceinline__ void load_bn_quad(BnQuad &q, const float *mean, const float *var, const float *scale,
                                             const float *bias, size_t c0, float eps) {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        q.mean[i] = mean[c0 + i];
        const float ve = var[c0 + i] + eps;
        q.rs[i] = 1.0 / sqrt((double)ve);
        q.scale[i] = (double)scale[c0 + i];
        q.bias[i] = (double)bias[c0 + i];
    }
}

template <bool RELU>
__device__ __forceinline__ float bn1(float x, const BnQuad &q, int i) {
    const float centred = x - q.mean[i];
    const float y = (float)((double)centred * q.rs[i] * q.scale[i] + q.bias[i]);
    return RELU ? ((y > 0.f) ? y : 0.f) : y;
}

template <bool RELU>
__device__ __forceinline__ float4 bn4(float4 x, const BnQuad &q) {
    return make_float4(bn1<RELU>(x.x, q, 0), bn1<RELU>(x.y, q, 1), bn1<RELU>(x.z, q, 2), bn1<RELU>(x.w, q, 3));
}

// The launch makes gridDim.x*kThreads a multiple of quads (= C/4), so the
// channel quad of a thread never changes while it strides through the tensor.
// Each trip issues kBnUnroll independent 128-bit loads before anything else, and
// the per-thread constants (four channels' parameters, a double 1/sqrt each) are
// computed while the first trip's loads are in flight.
constexpr int kBnUnroll = 4;
template <bool RELU, bool NT>
__global__ __launch_bounds__(kThreads) void bn_vec4(float *out, const float *in, const float *__restrict__ mean,
                                                    const float *__restrict__ var, const float *__restrict__ scale,
                                                    const float *__restrict__ bias, size_t total4, unsigned quads,
                                                    float eps) {
    const size_t g = (size_t)blockIdx.x * kThreads + threadIdx.x;
    const size_t step = (size_t)gridDim.x * kThreads;
    if (g >= total4) return;
    const float4 *i4 = reinterpret_cast<const float4 *>(in);
    float4 *o4 = reinterpret_cast<float4 *>(out);
    float4 x[kBnUnroll];
#pragma unroll
    for (int u = 0; u < kBnUnroll; ++u)
        if (g + u * step < total4) x[u] = ld4<NT>(i4 + g + u * step);
    BnQuad q;
    load_bn_quad(q, mean, var, scale, bias, (g % quads) * 4, eps);
    size_t i = g;
    while (true) {
#pragma unroll
        for (int u = 0; u < kBnUnroll; ++u)
            if (i + u * step < total4) st4<NT>(o4 + i + u * step, bn4<RELU>(x[u], q));
        i += kBnUnroll * step;
        if (i >= total4) break;
#pragma unroll
        for (int u = 0; u < kBnUnroll; ++u)
            if (i + u * step < total4) x[u] = ld4<NT>(i4 + i + u * step);
    }
}

template <bool RELU>
__global__ __launch_bounds__(kThreads) void bn_scalar(float *out, const float *in, const float *__restrict__ mean,
                                                      const float *__restrict__ var, const float *__restrict__ scale,
                                                      const float *__restrict__ bias, size_t total, size_t C,
                                                      float eps) {
    size_t i = (size_t)blockIdx.x * kThreads + threadIdx.x;
    const size_t step = (size_t)gridDim.x * kThreads;
    for (; i < total; i += step) {
        const size_t c = i % C;
        const float ve = var[c] + eps;
        const float centred = in[i] - mean[c];
        const float y = (float)((double)centred * (1.0 / sqrt((double)ve)) * (double)scale[c] + (double)bias[c]);
        out[i] = RELU ? ((y > 0.f) ? y : 0.f) : y;
    }
}

struct PoolGeom {
    int N, H, W, C, OH, OW, kh, kw, sh, sw, pt, pl;
};

// First in-bounds tap initialises, later taps replace only when strictly
// greater (kernels.h:362-366).  `BN` applies batchnorm+relu to each tap first.
template <bool ARGMAX, bool BN, bool NT>
__global__ __launch_bounds__(kThreads) void maxpool_vec4(const float *__restrict__ in, float *__restrict__ out,
                                                         int32_t *__restrict__ arg, PoolGeom g, size_t total4,
                                                         const float *__restrict__ mean, const float *__restrict__ var,
                                                         const float *__restrict__ scale,
                                                         const float *__restrict__ bias, float eps) {
    const unsigned quads = g.C / 4;
    const size_t gid = (size_t)blockIdx.x * kThreads + threadIdx.x;
    const size_t step = (size_t)gridDim.x * kThreads;
    if (gid >= total4) return;
    BnQuad q;
    if (BN) load_bn_quad(q, mean, var, scale, bias, (gid % quads) * 4, eps);
    const float4 *i4 = reinterpret_cast<const float4 *>(in);
    for (size_t o = gid; o < total4; o += step) {
        const unsigned cq = (unsigned)(o % quads);
        size_t r = o / quads;
        const int ox = (int)(r % g.OW);
        r /= g.OW;
        const int oy = (int)(r % g.OH);
        const int n = (int)(r / g.OH);
        float best[4] = {0.f, 0.f, 0.f, 0.f};
        int32_t where[4] = {-1, -1, -1, -1};
        bool have = false;
        for (int ky = 0; ky < g.kh; ++ky) {
            const int iy = oy * g.sh - g.pt + ky;
            if (iy < 0 || iy >= g.H) continue;
            for (int kx = 0; kx < g.kw; ++kx) {
                const int ix = ox * g.sw - g.pl + kx;
                if (ix < 0 || ix >= g.W) continue;
                const size_t pix = ((size_t)n * g.H + iy) * g.W + ix;
                float4 v4 = ld4<NT>(i4 + pix * quads + cq);
                if (BN) v4 = bn4<true>(v4, q);
                const float v[4] = {v4.x, v4.y, v4.z, v4.w};
                const int32_t flat = (int32_t)(pix * g.C + cq * 4);
#pragma unroll
                for (int c = 0; c < 4; ++c) {
                    if (!have || v[c] > best[c]) {
                        best[c] = v[c];
                        if (ARGMAX) where[c] = flat + c;
                    }
                }
                have = true;
            }
        }
        st4<NT>(reinterpret_cast<float4 *>(out) + o, make_float4(best[0], best[1], best[2], best[3]));
        if (ARGMAX) st4i<NT>(reinterpret_cast<int4 *>(arg) + o, make_int4(where[0], where[1], where[2], where[3]));
    }
}

// Windows that tile the image exactly (stride = kernel, no padding, H = OH*KH, W = OW*KW: the 2x2/2 pools of
// the configurations): every tap of every window is in bounds, so a thread — four channels of one window —
// requests all its taps at once and only then normalises and compares them.  blockIdx.y + row_base = n*OH + oy;
// blockIdx.x, threadIdx.x walk OW * C/4: 32-bit index arithmetic throughout.  The values and the first-maximum
// rule are those of maxpool_vec4.
template <int KH, int KW, bool BN, bool NT>
__global__ __launch_bounds__(kThreads) void maxpool_tiled(const float *__restrict__ in, float *__restrict__ out,
                                                          PoolGeom g, int row_base, const float *__restrict__ mean,
                                                          const float *__restrict__ var,
                                                          const float *__restrict__ scale,
                                                          const float *__restrict__ bias, float eps) {
    const int quads = g.C / 4;
    const int item = blockIdx.x * kThreads + threadIdx.x;
    if (item >= g.OW * quads) return;
    const int ox = item / quads, cq = item - ox * quads;
    const int window_row = row_base + blockIdx.y;
    const int oy = window_row % g.OH, n = window_row / g.OH;
    BnQuad q;
    if (BN) load_bn_quad(q, mean, var, scale, bias, (size_t)cq * 4, eps);
    const size_t row_pitch = (size_t)g.W * quads;   // in float4s
    const float4 *tap0 = reinterpret_cast<const float4 *>(in) + ((size_t)n * g.H + (size_t)oy * KH) * row_pitch +
                         (size_t)ox * KW * quads + cq;
    float4 t[KH * KW];
#pragma unroll
    for (int i = 0; i < KH * KW; ++i) t[i] = ld4<NT>(tap0 + (i / KW) * row_pitch + (size_t)(i % KW) * quads);
    float best[4];
#pragma unroll
    for (int i = 0; i < KH * KW; ++i) {
        const float4 v4 = BN ? bn4<true>(t[i], q) : t[i];
        const float v[4] = {v4.x, v4.y, v4.z, v4.w};
#pragma unroll
        for (int c = 0; c < 4; ++c)
            if (i == 0 || v[c] > best[c]) best[c] = v[c];
    }
    st4<NT>(reinterpret_cast<float4 *>(out) + ((size_t)window_row * g.OW + ox) * quads + cq,
            make_float4(best[0], best[1], best[2], best[3]));
}

template <bool ARGMAX, bool BN>
__global__ __launch_bounds__(kThreads) void maxpool_scalar(const float *__restrict__ in, float *__restrict__ out,
                                                           int32_t *__restrict__ arg, PoolGeom g, size_t total,
                                                           const float *__restrict__ mean,
                                                           const float *__restrict__ var,
                                                           const float *__restrict__ scale,
                                                           const float *__restrict__ bias, float eps) {
    size_t o = (size_t)blockIdx.x * kThreads + threadIdx.x;
    const size_t step = (size_t)gridDim.x * kThreads;
    for (; o < total; o += step) {
        const int c = (int)(o % g.C);
        size_t r = o / g.C;
        const int ox = (int)(r % g.OW);
        r /= g.OW;
        const int oy = (int)(r % g.OH);
        const int n = (int)(r / g.OH);
        float best = 0.f;
        int32_t where = -1;
        bool have = false;
        for (int ky = 0; ky < g.kh; ++ky) {
            const int iy = oy * g.sh - g.pt + ky;
            if (iy < 0 || iy >= g.H) continue;
            for (int kx = 0; kx < g.kw; ++kx) {
                const int ix = ox * g.sw - g.pl + kx;
                if (ix < 0 || ix >= g.W) continue;
                const size_t flat = (((size_t)n * g.H + iy) * g.W + ix) * g.C + c;
                float v = in[flat];
                if (BN) {
                    const float ve = var[c] + eps;
                    const float centred = v - mean[c];
                    v = (float)((double)centred * (1.0 / sqrt((double)ve)) * (double)scale[c] + (double)bias[c]);
                    v = (v > 0.f) ? v : 0.f;
                }
                if (!have || v > best) {
                    best = v;
                    where = (int32_t)flat;
                    have = true;
                }
            }
        }
        out[o] = best;
        if (ARGMAX) arg[o] = where;
    }
}

// avgpool_f (kernels.h:444-493): fp32 sum of the in-bounds taps in (ky, kx) scan
// order, divided by kh*kw (IEEE division) — the same operations in the same
// order as the reference, so the result is bit-exact.
template <bool NT>
__global__ __launch_bounds__(kThreads) void avgpool_vec4(const float *__restrict__ in, float *__restrict__ out,
                                                         PoolGeom g, size_t total4) {
    const unsigned quads = g.C / 4;
    const size_t step = (size_t)gridDim.x * kThreads;
    const float4 *i4 = reinterpret_cast<const float4 *>(in);
    const float count = (float)(g.kh * g.kw);
    for (size_t o = (size_t)blockIdx.x * kThreads + threadIdx.x; o < total4; o += step) {
        const unsigned cq = (unsigned)(o % quads);
        size_t r = o / quads;
        const int ox = (int)(r % g.OW);
        r /= g.OW;
        const int oy = (int)(r % g.OH);
        const int n = (int)(r / g.OH);
        float4 sum = make_float4(0.f, 0.f, 0.f, 0.f);
        for (int ky = 0; ky < g.kh; ++ky) {
            const int iy = oy * g.sh - g.pt + ky;
            if (iy < 0 || iy >= g.H) continue;
            // eight taps' loads in flight, then their adds in tap order; a tap outside the image adds +0, which
            // leaves the sum (never -0: it starts from +0) as skipping the tap does
            const float4 *row = i4 + ((size_t)n * g.H + iy) * g.W * quads + cq;
            for (int kx0 = 0; kx0 < g.kw; kx0 += 8) {
                float4 v[8];
#pragma unroll
                for (int u = 0; u < 8; ++u) {
                    const int ix = ox * g.sw - g.pl + kx0 + u;
                    const bool ok = kx0 + u < g.kw && ix >= 0 && ix < g.W;
                    v[u] = ok ? ld4<NT>(row + (size_t)ix * quads) : make_float4(0.f, 0.f, 0.f, 0.f);
                }
#pragma unroll
                for (int u = 0; u < 8; ++u) sum.x += v[u].x, sum.y += v[u].y, sum.z += v[u].z, sum.w += v[u].w;
            }
        }
        st4<NT>(reinterpret_cast<float4 *>(out) + o,
                make_float4(sum.x / count, sum.y / count, sum.z / count, sum.w / count));
    }
}

__global__ __launch_bounds__(kThreads) void avgpool_scalar(const float *__restrict__ in, float *__restrict__ out,
                                                           PoolGeom g, size_t total) {
    const size_t step = (size_t)gridDim.x * kThreads;
    const float count = (float)(g.kh * g.kw);
    for (size_t o = (size_t)blockIdx.x * kThreads + threadIdx.x; o < total; o += step) {
        const int c = (int)(o % g.C);
        size_t r = o / g.C;
        const int ox = (int)(r % g.OW);
        r /= g.OW;
        const int oy = (int)(r % g.OH);
        const int n = (int)(r / g.OH);
        float sum = 0.f;
        for (int ky = 0; ky < g.kh; ++ky) {
            const int iy = oy * g.sh - g.pt + ky;
            if (iy < 0 || iy >= g.H) continue;
            for (int kx = 0; kx < g.kw; ++kx) {
                const int ix = ox * g.sw - g.pl + kx;
                if (ix < 0 || ix >= g.W) continue;
                sum += in[(((size_t)n * g.H + iy) * g.W + ix) * g.C + c];
            }
        }
        out[o] = sum / count;
    }
}

// blocks such that blocks*kThreads is a multiple of `quads`
unsigned quad_stable_blocks(size_t total4, unsigned quads, unsigned max_blocks) {
    unsigned a = quads, b = kThreads;
    while (b) { unsigned t = a % b; a = b; b = t; }
    const unsigned unit = quads / a;  // blocks must be a multiple of this
    size_t need = (total4 + kThreads - 1) / kThreads;
    if (need > max_blocks) need = max_blocks;
    size_t blocks = ((need + unit - 1) / unit) * unit;
    if (blocks == 0) blocks = unit;
    return (unsigned)blocks;
}

int check_dims4(const char *who, const size_t *d) {
    for (int i = 0; i < 4; ++i)
        if (d[i] > 0x7fffffffu) return fail(SWC_HIP_EINVAL, "%s: dimension %d too large", who, i);
    return 0;
}

template <bool RELU>
int launch_bn(const char *who, float *output, const float *input, const float *mean, const float *var,
              const float *scale, const float *bias, const size_t *idims, float eps) {
    if (!idims) return fail(SWC_HIP_EINVAL, "%s: null idims", who);
    if (check_dims4(who, idims)) return SWC_HIP_EINVAL;
    const size_t C = idims[3];
    const size_t total = idims[0] * idims[1] * idims[2] * C;
    if (total == 0) return SWC_HIP_OK;
    if (!output || !input || !mean || !var || !scale || !bias) return fail(SWC_HIP_EINVAL, "%s: null pointer", who);
    if (C % 4 == 0 && aligned16(output) && aligned16(input)) {
        const size_t total4 = total / 4;
        const unsigned quads = (unsigned)(C / 4);
        const unsigned blocks = quad_stable_blocks((total4 + kBnUnroll - 1) / kBnUnroll, quads, (unsigned)num_cus() * 64u);
        if (total * sizeof(float) >= kStreamingBytes)
            bn_vec4<RELU, true><<<blocks, kThreads, 0, stream()>>>(output, input, mean, var, scale, bias, total4, quads, eps);
        else
            bn_vec4<RELU, false><<<blocks, kThreads, 0, stream()>>>(output, input, mean, var, scale, bias, total4, quads, eps);
    } else {
        size_t blocks = (total + kThreads - 1) / kThreads;
        if (blocks > 8192) blocks = 8192;
        bn_scalar<RELU><<<(unsigned)blocks, kThreads, 0, stream()>>>(output, input, mean, var, scale, bias, total, C, eps);
    }
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) return fail(SWC_HIP_ERUNTIME, "%s: launch failed: %s", who, hipGetErrorString(e));
    return SWC_HIP_OK;
}

template <bool ARGMAX, bool BN>
int launch_pool(const char *who, const float *input, float *output, int32_t *argmax, const size_t *idims,
                const size_t *odims, const size_t *kernels, const size_t *strides, const size_t *pads,
                const float *mean, const float *var, const float *scale, const float *bias, float eps) {
    if (!idims || !odims || !kernels || !strides || !pads) return fail(SWC_HIP_EINVAL, "%s: null shape array", who);
    if (check_dims4(who, idims) || check_dims4(who, odims)) return SWC_HIP_EINVAL;
    if (odims[0] != idims[0] || odims[3] != idims[3])
        return fail(SWC_HIP_EINVAL, "%s: output batch/channels differ from input", who);
    if (kernels[0] == 0 || kernels[1] == 0 || strides[0] == 0 || strides[1] == 0 || kernels[0] > 4096 ||
        kernels[1] > 4096 || strides[0] > 4096 || strides[1] > 4096 || pads[0] > 4096 || pads[1] > 4096)
        return fail(SWC_HIP_EINVAL, "%s: bad kernel/stride/pad", who);
    // every window must start inside the padded input, as in the reference's shape rule
    if (odims[1] && (odims[1] - 1) * strides[0] >= idims[1] + pads[0] + kernels[0])
        return fail(SWC_HIP_EINVAL, "%s: output height inconsistent with input", who);
    if (odims[2] && (odims[2] - 1) * strides[1] >= idims[2] + pads[1] + kernels[1])
        return fail(SWC_HIP_EINVAL, "%s: output width inconsistent with input", who);
    const size_t in_total = idims[0] * idims[1] * idims[2] * idims[3];
    const size_t total = odims[0] * odims[1] * odims[2] * odims[3];
    if (total == 0) return SWC_HIP_OK;
    if (ARGMAX && in_total > 0x7fffffffu) return fail(SWC_HIP_EUNSUPPORTED, "%s: input too large for int32 indices", who);
    if (!input || !output || (ARGMAX && !argmax)) return fail(SWC_HIP_EINVAL, "%s: null pointer", who);
    if (BN && (!mean || !var || !scale || !bias)) return fail(SWC_HIP_EINVAL, "%s: null batchnorm parameter", who);
    PoolGeom g{(int)idims[0], (int)idims[1], (int)idims[2], (int)idims[3], (int)odims[1], (int)odims[2],
               (int)kernels[0], (int)kernels[1], (int)strides[0], (int)strides[1], (int)pads[0], (int)pads[1]};
    const size_t C = idims[3];
    const bool vec = C % 4 == 0 && aligned16(input) && aligned16(output) && (!ARGMAX || aligned16(argmax));
    const bool tiles_exactly = g.sh == g.kh && g.sw == g.kw && g.pt == 0 && g.pl == 0 && (size_t)g.OH * g.kh == idims[1] &&
                               (size_t)g.OW * g.kw == idims[2];
    // (without batchnorm the strided kernel below is as fast or faster: 53 against 56 us on [256,32,32,256])
    if (BN && !ARGMAX && vec && tiles_exactly && g.kh == g.kw && (g.kh == 2 || g.kh == 3) && odims[0] * odims[1] <= 0x7fffffffu) {
        const size_t window_rows = odims[0] * odims[1];
        const unsigned blocks = (unsigned)(((size_t)g.OW * (C / 4) + kThreads - 1) / kThreads);
        const bool nt = in_total * sizeof(float) >= kStreamingBytes;
        auto kern = g.kh == 2 ? (nt ? maxpool_tiled<2, 2, BN, true> : maxpool_tiled<2, 2, BN, false>)
                              : (nt ? maxpool_tiled<3, 3, BN, true> : maxpool_tiled<3, 3, BN, false>);
        for (size_t r0 = 0; r0 < window_rows; r0 += 65535) {   // grid.y is limited to 65535
            const unsigned rows = (unsigned)(window_rows - r0 < 65535 ? window_rows - r0 : 65535);
            kern<<<dim3(blocks, rows), kThreads, 0, stream()>>>(input, output, g, (int)r0, mean, var, scale, bias, eps);
        }
    } else if (vec) {
        const size_t total4 = total / 4;
        const unsigned blocks = quad_stable_blocks(total4, (unsigned)(C / 4), (unsigned)num_cus() * 128u);
        if (in_total * sizeof(float) >= kStreamingBytes)
            maxpool_vec4<ARGMAX, BN, true><<<blocks, kThreads, 0, stream()>>>(input, output, argmax, g, total4, mean, var, scale, bias, eps);
        else
            maxpool_vec4<ARGMAX, BN, false><<<blocks, kThreads, 0, stream()>>>(input, output, argmax, g, total4, mean, var, scale, bias, eps);
    } else {
        size_t blocks = (total + kThreads - 1) / kThreads;
        if (blocks > 8192) blocks = 8192;
        maxpool_scalar<ARGMAX, BN><<<(unsigned)blocks, kThreads, 0, stream()>>>(input, output, argmax, g, total, mean, var, scale, bias, eps);
    }
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) return fail(SWC_HIP_ERUNTIME, "%s: launch failed: %s", who, hipGetErrorString(e));
    return SWC_HIP_OK;
}

} // namespace

extern "C" {

int swc_hip_batchnormalization_f(float *output, const float *input, const float *mean, const float *var,
                                 const float *scale, const float *bias, const size_t *idims, float epsilon) {
    SWC_REQUIRE_INIT();
    return launch_bn<false>("swc_hip_batchnormalization_f", output, input, mean, var, scale, bias, idims, epsilon);
}

int swc_hip_batchnormRelu_f(float *output, const float *input, const float *mean, const float *var,
                            const float *scale, const float *bias, const size_t *idims, float epsilon) {
    SWC_REQUIRE_INIT();
    return launch_bn<true>("swc_hip_batchnormRelu_f", output, input, mean, var, scale, bias, idims, epsilon);
}

int swc_hip_maxpool_f(const float *input, float *output, const size_t *idims, const size_t *odims,
                      const size_t *kernels, const size_t *strides, const size_t *pads) {
    SWC_REQUIRE_INIT();
    return launch_pool<false, false>("swc_hip_maxpool_f", input, output, nullptr, idims, odims, kernels, strides, pads,
                                     nullptr, nullptr, nullptr, nullptr, 0.f);
}

int swc_hip_maxpool_argmax_f(const float *input, float *output, int32_t *argmax, const size_t *idims,
                             const size_t *odims, const size_t *kernels, const size_t *strides, const size_t *pads) {
    SWC_REQUIRE_INIT();
    return launch_pool<true, false>("swc_hip_maxpool_argmax_f", input, output, argmax, idims, odims, kernels, strides,
                                    pads, nullptr, nullptr, nullptr, nullptr, 0.f);
}

int swc_hip_avgpool_f(const float *input, float *output, const size_t *idims, const size_t *odims,
                      const size_t *kernels, const size_t *strides, const size_t *pads) {
    SWC_REQUIRE_INIT();
    const char *who = "swc_hip_avgpool_f";
    if (!idims || !odims || !kernels || !strides || !pads) return fail(SWC_HIP_EINVAL, "%s: null shape array", who);
    if (check_dims4(who, idims) || check_dims4(who, odims)) return SWC_HIP_EINVAL;
    if (odims[0] != idims[0] || odims[3] != idims[3])
        return fail(SWC_HIP_EINVAL, "%s: output batch/channels differ from input", who);
    if (kernels[0] == 0 || kernels[1] == 0 || strides[0] == 0 || strides[1] == 0 || kernels[0] > 4096 ||
        kernels[1] > 4096 || strides[0] > 4096 || strides[1] > 4096 || pads[0] > 4096 || pads[1] > 4096)
        return fail(SWC_HIP_EINVAL, "%s: bad kernel/stride/pad", who);
    const size_t in_total = idims[0] * idims[1] * idims[2] * idims[3];
    const size_t total = odims[0] * odims[1] * odims[2] * odims[3];
    if (total == 0) return SWC_HIP_OK;
    SWC_ARG(input && output);
    PoolGeom g{(int)idims[0], (int)idims[1], (int)idims[2], (int)idims[3], (int)odims[1], (int)odims[2],
               (int)kernels[0], (int)kernels[1], (int)strides[0], (int)strides[1], (int)pads[0], (int)pads[1]};
    if (idims[3] % 4 == 0 && aligned16(input) && aligned16(output)) {
        const size_t total4 = total / 4;
        size_t blocks = (total4 + kThreads - 1) / kThreads;
        if (blocks > (size_t)num_cus() * 128) blocks = (size_t)num_cus() * 128;
        if (in_total * sizeof(float) >= kStreamingBytes)
            avgpool_vec4<true><<<(unsigned)blocks, kThreads, 0, stream()>>>(input, output, g, total4);
        else
            avgpool_vec4<false><<<(unsigned)blocks, kThreads, 0, stream()>>>(input, output, g, total4);
    } else {
        size_t blocks = (total + kThreads - 1) / kThreads;
        if (blocks > 8192) blocks = 8192;
        avgpool_scalar<<<(unsigned)blocks, kThreads, 0, stream()>>>(input, output, g, total);
    }
    SWC_LAUNCH_CHECK();
    return SWC_HIP_OK;
}

int swc_hip_batchnormReluMaxpool_f(float *output, const float *input, const float *mean, const float *var,
                                   const float *scale, const float *bias, const size_t *idims, float epsilon,
                                   const size_t *odims, const size_t *kernels, const size_t *strides,
                                   const size_t *pads) {
    SWC_REQUIRE_INIT();
    return launch_pool<false, true>("swc_hip_batchnormReluMaxpool_f", input, output, nullptr, idims, odims, kernels,
                                    strides, pads, mean, var, scale, bias, epsilon);
}

} // extern "C"
