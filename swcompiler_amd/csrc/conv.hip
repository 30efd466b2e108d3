// conv2d_f (kernels.h:177-243) as an implicit GEMM on fp32 MFMA, NHWC.
//
//   C[M, oC] = A[M, K] * F^T,  M = N*OH*OW (output pixels), K = kH*kW*iC,
//   A[m, (ky,kx,ci)] = in[n, oy*sh - pt + ky, ox*sw - pl + kx, ci] (0 outside),
//   F = filter viewed as [oC, K] — K is the contiguous axis of BOTH operands,
//   and the output tensor [N,OH,OW,oC] is exactly C row-major, so nothing is
//   ever materialised or transposed.  Bias, inference batchnorm and ReLU are
//   applied to the accumulators before the single store.
//
// The tile machinery is mfma_tile.hpp's; only the global->LDS gather differs
// from the FC GEMM.  When iC % 4 == 0 four consecutive k's lie in one tap, so
// the gather uses 128-bit loads; otherwise (first layer, iC = 1 or 3) 32-bit.
#include "common.hpp"
#include "mfma_dma.hpp"
#include "mfma_tile.hpp"
#include <cstdlib>
#include <cstring>

using namespace swc_hip;
using namespace swc_hip::mfma;

namespace {

struct ConvGeom {
    int N, H, W, C;      // input NHWC
    int OH, OW, OC;      // output
    int kh, kw, sh, sw, pt, pl;
    int M, K;            // GEMM view
};

template <int TM, int TN, bool VEC>
__global__ __launch_bounds__(kThreads) void conv_igemm(const float *__restrict__ in, const float *__restrict__ filt,
                                                       float *__restrict__ out, ConvGeom g, Epilogue ep) {
    using T = Tile<TM, TN, true>;
    extern __shared__ __align__(16) float lds[];
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = tid >> 6;
    const int wave_m = wave >> 1, wave_n = wave & 1;
    const int M = g.M, N = g.OC, K = g.K;

    int tile_m, tile_n;
    tile_coords((M + T::BM - 1) / T::BM, (N + T::BN - 1) / T::BN, tile_m, tile_n);
    const int m0 = tile_m * T::BM, n0 = tile_n * T::BN;

    v16f acc[TM][TN];
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j)
#pragma unroll
            for (int v = 0; v < 16; ++v) acc[i][j][v] = 0.f;

    // VEC: thread owns rows (tid>>3) + 32*i of the A tile and k quad (tid&7).
    // Per owned output pixel: element offset of its window's top-left tap
    // (channel 0) and that tap's input coordinates; rows >= M get coordinates
    // far outside the image so every tap fails the bounds test.
    long row_off[T::kAVec];
    int iy0[T::kAVec], ix0[T::kAVec];
    // The k position of this thread's quad, kept as (ky, kx, ci) and advanced by
    // BK per slice without divisions; tap_off = ((ky*W + kx)*C + ci).
    int ky = 0, kx = 0, ci = 0, kpos = 0;
    if (VEC) {
#pragma unroll
        for (int i = 0; i < T::kAVec; ++i) {
            const int m = m0 + (tid >> 3) + 32 * i;
            if (m < M) {
                const int ox = m % g.OW;
                const int t = m / g.OW;
                const int oy = t % g.OH;
                const int img = t / g.OH;
                iy0[i] = oy * g.sh - g.pt;
                ix0[i] = ox * g.sw - g.pl;
                row_off[i] = (((long)img * g.H + iy0[i]) * g.W + ix0[i]) * g.C;
            } else {
                iy0[i] = -(1 << 20);
                ix0[i] = -(1 << 20);
                row_off[i] = 0;
            }
        }
        kpos = (tid & 7) * 4;
        const int tap = kpos / g.C;
        ci = kpos - tap * g.C;
        ky = tap / g.kw;
        kx = tap - ky * g.kw;
    }

    constexpr int kAScalar = T::kAVec * 4, kBScalar = T::kBVec * 4;
    float4 ra[T::kAVec], rb[T::kBVec];
    float sa[VEC ? 1 : kAScalar], sb[VEC ? 1 : kBScalar];

    // VEC path: loads the slice at the thread's current (ky,kx,ci), then steps
    // the position by BK.  Slices are visited strictly in order.
    auto load_global = [&](int k0) {
        if (VEC) {
            const bool k_ok = kpos < K;
            const long tap_off = ((long)ky * g.W + kx) * g.C + ci;
#pragma unroll
            for (int i = 0; i < T::kAVec; ++i) {
                const int iy = iy0[i] + ky, ix = ix0[i] + kx;
                const bool ok = k_ok && (unsigned)iy < (unsigned)g.H && (unsigned)ix < (unsigned)g.W;
                ra[i] = ok ? *reinterpret_cast<const float4 *>(in + row_off[i] + tap_off)
                           : make_float4(0.f, 0.f, 0.f, 0.f);
            }
#pragma unroll
            for (int i = 0; i < T::kBVec; ++i) {
                const int col = n0 + (tid >> 3) + 32 * i;
                rb[i] = (col < N && k_ok) ? *reinterpret_cast<const float4 *>(filt + (size_t)col * K + kpos)
                                          : make_float4(0.f, 0.f, 0.f, 0.f);
            }
            kpos += BK;
            ci += BK;
            while (ci >= g.C) {
                ci -= g.C;
                if (++kx == g.kw) {
                    kx = 0;
                    ++ky;
                }
            }
        } else {
#pragma unroll
            for (int i = 0; i < kAScalar; ++i) {
                const int e = tid + kThreads * i;
                const int m = m0 + e / BK, k = k0 + e % BK;
                float v = 0.f;
                if (m < M && k < K) {
                    const int ox = m % g.OW;
                    const int t = m / g.OW;
                    const int oy = t % g.OH, n = t / g.OH;
                    const int tap = k / g.C, cc = k - tap * g.C;
                    const int kyy = tap / g.kw, kxx = tap - kyy * g.kw;
                    const int iy = oy * g.sh - g.pt + kyy, ix = ox * g.sw - g.pl + kxx;
                    if (iy >= 0 && iy < g.H && ix >= 0 && ix < g.W)
                        v = in[(((size_t)n * g.H + iy) * g.W + ix) * g.C + cc];
                }
                sa[i] = v;
            }
#pragma unroll
            for (int i = 0; i < kBScalar; ++i) {
                const int e = tid + kThreads * i;
                const int col = n0 + e / BK, k = k0 + e % BK;
                sb[i] = (col < N && k < K) ? filt[(size_t)col * K + k] : 0.f;
            }
        }
    };
    auto store_lds = [&](int stage) {
        float *As = lds + stage * T::kStageFloats;
        float *Bs = As + T::kAFloats;
        if (VEC) {
#pragma unroll
            for (int i = 0; i < T::kAVec; ++i)
                *reinterpret_cast<float4 *>(&As[((tid >> 3) + 32 * i) * kLdK + (tid & 7) * 4]) = ra[i];
#pragma unroll
            for (int i = 0; i < T::kBVec; ++i)
                *reinterpret_cast<float4 *>(&Bs[((tid >> 3) + 32 * i) * kLdK + (tid & 7) * 4]) = rb[i];
        } else {
#pragma unroll
            for (int i = 0; i < kAScalar; ++i) {
                const int e = tid + kThreads * i;
                As[(e / BK) * kLdK + e % BK] = sa[i];
            }
#pragma unroll
            for (int i = 0; i < kBScalar; ++i) {
                const int e = tid + kThreads * i;
                Bs[(e / BK) * kLdK + e % BK] = sb[i];
            }
        }
    };

    const int nk = (K + BK - 1) / BK;
    load_global(0);
    store_lds(0);
    __syncthreads();
    for (int kt = 0; kt < nk; ++kt) {
        const int cur = kt & 1;
        if (kt + 1 < nk) load_global((kt + 1) * BK);
        const float *As = lds + cur * T::kStageFloats;
        compute_slice<TM, TN, true>(As, As + T::kAFloats, acc, wave_m, wave_n, lane);
        if (kt + 1 < nk) store_lds(cur ^ 1);
        __syncthreads();
    }
    store_tile<TM, TN>(acc, out, (size_t)N, M, N, m0 + wave_m * 32 * TM, n0 + wave_n * 32 * TN, lane, ep);
}

// Direct-to-LDS variant (mfma_dma.hpp): the im2col gather is expressed as one
// 32-bit byte offset per lane per load — out-of-image taps and rows past M get
// the out-of-range offset and arrive in LDS as zeros.  Needs iC % 4 == 0,
// 16-byte-aligned tensors and input/filter below 2 GiB.
template <int TM, int TN, int STAGES, bool MID = false>
__global__ __launch_bounds__(kThreads) void conv_dma(const float *__restrict__ in, const float *__restrict__ filt,
                                                     float *__restrict__ out, ConvGeom g, unsigned in_bytes,
                                                     unsigned filt_bytes, Epilogue ep) {
#if __HIP_DEVICE_COMPILE__   // the host pass only needs the launch stub
    using T = DmaTile<TM, TN, true, STAGES>;
    extern __shared__ __align__(16) float lds[];
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = tid >> 6;
    const int M = g.M, N = g.OC, K = g.K;

    int tile_m, tile_n;
    tile_coords((M + T::BM - 1) / T::BM, (N + T::BN - 1) / T::BN, tile_m, tile_n);
    const int m0 = tile_m * T::BM, n0 = tile_n * T::BN;

    const __amdgpu_buffer_rsrc_t rsrc_a = make_rsrc(in, in_bytes);
    const __amdgpu_buffer_rsrc_t rsrc_b = make_rsrc(filt, filt_bytes);

    // Per load, the output pixel this lane gathers for: element offset of its
    // window's top-left tap (may be negative) and that tap's coordinates; rows
    // past M get coordinates no tap can bring back inside the image.
    int row_off[T::kALoads], iy0[T::kALoads], ix0[T::kALoads], f_base[T::kBLoads];
#pragma unroll
    for (int j = 0; j < T::kALoads; ++j) {
        const int m = m0 + (4 * j + wave) * 8 + kc_row_in_load(lane);
        if (m < M) {
            const int ox = m % g.OW;
            const int t = m / g.OW;
            const int oy = t % g.OH;
            const int img = t / g.OH;
            iy0[j] = oy * g.sh - g.pt;
            ix0[j] = ox * g.sw - g.pl;
            row_off[j] = ((img * g.H + iy0[j]) * g.W + ix0[j]) * g.C;
        } else {
            iy0[j] = ix0[j] = -(1 << 20);
            row_off[j] = 0;
        }
    }
#pragma unroll
    for (int j = 0; j < T::kBLoads; ++j) {
        const int n = n0 + (4 * j + wave) * 8 + kc_row_in_load(lane);
        f_base[j] = n < N ? n * K * 4 : kOutOfRange;
    }
    // k position of this lane's chunk, as (ky, kx, ci), stepped by BK per slice
    int kpos = kc_chunk(lane) * 4;
    int ky, kx, ci;
    {
        const int tap = kpos / g.C;
        ci = kpos - tap * g.C;
        ky = tap / g.kw;
        kx = tap - ky * g.kw;
    }
    int va[T::kALoads], vb[T::kBLoads];
    auto next_offsets = [&]() {   // offsets of the next slice in order
        const bool k_ok = kpos < K;
        const int tap_off = (ky * g.W + kx) * g.C + ci;
#pragma unroll
        for (int j = 0; j < T::kALoads; ++j) {
            const bool ok = k_ok && (unsigned)(iy0[j] + ky) < (unsigned)g.H && (unsigned)(ix0[j] + kx) < (unsigned)g.W;
            va[j] = ok ? (row_off[j] + tap_off) * 4 : kOutOfRange;
        }
#pragma unroll
        for (int j = 0; j < T::kBLoads; ++j)
            vb[j] = (k_ok && f_base[j] != kOutOfRange) ? f_base[j] + kpos * 4 : kOutOfRange;
        kpos += BK;
        ci += BK;
        while (ci >= g.C) {
            ci -= g.C;
            if (++kx == g.kw) {
                kx = 0;
                ++ky;
            }
        }
    };

    v16f acc[TM][TN];
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j)
#pragma unroll
            for (int v = 0; v < 16; ++v) acc[i][j][v] = 0.f;

#pragma unroll
    for (int s = 0; s < STAGES - 1; ++s) {
        next_offsets();
        float *wr = lds + s * T::kStageFloats;
#pragma unroll
        for (int j = 0; j < T::kALoads; ++j)
            __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrc_a, (lds_void_t *)(wr + (4 * j + wave) * 256), 16, va[j], 0, 0, 0);
#pragma unroll
        for (int j = 0; j < T::kBLoads; ++j)
            __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrc_b, (lds_void_t *)(wr + T::kAFloats + (4 * j + wave) * 256), 16,
                                                     vb[j], 0, 0, 0);
    }
    const int nk = (K + BK - 1) / BK;
    int rd_stage = 0, wr_stage = STAGES - 1;
    if constexpr (MID) {   // ring hand-over after the first MFMA group of a slice (dma_step_mid)
        ring_sync<(STAGES - 2) * T::kLoads>();   // slice 0 has landed
        Frag<TM, TN> frag[2];
        load_frag_swz<TM, TN, true>(frag[0], lds, lds + T::kAFloats, 0, wave >> 1, wave & 1, lane & 31, lane >> 5);
        for (int kt = 0; kt < nk; ++kt) {
            next_offsets();
            const int nx_stage = rd_stage + 1 == STAGES ? 0 : rd_stage + 1;
            dma_step_mid<TM, TN, true, STAGES>(lds + wr_stage * T::kStageFloats, lds + rd_stage * T::kStageFloats,
                                               lds + nx_stage * T::kStageFloats, rsrc_a, rsrc_b, va, vb, acc, frag,
                                               wave, lane);
            rd_stage = nx_stage;
            wr_stage = wr_stage + 1 == STAGES ? 0 : wr_stage + 1;
        }
    } else {
        for (int kt = 0; kt < nk; ++kt) {
            ring_sync<(STAGES - 2) * T::kLoads>();
            next_offsets();
            dma_step<TM, TN, true, STAGES>(lds + wr_stage * T::kStageFloats, lds + rd_stage * T::kStageFloats, rsrc_a,
                                           rsrc_b, va, vb, acc, wave, lane);
            rd_stage = rd_stage + 1 == STAGES ? 0 : rd_stage + 1;
            wr_stage = wr_stage + 1 == STAGES ? 0 : wr_stage + 1;
        }
    }
    wait_vmcnt<0>();   // the trailing dummy loads still target this workgroup's LDS
    acc_settle(acc);
    store_tile<TM, TN>(acc, out, (size_t)N, M, N, m0 + (wave >> 1) * 32 * TM, n0 + (wave & 1) * 32 * TN, lane, ep);
#endif
}

template <int TM, int TN, int STAGES, bool MID = false>
int launch_conv_dma(const float *in, const float *filt, float *out, const ConvGeom &g, size_t in_bytes,
                    size_t filt_bytes, const Epilogue &ep) {
    using T = DmaTile<TM, TN, true, STAGES>;
    const long tiles = (long)((g.M + T::BM - 1) / T::BM) * ((g.OC + T::BN - 1) / T::BN);
    auto kern = conv_dma<TM, TN, STAGES, MID>;
    static bool attr_set = false;
    if (!attr_set) {
        SWC_HIP_TRY(hipFuncSetAttribute(reinterpret_cast<const void *>(kern),
                                        hipFuncAttributeMaxDynamicSharedMemorySize, (int)T::kLdsBytes));
        attr_set = true;
    }
    kern<<<(unsigned)tiles, kThreads, T::kLdsBytes, stream()>>>(in, filt, out, g, (unsigned)in_bytes,
                                                                 (unsigned)filt_bytes, ep);
    SWC_LAUNCH_CHECK();
    return SWC_HIP_OK;
}

// ------------------------------------------------------------ small direct conv
// First layers (iC = 1 or 3, a handful of output channels) have K = kH*kW*iC of
// a few dozen: far too short for the MFMA pipeline, and iC % 4 != 0 rules out
// 128-bit gathers.  One thread per output pixel keeps all oC accumulators in
// registers, walks the taps in the reference's (ky, kx, ci) order and adds
// fl(x*w) with separate fp32 multiply and add starting from the bias — the very
// operation sequence of conv2d_f, so this path is bit-exact.  The filter is
// staged in LDS as [k][oC] and read as wavefront-uniform broadcasts.
constexpr int kDirectMaxK = 128;
constexpr int kDirectMaxOC = 32;

template <int OCQ>   // output channels rounded up to 4*OCQ
__global__ __launch_bounds__(256) void conv_direct(const float *__restrict__ in, const float *__restrict__ filt,
                                                   const float *__restrict__ bias, float *__restrict__ out,
                                                   ConvGeom g, Epilogue ep) {
#pragma clang fp contract(off)   // x*w and the add must round separately, as in the reference's -O2 x86 code
    constexpr int OCP = 4 * OCQ;
    __shared__ __align__(16) float w[kDirectMaxK * OCP];
    __shared__ float bsh[OCP], mean_sh[OCP], slope_sh[OCP], beta_sh[OCP];
    __shared__ float stage[256 * OCP];
    const int K = g.K, OC = g.OC;
    for (int i = threadIdx.x; i < K * OCP; i += 256) {
        const int k = i / OCP, oc = i - k * OCP;
        w[i] = oc < OC ? filt[(size_t)oc * K + k] : 0.f;
    }
    const bool bn = ep.bn_mean != nullptr;
    if (threadIdx.x < OCP) {
        const int oc = threadIdx.x;
        bsh[oc] = oc < OC ? bias[oc] : 0.f;
        if (bn && oc < OC) {
            mean_sh[oc] = ep.bn_mean[oc];
            slope_sh[oc] = (float)((double)ep.bn_scale[oc] / sqrt((double)(ep.bn_var[oc] + ep.eps)));
            beta_sh[oc] = ep.bn_bias[oc];
        }
    }
    __syncthreads();
    const int m = blockIdx.x * 256 + threadIdx.x;
    const bool active = m < g.M;
    const int mm = active ? m : 0;
    const int ox = mm % g.OW;
    const int t = mm / g.OW;
    const int oy = t % g.OH;
    const int img = t / g.OH;
    float acc[OCP];
#pragma unroll
    for (int oc = 0; oc < OCP; ++oc) acc[oc] = bsh[oc];
    // For a fixed ky the taps (kx, ci) are L = kw*C consecutive floats of one input
    // row (NHWC).  They are fetched eight at a time — all loads of a group issued
    // before the first multiply — so the pixel's ~K dependent load latencies
    // shrink to K/8.
    const int L = g.kw * g.C;
    const int ix0 = ox * g.sw - g.pl;
    for (int ky = 0; ky < g.kh; ++ky) {
        const int iy = oy * g.sh - g.pt + ky;
        if ((unsigned)iy >= (unsigned)g.H) continue;   // whole kernel row outside: skipped, as in the reference
        const float *row = in + (((long)img * g.H + iy) * g.W + ix0) * g.C;
        const int kbase = ky * L;
        for (int j0 = 0; j0 < L; j0 += 8) {
            float xv[8];
            bool ok[8];
            int kx = j0 / g.C, ci = j0 - kx * g.C;
#pragma unroll
            for (int u = 0; u < 8; ++u) {
                ok[u] = j0 + u < L && (unsigned)(ix0 + kx) < (unsigned)g.W;
                xv[u] = ok[u] ? row[j0 + u] : 0.f;
                if (++ci == g.C) {
                    ci = 0;
                    ++kx;
                }
            }
#pragma unroll
            for (int u = 0; u < 8; ++u) {
                if (!ok[u]) continue;
                const float x = xv[u];
                const float4 *wk = reinterpret_cast<const float4 *>(&w[(kbase + j0 + u) * OCP]);
#pragma unroll
                for (int q = 0; q < OCQ; ++q) {
                    const float4 wv = wk[q];
                    acc[4 * q + 0] += x * wv.x;
                    acc[4 * q + 1] += x * wv.y;
                    acc[4 * q + 2] += x * wv.z;
                    acc[4 * q + 3] += x * wv.w;
                }
            }
        }
    }
    // Results go through LDS as the [pixel][oC] block they form in the output, so
    // that the global stores are contiguous across the workgroup (a thread's own
    // oC values are only 4*oC bytes apart from its neighbour's).
    if (active) {
#pragma unroll
        for (int oc = 0; oc < OCP; ++oc) {
            if (oc >= OC) break;
            float v = acc[oc];
            if (bn) v = fmaf(v - mean_sh[oc], slope_sh[oc], beta_sh[oc]);
            if (ep.relu) v = (v > 0.f) ? v : 0.f;
            stage[threadIdx.x * OC + oc] = v;
        }
    }
    __syncthreads();
    const int first = blockIdx.x * 256;
    const int pixels = (g.M - first < 256) ? (g.M - first) : 256;
    float *o = out + (size_t)first * OC;
    for (int i = threadIdx.x; i < pixels * OC; i += 256) o[i] = stage[i];
}

int launch_conv_direct(const float *in, const float *filt, const float *bias, float *out, const ConvGeom &g,
                       const Epilogue &ep) {
    const unsigned blocks = ceil_div((size_t)g.M, 256);
    const int ocq = (g.OC + 3) / 4;
    switch (ocq) {
    case 1: conv_direct<1><<<blocks, 256, 0, stream()>>>(in, filt, bias, out, g, ep); break;
    case 2: conv_direct<2><<<blocks, 256, 0, stream()>>>(in, filt, bias, out, g, ep); break;
    case 3: conv_direct<3><<<blocks, 256, 0, stream()>>>(in, filt, bias, out, g, ep); break;
    case 4: conv_direct<4><<<blocks, 256, 0, stream()>>>(in, filt, bias, out, g, ep); break;
    case 5: conv_direct<5><<<blocks, 256, 0, stream()>>>(in, filt, bias, out, g, ep); break;
    case 6: conv_direct<6><<<blocks, 256, 0, stream()>>>(in, filt, bias, out, g, ep); break;
    case 7: conv_direct<7><<<blocks, 256, 0, stream()>>>(in, filt, bias, out, g, ep); break;
    default: conv_direct<8><<<blocks, 256, 0, stream()>>>(in, filt, bias, out, g, ep); break;
    }
    SWC_LAUNCH_CHECK();
    return SWC_HIP_OK;
}

template <int TM, int TN>
int launch_conv(bool vec, const float *in, const float *filt, float *out, const ConvGeom &g, const Epilogue &ep) {
    using T = Tile<TM, TN, true>;
    const long tiles = (long)((g.M + T::BM - 1) / T::BM) * ((g.OC + T::BN - 1) / T::BN);
    auto kern = vec ? conv_igemm<TM, TN, true> : conv_igemm<TM, TN, false>;
    static bool attr_set[2] = {false, false};
    if (!attr_set[vec]) {
        SWC_HIP_TRY(hipFuncSetAttribute(reinterpret_cast<const void *>(kern),
                                        hipFuncAttributeMaxDynamicSharedMemorySize, (int)T::kLdsBytes));
        attr_set[vec] = true;
    }
    kern<<<(unsigned)tiles, kThreads, T::kLdsBytes, stream()>>>(in, filt, out, g, ep);
    SWC_LAUNCH_CHECK();
    return SWC_HIP_OK;
}

int conv_dispatch(const char *who, float *output, const float *input, const float *filter, const float *bias,
                  const size_t *odims, const size_t *idims, const size_t *fdims, const size_t *kernels,
                  const size_t *strides, const size_t *pads, size_t group, const Epilogue &ep_in) {
    if (!odims || !idims || !fdims || !kernels || !strides || !pads)
        return fail(SWC_HIP_EINVAL, "%s: null shape array", who);
    if (group != 1) return fail(SWC_HIP_EUNSUPPORTED, "%s: group = %zu (only 1 is supported)", who, group);
    for (int i = 0; i < 4; ++i)
        if (odims[i] > 0x7fffffffu || idims[i] > 0x7fffffffu || fdims[i] > 0x7fffffffu)
            return fail(SWC_HIP_EINVAL, "%s: dimension too large", who);
    if (odims[0] != idims[0]) return fail(SWC_HIP_EINVAL, "%s: batch of output and input differ", who);
    if (fdims[0] != odims[3] || fdims[3] != idims[3] || fdims[1] != kernels[0] || fdims[2] != kernels[1])
        return fail(SWC_HIP_EINVAL, "%s: filter dims {%zu,%zu,%zu,%zu} do not match oC=%zu, kernels {%zu,%zu}, iC=%zu", who,
                    fdims[0], fdims[1], fdims[2], fdims[3], odims[3], kernels[0], kernels[1], idims[3]);
    if (strides[0] == 0 || strides[1] == 0 || strides[0] > 4096 || strides[1] > 4096 || pads[0] > 4096 ||
        pads[1] > 4096 || kernels[0] == 0 || kernels[1] == 0)
        return fail(SWC_HIP_EINVAL, "%s: bad kernel/stride/pad", who);
    const size_t M = odims[0] * odims[1] * odims[2];
    const size_t K = fdims[1] * fdims[2] * fdims[3];
    if (M > 0x7fffffffu || K > 0x7fffffffu || M * odims[3] > (size_t)1 << 40)
        return fail(SWC_HIP_EINVAL, "%s: problem too large", who);
    if (M == 0 || odims[3] == 0) return SWC_HIP_OK;
    if (!output || !input || !filter || !bias) return fail(SWC_HIP_EINVAL, "%s: null pointer", who);
    ConvGeom g{(int)idims[0], (int)idims[1], (int)idims[2], (int)idims[3], (int)odims[1], (int)odims[2],
               (int)odims[3], (int)kernels[0], (int)kernels[1], (int)strides[0], (int)strides[1], (int)pads[0],
               (int)pads[1], (int)M, (int)K};
    Epilogue ep = ep_in;
    ep.bias = bias;
    const bool vec = (g.C % 4 == 0) && aligned16(input) && aligned16(filter);
    const size_t in_bytes = idims[0] * idims[1] * idims[2] * idims[3] * 4, filt_bytes = odims[3] * K * 4;
    const bool dma_ok = vec && in_bytes < kMaxDmaBytes && filt_bytes < kMaxDmaBytes;
    const char *force = getenv("SWC_HIP_CONV");   // forces a kernel variant (tests, tuning): reg22 reg21 reg12 reg11 | 22_2 21_3 12_3 11_3 11_4 | 11_3m 21_3m 12_3m 22_3m (m: ring hand-over in mid-slice)
    if (force) {
        if (!strcmp(force, "reg22")) return launch_conv<2, 2>(vec, input, filter, output, g, ep);
        if (!strcmp(force, "reg21")) return launch_conv<2, 1>(vec, input, filter, output, g, ep);
        if (!strcmp(force, "reg12")) return launch_conv<1, 2>(vec, input, filter, output, g, ep);
        if (!strcmp(force, "reg11")) return launch_conv<1, 1>(vec, input, filter, output, g, ep);
        if (dma_ok) {
            if (!strcmp(force, "22_2")) return launch_conv_dma<2, 2, 2>(input, filter, output, g, in_bytes, filt_bytes, ep);
            if (!strcmp(force, "21_3")) return launch_conv_dma<2, 1, 3>(input, filter, output, g, in_bytes, filt_bytes, ep);
            if (!strcmp(force, "12_3")) return launch_conv_dma<1, 2, 3>(input, filter, output, g, in_bytes, filt_bytes, ep);
            if (!strcmp(force, "11_3")) return launch_conv_dma<1, 1, 3>(input, filter, output, g, in_bytes, filt_bytes, ep);
            if (!strcmp(force, "11_4")) return launch_conv_dma<1, 1, 4>(input, filter, output, g, in_bytes, filt_bytes, ep);
            if (!strcmp(force, "11_3m")) return launch_conv_dma<1, 1, 3, true>(input, filter, output, g, in_bytes, filt_bytes, ep);
            if (!strcmp(force, "21_3m")) return launch_conv_dma<2, 1, 3, true>(input, filter, output, g, in_bytes, filt_bytes, ep);
            if (!strcmp(force, "12_3m")) return launch_conv_dma<1, 2, 3, true>(input, filter, output, g, in_bytes, filt_bytes, ep);
            if (!strcmp(force, "22_3m")) return launch_conv_dma<2, 2, 3, true>(input, filter, output, g, in_bytes, filt_bytes, ep);
        }
    }
    if (!(force && !strncmp(force, "reg", 3)) && g.K <= kDirectMaxK && g.OC <= kDirectMaxOC && g.C % 4 != 0)
        return launch_conv_direct(input, filter, bias, output, g, ep);
    if (dma_ok) {
        // These layers last 80-160 us: how evenly the tiles divide over the 256 CUs matters as much as
        // the tile's own efficiency.  64x64 tiles (ring hand-over in mid-slice) while there are at least
        // eight of them per CU; below that 64x128 tiles for wide layers, which halve the count but keep
        // two workgroups per CU busy to the end (measured: 105 vs 100 TFLOP/s for 56x56x64->128,
        // 85 vs 90 for 28x28x128->128).
        const size_t tiles64 = ((M + 63) / 64) * ((g.OC + 63) / 64);
        if (tiles64 < 8 * (size_t)num_cus() && g.OC > 64 && ((M + 63) / 64) * ((g.OC + 127) / 128) >= (size_t)num_cus())
            return launch_conv_dma<1, 2, 3>(input, filter, output, g, in_bytes, filt_bytes, ep);
        return launch_conv_dma<1, 1, 3, true>(input, filter, output, g, in_bytes, filt_bytes, ep);
    }
    const long tiles_m128 = (M + 127) / 128;
    if (g.OC > 64 && tiles_m128 * ((g.OC + 127) / 128) >= num_cus())
        return launch_conv<2, 2>(vec, input, filter, output, g, ep);
    if (tiles_m128 * ((g.OC + 63) / 64) >= num_cus()) return launch_conv<2, 1>(vec, input, filter, output, g, ep);
    return launch_conv<1, 1>(vec, input, filter, output, g, ep);
}

} // namespace

extern "C" {

int swc_hip_conv2d_f(float *output, const float *input, const float *filter, const float *bias, const size_t *odims,
                     const size_t *idims, const size_t *fdims, const size_t *bdims, const size_t *kernels,
                     const size_t *strides, const size_t *pads, size_t group) {
    SWC_REQUIRE_INIT();
    (void)bdims;
    Epilogue ep{nullptr, nullptr, nullptr, nullptr, nullptr, 0.f, 0};
    return conv_dispatch("swc_hip_conv2d_f", output, input, filter, bias, odims, idims, fdims, kernels, strides, pads,
                         group, ep);
}

int swc_hip_conv2dFused_f(float *output, const float *input, const float *filter, const float *bias,
                          const size_t *odims, const size_t *idims, const size_t *fdims, const size_t *bdims,
                          const size_t *kernels, const size_t *strides, const size_t *pads, size_t group,
                          const float *bn_mean, const float *bn_var, const float *bn_scale, const float *bn_bias,
                          float epsilon, int relu) {
    SWC_REQUIRE_INIT();
    (void)bdims;
    if (bn_mean || bn_var || bn_scale || bn_bias)
        SWC_ARG(bn_mean && bn_var && bn_scale && bn_bias);
    Epilogue ep{nullptr, bn_mean, bn_var, bn_scale, bn_bias, epsilon, relu};
    return conv_dispatch("swc_hip_conv2dFused_f", output, input, filter, bias, odims, idims, fdims, kernels, strides,
                         pads, group, ep);
}

} // extern "C"
