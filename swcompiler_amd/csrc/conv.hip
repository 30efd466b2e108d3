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
#include "mfma_dma2.hpp"
#include "mfma_tile.hpp"
#include <algorithm>
#include <cstdlib>
#include <cstring>
#include <type_traits>

using namespace swc_hip;
using namespace swc_hip::mfma;

namespace {

struct ConvGeom {
    int N, H, W, C;      // input NHWC
    int OH, OW, OC;      // output
    int kh, kw, sh, sw, pt, pl;
    int M, K;            // GEMM view: output pixels, kh*kw*C
    // Order in which the rows of the GEMM view walk the output pixels.  0: raster order (image, row, column).
    // 1: by 2 x 2 windows — row m is pixel (2py + d/2, 2px + d%2) of window m/4 = (image, py, px) in raster order
    // of the windows, d = m%4 — so that every aligned group of four rows is one window of a 2 x 2 / stride 2
    // pooling (even OH and OW only).
    int win = 0;
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

// Row m of the GEMM view -> output pixel (see ConvGeom::win).
__device__ __forceinline__ void pixel_of_row(const ConvGeom &g, int m, int &img, int &oy, int &ox) {
    if (g.win) {
        const int w = m >> 2, d = m & 3, pw = g.OW >> 1, ph = g.OH >> 1;
        const int px = w % pw, t = w / pw;
        const int py = t % ph;
        img = t / ph;
        oy = 2 * py + (d >> 1);
        ox = 2 * px + (d & 1);
    } else {
        ox = m % g.OW;
        const int t = m / g.OW;
        oy = t % g.OH;
        img = t / g.OH;
    }
}

// The per-element epilogue of every convolution kernel here: bias, folded batchnorm, second summand, ReLU.
struct ColumnParams {
    float bias, mean, slope, beta;
};
__device__ __forceinline__ ColumnParams column_params(const Epilogue &ep, int col, bool ok) {
    ColumnParams c{(ep.bias && ok) ? ep.bias[col] : 0.f, 0.f, 1.f, 0.f};
    if (ep.bn_mean && ok) {   // slope formed in double and rounded once, as store_tile_impl
        c.mean = ep.bn_mean[col];
        c.slope = (float)((double)ep.bn_scale[col] / sqrt((double)(ep.bn_var[col] + ep.eps)));
        c.beta = ep.bn_bias[col];
    }
    return c;
}
// The same in two steps, for a kernel that requests the parameters at its start and needs them at its end: the raw
// loads (nothing waits for them), and, once they have arrived, the arithmetic.
struct ColumnRaw {
    float bias, mean, var, scale, beta;
};
__device__ __forceinline__ ColumnRaw column_raw(const Epilogue &ep, int col, bool ok) {
    ColumnRaw r{(ep.bias && ok) ? ep.bias[col] : 0.f, 0.f, 1.f, 1.f, 0.f};
    if (ep.bn_mean && ok) {
        r.mean = ep.bn_mean[col];
        r.var = ep.bn_var[col];
        r.scale = ep.bn_scale[col];
        r.beta = ep.bn_bias[col];
    }
    return r;
}
__device__ __forceinline__ ColumnParams column_params(const Epilogue &ep, const ColumnRaw &r) {
    ColumnParams c{r.bias, 0.f, 1.f, 0.f};
    if (ep.bn_mean) {
        c.mean = r.mean;
        c.slope = (float)((double)r.scale / sqrt((double)(r.var + ep.eps)));
        c.beta = r.beta;
    }
    return c;
}
// maxpool_f's choice among the taps of a window in its order (kernels.h:343-383: the first, then whatever is greater)
__device__ __forceinline__ float window_max(float a, float b, float c, float d) {
    float best = a;
    if (b > best) best = b;
    if (c > best) best = c;
    if (d > best) best = d;
    return best;
}

// A wavefront's 32 TM x 32 TN part of a tile whose rows are in window order (ConvGeom::win).  The four rows that a
// lane holds in accumulator registers 4g .. 4g + 3 are the four pixels of one window.
//   POOL == false: each goes to its own pixel of the [N, OH, OW, OC] output (the arithmetic of store_tile_impl);
//   POOL == true:  the epilogue of each, then their maximum to the window's place in the [N, OH/2, OW/2, OC] output.
// M is a multiple of 4 here, so a window is wholly inside or outside.
template <int TM, int TN, bool POOL>
__device__ __forceinline__ void store_tile_windows(const v16f (&acc)[TM][TN], float *__restrict__ out, const ConvGeom &g,
                                                   int row0, int col0, int lane, const Epilogue &ep,
                                                   const ColumnParams (&cp)[TN]) {
    const int l32 = lane & 31, h = lane >> 5;
    const int N = g.OC, pw = g.OW >> 1, ph = g.OH >> 1;
    const bool bn = ep.bn_mean != nullptr;
    // this lane's windows: w0, w0 + 2, w0 + 4, ... (rows row0 + 4h + 8 * (g + 4 tm))
    int w = (row0 >> 2) + h;
    int px = w % pw, t = w / pw;
    int py = t % ph, img = t / ph;
#pragma unroll
    for (int tm = 0; tm < TM; ++tm) {
#pragma unroll
        for (int q = 0; q < 4; ++q) {
            if (4 * w < g.M) {
                const size_t pix = ((size_t)(img * g.OH + 2 * py) * g.OW + 2 * px);
#pragma unroll
                for (int tn = 0; tn < TN; ++tn) {
                    const int col = col0 + tn * 32 + l32;
                    if (col >= N) continue;
                    float x[4];
#pragma unroll
                    for (int d = 0; d < 4; ++d) {
                        x[d] = acc[tm][tn][4 * q + d] + cp[tn].bias;
                        if (bn) x[d] = fmaf(x[d] - cp[tn].mean, cp[tn].slope, cp[tn].beta);
                    }
                    if (ep.residual) {
#pragma unroll
                        for (int d = 0; d < 4; ++d) x[d] += ep.residual[(pix + (d >> 1) * g.OW + (d & 1)) * N + col];
                    }
                    if (ep.relu) {
#pragma unroll
                        for (int d = 0; d < 4; ++d) x[d] = (x[d] > 0.f) ? x[d] : 0.f;
                    }
                    if (POOL) {
                        out[(size_t)w * N + col] = window_max(x[0], x[1], x[2], x[3]);
                    } else {
#pragma unroll
                        for (int d = 0; d < 4; ++d) out[(pix + (d >> 1) * g.OW + (d & 1)) * N + col] = x[d];
                    }
                }
            }
            w += 2;
            px += 2;
            while (px >= pw) {
                px -= pw;
                if (++py == ph) py = 0, ++img;
            }
        }
    }
}

// Direct-to-LDS variant (mfma_dma.hpp): the im2col gather is expressed as one
// 32-bit byte offset per lane per load — out-of-image taps and rows past M get
// the out-of-range offset and arrive in LDS as zeros.  Needs iC % 4 == 0,
// 16-byte-aligned tensors and input/filter below 2 GiB.
//
// Work is counted in units of one K slice of one tile.  `dp_tiles` workgroups
// each take a whole tile.  The tiles that are left — fewer than the chip holds
// workgroups at a time, so that handing them out whole would leave most CUs
// idle while a few finish — are cut along K: their units form one sequence
// that `sk_wgs` further workgroups share evenly (the first `r` take q + 1
// units, the others q).  The sharing workgroups have the LOWEST workgroup
// numbers: they start first, are done after a few slices, and whole tiles take
// their places, so that the kernel ends with every slot finishing a whole tile
// at about the same time.  (With the short pieces last, most of the chip idled
// while they ran: 85 / 153 / 77 / 77 us against 80 / 136 / 70 / 67 us for the
// four layers of the ResNet-like block, 84 against 71 us for 7x7x512->512.)  A workgroup whose share covers a whole tile
// stores it as usual; otherwise it stores the raw partial sums of its piece in
// slot 2s (the piece its share begins with) or 2s + 1 (the piece it ends with)
// of `part`, and conv_sk_finish adds the pieces of each tile in K order.
struct SkPlan {
    int dp_tiles;   // tiles computed whole, one workgroup each
    int sk_wgs;     // workgroups sharing the remaining tiles (0: none remain)
    int q, r;       // units per sharing workgroup: q, and one more for the first r
};

// Tile number -> tile coordinates.  Workgroups are dealt round-robin to the 8 XCDs, each with its own L2; the whole
// tiles (all but the last few) are renumbered so that the ones one XCD works on are consecutive; consecutive numbers
// walk the column tiles of one block of rows, then the next block of rows: the tiles an XCD holds at a time share
// their rows of the gathered operand (the filter, a few hundred KB, stays in every L2 anyway).  The shared tiles are
// taken in order.
__device__ __forceinline__ int xcd_renumbered(int pid, int dp_tiles) {
    constexpr int kXcd = Device::xcds;
    const int full = dp_tiles - dp_tiles % kXcd;
    return pid < full ? (pid % kXcd) * (full / kXcd) + pid / kXcd : pid;
}
__device__ __forceinline__ void sk_tile_coords(int pid, int dp_tiles, int tiles_m, int tiles_n, int &tile_m, int &tile_n) {
    (void)tiles_m;
    pid = xcd_renumbered(pid, dp_tiles);
    tile_m = pid / tiles_n;
    tile_n = pid - tile_m * tiles_n;
}

template <int TM, int TN, int STAGES, bool MID = false>
__global__ __launch_bounds__(kThreads) void conv_dma(const float *__restrict__ in, const float *__restrict__ filt,
                                                     float *__restrict__ out, ConvGeom g, unsigned in_bytes,
                                                     unsigned filt_bytes, Epilogue ep, SkPlan sk,
                                                     float *__restrict__ part, int pool) {
#if __HIP_DEVICE_COMPILE__   // the host pass only needs the launch stub
    using T = DmaTile<TM, TN, true, STAGES>;
    extern __shared__ __align__(16) float lds[];
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int M = g.M, N = g.OC, K = g.K;
    const int tiles_m = (M + T::BM - 1) / T::BM, tiles_n = (N + T::BN - 1) / T::BN;
    const int nk = (K + BK - 1) / BK;

    const __amdgpu_buffer_rsrc_t rsrc_a = make_rsrc(in, in_bytes);
    const __amdgpu_buffer_rsrc_t rsrc_b = make_rsrc(filt, filt_bytes);

    // this workgroup's units [u0, u1) of the sequence (tile 0: units 0..nk-1, tile 1: nk..2nk-1, ...)
    int u0, u1, share = -1;
    if ((int)blockIdx.x >= sk.sk_wgs) {
        u0 = ((int)blockIdx.x - sk.sk_wgs) * nk;
        u1 = u0 + nk;
    } else {
        share = blockIdx.x;
        u0 = sk.dp_tiles * nk + share * sk.q + (share < sk.r ? share : sk.r);
        u1 = u0 + sk.q + (share < sk.r ? 1 : 0);
    }
    for (int piece = 0; u0 < u1; ++piece) {
        const int pid = u0 / nk;
        const int kt_begin = u0 - pid * nk;
        const int kt_end = (u1 - u0 < nk - kt_begin) ? kt_begin + (u1 - u0) : nk;
        const bool whole = kt_begin == 0 && kt_end == nk;
        u0 += kt_end - kt_begin;
        if (piece) __builtin_amdgcn_s_barrier();   // every wavefront is done reading the ring of the previous piece

        int tile_m, tile_n;
        sk_tile_coords(pid, sk.dp_tiles, tiles_m, tiles_n, tile_m, tile_n);
        const int m0 = tile_m * T::BM, n0 = tile_n * T::BN;
        const int k_limit = (kt_end * BK < K) ? kt_end * BK : K;
        // The three workgroups of a CU run in step (they start together and take equally long), so the start and
        // the end of a tile are not covered by the others' matrix work: both are kept short and run at a raised
        // wavefront priority, the K loop at the lowest.  The epilogue's per-column parameters are requested here,
        // ahead of the ring's loads (older loads complete first, so the ring's counts are unaffected), and
        // turned into bias / slope / offset after the first slice has landed.
        __builtin_amdgcn_s_setprio(3);
        const int col_first = n0 + (wave & 1) * 32 * TN + (lane & 31);
        ColumnRaw raw[TN];
        ColumnParams cp[TN];
        if (whole && g.win) {
#pragma unroll
            for (int tn = 0; tn < TN; ++tn) raw[tn] = column_raw(ep, col_first + tn * 32, col_first + tn * 32 < N);
        }
        __builtin_amdgcn_sched_barrier(0);
        auto first_slice_landed = [&]() {
            if (whole && g.win) {
#pragma unroll
                for (int tn = 0; tn < TN; ++tn) cp[tn] = column_params(ep, raw[tn]);
            }
            __builtin_amdgcn_s_setprio(0);
        };

        // Per load, the output pixel this lane gathers for: element offset of its
        // window's top-left tap (may be negative) and that tap's coordinates; rows
        // past M get coordinates no tap can bring back inside the image.
        int row_off[T::kALoads], iy0[T::kALoads], ix0[T::kALoads], f_base[T::kBLoads];
#pragma unroll
        for (int j = 0; j < T::kALoads; ++j) {
            const int m = m0 + (4 * j + wave) * 8 + kc_row_in_load(lane);
            if (m < M) {
                int img, oy, ox;
                pixel_of_row(g, m, img, oy, ox);
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
        int kpos = kt_begin * BK + kc_chunk(lane, wave) * 4;
        int ky, kx, ci;
        {
            const int tap = kpos / g.C;
            ci = kpos - tap * g.C;
            ky = tap / g.kw;
            kx = tap - ky * g.kw;
        }
        int va[T::kALoads], vb[T::kBLoads];
        auto next_offsets = [&]() {   // offsets of the next slice in order
            const bool k_ok = kpos < k_limit;
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
                __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrc_a, (lds_void_t *)(wr + (4 * j + wave) * 256), 16, va[j], 0, 0,
                                                         0);
#pragma unroll
            for (int j = 0; j < T::kBLoads; ++j)
                __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrc_b, (lds_void_t *)(wr + T::kAFloats + (4 * j + wave) * 256),
                                                         16, vb[j], 0, 0, 0);
        }
        int rd_stage = 0, wr_stage = STAGES - 1;
        if constexpr (MID) {   // ring hand-over after the first MFMA group of a slice (dma_step_mid)
            ring_sync<(STAGES - 2) * T::kLoads>();   // the first slice has landed
            first_slice_landed();
            Frag<TM, TN> frag[2];
            load_frag_swz<TM, TN, true>(frag[0], lds, lds + T::kAFloats, 0, wave >> 1, wave & 1, lane & 31, lane >> 5);
            for (int kt = kt_begin; kt < kt_end; ++kt) {
                next_offsets();
                const int nx_stage = rd_stage + 1 == STAGES ? 0 : rd_stage + 1;
                dma_step_mid<TM, TN, true, STAGES>(lds + wr_stage * T::kStageFloats, lds + rd_stage * T::kStageFloats,
                                                   lds + nx_stage * T::kStageFloats, rsrc_a, rsrc_b, va, vb, acc, frag,
                                                   wave, lane);
                rd_stage = nx_stage;
                wr_stage = wr_stage + 1 == STAGES ? 0 : wr_stage + 1;
            }
        } else {
            for (int kt = kt_begin; kt < kt_end; ++kt) {
                ring_sync<(STAGES - 2) * T::kLoads>();
                if (kt == kt_begin) first_slice_landed();
                next_offsets();
                dma_step<TM, TN, true, STAGES>(lds + wr_stage * T::kStageFloats, lds + rd_stage * T::kStageFloats, rsrc_a,
                                               rsrc_b, va, vb, acc, wave, lane);
                rd_stage = rd_stage + 1 == STAGES ? 0 : rd_stage + 1;
                wr_stage = wr_stage + 1 == STAGES ? 0 : wr_stage + 1;
            }
        }
        __builtin_amdgcn_s_setprio(3);
        wait_vmcnt<0>();   // the trailing dummy loads still target this workgroup's LDS
        acc_settle(acc);
        if (whole) {
            const int row0 = m0 + (wave >> 1) * 32 * TM, col0 = n0 + (wave & 1) * 32 * TN;
            if (!g.win) store_tile<TM, TN>(acc, out, (size_t)N, M, N, row0, col0, lane, ep);
            else if (pool) store_tile_windows<TM, TN, true>(acc, out, g, row0, col0, lane, ep, cp);
            else store_tile_windows<TM, TN, false>(acc, out, g, row0, col0, lane, ep, cp);
        } else {
            float *slot = part + (size_t)(2 * share + (piece ? 1 : 0)) * (T::BM * T::BN);
            store_tile_impl<TM, TN, false, false>(acc, slot, (size_t)T::BN, T::BM, T::BN, (wave >> 1) * 32 * TM,
                                           (wave & 1) * 32 * TN, lane, Epilogue{});
        }
    }
#endif
}

#if __HIP_DEVICE_COMPILE__
// store_tile_windows with as few vector instructions as the arithmetic allows (they are paid for in matrix-core time):
// stores through a buffer descriptor of the output — one 32-bit offset per window and column block, the four pixels of
// a window at scalar offsets from it — and the window's coordinates from one division on scalars.  No second summand;
// the output below 2 GiB.
template <int TM, int TN, bool POOL>
__device__ __forceinline__ void store_tile_windows_buf(const v16f (&acc)[TM][TN], __amdgpu_buffer_rsrc_t rsrc_out,
                                                       const ConvGeom &g, int row0, int col0, int lane, const Epilogue &ep,
                                                       const ColumnParams (&cp)[TN]) {
    const int l32 = lane & 31, h = lane >> 5;
    const int N = g.OC, pw = g.OW >> 1, ph = g.OH >> 1;
    const bool bn = ep.bn_mean != nullptr;
    const int s_px = N * 4, s_row = g.OW * N * 4;   // byte steps to the window's right and lower pixels
    // this lane's windows: w0, w0 + 2, ... with w0 = row0 / 4 + h (row0 is the same for the whole wavefront)
    int w = row0 >> 2;
    int px, py, img;
    {
        const int t = w / pw;
        px = w - t * pw;
        img = t / ph;
        py = t - img * ph;
    }
    w += h;
    px += h;
    if (px >= pw) {
        px -= pw;
        if (++py == ph) py = 0, ++img;
    }
#pragma unroll
    for (int tm = 0; tm < TM; ++tm) {
#pragma unroll
        for (int q = 0; q < 4; ++q) {
            if (4 * w < g.M) {
                const int base = POOL ? w * N : ((img * g.OH + 2 * py) * g.OW + 2 * px) * N;
#pragma unroll
                for (int tn = 0; tn < TN; ++tn) {
                    const int col = col0 + tn * 32 + l32;
                    if (col >= N) continue;
                    const int voff = (base + col) * 4;
                    float x[4];
#pragma unroll
                    for (int d = 0; d < 4; ++d) {
                        x[d] = acc[tm][tn][4 * q + d] + cp[tn].bias;
                        if (bn) x[d] = fmaf(x[d] - cp[tn].mean, cp[tn].slope, cp[tn].beta);
                    }
                    if (ep.relu) {
#pragma unroll
                        for (int d = 0; d < 4; ++d) x[d] = (x[d] > 0.f) ? x[d] : 0.f;
                    }
                    if (POOL) {
                        __builtin_amdgcn_raw_buffer_store_b32(__builtin_bit_cast(unsigned, window_max(x[0], x[1], x[2], x[3])),
                                                              rsrc_out, voff, 0, 0);
                    } else {
                        __builtin_amdgcn_raw_buffer_store_b32(__builtin_bit_cast(unsigned, x[0]), rsrc_out, voff, 0, 0);
                        __builtin_amdgcn_raw_buffer_store_b32(__builtin_bit_cast(unsigned, x[1]), rsrc_out, voff, s_px, 0);
                        __builtin_amdgcn_raw_buffer_store_b32(__builtin_bit_cast(unsigned, x[2]), rsrc_out, voff, s_row, 0);
                        __builtin_amdgcn_raw_buffer_store_b32(__builtin_bit_cast(unsigned, x[3]), rsrc_out, voff, s_row + s_px, 0);
                    }
                }
            }
            w += 2;
            px += 2;
            while (px >= pw) {
                px -= pw;
                if (++py == ph) py = 0, ++img;
            }
        }
    }
}

// The four loads of a wavefront for one slice of a 64 x 64 tile into stage `wr` (conv_dma_lean): per-lane offsets
// va/vb, the position inside the tap (A) and along K (B) as scalar offsets.
__device__ __forceinline__ void lean_request(char *__restrict__ wr, __amdgpu_buffer_rsrc_t rsrc_a, __amdgpu_buffer_rsrc_t rsrc_b,
                                             int va0, int va1, int vb0, int vb1, int soff_a, int soff_b, int wave) {
    __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrc_a, (lds_void_t *)(wr + wave * 1024), 16, va0, soff_a, 0, 0);
    __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrc_a, (lds_void_t *)(wr + (4 + wave) * 1024), 16, va1, soff_a, 0, 0);
    __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrc_b, (lds_void_t *)(wr + 8192 + wave * 1024), 16, vb0, soff_b, 0, 0);
    __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrc_b, (lds_void_t *)(wr + 8192 + (4 + wave) * 1024), 16, vb1, soff_b, 0, 0);
}
__device__ __forceinline__ void lean_read(Frag<1, 1> &f, const char *__restrict__ stage, int a_addr, int b_addr) {
    const float4 a = *reinterpret_cast<const float4 *>(stage + a_addr);
    const float4 b = *reinterpret_cast<const float4 *>(stage + b_addr);
    f.a[0][0] = a.x, f.a[0][1] = a.y, f.a[0][2] = a.z, f.a[0][3] = a.w;
    f.b[0][0] = b.x, f.b[0][1] = b.y, f.b[0][2] = b.z, f.b[0][3] = b.w;
}
// One slice out of stage `rd`; behind the barrier the loads of the slice two on go into `wr`; the first fragments of
// the next slice come out of `nx` (see dma_step_mid).  The three stages are distinct, which is what __restrict__ says:
// without it every LDS read behind a load would wait for ALL outstanding loads.
__device__ __forceinline__ void lean_step(char *__restrict__ wr, const char *__restrict__ rd, const char *__restrict__ nx,
                                          __amdgpu_buffer_rsrc_t rsrc_a, __amdgpu_buffer_rsrc_t rsrc_b, int va0, int va1,
                                          int vb0, int vb1, int soff_a, int soff_b, const int (&a_addr)[4],
                                          const int (&b_addr)[4], v16f (&acc)[1][1], Frag<1, 1> (&frag)[2], int wave) {
#pragma unroll
    for (int gq = 0; gq < 4; ++gq) {
        if (gq == 1) {
            ring_sync<0>();
            lean_request(wr, rsrc_a, rsrc_b, va0, va1, vb0, vb1, soff_a, soff_b, wave);
        }
        if (gq < 3) lean_read(frag[(gq + 1) & 1], rd, a_addr[gq + 1], b_addr[gq + 1]);
        else lean_read(frag[0], nx, a_addr[0], b_addr[0]);
        __builtin_amdgcn_sched_barrier(0);
        const Frag<1, 1> &f = frag[gq & 1];
#pragma unroll
        for (int s4 = 0; s4 < 4; ++s4) mfma_acc(acc[0][0], f.a[0][s4], f.b[0][s4]);
        __builtin_amdgcn_sched_barrier(0);
    }
}
#endif

// conv_dma<1,1,3,true> with next to no vector-ALU work in its K loop, for layers whose channel count is a multiple
// of 32 (a K slice then lies inside one filter tap, the same for every lane).
// Why.  On this chip the vector ALU and the matrix pipe of a SIMD do not run side by side: a microbenchmark of three
// wavefronts per SIMD, each issuing 16 dependent v_mfma_f32_32x32x2_f32 per iteration, loses 2 - 5 cycles of MFMA
// throughput for every VALU instruction that any of the three executes (v_mov 2.2, v_fma 3.1, v_cmp 4.9; LDS reads
// and scalar instructions under half a cycle).  conv_dma spends about 60 VALU instructions per slice of 16 MFMAs
// on gather offsets (bounds tests, tap stepping) and LDS addresses — a fifth of the slice's 1024 MFMA cycles — and
// that, not its memory traffic, is most of what its matrix cores wait for.
// What differs here:
//   * the gather offset of a row changes with the tap only: within a tap the channel position travels in the load's
//     scalar offset, so the per-lane offsets (with their bounds tests) are recomputed once per tap, C/32 slices;
//   * the filter rows' offsets never change (the k position is the scalar offset);
//   * the K loop is unrolled over the three ring stages, so every LDS address is a lane constant (eight registers,
//     one per operand and group of 8 k) plus an immediate.
// Pieces, slots, ring discipline, epilogues and results are conv_dma's.
__global__ __launch_bounds__(kThreads) void conv_dma_lean(const float *__restrict__ in, const float *__restrict__ filt,
                                                          float *__restrict__ out, ConvGeom g, unsigned in_bytes,
                                                          unsigned filt_bytes, Epilogue ep, SkPlan sk,
                                                          float *__restrict__ part, int pool, unsigned out_bytes) {
#if __HIP_DEVICE_COMPILE__
    // out_bytes: size of the output if it is below 2 GiB (stores then go through a buffer descriptor), else 0
    constexpr int TM = 1, TN = 1, STAGES = 3;
    using T = DmaTile<TM, TN, true, STAGES>;
    static_assert(T::kALoads == 2 && T::kBLoads == 2, "");
    extern __shared__ __align__(16) float lds[];
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int M = g.M, N = g.OC, K = g.K;
    const int tiles_m = (M + T::BM - 1) / T::BM, tiles_n = (N + T::BN - 1) / T::BN;
    const int nk = K / BK;   // C % 32 == 0
    const __amdgpu_buffer_rsrc_t rsrc_a = make_rsrc(in, in_bytes);
    const __amdgpu_buffer_rsrc_t rsrc_b = make_rsrc(filt, filt_bytes);
    char *const lds_b = reinterpret_cast<char *>(lds);

    // LDS byte addresses of this lane's fragments inside a stage, per group of 8 k (see load_frag_swz)
    int a_addr[4], b_addr[4];
    {
        const int l32 = lane & 31, h = lane >> 5, swz = (l32 >> 1) & 7;
        const int row_a = (wave >> 1) * 32 + l32, row_b = (wave & 1) * 32 + l32;
#pragma unroll
        for (int gq = 0; gq < 4; ++gq) {
            a_addr[gq] = (row_a * BK + (((2 * gq + h) ^ swz) << 2)) * 4;
            b_addr[gq] = (T::kAFloats + row_b * BK + (((2 * gq + h) ^ swz) << 2)) * 4;
        }
    }
    const int chunk16 = kc_chunk(lane, wave) * 16;   // byte position of this lane's 16 bytes inside a slice of a row

    int u0, u1, share = -1;
    if ((int)blockIdx.x >= sk.sk_wgs) {
        u0 = ((int)blockIdx.x - sk.sk_wgs) * nk;
        u1 = u0 + nk;
    } else {
        share = blockIdx.x;
        u0 = sk.dp_tiles * nk + share * sk.q + (share < sk.r ? share : sk.r);
        u1 = u0 + sk.q + (share < sk.r ? 1 : 0);
    }
    for (int piece = 0; u0 < u1; ++piece) {
        const int pid = u0 / nk;
        const int kt_begin = u0 - pid * nk;
        const int kt_end = (u1 - u0 < nk - kt_begin) ? kt_begin + (u1 - u0) : nk;
        const bool whole = kt_begin == 0 && kt_end == nk;
        u0 += kt_end - kt_begin;
        if (piece) __builtin_amdgcn_s_barrier();   // every wavefront is done reading the ring of the previous piece

        int tile_m, tile_n;
        sk_tile_coords(pid, sk.dp_tiles, tiles_m, tiles_n, tile_m, tile_n);
        const int m0 = tile_m * T::BM, n0 = tile_n * T::BN;
        __builtin_amdgcn_s_setprio(3);
        const int col_first = n0 + (wave & 1) * 32 + (lane & 31);
        ColumnRaw raw[TN];
        ColumnParams cp[TN];
        if (whole && g.win) raw[0] = column_raw(ep, col_first, col_first < N);
        __builtin_amdgcn_sched_barrier(0);

        // per-lane constants of the two rows of A and of B that this lane gathers for.  In window order with at
        // least eight windows per output row the pixel of row m0 + r follows from the tile's first window (one
        // division on scalars) by at most two carries — the general map costs four divisions per row, and vector
        // instructions here are paid for in matrix-core time.
        const int pw = g.OW >> 1, ph = g.OH >> 1;
        const bool near = g.win && pw >= 8;
        int img_t = 0, py_t = 0, px_t = 0;
        if (near) {
            const int w0 = m0 >> 2, t0 = w0 / pw;
            px_t = w0 - t0 * pw;
            img_t = t0 / ph;
            py_t = t0 - img_t * ph;
        }
        int row_off[2], iy0[2], ix0[2], vb[2];
#pragma unroll
        for (int j = 0; j < 2; ++j) {
            const int r = (4 * j + wave) * 8 + kc_row_in_load(lane);
            const int m = m0 + r;
            if (m < M) {
                int img, oy, ox;
                if (near) {
                    int px = px_t + (r >> 2), py = py_t;
                    img = img_t;
#pragma unroll
                    for (int c = 0; c < 2; ++c)
                        if (px >= pw) {
                            px -= pw;
                            if (++py == ph) py = 0, ++img;
                        }
                    oy = 2 * py + ((r >> 1) & 1);
                    ox = 2 * px + (r & 1);
                } else {
                    pixel_of_row(g, m, img, oy, ox);
                }
                iy0[j] = oy * g.sh - g.pt;
                ix0[j] = ox * g.sw - g.pl;
                row_off[j] = (((img * g.H + iy0[j]) * g.W + ix0[j]) * g.C) * 4 + chunk16;
            } else {
                iy0[j] = ix0[j] = -(1 << 20);
                row_off[j] = 0;
            }
            const int n = n0 + (4 * j + wave) * 8 + kc_row_in_load(lane);
            vb[j] = n < N ? n * K * 4 + chunk16 : kOutOfRange;
        }
        // the loads' position: slice lk of the piece = tap (ky, kx), channels ci .. ci + 31
        int lk = kt_begin, ky, kx, ci;
        {
            const int tap = (lk * BK) / g.C;
            ci = lk * BK - tap * g.C;
            ky = tap / g.kw;
            kx = tap - ky * g.kw;
        }
        int va[2];
        auto retap = [&]() {   // the rows' offsets under tap (ky, kx), or out of range
            const int tap_off = (ky * g.W + kx) * g.C * 4;
#pragma unroll
            for (int j = 0; j < 2; ++j) {
                const bool ok = (unsigned)(iy0[j] + ky) < (unsigned)g.H && (unsigned)(ix0[j] + kx) < (unsigned)g.W;
                va[j] = ok ? row_off[j] + tap_off : kOutOfRange;
            }
        };
        retap();
        // moves the loads' position on by a slice; past the piece's end the loads are empty
        auto advance = [&]() {
            ++lk;
            ci += BK;
            if (lk == kt_end) {
                va[0] = va[1] = vb[0] = vb[1] = kOutOfRange;
            } else if (ci == g.C) {
                asm volatile("" ::: "memory");   // keeps this a (wavefront-uniform) branch: as selects it would run every slice
                ci = 0;
                if (++kx == g.kw) {
                    kx = 0;
                    ++ky;
                }
                retap();
            }
        };
        constexpr int kStageBytes = T::kStageFloats * 4;
        char *const st0 = lds_b, *const st1 = lds_b + kStageBytes, *const st2 = lds_b + 2 * kStageBytes;

        v16f acc[1][1];
#pragma unroll
        for (int v = 0; v < 16; ++v) acc[0][0][v] = 0.f;
        Frag<1, 1> frag[2];
        // a step out of stage RD: its loads go into stage (RD + 2) % 3, the next slice sits in (RD + 1) % 3
        auto step = [&](char *wr, const char *rd, const char *nx) {
            lean_step(wr, rd, nx, rsrc_a, rsrc_b, va[0], va[1], vb[0], vb[1], ci * 4, lk * BK * 4, a_addr, b_addr, acc, frag, wave);
            advance();
        };

        lean_request(st0, rsrc_a, rsrc_b, va[0], va[1], vb[0], vb[1], ci * 4, lk * BK * 4, wave);
        advance();
        lean_request(st1, rsrc_a, rsrc_b, va[0], va[1], vb[0], vb[1], ci * 4, lk * BK * 4, wave);
        advance();
        ring_sync<T::kLoads>();   // the first slice has landed
        if (whole && g.win) cp[0] = column_params(ep, raw[0]);
        __builtin_amdgcn_s_setprio(0);
        lean_read(frag[0], st0, a_addr[0], b_addr[0]);
        int kt = kt_begin;
        for (; kt + 3 <= kt_end; kt += 3) {
            step(st2, st0, st1);
            step(st0, st1, st2);
            step(st1, st2, st0);
        }
        if (kt < kt_end) step(st2, st0, st1);
        if (kt + 1 < kt_end) step(st0, st1, st2);

        __builtin_amdgcn_s_setprio(3);
        wait_vmcnt<0>();   // the trailing empty loads still target this workgroup's LDS
        acc_settle(acc);
        if (whole) {
            const int row0 = m0 + (wave >> 1) * 32, col0 = n0 + (wave & 1) * 32;
            if (!g.win) {
                store_tile<1, 1>(acc, out, (size_t)N, M, N, row0, col0, lane, ep);
            } else if (out_bytes && !ep.residual) {
                const __amdgpu_buffer_rsrc_t rsrc_out = make_rsrc(out, out_bytes);
                if (pool) store_tile_windows_buf<1, 1, true>(acc, rsrc_out, g, row0, col0, lane, ep, cp);
                else store_tile_windows_buf<1, 1, false>(acc, rsrc_out, g, row0, col0, lane, ep, cp);
            } else if (pool) {
                store_tile_windows<1, 1, true>(acc, out, g, row0, col0, lane, ep, cp);
            } else {
                store_tile_windows<1, 1, false>(acc, out, g, row0, col0, lane, ep, cp);
            }
        } else {
            float *slot = part + (size_t)(2 * share + (piece ? 1 : 0)) * (T::BM * T::BN);
            store_tile_impl<1, 1, false, false>(acc, slot, (size_t)T::BN, T::BM, T::BN, (wave >> 1) * 32, (wave & 1) * 32, lane,
                                                Epilogue{});
        }
    }
#endif
}

// ------------------------------------------------------------------------------------------------ conv_win
// The tile kernel of the layers that matter most: output with whole 2 x 2 windows (rows in window order), a channel
// count that is a multiple of 32, tensors below 2 GiB.  Tile (64 x 64), ring, swizzle, MFMA order, pieces, slots and
// epilogue arithmetic are conv_dma<1,1,3,true>'s — the same bits — but a vector-ALU instruction issued by ANY
// wavefront of a SIMD costs that SIMD 2-5 cycles of matrix throughput, so everything around the MFMAs is cut down to
// what the arithmetic needs:
//   * all geometry comes from one argument record in the kernel-argument segment; tile and window coordinates are
//     scalar arithmetic with precomputed multiply-shift divisions (no division runs in the vector unit, no
//     argument is kept in a vector register across the K loop);
//   * the gather offset of a row is lane constant + scalar: the descriptor starts (pt*W + pl) pixels below the
//     input, which makes a row's top-left tap offset non-negative, and the tap position travels in the load's
//     scalar offset with the channel position.  A change of filter tap only re-selects between that constant and
//     "out of range" (3 instructions per row: the column test; the row test is a lane mask kept per filter row);
//   * the K loop holds no vector-ALU instruction at all: its LDS reads are assembly with immediate offsets;
//   * the pixel of a window follows from its number w by one division: 2 x 2 windows in raster order make the
//     output offset of window w's first pixel 2 OC (w + floor(w / pw) pw) — no image or row coordinates.
// Measured against conv_dma_lean in alternating runs on one box, the four layers of the ResNet-like block:
// 73.5 / 133.2 / 69.1 / 67.5 -> 68.2 / 120.2 / 64.9 / 63.7 us.  Tried with it and dropped: 128 x 64 tiles (a wavefront
// owning 64 x 32; three ring stages with two workgroups per CU, or two stages with three): 77.4 / 123.8 / 72.2 / 71.4 and
// 71.4 / 122.9 / 75.2 / 74.1 us — fewer bytes per MFMA buy nothing here.
struct Magic {   // x / d for 0 <= x < 2^31 as (umulhi(x, mul) + x) >> shift
    unsigned mul, shift;
};
Magic magic_of(unsigned d) {
    unsigned shift = 0;
    while ((1ull << shift) < d) ++shift;
    return Magic{(unsigned)(((1ull << 32) * ((1ull << shift) - d)) / d + 1), shift};
}
__device__ __forceinline__ int magic_div(int x, Magic m) { return (int)((__umulhi((unsigned)x, m.mul) + (unsigned)x) >> m.shift); }

struct WinArgs {
    const float *in, *filt;
    float *out;
    float *part;                        // slots for the pieces of tiles cut along K
    Epilogue ep;
    SkPlan sk;
    unsigned in_bytes, filt_bytes, out_bytes;   // out_bytes: of the tensor that is written (pooled or not)
    int shift_bytes;                    // (pt * W + pl) * C * 4: how far below the input its descriptor starts
    int N, K, C, H, W, kw, sh, sw, pt, pl, OW;
    int pw, ph, nwin;                   // windows per output row and column, windows in all (M / 4)
    int tiles_n, nk, cpt;               // column tiles, K slices per tile, slices per filter tap (C / 32)
    Magic d_pw, d_ph, d_tn;
    int last_round;                     // workgroups from this number on finish together (see the K loop)
};

#if __HIP_DEVICE_COMPILE__
// The K loop's LDS reads are written as assembly: the compiler cannot tell which ring stage a direct-to-LDS load
// targets and would make every LDS read behind one wait for ALL outstanding loads; it also re-derives addresses
// it could keep.  The ring's real ordering is the explicit s_waitcnt vmcnt + s_barrier (ring_sync); these reads are
// ordered among themselves and against the MFMAs by lds_wait, which takes the fragments as operands.
typedef float f4v __attribute__((ext_vector_type(4)));
template <int OFF> __device__ __forceinline__ void lds_read128(f4v &dst, int addr) {   // addr + OFF: LDS byte address
    static_assert(OFF >= 0 && OFF < 65536, "the instruction's offset field has 16 bits");
    asm volatile("ds_read_b128 %0, %1 offset:%2" : "=v"(dst) : "v"(addr), "n"(OFF));
}
struct WinFrag {
    f4v a, b;
};
// waits until at most PENDING LDS reads are outstanding; the fragments' registers are operands so that no use of
// them moves above the wait
template <int PENDING> __device__ __forceinline__ void lds_wait(WinFrag &f) {
    asm volatile("s_waitcnt lgkmcnt(%2)" : "+v"(f.a), "+v"(f.b) : "n"(PENDING));
}
// if_set where the lane's bit of `mask` is set, else if_clear (the mask stays in scalar registers)
__device__ __forceinline__ int select_by_mask(unsigned long long mask, int if_set, int if_clear) {
    int r;
    asm("v_cndmask_b32_e64 %0, %1, %2, %3" : "=v"(r) : "v"(if_clear), "v"(if_set), "s"(mask));
    return r;
}
#endif

// The argument record as it lies in the kernel-argument segment, for the fields that are needed only once the K loop
// is over: read again there (scalar loads that hit the scalar cache) instead of kept in scalar registers across the
// loop, which has none to spare — the compiler parked them in lanes of a vector register (44 v_writelane at the
// start, some 60 v_readlane behind the loop, per workgroup: vector instructions that take matrix-pipe cycles).
typedef const __attribute__((address_space(4))) WinArgs *WinArgsInSegment;
__device__ __forceinline__ WinArgsInSegment win_args_again() {
    WinArgsInSegment p = (WinArgsInSegment)__builtin_amdgcn_kernarg_segment_ptr();
    asm volatile("" : "+s"(p));   // a value the compiler cannot trace back to the loads at the kernel's entry
    return p;
}

template <bool POOL, bool RES>
__global__ __launch_bounds__(kThreads) void conv_win(const WinArgs a) {
#if __HIP_DEVICE_COMPILE__
    // A new wavefront is the youngest on its SIMD and the CU serves the oldest first: without a raised priority its
    // first instructions wait behind the MFMAs of the workgroups that are in their K loops.
    __builtin_amdgcn_s_setprio(3);
    constexpr int BM = 64, BN = 64;
    constexpr int kLoads = 4;                                // 1-KiB loads per wavefront per slice: two of A, two of B
    constexpr int kBBytes = BN * 128, kABytes = BM * 128;   // a stage: the filter rows, then the gathered rows
    constexpr int kStageBytes = kABytes + kBBytes;
    extern __shared__ __align__(16) float lds[];
    char *const lds_b = reinterpret_cast<char *>(lds);
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int l32 = lane & 31, h = lane >> 5;
    const int wave_m = wave >> 1, wave_n = wave & 1;
    const int nk = a.nk;
    const int chunk16 = kc_chunk(lane, wave) * 16;   // byte position of this lane's 16 bytes inside a slice of a row
    const int row_in_load = kc_row_in_load(lane);
    const __amdgpu_buffer_rsrc_t rsrc_a = make_rsrc(reinterpret_cast<const char *>(a.in) - a.shift_bytes, a.in_bytes + a.shift_bytes);
    const __amdgpu_buffer_rsrc_t rsrc_b = make_rsrc(a.filt, a.filt_bytes);

    int u0, u1, share = -1;
    if ((int)blockIdx.x >= a.sk.sk_wgs) {
        u0 = ((int)blockIdx.x - a.sk.sk_wgs) * nk;
        u1 = u0 + nk;
    } else {
        share = blockIdx.x;
        u0 = a.sk.dp_tiles * nk + share * a.sk.q + (share < a.sk.r ? share : a.sk.r);
        u1 = u0 + a.sk.q + (share < a.sk.r ? 1 : 0);
    }
    for (int piece = 0; u0 < u1; ++piece) {
        int pid, kt_begin, kt_end;
        if (share < 0) {
            pid = (int)blockIdx.x - a.sk.sk_wgs, kt_begin = 0, kt_end = nk;
        } else {
            pid = u0 / nk;
            kt_begin = u0 - pid * nk;
            kt_end = (u1 - u0 < nk - kt_begin) ? kt_begin + (u1 - u0) : nk;
        }
        const bool whole = kt_begin == 0 && kt_end == nk;
        u0 += kt_end - kt_begin;
        if (piece) {
            __builtin_amdgcn_s_barrier();   // every wavefront is done reading the ring of the previous piece
            __builtin_amdgcn_s_setprio(3);
        }
        pid = xcd_renumbered(pid, a.sk.dp_tiles);
        const int tile_m = magic_div(pid, a.d_tn), tile_n = pid - tile_m * a.tiles_n;
        const int m0 = tile_m * BM, n0 = tile_n * BN;

        // The filter rows' loads of the first two slices go out before anything else is computed (load j of a
        // wavefront fills the 1-KiB block 4j + wave of its operand's part of a stage).
        int vb[2];
#pragma unroll
        for (int j = 0; j < 2; ++j) {
            const int n = n0 + (4 * j + wave) * 8 + row_in_load;
            vb[j] = n < a.N ? n * a.K * 4 + chunk16 : kOutOfRange;
        }
        int soff_b = kt_begin * BK * 4;
        auto request_b = [&](int stage, int soff) {
            char *const wr = lds_b + stage * kStageBytes;
#pragma unroll
            for (int j = 0; j < 2; ++j)
                __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrc_b, (lds_void_t *)(wr + (4 * j + wave) * 1024), 16, vb[j], soff, 0, 0);
        };
        const bool two = kt_begin + 1 < kt_end;
        request_b(0, soff_b);
        if (two) request_b(1, soff_b + BK * 4);
        // the epilogue's per-column parameters (a whole tile's): requested here — older loads complete first, so the
        // count below of the loads that may still be pending is unaffected — and turned into bias / slope / offset
        // once the first slice has landed
        const int col = n0 + wave_n * 32 + l32;
        ColumnRaw raw;
        ColumnParams cp;
        if (whole) raw = column_raw(a.ep, col, col < a.N);
        __builtin_amdgcn_sched_barrier(0);

        // per A load: the lane's row is row (4j + wave) * 8 + lane / 8 of the tile = pixel d of window w
        int row_off[2], iy0[2], ix0[2], va[2];
        const int d = row_in_load & 3;
#pragma unroll
        for (int j = 0; j < 2; ++j) {
            const int w = (m0 >> 2) + 8 * j + 2 * wave + (row_in_load >> 2);
            const int t = magic_div(w, a.d_pw), px = w - t * a.pw;
            const int img = magic_div(t, a.d_ph), py = t - img * a.ph;
            const int y = (2 * py + (d >> 1)) * a.sh - a.pt;
            ix0[j] = (2 * px + (d & 1)) * a.sw - a.pl;
            iy0[j] = w < a.nwin ? y : -(1 << 20);   // rows past M: no filter row brings them inside the image
            row_off[j] = ((img * a.H + y) * a.W + ix0[j]) * a.C * 4 + chunk16 + a.shift_bytes;
        }
        // the loads' position: slice lk = slice cs of tap (ky, kx)
        int lk = kt_begin, ky = 0, kx = 0, cs = 0;
        if (kt_begin) {
            const int tap = kt_begin / a.cpt;
            cs = kt_begin - tap * a.cpt;
            ky = tap / a.kw;
            kx = tap - ky * a.kw;
        }
        unsigned long long y_ok[2];
        auto refilter_row = [&]() {
#pragma unroll
            for (int j = 0; j < 2; ++j) y_ok[j] = __builtin_amdgcn_ballot_w64((unsigned)(iy0[j] + ky) < (unsigned)a.H);
        };
        auto retap = [&]() {
#pragma unroll
            for (int j = 0; j < 2; ++j) {
                const unsigned long long ok = y_ok[j] & __builtin_amdgcn_ballot_w64((unsigned)(ix0[j] + kx) < (unsigned)a.W);
                va[j] = select_by_mask(ok, row_off[j], kOutOfRange);
            }
        };
        refilter_row();
        retap();
        int soff_a = ((ky * a.W + kx) * a.C + cs * BK) * 4;
        // moves the loads' position on by a slice (the array va has ONE place that writes it: two would be merged
        // into a store at a variable index, and the array would live in scratch memory)
        auto advance = [&]() {
            ++lk, ++cs;
            soff_a += BK * 4, soff_b += BK * 4;
            if (lk < kt_end && cs == a.cpt) {
                cs = 0;
                asm volatile("" : "+s"(cs));   // keeps this a (wavefront-uniform) branch: as selects it would run every slice
                if (++kx == a.kw) {
                    kx = 0, ++ky;
                    refilter_row();
                }
                soff_a = (ky * a.W + kx) * a.C * 4;
                retap();
            }
        };
        auto request_a = [&](int stage) {
            char *const wr = lds_b + stage * kStageBytes + kBBytes;
#pragma unroll
            for (int j = 0; j < 2; ++j)
                __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrc_a, (lds_void_t *)(wr + (4 * j + wave) * 1024), 16, va[j], soff_a, 0, 0);
        };
        request_a(0);
        advance();
        if (two) request_a(1);
        advance();
        __builtin_amdgcn_sched_barrier(0);

        // LDS byte addresses of this lane's fragments in stage 0, per group of 8 k (see load_frag_swz)
        int a_addr[4], b_addr[4];
        {
            const int base = (int)(unsigned)(uintptr_t)(lds_void_t *)lds_b, swz = (l32 >> 1) & 7;
#pragma unroll
            for (int gq = 0; gq < 4; ++gq) {
                const int chunk = ((2 * gq + h) ^ swz) << 4;
                a_addr[gq] = base + kBBytes + (wave_m * 32 + l32) * 128 + chunk;
                b_addr[gq] = base + (wave_n * 32 + l32) * 128 + chunk;
                asm volatile("" : "+v"(a_addr[gq]), "+v"(b_addr[gq]));   // eight registers, kept: not re-derived from shared parts at every use
            }
        }

        v16f acc[1][1];
#pragma unroll
        for (int v = 0; v < 16; ++v) acc[0][0][v] = 0.f;
        WinFrag frag[2];
        auto read_frags = [&](WinFrag &f, auto stage_c, auto gq_c) {
            constexpr int kStage = decltype(stage_c)::value * kStageBytes, GQ = decltype(gq_c)::value;
            lds_read128<kStage>(f.a, a_addr[GQ]);
            lds_read128<kStage>(f.b, b_addr[GQ]);
        };
        using G0 = std::integral_constant<int, 0>;
        using G1 = std::integral_constant<int, 1>;
        using G2 = std::integral_constant<int, 2>;
        using G3 = std::integral_constant<int, 3>;
        // the MFMAs of group GQ of a slice out of frag[GQ & 1], behind the reads of the next group's fragments
        auto group = [&](auto gq_c, auto rd_c, auto nx_c) {
            constexpr int GQ = decltype(gq_c)::value;
            if constexpr (GQ == 0) read_frags(frag[1], rd_c, G1{});
            else if constexpr (GQ == 1) read_frags(frag[0], rd_c, G2{});
            else if constexpr (GQ == 2) read_frags(frag[1], rd_c, G3{});
            else read_frags(frag[0], nx_c, G0{});
            WinFrag &f = frag[GQ & 1];
            lds_wait<2>(f);   // the fragments read a group ago are here
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int s4 = 0; s4 < 4; ++s4) mfma_acc(acc[0][0], f.a[s4], f.b[s4]);
            __builtin_amdgcn_sched_barrier(0);
        };
        // A CU serves its wavefronts by priority, then oldest first: left alone, the workgroups of a CU finish one
        // after the other and the last runs by itself for a third of its K range — and a single workgroup cannot
        // hide the loads' latency behind one slice.  Where all whole tiles are on the chip at once (a single round)
        // they therefore lower their priority as they get on (3, 2, 1, 0 by quarters of the K range): whoever is
        // behind is served first and they finish together (2 % on the 28 x 28 x 128 layers).  With several rounds the
        // staggered ends are wanted — they hide the starts of the workgroups that follow (the same rule there: 68 ->
        // 75 us on 56 x 56 x 64 -> 64) — and every K loop runs at the lowest priority.
        const bool fair = (int)blockIdx.x >= a.last_round;
        const int quarter = (kt_end - kt_begin + 3) >> 2;
        int done = 0, next_drop = quarter;
        // One slice out of stage RD.  Behind the barrier (every wavefront's part of the next slice has landed,
        // nobody reads the slice before this one any more) the loads of the slice two on go into stage WR; the
        // first fragments of the next slice come out of stage NX.
        auto step = [&](auto rd_c, auto wr_c, auto nx_c) {
            group(G0{}, rd_c, nx_c);
            ring_sync<0>();
            if (lk < kt_end) {   // (past the piece's end there is nothing to load)
                request_a(decltype(wr_c)::value);
                request_b(decltype(wr_c)::value, soff_b);
            }
            __builtin_amdgcn_sched_barrier(0);
            group(G1{}, rd_c, nx_c);
            group(G2{}, rd_c, nx_c);
            group(G3{}, rd_c, nx_c);
            advance();
            if (fair && ++done == next_drop) {
                next_drop += quarter;
                if (done == quarter) __builtin_amdgcn_s_setprio(2);
                else if (done == 2 * quarter) __builtin_amdgcn_s_setprio(1);
                else __builtin_amdgcn_s_setprio(0);
            }
        };
        using S0 = std::integral_constant<int, 0>;
        using S1 = std::integral_constant<int, 1>;
        using S2 = std::integral_constant<int, 2>;
        if (two) ring_sync<2>();   // all but the second slice's gathered rows — the last two loads — have landed
        else ring_sync<0>();
        if (whole) cp = column_params(a.ep, raw);
        if (!fair) __builtin_amdgcn_s_setprio(0);
        read_frags(frag[0], S0{}, G0{});
        int kt = kt_begin;
        for (; kt + 3 <= kt_end; kt += 3) {
            step(S0{}, S2{}, S1{});
            step(S1{}, S0{}, S2{});
            step(S2{}, S1{}, S0{});
        }
        if (kt < kt_end) step(S0{}, S2{}, S1{});
        if (kt + 1 < kt_end) step(S1{}, S0{}, S2{});

        __builtin_amdgcn_s_setprio(3);
        lds_wait<0>(frag[0]);   // the fragments read ahead for a slice that does not follow
        acc_settle(acc);
        if (whole) {
            // Lane (l32, h) holds column `col` of the windows wbase + 2 q, four pixels each (accumulator registers
            // 4q .. 4q + 3).  One 32-bit offset per window; the window's other pixels (and those of the second
            // summand) at scalar offsets from it.
            const WinArgsInSegment z = win_args_again();
            const Magic d_pw{z->d_pw.mul, z->d_pw.shift};
            const int pw = z->pw, nwin = z->nwin;
            const bool relu = z->ep.relu != 0;
            const __amdgpu_buffer_rsrc_t rsrc_out = make_rsrc(z->out, z->out_bytes);
            const int N = z->N, s_px = N * 4, s_row = z->OW * N * 4;
            const int wbase = (m0 >> 2) + wave_m * 8 + h;
            const bool bn = z->ep.bn_mean != nullptr;
            int voff[4];
#pragma unroll
            for (int q = 0; q < 4; ++q) {
                const int w = wbase + 2 * q;
                const int at = POOL ? (w * N + col) * 4 : ((w + magic_div(w, d_pw) * pw) * 2 * N + col) * 4;
                voff[q] = (w < nwin && col < N) ? at : kOutOfRange;
            }
            float add[4][4];
            if constexpr (RES) {
                const __amdgpu_buffer_rsrc_t rsrc_res = make_rsrc(z->ep.residual, (unsigned)nwin * 16u * (unsigned)N);
#pragma unroll
                for (int q = 0; q < 4; ++q) {
                    add[q][0] = __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(rsrc_res, voff[q], 0, 0));
                    add[q][1] = __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(rsrc_res, voff[q], s_px, 0));
                    add[q][2] = __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(rsrc_res, voff[q], s_row, 0));
                    add[q][3] = __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(rsrc_res, voff[q], s_row + s_px, 0));
                }
            }
            // (batchnorm and ReLU or not: four straight-line copies behind wavefront-uniform branches — as selects on the
            // two flags they were two more vector instructions for every one of the 16 elements)
            auto finish = [&](auto bn_c, auto relu_c) {
#pragma unroll
                for (int q = 0; q < 4; ++q) {
                    float x[4];
#pragma unroll
                    for (int e = 0; e < 4; ++e) {
                        x[e] = acc[0][0][4 * q + e] + cp.bias;
                        if constexpr (decltype(bn_c)::value) x[e] = fmaf(x[e] - cp.mean, cp.slope, cp.beta);
                        if constexpr (RES) x[e] += add[q][e];
                        if constexpr (decltype(relu_c)::value) x[e] = (x[e] > 0.f) ? x[e] : 0.f;
                    }
                    if constexpr (POOL) {
                        __builtin_amdgcn_raw_buffer_store_b32(__builtin_bit_cast(unsigned, window_max(x[0], x[1], x[2], x[3])), rsrc_out, voff[q], 0, 0);
                    } else {
                        __builtin_amdgcn_raw_buffer_store_b32(__builtin_bit_cast(unsigned, x[0]), rsrc_out, voff[q], 0, 0);
                        __builtin_amdgcn_raw_buffer_store_b32(__builtin_bit_cast(unsigned, x[1]), rsrc_out, voff[q], s_px, 0);
                        __builtin_amdgcn_raw_buffer_store_b32(__builtin_bit_cast(unsigned, x[2]), rsrc_out, voff[q], s_row, 0);
                        __builtin_amdgcn_raw_buffer_store_b32(__builtin_bit_cast(unsigned, x[3]), rsrc_out, voff[q], s_row + s_px, 0);
                    }
                }
            };
            if (bn) {
                if (relu) finish(std::true_type{}, std::true_type{});
                else finish(std::true_type{}, std::false_type{});
            } else {
                if (relu) finish(std::false_type{}, std::true_type{});
                else finish(std::false_type{}, std::false_type{});
            }
        } else {
            float *slot = win_args_again()->part + (size_t)(2 * share + (piece ? 1 : 0)) * (BM * BN);
            store_tile_impl<1, 1, false, false>(acc, slot, (size_t)BN, BM, BN, wave_m * 32, wave_n * 32, lane, Epilogue{});
        }
    }
#endif
}

// Adds the pieces of every shared tile that more than one workgroup worked on (see conv_dma) in K order and
// applies the epilogue.  blockIdx.x = shared tile, blockIdx.y = block of 16 rows of it.  With `pool` (rows in window
// order) the finished values of a window's four rows meet in LDS and their maximum is stored.
template <int BM, int BN>
__global__ __launch_bounds__(256) void conv_sk_finish(float *__restrict__ out, const float *__restrict__ part, ConvGeom g,
                                                      int nk, SkPlan sk, Epilogue ep, int vec_ok, int pool) {
    const int M = g.M, N = g.OC;
    const int t = blockIdx.x;
    const int first = t * nk, last = first + nk - 1;   // this tile's units, counted from the first shared unit
    const int big = sk.r * (sk.q + 1);                 // units held by the shares of q + 1
    auto share_of = [&](int u) { return u < big ? u / (sk.q + 1) : sk.r + (u - big) / sk.q; };
    const int s_lo = share_of(first), s_hi = share_of(last);
    if (s_lo == s_hi) return;   // one workgroup had the whole tile and stored it
    const int tiles_m = (M + BM - 1) / BM, tiles_n = (N + BN - 1) / BN;
    int tile_m, tile_n;
    sk_tile_coords(sk.dp_tiles + t, sk.dp_tiles, tiles_m, tiles_n, tile_m, tile_n);
    // the sum over the pieces of columns c .. c + 3 of row r of the tile
    auto sum_pieces = [&](int r, int c) {
        float4 sum = {0.f, 0.f, 0.f, 0.f};
        // sixteen pieces' loads in flight (a tile is cut into 8 or 16 pieces on a whole chip: one round trip to memory
        // instead of two to four, in a kernel that is little else), added in K order
        constexpr int kAtOnce = 16;
        for (int s0 = s_lo; s0 <= s_hi; s0 += kAtOnce) {
            float4 v[kAtOnce];
#pragma unroll
            for (int i = 0; i < kAtOnce; ++i) {
                const int s = s0 + i;
                const int begin = s * sk.q + (s < sk.r ? s : sk.r);
                const float *slot = part + (size_t)(2 * s + (begin < first ? 1 : 0)) * (BM * BN);
                v[i] = s <= s_hi ? *reinterpret_cast<const float4 *>(slot + r * BN + c) : make_float4(0.f, 0.f, 0.f, 0.f);
            }
#pragma unroll
            for (int i = 0; i < kAtOnce; ++i)
                if (s0 + i <= s_hi) sum.x += v[i].x, sum.y += v[i].y, sum.z += v[i].z, sum.w += v[i].w;
        }
        return sum;
    };
    // the epilogue of store_tile_impl on the four columns; `pix` = the row's pixel in the output.  The columns'
    // parameters are fetched (and the batchnorm slope formed) before the pieces are asked for, so that their latency
    // and arithmetic run beside the pieces' loads instead of behind them.
    struct Columns {
        float bias[4], mean[4], slope[4], beta[4];
    };
    auto columns = [&](int col) {
        Columns p;
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            const bool in = col + e < N;
            p.bias[e] = (in && ep.bias) ? ep.bias[col + e] : 0.f;
            p.mean[e] = p.beta[e] = 0.f, p.slope[e] = 1.f;
            if (in && ep.bn_mean) {
                const float ve = ep.bn_var[col + e] + ep.eps;
                p.slope[e] = (float)((double)ep.bn_scale[col + e] / sqrt((double)ve));
                p.mean[e] = ep.bn_mean[col + e], p.beta[e] = ep.bn_bias[col + e];
            }
        }
        return p;
    };
    auto finish = [&](float4 sum, const Columns &p, int col, size_t pix, float (&x)[4]) {
        x[0] = sum.x, x[1] = sum.y, x[2] = sum.z, x[3] = sum.w;
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            if (col + e >= N) break;
            float y = x[e] + p.bias[e];
            if (ep.bn_mean) y = fmaf(y - p.mean[e], p.slope[e], p.beta[e]);
            if (ep.residual) y += ep.residual[pix * N + col + e];
            if (ep.relu) y = (y > 0.f) ? y : 0.f;
            x[e] = y;
        }
    };
    auto pixel = [&](int row) -> size_t {
        if (!g.win) return (size_t)row;
        int img, oy, ox;
        pixel_of_row(g, row, img, oy, ox);
        return ((size_t)img * g.OH + oy) * g.OW + ox;
    };
    auto store4 = [&](float *dst, int col, const float (&x)[4]) {
        if (vec_ok && col + 3 < N) {
            *reinterpret_cast<float4 *>(dst) = make_float4(x[0], x[1], x[2], x[3]);
        } else {
            for (int e = 0; e < 4 && col + e < N; ++e) dst[e] = x[e];
        }
    };
    if (!pool) {
        constexpr int kQuads = 16 * BN / 4;   // float4s in a block of 16 rows
        for (int i = threadIdx.x; i < kQuads; i += 256) {
            const int r = blockIdx.y * 16 + i / (BN / 4), c = (i % (BN / 4)) * 4;
            const int row = tile_m * BM + r, col = tile_n * BN + c;
            if (row >= M || col >= N) continue;
            const Columns p = columns(col);
            const size_t pix = pixel(row);
            float x[4];
            finish(sum_pieces(r, c), p, col, pix, x);
            store4(out + pix * N + col, col, x);
        }
    } else {
        // every thread finishes one row x four columns as above, into LDS; then the four rows of each window meet
        __shared__ float done[16][BN];
        constexpr int kQuads = 16 * BN / 4;
        for (int i = threadIdx.x; i < kQuads; i += 256) {
            const int rl = i / (BN / 4), c = (i % (BN / 4)) * 4;
            const int r = blockIdx.y * 16 + rl;
            const int row = tile_m * BM + r, col = tile_n * BN + c;
            if (row >= M || col >= N) continue;
            const Columns p = columns(col);
            float x[4];
            finish(sum_pieces(r, c), p, col, pixel(row), x);
#pragma unroll
            for (int e = 0; e < 4; ++e) done[rl][c + e] = x[e];
        }
        __syncthreads();
        constexpr int kWindowQuads = 4 * BN / 4;
        for (int i = threadIdx.x; i < kWindowQuads; i += 256) {
            const int rl = 4 * (i / (BN / 4)), c = (i % (BN / 4)) * 4;
            const int row = tile_m * BM + blockIdx.y * 16 + rl, col = tile_n * BN + c;
            if (row >= M || col >= N) continue;
            float best[4];
#pragma unroll
            for (int e = 0; e < 4; ++e) best[e] = window_max(done[rl][c + e], done[rl + 1][c + e], done[rl + 2][c + e], done[rl + 3][c + e]);
            store4(out + (size_t)(row >> 2) * N + col, col, best);
        }
    }
}

// How the tiles of an M x OC output are handed out (see conv_dma): whole tiles while they fill every
// workgroup slot of the chip (`slots` = CUs x workgroups resident per CU), the rest cut along K — when at
// least one full round of whole tiles precedes them and they would fill less than half of the last round;
// otherwise (small layers, nearly full last rounds) the pieces and the second kernel cost more than the idle
// CUs (LeNet's 12x12x20 -> 50 layer: 20 us whole, 28 us cut).
// A layer with fewer tiles than slots and a long K (the late stages of a residual network at a moderate
// batch: 32 x 7 x 7 x 512 -> 512 has 200 tiles of 144 slices each) would leave CUs idle for its whole
// duration: all of its tiles are cut, into as many shares as there are slots.  With a twelfth of a round or
// less (one image: 16 tiles of 32 slices for 14 x 14 x 1024 -> 256, 24 us as whole tiles) K = 512 is long enough.
constexpr int kShareAllMinSlices = 64;   // K >= 2048: below that the pieces and the second kernel cost what the idle CUs do
int share_all_min_slices() {
    const int n = switches().conv_share_all;   // tuning: slices per tile from which a short layer is cut
    return n > 0 ? n : n < 0 ? 1 << 30 : kShareAllMinSlices;
}

// A compute unit serves its resident workgroups oldest first at the rate of its matrix cores: what has to be even
// is the work per CU.  With at least as many tiles as CUs, every CU gets the same number of whole tiles (the
// dispatcher refills slots as they free up) and the tiles beyond a multiple of the CU count are cut into one piece
// per CU, started first (the first workgroups of a launch land on distinct CUs): with pieces of four slices or more on
// only some CUs those CUs finished 4-5 us after the others (traced per workgroup: 65.5 against 61 us on 28x28x128->128).
constexpr int kPieceMinSlices = 2;   // a piece costs a ring start and a tile store
// The pieces need a second kernel (5-6 us with the gap before it) and their own stores, the more of them the more
// tiles are cut: cutting pays only if whole tiles would leave the average CU idle for longer than that while the
// busiest one works through its last tile.  Idle time in slices = (rounds of the busiest CU - tiles per CU) x slices
// per tile; tiles are cut from 12 slices + 1/16 per cut tile on.  Measured at batch 32, whole against cut (idle
// slices, cut tiles): 28x28x512 -> 256 1x1/2 (7.5, 136) 21.0 / 26.4 us; 14x14x1024 -> 256 1x1 (15, 136) 37.5 / 39.4;
// 7x7x2048 -> 512 1x1 (14, 200) 41.2 / 44.3; 56x56x64 -> 128 3x3 (13.5, 64) 125.9 / 124.0; 7x7x512 -> 2048 1x1 (14, 32)
// 44.0 / 40.8; 56x56x64 -> 64 3x3 (15.8, 32) 74.1 / 71.9; 14x14x1024 -> 2048 1x1/2 (28, 32) 78.1 / 65.7; 28x28x128 -> 128 3x3
// (34, 16) 77.7 / 67.6; 14x14x256 -> 256 3x3 (34, 136) 75.5 / 69.7; 14x14x512 -> 512 3x3 (68, 136) 271 / 215.
constexpr int kMinIdleSlices = 12;
SkPlan sk_plan(long tiles, int nk, int slots, bool allow_shared) {
    SkPlan p{(int)tiles, 0, 0, 0};
    if (!allow_shared || tiles == 0) return p;
    const int piece_min = switches().conv_piece_min > 0 ? switches().conv_piece_min : kPieceMinSlices;
    const long cus = num_cus() < slots ? num_cus() : slots;   // (tests pretend a smaller chip through `slots`)
    const int min_idle = switches().conv_min_idle >= 0 ? switches().conv_min_idle : kMinIdleSlices;
    const long cut = tiles < cus ? tiles : tiles % cus;
    if (min_idle > 0 && ((tiles + cus - 1) / cus * cus - tiles) * nk * 16 < (min_idle * 16 + cut) * cus) return p;
    long rest, wgs;
    if (tiles < cus) {
        // fewer tiles than CUs: all are cut if K is long (a nearly full round: leave it; a twelfth of a round or
        // less — single images — is cut from K = 512 on), into as many pieces as the chip holds workgroups
        const int min_slices = share_all_min_slices();
        const bool long_k = nk >= min_slices || (min_slices == kShareAllMinSlices && 12 * tiles <= slots && nk >= 16);
        if (!long_k) return p;
        rest = tiles;
        wgs = slots;
        if (rest * nk < 4 * wgs) wgs = rest * nk / 4;
    } else {
        rest = tiles % cus;
        if (rest == 0 || nk < 8) return p;
        wgs = cus;
        if (rest * nk < piece_min * wgs) wgs = rest * nk / piece_min;
    }
    const long units = rest * nk;
    if (wgs <= rest) return p;              // shares of a tile or more each: nothing to gain
    p.dp_tiles = (int)(tiles - rest);
    p.sk_wgs = (int)wgs;
    p.q = (int)(units / wgs);
    p.r = (int)(units % wgs);
    return p;
}

// Workgroups of one kernel variant that the chip holds at a time (its LDS and registers decide).
template <int TM, int TN, int STAGES, bool MID>
int conv_dma_slots() {
    if (switches().conv_slots > 0) return switches().conv_slots;   // tests: pretend the chip holds this many workgroups
    static int per_cu = 0;
    if (!per_cu) {
        using T = DmaTile<TM, TN, true, STAGES>;
        auto kern = conv_dma<TM, TN, STAGES, MID>;
        (void)hipFuncSetAttribute(reinterpret_cast<const void *>(kern), hipFuncAttributeMaxDynamicSharedMemorySize,
                                  (int)T::kLdsBytes);
        int n = 0;
        if (hipOccupancyMaxActiveBlocksPerMultiprocessor(&n, kern, kThreads, T::kLdsBytes) != hipSuccess || n < 1) {
            (void)hipGetLastError();
            n = 1;
        }
        per_cu = n;
    }
    return per_cu * num_cus();
}

template <int TM, int TN, int STAGES, bool MID>
SkPlan conv_dma_plan(const ConvGeom &g, bool allow_shared) {
    using T = DmaTile<TM, TN, true, STAGES>;
    const long tiles = (long)((g.M + T::BM - 1) / T::BM) * ((g.OC + T::BN - 1) / T::BN);
    return sk_plan(tiles, (g.K + BK - 1) / BK, conv_dma_slots<TM, TN, STAGES, MID>(), allow_shared);
}

template <int TM, int TN, int STAGES, bool MID>
size_t conv_dma_scratch_bytes(const ConvGeom &g) {
    using T = DmaTile<TM, TN, true, STAGES>;
    return (size_t)2 * conv_dma_plan<TM, TN, STAGES, MID>(g, true).sk_wgs * T::BM * T::BN * sizeof(float);
}

// `scratch` (may be null) receives the pieces of shared tiles; without it every tile is computed whole.
template <int TM, int TN, int STAGES, bool MID = false>
int launch_conv_dma(const float *in, const float *filt, float *out, const ConvGeom &g, size_t in_bytes,
                    size_t filt_bytes, const Epilogue &ep, float *scratch = nullptr, bool pool = false) {
    using T = DmaTile<TM, TN, true, STAGES>;
    const long tiles = (long)((g.M + T::BM - 1) / T::BM) * ((g.OC + T::BN - 1) / T::BN);
    const int nk = (g.K + BK - 1) / BK;
    const SkPlan p = conv_dma_plan<TM, TN, STAGES, MID>(g, scratch != nullptr);
    bool lean = false;   // the variant with a K loop free of vector-ALU work (conv_dma_lean); SWC_HIP_CONV_LEAN=0 (test-only) rules it out
    if constexpr (TM == 1 && TN == 1 && STAGES == 3 && MID) {
        lean = g.C % BK == 0 && switches().conv_lean;
        if (lean) {
            note_kernel("conv_dma_lean%s%s", p.sk_wgs ? " + conv_sk_finish" : "", pool ? " (pooled)" : "");
            const size_t out_bytes = (size_t)(pool ? g.M / 4 : g.M) * g.OC * 4;
            conv_dma_lean<<<(unsigned)(p.dp_tiles + p.sk_wgs), kThreads, T::kLdsBytes, stream()>>>(
                in, filt, out, g, (unsigned)in_bytes, (unsigned)filt_bytes, ep, p, scratch, pool ? 1 : 0,
                out_bytes < kMaxDmaBytes ? (unsigned)out_bytes : 0u);
            SWC_LAUNCH_CHECK();
        }
    }
    if (!lean) {
        note_kernel("conv_dma<%d,%d,%d,%s>%s%s", TM, TN, STAGES, MID ? "true" : "false", p.sk_wgs ? " + conv_sk_finish" : "",
                    pool ? " (pooled)" : "");
        auto kern = conv_dma<TM, TN, STAGES, MID>;
        kern<<<(unsigned)(p.dp_tiles + p.sk_wgs), kThreads, T::kLdsBytes, stream()>>>(
            in, filt, out, g, (unsigned)in_bytes, (unsigned)filt_bytes, ep, p, scratch, pool ? 1 : 0);
        SWC_LAUNCH_CHECK();
    }
    if (p.sk_wgs) {
        conv_sk_finish<T::BM, T::BN><<<dim3((unsigned)(tiles - p.dp_tiles), T::BM / 16), 256, 0, stream()>>>(
            out, scratch, g, nk, p, ep, (g.OC % 4 == 0 && aligned16(out)) ? 1 : 0, pool ? 1 : 0);
        SWC_LAUNCH_CHECK();
    }
    return SWC_HIP_OK;
}

// ------------------------------------------------------------ conv_win: host side
constexpr size_t kWinLdsBytes = 3 * (64 + 64) * 128;

int conv_win_slots() {
    if (switches().conv_slots > 0) return switches().conv_slots;   // tests: pretend the chip holds this many workgroups
    static int per_cu = 0;
    if (!per_cu) {
        int n = 0;
        if (hipOccupancyMaxActiveBlocksPerMultiprocessor(&n, conv_win<false, false>, kThreads, kWinLdsBytes) != hipSuccess || n < 1) {
            (void)hipGetLastError();
            n = 1;
        }
        per_cu = n;
    }
    return per_cu * num_cus();
}

SkPlan conv_win_plan(const ConvGeom &g, bool allow_shared) {
    const long tiles = (long)((g.M + 63) / 64) * ((g.OC + 63) / 64);
    return sk_plan(tiles, g.K / BK, conv_win_slots(), allow_shared);
}

size_t conv_win_scratch_bytes(const ConvGeom &g) { return (size_t)2 * conv_win_plan(g, true).sk_wgs * 64 * 64 * sizeof(float); }

// Whether a layer runs on conv_win.  SWC_HIP_CONV=win forces it where it applies (test-only); any other forced variant,
// or SWC_HIP_CONV_LEAN=0, rules the kernel out.  `g.win` must have been set.
bool takes_win(const ConvGeom &g, const void *input, const void *filter) {
    const char *force = switches().conv;
    if ((force && strcmp(force, "win")) || !switches().conv_lean) return false;
    if (!g.win || g.C % BK != 0 || g.M % 4 != 0 || (g.OW >> 1) < 1) return false;
    const size_t in_bytes = (size_t)g.N * g.H * g.W * g.C * 4, filt_bytes = (size_t)g.OC * g.K * 4;
    const size_t out_bytes = (size_t)g.M * g.OC * 4, shift = ((size_t)g.pt * g.W + g.pl) * g.C * 4;
    return aligned16(input) && aligned16(filter) && in_bytes + shift < kMaxDmaBytes && filt_bytes < kMaxDmaBytes &&
           out_bytes < kMaxDmaBytes;
}

int launch_conv_win(const float *in, const float *filt, float *out, const ConvGeom &g, const Epilogue &ep, float *scratch, bool pool) {
    constexpr int BM = 64, BN = 64;
    const long tiles = (long)((g.M + BM - 1) / BM) * ((g.OC + BN - 1) / BN);
    const SkPlan p = conv_win_plan(g, scratch != nullptr);
    WinArgs a{};
    a.in = in, a.filt = filt, a.out = out, a.part = scratch, a.ep = ep, a.sk = p;
    a.in_bytes = (unsigned)((size_t)g.N * g.H * g.W * g.C * 4);
    a.filt_bytes = (unsigned)((size_t)g.OC * g.K * 4);
    a.out_bytes = (unsigned)((size_t)(pool ? g.M / 4 : g.M) * g.OC * 4);
    a.shift_bytes = (g.pt * g.W + g.pl) * g.C * 4;
    a.N = g.OC, a.K = g.K, a.C = g.C, a.H = g.H, a.W = g.W, a.kw = g.kw, a.sh = g.sh, a.sw = g.sw, a.pt = g.pt, a.pl = g.pl;
    a.OW = g.OW, a.pw = g.OW >> 1, a.ph = g.OH >> 1, a.nwin = g.M >> 2;
    a.tiles_n = (g.OC + BN - 1) / BN, a.nk = g.K / BK, a.cpt = g.C / BK;
    a.d_pw = magic_of((unsigned)a.pw), a.d_ph = magic_of((unsigned)a.ph), a.d_tn = magic_of((unsigned)a.tiles_n);
    a.last_round = switches().conv_fair && p.dp_tiles <= conv_win_slots() ? p.sk_wgs : 1 << 30;
    note_kernel("conv_win%s%s", p.sk_wgs ? " + conv_sk_finish" : "", pool ? " (pooled)" : "");
    const unsigned grid = (unsigned)(p.dp_tiles + p.sk_wgs);
    if (pool) conv_win<true, false><<<grid, kThreads, kWinLdsBytes, stream()>>>(a);
    else if (ep.residual) conv_win<false, true><<<grid, kThreads, kWinLdsBytes, stream()>>>(a);
    else conv_win<false, false><<<grid, kThreads, kWinLdsBytes, stream()>>>(a);
    SWC_LAUNCH_CHECK();
    if (p.sk_wgs) {
        conv_sk_finish<BM, BN><<<dim3((unsigned)(tiles - p.dp_tiles), BM / 16), 256, 0, stream()>>>(
            out, scratch, g, a.nk, p, ep, (g.OC % 4 == 0 && aligned16(out)) ? 1 : 0, pool ? 1 : 0);
        SWC_LAUNCH_CHECK();
    }
    return SWC_HIP_OK;
}

// ------------------------------------------------------------ small direct conv
// First layers (iC = 1 or 3, a handful of output channels) have K = kH*kW*iC of
// a few dozen: far too short for the MFMA pipeline, and iC % 4 != 0 rules out
// 128-bit gathers.  A thread computes P output pixels with all their oC
// accumulators in registers, walks the taps in the reference's (ky, kx, ci)
// order and adds fl(x*w) with separate fp32 multiply and add starting from the
// bias — the very operation sequence of conv2d_f, so this path is bit-exact.
// The filter is staged in LDS as [k][oC] and read as wavefront-uniform 128-bit
// broadcasts; each such read feeds 8*P VALU operations (with P = 1 the kernel
// needed the whole LDS bandwidth and ran at half the VALU rate).
constexpr int kDirectMaxK = 128;
constexpr int kDirectMaxOC = 32;

// POOL (OH and OW even): the pixels are numbered in 2 x 2 window order (pixel m is pixel m % 4 of window m / 4), so
// four neighbouring threads hold a window; their finished values meet in the staging block, and what is stored is
// maxpool_f's choice among them, at the window's place in the pooled tensor.
template <int OCQ, int P, bool POOL = false>   // output channels rounded up to 4*OCQ; pixels per thread
__global__ __launch_bounds__(256) void conv_direct(const float *__restrict__ in, const float *__restrict__ filt,
                                                   const float *__restrict__ bias, float *__restrict__ out,
                                                   ConvGeom g, Epilogue ep) {
#pragma clang fp contract(off)   // x*w and the add must round separately, as in the reference's -O2 x86 code
    constexpr int OCP = 4 * OCQ;
    __shared__ __align__(16) float w[kDirectMaxK * OCP];
    __shared__ float bsh[OCP], mean_sh[OCP], slope_sh[OCP], beta_sh[OCP];
    __shared__ float stage[256 * (OCP + 1)];
    const int K = g.K, OC = g.OC;
    for (int i = threadIdx.x; i < K * OCP; i += 256) {
        const int k = i / OCP, oc = i - k * OCP;
        w[i] = oc < OC ? filt[(size_t)oc * K + k] : 0.f;
    }
    const bool bn = ep.bn_mean != nullptr;
    if (threadIdx.x < OCP) {
        const int oc = threadIdx.x;
        bsh[oc] = (oc < OC && bias) ? bias[oc] : 0.f;
        if (bn && oc < OC) {
            mean_sh[oc] = ep.bn_mean[oc];
            slope_sh[oc] = (float)((double)ep.bn_scale[oc] / sqrt((double)(ep.bn_var[oc] + ep.eps)));
            beta_sh[oc] = ep.bn_bias[oc];
        }
    }
    __syncthreads();
    // pixel p of this thread: first + p*256 + threadIdx.x (consecutive lanes, consecutive pixels)
    const int first = blockIdx.x * (256 * P);
    int iy0[P], ix0[P];
    long img_base[P];
#pragma unroll
    for (int p = 0; p < P; ++p) {
        const int m = first + p * 256 + threadIdx.x;
        const int mm = m < g.M ? m : 0;
        int ox, oy, img;
        if (POOL) {   // pixel mm % 4 of window mm / 4: (2 py + d / 2, 2 px + d % 2)
            const int w = mm >> 2, d = mm & 3, pw = g.OW >> 1, ph = g.OH >> 1;
            const int px = w % pw, t = w / pw;
            ox = 2 * px + (d & 1);
            oy = 2 * (t % ph) + (d >> 1);
            img = t / ph;
        } else {
            ox = mm % g.OW;
            const int t = mm / g.OW;
            oy = t % g.OH;
            img = t / g.OH;
        }
        iy0[p] = m < g.M ? oy * g.sh - g.pt : -(1 << 20);   // pixels past M: no tap in bounds
        ix0[p] = ox * g.sw - g.pl;
        img_base[p] = (long)img * g.H;
    }
    float acc[P][OCP];
#pragma unroll
    for (int p = 0; p < P; ++p)
#pragma unroll
        for (int oc = 0; oc < OCP; ++oc) acc[p][oc] = bsh[oc];
    // For a fixed ky the taps (kx, ci) are L = kw*C consecutive floats of one input
    // row (NHWC).  They are fetched eight at a time — all loads of a group issued
    // before the first multiply.
    const int L = g.kw * g.C;
    for (int ky = 0; ky < g.kh; ++ky) {
        for (int j0 = 0; j0 < L; j0 += 8) {
            float xv[P][8];
            unsigned ok[P];
#pragma unroll
            for (int p = 0; p < P; ++p) {
                const int iy = iy0[p] + ky;
                const bool row_ok = (unsigned)iy < (unsigned)g.H;   // whole kernel row outside: skipped, as in the reference
                const float *row = in + ((img_base[p] + iy) * g.W + ix0[p]) * g.C;
                int kx = j0 / g.C, ci = j0 - kx * g.C;
                ok[p] = 0;
#pragma unroll
                for (int u = 0; u < 8; ++u) {
                    const bool tap_ok = row_ok && j0 + u < L && (unsigned)(ix0[p] + kx) < (unsigned)g.W;
                    xv[p][u] = tap_ok ? row[j0 + u] : 0.f;
                    ok[p] |= tap_ok ? 1u << u : 0u;
                    if (++ci == g.C) {
                        ci = 0;
                        ++kx;
                    }
                }
            }
            const int taps = L - j0 < 8 ? L - j0 : 8;            // uniform
            const unsigned in_group = (1u << taps) - 1u;
            bool skips = false;
#pragma unroll
            for (int p = 0; p < P; ++p) skips |= ok[p] != in_group;
            const float *wk0 = &w[(ky * L + j0) * OCP];
            if (__builtin_amdgcn_ballot_w64(skips) == 0) {       // no lane of the wavefront skips a tap
#pragma unroll
                for (int u = 0; u < 8; ++u) {
                    if (u >= taps) break;
#pragma unroll
                    for (int q = 0; q < OCQ; ++q) {
                        const float4 wv = *reinterpret_cast<const float4 *>(wk0 + u * OCP + 4 * q);
#pragma unroll
                        for (int p = 0; p < P; ++p) {
                            const float x = xv[p][u];
                            acc[p][4 * q + 0] += x * wv.x;
                            acc[p][4 * q + 1] += x * wv.y;
                            acc[p][4 * q + 2] += x * wv.z;
                            acc[p][4 * q + 3] += x * wv.w;
                        }
                    }
                }
            } else {   // padding taps are skipped, not added as zeros (a skipped tap leaves -0 and NaN cases alone)
#pragma unroll
                for (int u = 0; u < 8; ++u) {
                    if (u >= taps) break;
#pragma unroll
                    for (int q = 0; q < OCQ; ++q) {
                        const float4 wv = *reinterpret_cast<const float4 *>(wk0 + u * OCP + 4 * q);
#pragma unroll
                        for (int p = 0; p < P; ++p) {
                            const bool use = ok[p] >> u & 1;
                            const float x = xv[p][u];
                            acc[p][4 * q + 0] = use ? acc[p][4 * q + 0] + x * wv.x : acc[p][4 * q + 0];
                            acc[p][4 * q + 1] = use ? acc[p][4 * q + 1] + x * wv.y : acc[p][4 * q + 1];
                            acc[p][4 * q + 2] = use ? acc[p][4 * q + 2] + x * wv.z : acc[p][4 * q + 2];
                            acc[p][4 * q + 3] = use ? acc[p][4 * q + 3] + x * wv.w : acc[p][4 * q + 3];
                        }
                    }
                }
            }
        }
    }
    // Results go through LDS so that the global stores are contiguous across the workgroup (a thread's own oC
    // values are only 4*oC bytes apart from its neighbour's).  Rows of the staging block have an odd stride: the
    // threads of a wavefront, each writing its own row, then hit distinct banks.  On the way out a wavefront
    // moves 64/oC whole pixels per step, lane = (pixel in step, channel).
    const int stride = OC | 1;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int per_step = 64 / OC;   // OC <= kDirectMaxOC: at least two
    const int lane_px = lane / OC, lane_oc = lane - lane_px * OC;
#pragma unroll
    for (int p = 0; p < P; ++p) {
        const int base = first + p * 256;   // (past M: nothing is staged or stored; the barriers are still met)
        if (p) __syncthreads();
        if (base + (int)threadIdx.x < g.M) {
#pragma unroll
            for (int oc = 0; oc < OCP; ++oc) {
                if (oc >= OC) continue;   // (not "break": an early exit keeps the compiler from unrolling the pixel loop)
                float v = acc[p][oc];
                if (bn) v = fmaf(v - mean_sh[oc], slope_sh[oc], beta_sh[oc]);
                if (ep.relu && !ep.residual) v = (v > 0.f) ? v : 0.f;
                stage[threadIdx.x * stride + oc] = v;
            }
        }
        __syncthreads();
        const int pixels = (g.M - base < 256) ? (g.M - base) : 256;   // may be <= 0
        if (POOL) {   // (M is a multiple of 4: whole windows only)
            float *o = out + (size_t)(base >> 2) * OC;
            if (lane_px < per_step)
                for (int wl = wave * per_step + lane_px; 4 * wl < pixels; wl += 4 * per_step) {
                    const float *q = &stage[4 * wl * stride + lane_oc];
                    o[wl * OC + lane_oc] = window_max(q[0], q[stride], q[2 * stride], q[3 * stride]);
                }
            continue;
        }
        float *o = out + (size_t)base * OC;
        const float *res = ep.residual ? ep.residual + (size_t)base * OC : nullptr;
        if (lane_px < per_step)
            for (int px = wave * per_step + lane_px; px < pixels; px += 4 * per_step) {
                float v = stage[px * stride + lane_oc];
                if (res) {
                    v += res[px * OC + lane_oc];
                    if (ep.relu) v = (v > 0.f) ? v : 0.f;
                }
                o[px * OC + lane_oc] = v;
            }
    }
}

// Whether the direct kernel can take the 2 x 2 / stride 2 pooling of its layer along.
bool direct_pools(const ConvGeom &g) { return g.OH % 2 == 0 && g.OW % 2 == 0 && g.OH > 0 && g.OW > 0; }

int launch_conv_direct(const float *in, const float *filt, const float *bias, float *out, const ConvGeom &g,
                       const Epilogue &ep, bool pool = false) {
    const int ocq = (g.OC + 3) / 4;
    // four (two) pixels per thread while that leaves at least two workgroups per CU; four only while the
    // accumulators leave room for two wavefronts per SIMD
    const bool four = ocq <= 5 && (size_t)g.M >= (size_t)2048 * num_cus();
    const bool two = !four && (size_t)g.M >= (size_t)1024 * num_cus();
    const int pixels = four ? 4 : two ? 2 : 1;
    const unsigned blocks = ceil_div((size_t)g.M, (size_t)256 * pixels);
    note_kernel("conv_direct<%d,%d>%s", ocq, pixels, pool ? " (pooled)" : "");
    auto launch = [&]<int OCQ>() {
        auto with_pool = [&]<bool POOL>() {
            if constexpr (OCQ <= 5)
                if (four) return conv_direct<OCQ, 4, POOL><<<blocks, 256, 0, stream()>>>(in, filt, bias, out, g, ep);
            if (two) return conv_direct<OCQ, 2, POOL><<<blocks, 256, 0, stream()>>>(in, filt, bias, out, g, ep);
            return conv_direct<OCQ, 1, POOL><<<blocks, 256, 0, stream()>>>(in, filt, bias, out, g, ep);
        };
        if (pool) with_pool.template operator()<true>();
        else with_pool.template operator()<false>();
    };
    switch (ocq) {
    case 1: launch.template operator()<1>(); break;
    case 2: launch.template operator()<2>(); break;
    case 3: launch.template operator()<3>(); break;
    case 4: launch.template operator()<4>(); break;
    case 5: launch.template operator()<5>(); break;
    case 6: launch.template operator()<6>(); break;
    case 7: launch.template operator()<7>(); break;
    default: launch.template operator()<8>(); break;
    }
    SWC_LAUNCH_CHECK();
    return SWC_HIP_OK;
}

template <int TM, int TN>
int launch_conv(bool vec, const float *in, const float *filt, float *out, const ConvGeom &g, const Epilogue &ep) {
    using T = Tile<TM, TN, true>;
    const long tiles = (long)((g.M + T::BM - 1) / T::BM) * ((g.OC + T::BN - 1) / T::BN);
    note_kernel("conv_igemm<%d,%d,%s>", TM, TN, vec ? "true" : "false");
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

// The direct-to-LDS variants by name ("TMTN_S", m = ring hand-over in mid-slice).
enum DmaVariant { kV22_2, kV21_3, kV12_3, kV11_3, kV11_4, kV11_3m, kV21_3m, kV12_3m, kV22_3m, kVariants };
const char *const kDmaVariantName[kVariants] = {"22_2", "21_3", "12_3", "11_3", "11_4", "11_3m", "21_3m", "12_3m", "22_3m"};

// Calls f.template operator()<TM, TN, STAGES, MID>() for the variant.
template <class F> auto with_dma_variant(int v, F &&f) {
    switch (v) {
    case kV22_2: return f.template operator()<2, 2, 2, false>();
    case kV21_3: return f.template operator()<2, 1, 3, false>();
    case kV12_3: return f.template operator()<1, 2, 3, false>();
    case kV11_3: return f.template operator()<1, 1, 3, false>();
    case kV11_4: return f.template operator()<1, 1, 4, false>();
    case kV21_3m: return f.template operator()<2, 1, 3, true>();
    case kV12_3m: return f.template operator()<1, 2, 3, true>();
    case kV22_3m: return f.template operator()<2, 2, 3, true>();
    default: return f.template operator()<1, 1, 3, true>();
    }
}

// Whether the leftover tiles are cut along K (SWC_HIP_CONV_SHARE=0 turns it off; read per call).
bool share_tiles() {
    return switches().conv_share;
}

// Variant for a geometry the direct-to-LDS kernels can take; `forced` = SWC_HIP_CONV.
int pick_dma_variant(const ConvGeom &g, const char *forced, bool shared) {
    if (forced)
        for (int v = 0; v < kVariants; ++v)
            if (!strcmp(forced, kDmaVariantName[v])) return v;
    // These layers last 80-160 us: how evenly the work divides over the 256 CUs matters as much as the
    // tile's own efficiency.  With the leftover tiles cut along K, 64x64 tiles (ring hand-over in
    // mid-slice, three workgroups per CU) were the fastest or within 1 % of it for every layer shape
    // measured (56x56x64->64: 88 TFLOP/s against 84 for 128x64 tiles; 28x28x128->128: 98 against 92-95).
    if (shared) return kV11_3m;
    // All tiles whole: 64x64 tiles while there are at least eight of them per CU; below that 64x128 tiles
    // for wide layers, which halve the count but keep two workgroups per CU busy to the end.
    const size_t M = (size_t)g.M;
    const size_t tiles64 = ((M + 63) / 64) * ((g.OC + 63) / 64);
    if (tiles64 < 8 * (size_t)num_cus() && g.OC > 64 && ((M + 63) / 64) * ((g.OC + 127) / 128) >= (size_t)num_cus())
        return kV12_3;
    return kV11_3m;
}

struct ConvScratch {   // where a convolution may keep the pieces of shared tiles
    float *ptr;        // null: take the library's workspace
    size_t bytes;
};

bool conv_uses_dma(const ConvGeom &g, const void *input, const void *filter, const char *force) {
    const size_t in_bytes = (size_t)g.N * g.H * g.W * g.C * 4, filt_bytes = (size_t)g.OC * g.K * 4;
    if (!(g.C % 4 == 0 && aligned16(input) && aligned16(filter) && in_bytes < kMaxDmaBytes && filt_bytes < kMaxDmaBytes))
        return false;
    if (force && !strncmp(force, "reg", 3)) return false;
    return true;
}

// dst[m][0..OCP) = src[m][0..OC), zeros behind: rows of a channel count the 128-bit gathers can take
__global__ __launch_bounds__(256) void pad_channels(float *__restrict__ dst, const float *__restrict__ src, size_t rows,
                                                    int OC, int OCP) {
    const size_t total = rows * OCP;
    for (size_t i = (size_t)blockIdx.x * 256 + threadIdx.x; i < total; i += (size_t)gridDim.x * 256) {
        const size_t m = i / OCP;
        const int co = (int)(i - m * OCP);
        dst[i] = co < OC ? src[m * OC + co] : 0.f;
    }
}

// Grouped convolution as the reference indexes it (kernels.h:177-243: the filter keeps all iC channels per tap and
// output channel co of group g reads only channels [g*iC/group, (g+1)*iC/group) of input and filter): a copy of
// the filter with every other channel set to zero makes it an ordinary convolution over all channels, whose
// extra terms are products with zero.
__global__ __launch_bounds__(256) void mask_filter_groups(float *dst, const float *src, int OC, int taps, int C,
                                                          int group) {   // dst may be src
    const size_t total = (size_t)OC * taps * C;
    const int ocg = OC / group, cg = C / group;
    for (size_t i = (size_t)blockIdx.x * 256 + threadIdx.x; i < total; i += (size_t)gridDim.x * 256) {
        const int ci = (int)(i % C);
        const int co = (int)(i / ((size_t)taps * C));
        dst[i] = ci / cg == co / ocg ? src[i] : 0.f;
    }
}

bool window_order(const ConvGeom &g);

// Scratch bytes the forward convolution of this geometry uses (0: none).
size_t conv_scratch_bytes(const ConvGeom &g, const void *input, const void *filter) {
    const char *force = switches().conv;
    if (!share_tiles() || !conv_uses_dma(g, input, filter, force)) return 0;
    ConvGeom gw = g;
    gw.win = window_order(g) ? 1 : 0;
    if (takes_win(gw, input, filter)) return conv_win_scratch_bytes(gw);
    return with_dma_variant(pick_dma_variant(g, force, true), [&]<int TM, int TN, int STAGES, bool MID>() {
        return conv_dma_scratch_bytes<TM, TN, STAGES, MID>(g);
    });
}

size_t align256(size_t b) { return (b + 255) & ~(size_t)255; }

// An input-channel count that is no multiple of 4 keeps a layer off the 128-bit gathers of the MFMA kernels
// (the register-staged fallback reaches a tenth of their rate).  Such a layer — unless it is one for the direct
// kernel — is computed on zero-padded copies of input and filter instead: this returns the padded count, or 0.
int padded_channels(const ConvGeom &g, const char *force) {
    if (g.C % 4 == 0 || (force && !strncmp(force, "reg", 3))) return 0;
    if (g.K <= kDirectMaxK && g.OC <= kDirectMaxOC) return 0;   // the direct kernel's
    const int cp = (g.C + 3) & ~3;
    const size_t in_bytes = (size_t)g.N * g.H * g.W * cp * 4, filt_bytes = (size_t)g.OC * g.kh * g.kw * cp * 4;
    return in_bytes < kMaxDmaBytes && filt_bytes < kMaxDmaBytes ? cp : 0;
}

ConvGeom with_channels(ConvGeom g, int c) {
    g.C = c;
    g.K = g.kh * g.kw * c;
    return g;
}

// Scratch bytes a forward convolution uses in all: padded copies (if any) and the pieces of shared tiles.
size_t conv_total_scratch(const ConvGeom &g, const void *input, const void *filter) {
    const int cp = padded_channels(g, switches().conv);
    if (!cp) return conv_scratch_bytes(g, input, filter);
    return align256((size_t)g.N * g.H * g.W * cp * 4) + align256((size_t)g.OC * g.kh * g.kw * cp * 4) +
           conv_scratch_bytes(with_channels(g, cp), nullptr, nullptr);
}

// Rows of the GEMM view in 2 x 2 window order (ConvGeom::win) wherever the output has whole windows: a pooled
// convolution needs it, and the plain one takes the same order so that the two put every pixel into the same tile
// and add its products in the same sequence — the pooled result is then bit for bit the maximum of the plain one's.
// SWC_HIP_CONV_ORDER=raster (test-only) keeps raster order.
bool window_order(const ConvGeom &g) {
    return g.OH % 2 == 0 && g.OW % 2 == 0 && g.OH > 0 && g.OW > 0 && !switches().conv_raster;
}

// Whether conv_dispatch would run this layer on the direct-to-LDS tile kernels, the ones that can pool in their
// epilogue (the same tests in the same order as conv_dispatch).
bool conv_pool_fusable(ConvGeom g, const void *input, const void *filter, const void *output) {
    const char *force = switches().conv;
    if (!window_order(g)) return false;
    if (force && !strncmp(force, "reg", 3)) return false;
    bool forced_dma = false;
    if (force)
        for (int v = 0; v < kVariants; ++v) forced_dma |= !strcmp(force, kDmaVariantName[v]);
    if (!forced_dma && g.K <= kDirectMaxK && g.OC <= kDirectMaxOC && g.C % 4 != 0) return direct_pools(g);   // the direct kernel's layer
    if (const int cp = padded_channels(g, force)) {
        g = with_channels(g, cp);
        input = filter = nullptr;   // the padded copies are aligned
    }
    return conv_uses_dma(g, input, filter, force);
}

int check_conv_dims(const char *who, const size_t *odims, const size_t *idims, const size_t *fdims,
                    const size_t *kernels, const size_t *strides, const size_t *pads, size_t group,
                    bool groups_ok = false) {
    if (!odims || !idims || !fdims || !kernels || !strides || !pads)
        return fail(SWC_HIP_EINVAL, "%s: null shape array", who);
    if (group != 1 && !groups_ok) return fail(SWC_HIP_EUNSUPPORTED, "%s: group = %zu (only 1 is supported)", who, group);
    if (group == 0 || odims[3] % group || idims[3] % group)
        return fail(SWC_HIP_EINVAL, "%s: group = %zu does not divide oC = %zu and iC = %zu", who, group, odims[3], idims[3]);
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
    return SWC_HIP_OK;
}

ConvGeom make_geom(const size_t *odims, const size_t *idims, const size_t *fdims, const size_t *kernels,
                   const size_t *strides, const size_t *pads) {
    return ConvGeom{(int)idims[0],   (int)idims[1],   (int)idims[2],   (int)idims[3], (int)odims[1],
                    (int)odims[2],   (int)odims[3],   (int)kernels[0], (int)kernels[1], (int)strides[0],
                    (int)strides[1], (int)pads[0],    (int)pads[1],    (int)(odims[0] * odims[1] * odims[2]),
                    (int)(fdims[1] * fdims[2] * fdims[3])};
}

int conv_dispatch(const char *who, float *output, const float *input, const float *filter, const float *bias,
                  const size_t *odims, const size_t *idims, const size_t *fdims, const size_t *kernels,
                  const size_t *strides, const size_t *pads, size_t group, const Epilogue &ep_in,
                  bool bias_optional = false, ConvScratch scratch = {nullptr, 0}, bool pooled = false) {
    // pooled: `output` is the [N, OH/2, OW/2, OC] result of a 2 x 2 / stride 2 max-pooling of the convolution, and
    // the caller has made sure (conv_pool_fusable) that the layer runs on the direct-to-LDS tile kernels
    if (int rc = check_conv_dims(who, odims, idims, fdims, kernels, strides, pads, group, true)) return rc;
    ConvGeom g = make_geom(odims, idims, fdims, kernels, strides, pads);
    g.win = window_order(g) ? 1 : 0;
    const auto not_pooled = [&]() { return fail(SWC_HIP_EUNSUPPORTED, "%s: this kernel does not pool (internal error)", who); };
    const size_t M = (size_t)g.M;
    if (M == 0 || odims[3] == 0) return SWC_HIP_OK;
    if (!output || !input || !filter || (!bias && !bias_optional)) return fail(SWC_HIP_EINVAL, "%s: null pointer", who);
    if (group > 1) {
        // the filter with the channels of other groups zeroed, then the layer as one group
        const size_t f_b = align256((size_t)g.OC * g.K * 4);
        const size_t need = f_b + conv_total_scratch(g, input, nullptr);
        char *base = nullptr;
        if (scratch.ptr && scratch.bytes >= need) base = reinterpret_cast<char *>(scratch.ptr);
        else if (!scratch.ptr) base = static_cast<char *>(workspace(need, who));
        if (!base) return scratch.ptr ? fail(SWC_HIP_EINVAL, "%s: scratch region too small for %zu groups", who, group)
                                      : fail_code();
        float *masked = reinterpret_cast<float *>(base);
        const unsigned blocks = ceil_div((size_t)g.OC * g.K, 256);
        mask_filter_groups<<<blocks > 16384 ? 16384 : blocks, 256, 0, stream()>>>(masked, filter, g.OC, g.kh * g.kw, g.C,
                                                                                 (int)group);
        SWC_LAUNCH_CHECK();
        return conv_dispatch(who, output, input, masked, bias, odims, idims, fdims, kernels, strides, pads, 1, ep_in,
                             bias_optional, ConvScratch{reinterpret_cast<float *>(base + f_b), need - f_b}, pooled);
    }
    Epilogue ep = ep_in;
    ep.bias = bias;
    const bool vec = (g.C % 4 == 0) && aligned16(input) && aligned16(filter);
    const size_t M_in = idims[0] * idims[1] * idims[2];
    const size_t in_bytes = M_in * idims[3] * 4, filt_bytes = odims[3] * (size_t)g.K * 4;
    const char *force = switches().conv;   // forces a kernel variant (tests, tuning): reg22 reg21 reg12 reg11 | 22_2 21_3 12_3 11_3 11_4 | 11_3m 21_3m 12_3m 22_3m (m: ring hand-over in mid-slice)
    if (force && pooled && !strncmp(force, "reg", 3)) return not_pooled();
    if (force) {
        if (!strcmp(force, "reg22")) return launch_conv<2, 2>(vec, input, filter, output, g, ep);
        if (!strcmp(force, "reg21")) return launch_conv<2, 1>(vec, input, filter, output, g, ep);
        if (!strcmp(force, "reg12")) return launch_conv<1, 2>(vec, input, filter, output, g, ep);
        if (!strcmp(force, "reg11")) return launch_conv<1, 1>(vec, input, filter, output, g, ep);
    }
    bool forced_dma = false;
    if (force)
        for (int v = 0; v < kVariants; ++v) forced_dma |= !strcmp(force, kDmaVariantName[v]);
    if (!forced_dma && !(force && !strncmp(force, "reg", 3)) && g.K <= kDirectMaxK && g.OC <= kDirectMaxOC && g.C % 4 != 0)
        return pooled && !direct_pools(g) ? not_pooled() : launch_conv_direct(input, filter, bias, output, g, ep, pooled);
    if (const int cp = forced_dma || !(force && !strncmp(force, "reg", 3)) ? padded_channels(g, force) : 0) {
        // zero-padded copies of input and filter, then the same convolution with a channel count of cp
        const size_t in_b = align256(M_in * cp * 4), f_b = align256((size_t)g.OC * g.kh * g.kw * cp * 4);
        const ConvGeom gp = with_channels(g, cp);
        const size_t need = in_b + f_b + conv_scratch_bytes(gp, nullptr, nullptr);
        char *base = nullptr;
        if (scratch.ptr && scratch.bytes >= need) base = reinterpret_cast<char *>(scratch.ptr);
        else if (!scratch.ptr) base = static_cast<char *>(workspace(need, who));
        if (!base && !scratch.ptr) return fail_code();
        if (base) {
            float *in_p = reinterpret_cast<float *>(base), *f_p = reinterpret_cast<float *>(base + in_b);
            unsigned blocks = ceil_div(M_in * cp, 256);
            pad_channels<<<blocks > 16384 ? 16384 : blocks, 256, 0, stream()>>>(in_p, input, M_in, g.C, cp);
            SWC_LAUNCH_CHECK();
            blocks = ceil_div((size_t)g.OC * g.kh * g.kw * cp, 256);
            pad_channels<<<blocks > 16384 ? 16384 : blocks, 256, 0, stream()>>>(f_p, filter, (size_t)g.OC * g.kh * g.kw, g.C, cp);
            SWC_LAUNCH_CHECK();
            const size_t p_idims[4] = {idims[0], idims[1], idims[2], (size_t)cp};
            const size_t p_fdims[4] = {fdims[0], fdims[1], fdims[2], (size_t)cp};
            return conv_dispatch(who, output, in_p, f_p, bias, odims, p_idims, p_fdims, kernels, strides, pads, group, ep_in,
                                 bias_optional, ConvScratch{reinterpret_cast<float *>(base + in_b + f_b), need - in_b - f_b},
                                 pooled);
        }
    }
    if (conv_uses_dma(g, input, filter, force)) {
        // the pieces of shared tiles go into the caller's region when it gave one (and none are made if that
        // is too small), else into the library workspace
        float *pieces = nullptr;
        bool shared = share_tiles();
        if (shared) {
            const size_t need = conv_scratch_bytes(g, input, filter);
            if (!need || (scratch.ptr && scratch.bytes < need)) {
                shared = false;
            } else if (scratch.ptr) {
                pieces = scratch.ptr;
            } else {
                pieces = static_cast<float *>(workspace(need, who));
                if (!pieces) return fail_code();
            }
        }
        if (takes_win(g, input, filter)) return launch_conv_win(input, filter, output, g, ep, pieces, pooled);
        return with_dma_variant(pick_dma_variant(g, force, shared), [&]<int TM, int TN, int STAGES, bool MID>() {
            return launch_conv_dma<TM, TN, STAGES, MID>(input, filter, output, g, in_bytes, filt_bytes, ep, pieces, pooled);
        });
    }
    if (pooled) return not_pooled();
    const long tiles_m128 = (M + 127) / 128;
    if (g.OC > 64 && tiles_m128 * ((g.OC + 127) / 128) >= num_cus())
        return launch_conv<2, 2>(vec, input, filter, output, g, ep);
    if (tiles_m128 * ((g.OC + 63) / 64) >= num_cus()) return launch_conv<2, 1>(vec, input, filter, output, g, ep);
    return launch_conv<1, 1>(vec, input, filter, output, g, ep);
}

// =================================================================== gradients
// conv2dGrad_f (kernels.h:245-319), group 1.  Three independent results:
//
//   inputG  [N,H,W,iC]   = sum over (co,ky,kx) filter[co,ky,kx,ci] * outputG[n,oy,ox,co]
//       For stride 1 this is itself a convolution — of outputG with the filter
//       turned by 180 degrees and its channel axes swapped, padded by
//       (kh-1-pt, kw-1-pl) — and runs on the forward kernels above; the turned
//       filter is built in the workspace.  Other strides: a direct gather.
//   filterG [oC,kh,kw,iC] = outputG^T [oC, M] * im2col(input) [M, kh*kw*iC]
//       A GEMM whose K is the pixel count M (10^4..10^5) and whose result is
//       small: it runs on the column-interleaved kernel body (mfma_dma2.hpp)
//       with the im2col matrix gathered on the fly as the B operand, outputG
//       transposed once into the workspace so that M is the contiguous axis of
//       the A operand, and K split over blockIdx.y; the splits' partial results
//       are summed in split order by a second kernel (deterministic).
//   biasG   [oC]          = column sums of outputG over the pixels whose first
//       tap (0,0) is inside the image (the reference adds it after the bounds
//       test of that tap); two passes, partial sums in the workspace.
//
// inputG and filterG are sums of the same fp32 products as the reference's, in
// a different order.

// turned[ci][ky][kx][co] = filter[co][kh-1-ky][kw-1-kx][ci]; rows of OCP >= OC floats, the tail zero
struct TurnJob {
    const float *filt;
    float *turned;
    int OC, OCP, kh, kw, C;
};
// (block `block` of `blocks` workgroups of 256 threads)
__device__ __forceinline__ void turn_filter_part(const TurnJob &j, int block, int blocks) {
    const int total = j.OCP * j.kh * j.kw * j.C;
    for (int i = block * 256 + threadIdx.x; i < total; i += blocks * 256) {
        const int co = i % j.OCP;
        int t = i / j.OCP;
        const int kx = t % j.kw;
        t /= j.kw;
        const int ky = t % j.kh;
        const int ci = t / j.kh;
        j.turned[i] = co < j.OC ? j.filt[((co * j.kh + (j.kh - 1 - ky)) * j.kw + (j.kw - 1 - kx)) * j.C + ci] : 0.f;
    }
}
__global__ __launch_bounds__(256) void turn_filter(TurnJob j) { turn_filter_part(j, blockIdx.x, gridDim.x); }

// any stride: one thread per input element gathers the taps that reach it
__global__ __launch_bounds__(256) void dgrad_direct(float *__restrict__ ig, const float *__restrict__ og,
                                                    const float *__restrict__ filt, ConvGeom g) {
    const size_t total = (size_t)g.N * g.H * g.W * g.C;
    for (size_t i = (size_t)blockIdx.x * 256 + threadIdx.x; i < total; i += (size_t)gridDim.x * 256) {
        const int ci = (int)(i % g.C);
        size_t t = i / g.C;
        const int ix = (int)(t % g.W);
        t /= g.W;
        const int iy = (int)(t % g.H);
        const int n = (int)(t / g.H);
        float sum = 0.f;
        for (int ky = 0; ky < g.kh; ++ky) {
            const int ny = iy + g.pt - ky;
            if (ny < 0 || ny % g.sh != 0 || ny / g.sh >= g.OH) continue;
            for (int kx = 0; kx < g.kw; ++kx) {
                const int nx = ix + g.pl - kx;
                if (nx < 0 || nx % g.sw != 0 || nx / g.sw >= g.OW) continue;
                const float *o = og + (((size_t)n * g.OH + ny / g.sh) * g.OW + nx / g.sw) * g.OC;
                const float *f = filt + ((size_t)ky * g.kw + kx) * g.C + ci;
                for (int co = 0; co < g.OC; ++co) sum += f[(size_t)co * g.K] * o[co];
            }
        }
        ig[i] = sum;
    }
}

// Up to four input channels (first layers), any stride: one thread per input pixel gathers the taps that reach
// it for all its channels.  The filter sits in LDS as [ky][kx][ci][co] (rows of OCP floats, a multiple of 4), read
// as wavefront-uniform 128-bit broadcasts; outputG is read four output channels at a time where it can be.
template <int CI, bool VEC>
__global__ __launch_bounds__(256) void dgrad_few_channels(float *__restrict__ ig, const float *__restrict__ og,
                                                          const float *__restrict__ filt, ConvGeom g, int OCP) {
    extern __shared__ __align__(16) float f_s[];   // [kh][kw][CI][OCP]
    const int taps = g.kh * g.kw;
    for (int i = threadIdx.x; i < taps * CI * OCP; i += 256) {
        const int co = i % OCP;
        int t = i / OCP;
        const int ci = t % CI;
        t /= CI;   // ky*kw + kx
        f_s[i] = co < g.OC ? filt[((size_t)co * taps + t) * CI + ci] : 0.f;
    }
    __syncthreads();
    const size_t pixels = (size_t)g.N * g.H * g.W;
    for (size_t p = (size_t)blockIdx.x * 256 + threadIdx.x; p < pixels; p += (size_t)gridDim.x * 256) {
        const int ix = (int)(p % g.W);
        const size_t t = p / g.W;
        const int iy = (int)(t % g.H), n = (int)(t / g.H);
        float sum[CI];
#pragma unroll
        for (int c = 0; c < CI; ++c) sum[c] = 0.f;
        for (int ky = 0; ky < g.kh; ++ky) {
            const int ny = iy + g.pt - ky;
            if (ny < 0 || ny % g.sh != 0 || ny / g.sh >= g.OH) continue;
            for (int kx = 0; kx < g.kw; ++kx) {
                const int nx = ix + g.pl - kx;
                if (nx < 0 || nx % g.sw != 0 || nx / g.sw >= g.OW) continue;
                const float *o = og + (((size_t)n * g.OH + ny / g.sh) * g.OW + nx / g.sw) * g.OC;
                const float *f = f_s + (ky * g.kw + kx) * CI * OCP;
                if (VEC) {   // OC % 4 == 0, outputG 16-byte aligned
                    for (int co = 0; co < g.OC; co += 4) {
                        const float4 ov = *reinterpret_cast<const float4 *>(o + co);
#pragma unroll
                        for (int c = 0; c < CI; ++c) {
                            const float4 fv = *reinterpret_cast<const float4 *>(f + c * OCP + co);
                            sum[c] += fv.x * ov.x;
                            sum[c] += fv.y * ov.y;
                            sum[c] += fv.z * ov.z;
                            sum[c] += fv.w * ov.w;
                        }
                    }
                } else {
                    for (int co = 0; co < g.OC; ++co) {
                        const float ov = o[co];
#pragma unroll
                        for (int c = 0; c < CI; ++c) sum[c] += f[c * OCP + co] * ov;
                    }
                }
            }
        }
#pragma unroll
        for (int c = 0; c < CI; ++c) ig[p * CI + c] = sum[c];
    }
}

// ---- filter gradient: B operand = im2col(input), gathered
// (Tried and dropped: the pixel arithmetic on the scalar unit — a load instruction covers one or two pixels of the
// [32 pixels][BN columns] tile, so coordinates, bounds tests and the pixel's offset are wavefront-uniform, and per lane
// a load needs an add and a select instead of some twenty vector instructions.  Bit-identical, but the scalar chains
// (a wavefront issues in order: its MFMAs wait behind them) and the spilled scalar registers cost more than the
// vector instructions saved: 215.6 / 339.6 / 182.0 us against 174.6 / 299.8 / 166.2 us for conv2dGrad_f on the three
// layer shapes of the ResNet-like block, alternating runs on one box.)
struct Im2colB {
    const float *in;
    unsigned bytes;
    int H, W, nimg, kw, C, OH, OW, sh, sw, pt, pl;
    // A lane follows its pixel from slice to slice (+32 pixels) by additions and selects only: multiplications, and
    // divergent branches between the MFMAs of a slice, cost the matrix pipe more than the loads they feed.
    int ys_end, xs_end;          // OH * sh, OW * sw: where the scaled row / column wraps
    int dxs, dys, doff;          // a slice's step: columns (x sw), rows (x sh), bytes (whole images included) — before carries
    int row_carry, img_carry;    // bytes added when the column wraps into the next row / the row into the next image
    struct Lane {
        int ys, xs, off;         // oy * sh, ox * sw, byte offset of the input pixel (image, ys, xs)
        int ty, tx, tap, krow;   // tap row - pt, tap column - pl, byte offset of the tap and channel (+ descriptor shift), row in the slice
        bool ok;
    };
    static Im2colB of(const float *in, size_t in_bytes, const ConvGeom &g) {
        Im2colB b{};
        b.in = in, b.bytes = (unsigned)in_bytes;
        b.H = g.H, b.W = g.W, b.nimg = g.N, b.kw = g.kw, b.C = g.C, b.OH = g.OH, b.OW = g.OW;
        b.sh = g.sh, b.sw = g.sw, b.pt = g.pt, b.pl = g.pl;
        b.ys_end = g.OH * g.sh, b.xs_end = g.OW * g.sw;
        const int per_img = g.OH * g.OW, qi = BK / per_img, qy = BK % per_img / g.OW, rx = BK % per_img % g.OW;
        const int px = g.C * 4;   // bytes per input pixel
        b.dxs = rx * g.sw, b.dys = qy * g.sh;
        b.doff = ((qi * g.H + qy * g.sh) * g.W + rx * g.sw) * px;
        b.row_carry = (g.sh * g.W - g.OW * g.sw) * px;
        b.img_carry = (g.H - g.OH * g.sh) * g.W * px;
        return b;
    }
#if __HIP_DEVICE_COMPILE__
    __device__ __forceinline__ __amdgpu_buffer_rsrc_t rsrc() const {
        return make_rsrc(reinterpret_cast<const char *>(in) - kImmSpan, bytes + kImmSpan);
    }
    // row krow of a slice is output pixel k_begin + krow (+32 per slice); column col is (ky, kx, ci)
    __device__ __forceinline__ Lane init(int krow, int col, bool col_ok, int imm, int k_begin) const {
        Lane s;
        const int pix = k_begin + krow;
        const int ox = pix % OW, t = pix / OW, oy = t % OH, img = t / OH;
        s.ys = oy * sh;
        s.xs = ox * sw;
        s.off = ((img * H + s.ys) * W + s.xs) * C * 4;
        const int tap = col / C, ky = tap / kw;
        s.ty = ky - pt;
        s.tx = tap - ky * kw - pl;
        s.tap = ((s.ty * W + s.tx) * C + (col - tap * C)) * 4 + kImmSpan - imm;
        s.krow = krow;
        s.ok = col_ok;
        return s;
    }
    __device__ __forceinline__ int voffset(const Lane &s, int k0, int k_end) const {
        const int iy = s.ys + s.ty, ix = s.xs + s.tx;
        // (k_end is at most the pixel count, so a row of the slice below k_end lies in one of the images)
        const bool valid = s.ok & (s.krow < k_end - k0) & ((unsigned)iy < (unsigned)H) & ((unsigned)ix < (unsigned)W);   // (k_end - k0: scalar)
        const int off = s.off + s.tap;
        return valid ? off : kOutOfRange;
    }
    __device__ __forceinline__ int soffset(int) const { return 0; }
    __device__ __forceinline__ void advance(Lane &s) const {
        s.xs += dxs;
        s.off += doff;
        const bool cx = s.xs >= xs_end;
        s.xs -= cx ? xs_end : 0;
        s.off += cx ? row_carry : 0;
        s.ys += dys + (cx ? sh : 0);
        const bool cy = s.ys >= ys_end;
        s.ys -= cy ? ys_end : 0;
        s.off += cy ? img_carry : 0;
    }
#endif
};

template <int TM, int TN, int WM, int STAGES, bool MID, int NW, class BSrc>
__global__ __launch_bounds__(64 * NW) void conv_wgrad(const float *__restrict__ ogT, unsigned a_bytes, int lda,
                                                       BSrc bsrc, float *__restrict__ part, size_t split_stride,
                                                       int OC, int Kf, int M, int slices_per_split) {
#if __HIP_DEVICE_COMPILE__
    const int k_begin = blockIdx.y * slices_per_split * BK;
    const int k_stop = k_begin + slices_per_split * BK;
    const Epilogue ep{nullptr, nullptr, nullptr, nullptr, nullptr, 0.f, 0};
    dma2_tile_body<TM, TN, WM, STAGES, MID, NW, BSrc, true>(ogT, a_bytes, lda, bsrc, part + blockIdx.y * split_stride, (size_t)Kf,
                                                            OC, Kf, k_begin, k_stop < M ? k_stop : M, ep);
#endif
}

template <int TM, int TN, int WM, int STAGES, bool MID, int NW, class BSrc>
int launch_wgrad_as(const float *ogT, size_t a_bytes, int lda, const BSrc &bsrc, float *part, int OC, int Kf, int M, int splits,
                    int sps) {
    using T = Dma2Tile<TM, TN, WM, STAGES, NW>;
    auto kern = conv_wgrad<TM, TN, WM, STAGES, MID, NW, BSrc>;
    static bool attr_set = false;
    if (!attr_set) {
        SWC_HIP_TRY(hipFuncSetAttribute(reinterpret_cast<const void *>(kern),
                                        hipFuncAttributeMaxDynamicSharedMemorySize, (int)T::kLdsBytes));
        attr_set = true;
    }
    const unsigned tiles = (unsigned)(((OC + T::BM - 1) / T::BM) * ((Kf + T::BN - 1) / T::BN));
    kern<<<dim3(tiles, splits), T::kThreadsWg, T::kLdsBytes, stream()>>>(ogT, (unsigned)a_bytes, lda, bsrc, part,
                                                                         (size_t)OC * Kf, OC, Kf, M, sps);
    SWC_LAUNCH_CHECK();
    return SWC_HIP_OK;
}

template <int TM, int TN, int WM, int STAGES, bool MID, int NW>
int launch_wgrad(const float *ogT, size_t a_bytes, int lda, const Im2colB &b, float *part, int OC, int Kf, int M, int splits, int sps) {
    note_kernel("conv_wgrad<%d,%d,%d,%d,%s,%d>", TM, TN, WM, STAGES, MID ? "true" : "false", NW);
    return launch_wgrad_as<TM, TN, WM, STAGES, MID, NW>(ogT, a_bytes, lda, b, part, OC, Kf, M, splits, sps);
}

// out[i] = sum over splits of part[split][i], in a fixed order: PH threads share an element, thread p adds
// splits p, p+PH, p+2PH, ... four loads at a time (PH independent chains instead of one long one), then the PH
// partial sums are added in order.  PH = 8 for a few splits of many elements, 32 for hundreds of splits.
struct SumJob {
    float *out;
    const float *part;
    size_t n;
    int splits;
};
template <int PH>
__device__ __forceinline__ void sum_splits_part(const SumJob &j, unsigned block, unsigned blocks) {
    __shared__ float red[PH][33];
    const int e = threadIdx.x & 31, p = threadIdx.x >> 5;
    const float *__restrict__ part = j.part;
    const size_t n = j.n;
    const int splits = j.splits;
    for (size_t base = (size_t)block * 32; base < n; base += (size_t)blocks * 32) {
        const size_t i = base + e;
        float s = 0.f;
        if (i < n) {
            int k = p;
            for (; k + 3 * PH < splits; k += 4 * PH) {
                const float v0 = part[(size_t)k * n + i], v1 = part[(size_t)(k + PH) * n + i];
                const float v2 = part[(size_t)(k + 2 * PH) * n + i], v3 = part[(size_t)(k + 3 * PH) * n + i];
                s += v0, s += v1, s += v2, s += v3;
            }
            for (; k < splits; k += PH) s += part[(size_t)k * n + i];
        }
        red[p][e] = s;
        __syncthreads();
        if (p == 0 && i < n) {
            float t = red[0][e];
#pragma unroll
            for (int q = 1; q < PH; ++q) t += red[q][e];
            j.out[i] = t;
        }
        __syncthreads();
    }
}
// The first blocks_a workgroups sum job a, the others (if any) job b: two reductions of one call in one launch.
template <int PH>
__global__ __launch_bounds__(32 * PH) void sum_splits(SumJob a, SumJob b, unsigned blocks_a) {
    if (blockIdx.x < blocks_a) sum_splits_part<PH>(a, blockIdx.x, blocks_a);
    else sum_splits_part<PH>(b, blockIdx.x - blocks_a, gridDim.x - blocks_a);
}

// launches sum_splits with the number of chains that suits the number of splits; `also`: a second reduction for
// the same launch
int launch_sum_splits(float *out, const float *part, size_t n, int splits, const SumJob *also = nullptr) {
    unsigned blocks = ceil_div(n, 32);
    blocks = blocks > 16384 ? 16384 : blocks;
    unsigned more = also ? ceil_div(also->n, 32) : 0;
    more = more > 16384 ? 16384 : more;
    const SumJob a{out, part, n, splits}, b = also ? *also : SumJob{nullptr, nullptr, 0, 0};
    if (splits >= 128 || b.splits >= 128) sum_splits<32><<<blocks + more, 1024, 0, stream()>>>(a, b, blocks);
    else sum_splits<8><<<blocks + more, 256, 0, stream()>>>(a, b, blocks);
    SWC_LAUNCH_CHECK();
    return SWC_HIP_OK;
}

// any shape: one workgroup per filter element, pixels strided over its threads
__global__ __launch_bounds__(256) void wgrad_direct(float *__restrict__ fg, const float *__restrict__ og,
                                                    const float *__restrict__ in, ConvGeom g) {
    __shared__ float red[256];
    const int e = blockIdx.x;   // (co, ky, kx, ci)
    const int ci = e % g.C;
    int t = e / g.C;
    const int kx = t % g.kw;
    t /= g.kw;
    const int ky = t % g.kh;
    const int co = t / g.kh;
    float sum = 0.f;
    for (int m = threadIdx.x; m < g.M; m += 256) {
        const int ox = m % g.OW;
        const int t2 = m / g.OW;
        const int oy = t2 % g.OH;
        const int n = t2 / g.OH;
        const int iy = oy * g.sh - g.pt + ky, ix = ox * g.sw - g.pl + kx;
        if ((unsigned)iy < (unsigned)g.H && (unsigned)ix < (unsigned)g.W)
            sum += in[(((size_t)n * g.H + iy) * g.W + ix) * g.C + ci] * og[(size_t)m * g.OC + co];
    }
    red[threadIdx.x] = sum;
    __syncthreads();
    for (int s = 128; s > 0; s >>= 1) {
        if ((int)threadIdx.x < s) red[threadIdx.x] += red[threadIdx.x + s];
        __syncthreads();
    }
    if (threadIdx.x == 0) fg[e] = red[0];
}

// Small filters that the MFMA path cannot take (first layers: iC = 1 or 3): one thread per filter element
// (co, ky, kx, ci), a workgroup per block of `rows` output rows of one image.  The block's outputG rows and
// the input rows under them are staged in LDS, where the many threads that need the same value read it as a
// broadcast; partial sums per block go to `part`, sum_splits adds them.  blockIdx.x = image, blockIdx.y = row block.
__global__ __launch_bounds__(1024) void wgrad_small(float *__restrict__ part, const float *__restrict__ og,
                                                    const float *__restrict__ in, ConvGeom g, int rows) {
    extern __shared__ float wg_lds[];
    const int n = blockIdx.x, oy0 = blockIdx.y * rows;
    const int oy1 = oy0 + rows < g.OH ? oy0 + rows : g.OH;
    const int iy_first = oy0 * g.sh - g.pt;                           // input row under tap row 0 of the first output row
    const int in_rows = (oy1 - 1 - oy0) * g.sh + g.kh;
    float *og_s = wg_lds;                                             // [oy1-oy0][OW][OC]
    float *in_s = wg_lds + (size_t)rows * g.OW * g.OC;                // [in_rows][W][C], rows outside the image zero
    const int og_count = (oy1 - oy0) * g.OW * g.OC, row_len = g.W * g.C;
    const float *og_src = og + ((size_t)n * g.OH + oy0) * g.OW * g.OC;
    for (int i = threadIdx.x; i < og_count; i += blockDim.x) og_s[i] = og_src[i];
    for (int i = threadIdx.x; i < in_rows * row_len; i += blockDim.x) {
        const int r = i / row_len, iy = iy_first + r;
        in_s[i] = (unsigned)iy < (unsigned)g.H ? in[((size_t)n * g.H + iy) * row_len + (i - r * row_len)] : 0.f;
    }
    __syncthreads();
    const int e = threadIdx.x;
    const int elems = g.OC * g.K;
    if (e >= elems) return;
    const int ci = e % g.C;
    int t = e / g.C;
    const int kx = t % g.kw;
    t /= g.kw;
    const int ky = t % g.kh;
    const int co = t / g.kh;
    // output columns whose tap kx lies inside the image
    int ox_lo = 0, ox_hi = g.OW;
    while (ox_lo < ox_hi && ox_lo * g.sw - g.pl + kx < 0) ++ox_lo;
    while (ox_hi > ox_lo && (ox_hi - 1) * g.sw - g.pl + kx >= g.W) --ox_hi;
    float acc[2] = {0.f, 0.f};
    for (int oy = oy0; oy < oy1; ++oy) {
        const float *o = og_s + ((oy - oy0) * g.OW) * g.OC + co;
        const float *x = in_s + ((oy - oy0) * g.sh + ky) * row_len + (kx - g.pl) * g.C + ci;   // rows outside hold zeros
        int ox = ox_lo;
        for (; ox + 1 < ox_hi; ox += 2) {
            acc[0] += x[ox * g.sw * g.C] * o[ox * g.OC];
            acc[1] += x[(ox + 1) * g.sw * g.C] * o[(ox + 1) * g.OC];
        }
        if (ox < ox_hi) acc[0] += x[ox * g.sw * g.C] * o[ox * g.OC];
    }
    part[((size_t)n * gridDim.y + blockIdx.y) * elems + e] = acc[0] + acc[1];
}

// ---- bias gradient: masked column sums of outputG [M, OC]
constexpr int kBiasRows = 128;   // rows per partial sum: 128 measured best on the cfg4 layers (256: 183 / 307 / 169 us for conv2dGrad, 128: 181 / 304 / 163, 64: 184 / 304 / 160)
// A workgroup sums kBiasRows rows: thread = (VEC columns, row phase), the pixel coordinates of its rows kept
// incrementally (no division in the loop); the 256/colsq phases of a column are combined in a fixed order.
// colsq * VEC columns per workgroup in x (colsq a power of two), row chunks in y.
template <int VEC>
__global__ __launch_bounds__(256) void bias_partials(float *__restrict__ part, const float *__restrict__ og, ConvGeom g,
                                                     int colsq, int phases) {
    __shared__ float red[256 * VEC];
    const int c_local = threadIdx.x % colsq, phase = threadIdx.x / colsq;
    const int co = (blockIdx.x * colsq + c_local) * VEC;
    const int m0 = blockIdx.y * kBiasRows;
    const int m1 = m0 + kBiasRows < g.M ? m0 + kBiasRows : g.M;
    float acc[VEC];
#pragma unroll
    for (int v = 0; v < VEC; ++v) acc[v] = 0.f;
    if (co < g.OC && phase < phases) {
        int m = m0 + phase;
        int ox = m % g.OW, oy = (m / g.OW) % g.OH;
        const int step_y = phases / g.OW, step_x = phases - step_y * g.OW;   // phases rows further on
#pragma unroll 4
        for (; m < m1; m += phases) {
            // the reference adds outputG at tap (0,0) after that tap's bounds test: pixels whose first tap lies
            // in the padding do not contribute
            const bool counts = (unsigned)(oy * g.sh - g.pt) < (unsigned)g.H && (unsigned)(ox * g.sw - g.pl) < (unsigned)g.W;
            const float *p = og + (size_t)m * g.OC + co;
            if (VEC == 4) {
                const float4 q = *reinterpret_cast<const float4 *>(p);
                if (counts) acc[0] += q.x, acc[VEC > 1 ? 1 : 0] += q.y, acc[VEC > 2 ? 2 : 0] += q.z, acc[VEC > 3 ? 3 : 0] += q.w;
            } else {
                const float q = *p;
                if (counts) acc[0] += q;
            }
            ox += step_x;
            oy += step_y;
            if (ox >= g.OW) ox -= g.OW, ++oy;
            while (oy >= g.OH) oy -= g.OH;
        }
    }
#pragma unroll
    for (int v = 0; v < VEC; ++v) red[threadIdx.x * VEC + v] = acc[v];
    __syncthreads();
    if (phase == 0 && co < g.OC) {
#pragma unroll
        for (int v = 0; v < VEC; ++v) {
            float t = red[c_local * VEC + v];
            for (int q = 1; q < phases; ++q) t += red[(q * colsq + c_local) * VEC + v];
            if (co + v < g.OC) part[(size_t)blockIdx.y * g.OC + co + v] = t;
        }
    }
}

// outputG [M, OC] -> its transpose ogT [OC, lda] (what the filter gradient's GEMM reads), and in the same pass over
// outputG the bias gradient's masked column sums of chunks of kBiasRows rows (see bias_partials for the mask): one read
// of outputG instead of two.  A workgroup moves kBiasRows / 32 tiles of 32 rows x 32 columns through a 32 x 33 LDS tile
// (matrix_trans's); thread (tx, ty) sees rows ty, ty + 8, ... of column tx and keeps its pixel coordinates
// incrementally; the eight partial sums of a column are added in order.  grid: (chunks, OC / 32 rounded up).
// Workgroups with blockIdx.x >= chunks (if any) turn the filter for the input gradient's convolution instead: one
// launch of a few microseconds less in a call whose small kernels add up to a sixth of its time.
__global__ __launch_bounds__(256) void trans_bias_partials(float *__restrict__ ogT, size_t lda, float *__restrict__ part,
                                                           const float *__restrict__ og, ConvGeom g, int chunks, TurnJob turn) {
    if ((int)blockIdx.x >= chunks) {
        turn_filter_part(turn, ((int)blockIdx.x - chunks) * gridDim.y + blockIdx.y, ((int)gridDim.x - chunks) * gridDim.y);
        return;
    }
    __shared__ float tile[32][33];
    __shared__ float red[8][33];
    const int tx = threadIdx.x & 31, ty = threadIdx.x >> 5;   // 32 x 8
    const int c0 = blockIdx.y * 32, m0 = blockIdx.x * kBiasRows;
    int m = m0 + ty;
    int ox = m % g.OW, oy = (m / g.OW) % g.OH;
    const int step_y = 8 / g.OW, step_x = 8 - step_y * g.OW;   // eight rows further on
    float acc = 0.f;
    for (int r0 = m0; r0 < m0 + kBiasRows && r0 < g.M; r0 += 32) {
#pragma unroll
        for (int k = 0; k < 4; ++k) {
            const int r = r0 + ty + 8 * k, c = c0 + tx;
            if (r < g.M && c < g.OC) {
                const float v = og[(size_t)r * g.OC + c];
                tile[ty + 8 * k][tx] = v;
                const bool counts = (unsigned)(oy * g.sh - g.pt) < (unsigned)g.H && (unsigned)(ox * g.sw - g.pl) < (unsigned)g.W;
                if (counts) acc += v;
            }
            ox += step_x;
            oy += step_y;
            if (ox >= g.OW) ox -= g.OW, ++oy;
            while (oy >= g.OH) oy -= g.OH;
        }
        __syncthreads();
#pragma unroll
        for (int k = 0; k < 4; ++k) {
            const int c = c0 + ty + 8 * k, r = r0 + tx;   // output row c, column r
            if (c < g.OC && r < g.M) ogT[(size_t)c * lda + r] = tile[tx][ty + 8 * k];
        }
        __syncthreads();
    }
    red[ty][tx] = acc;
    __syncthreads();
    if (ty == 0 && c0 + tx < g.OC) {
        float t = red[0][tx];
        for (int q = 1; q < 8; ++q) t += red[q][tx];
        part[(size_t)blockIdx.x * g.OC + c0 + tx] = t;
    }
}

size_t wgrad_small_lds(const ConvGeom &g, int rows) {
    return ((size_t)rows * g.OW * g.OC + ((size_t)(rows - 1) * g.sh + g.kh) * g.W * g.C) * sizeof(float);
}

// Where conv_grad keeps its intermediate results in the workspace, and the kernel choices that decide their
// sizes; a pure function of the shapes, the device and the operands' alignment, shared by the call and by
// swc_hip_conv2dGrad_workspace_bytes.
struct GradLayout {
    bool dgrad_conv, wgrad_mfma, narrow, narrow128;
    int lda, bias_chunks, splits, sps, wgrad_rows;
    size_t ocp, turned_b, ogp_b, dgrad_b, ogt_b, part_b, bias_b;
    size_t t_odims[4], t_idims[4], t_fdims[4], t_strides[2], t_pads[4];
    size_t total() const { return turned_b + ogt_b + part_b + bias_b + dgrad_b + ogp_b; }
};

GradLayout grad_layout(const ConvGeom &g, const size_t *odims, const size_t *idims, const size_t *fdims,
                       const size_t *kernels, bool input_aligned, bool og_aligned, bool fg_aligned) {
    GradLayout L{};
    const size_t M = (size_t)g.M, Kf = (size_t)g.K;
    const size_t in_elems = idims[0] * idims[1] * idims[2] * idims[3], f_elems = fdims[0] * Kf;
    // (an input of very few channels leaves the GEMM form with a handful of columns: the gather is faster there)
    L.dgrad_conv = g.sh == 1 && g.sw == 1 && g.pt <= g.kh - 1 && g.pl <= g.kw - 1 && g.C >= 8;
    // (the column-interleaved kernel body starts its descriptors 4 KiB early: operands stay below 2 GiB - 64 KiB)
    L.wgrad_mfma = g.C % 4 == 0 && input_aligned && og_aligned && fg_aligned && in_elems * 4 < 0x7fff0000u &&
                   (M + 4) * odims[3] * 4 < 0x7fff0000u;
    L.lda = (int)((M + 3) & ~(size_t)3);   // row length of the transposed outputG
    L.bias_chunks = (int)((M + kBiasRows - 1) / kBiasRows);
    // filter-gradient tiles and splits: about two workgroups per CU (what fits at once)
    // (up to 64 output channels: tiles of 64 rows, 256 columns wide — or 128 where that covers the kh*kw*iC columns
    // with over a tenth fewer: 576 columns are 768 on three wide tiles, 640 on five narrow ones)
    L.narrow = g.OC <= 64;
    L.narrow128 = L.narrow && ((Kf + 127) / 128 * 128) * 11 < ((Kf + 255) / 256 * 256) * 10;
    if (switches().wgrad_bn)   // test-only: 128 or 256 forces the width for narrow layers
        L.narrow128 = L.narrow && switches().wgrad_bn == 128;
    const int bm = L.narrow ? 64 : 128, bn = L.narrow && !L.narrow128 ? 256 : 128;
    const int tiles = ((g.OC + bm - 1) / bm) * (int)((Kf + bn - 1) / bn);
    const int nk = (int)((M + BK - 1) / BK);
    int splits = (2 * num_cus() + tiles - 1) / tiles;
    splits = splits < 1 ? 1 : (splits > nk ? nk : splits);
    L.sps = (nk + splits - 1) / splits;
    L.splits = (nk + L.sps - 1) / L.sps;
    // the input gradient as a convolution of outputG with the turned filter
    // (its channel count is OC: padded to a multiple of 4 with zeros where needed, so that the 128-bit gathers
    // of the MFMA kernels apply — 50 channels: 230 us on the scalar path, 30 with two small copies)
    L.ocp = (odims[3] + 3) & ~(size_t)3;
    const size_t t_odims[4] = {idims[0], idims[1], idims[2], idims[3]};
    const size_t t_idims[4] = {odims[0], odims[1], odims[2], L.ocp};
    const size_t t_fdims[4] = {idims[3], kernels[0], kernels[1], L.ocp};
    const size_t t_pads[4] = {(size_t)(g.kh - 1 - g.pt), (size_t)(g.kw - 1 - g.pl), 0, 0};
    for (int i = 0; i < 4; ++i) L.t_odims[i] = t_odims[i], L.t_idims[i] = t_idims[i], L.t_fdims[i] = t_fdims[i], L.t_pads[i] = t_pads[i];
    L.t_strides[0] = L.t_strides[1] = 1;
    L.turned_b = L.dgrad_conv ? align256(idims[3] * fdims[1] * fdims[2] * L.ocp * 4) : 0;
    L.ogp_b = L.dgrad_conv && L.ocp != odims[3] ? align256(M * L.ocp * 4) : 0;   // outputG with padded channels
    // (the turned filter lies at the start of the workspace, which is 256-byte aligned like outputG must be)
    L.dgrad_b = L.dgrad_conv ? align256(conv_scratch_bytes(make_geom(t_odims, t_idims, t_fdims, kernels, L.t_strides, t_pads),
                                                           og_aligned ? nullptr : reinterpret_cast<const void *>(4), nullptr))
                             : 0;
    L.ogt_b = L.wgrad_mfma ? align256((size_t)g.OC * L.lda * 4) : 0;
    // small filters off the MFMA path: row blocks of about three workgroups per CU, as LDS allows
    if (!L.wgrad_mfma && f_elems <= 1024 && g.OH > 0 && g.N <= 65535) {
        int rows = (int)((size_t)g.N * g.OH / (3 * (size_t)num_cus()));
        rows = rows < 1 ? 1 : (rows > g.OH ? g.OH : rows);
        while (rows > 1 && wgrad_small_lds(g, rows) > 64 * 1024) --rows;
        if (wgrad_small_lds(g, rows) <= 64 * 1024 && (g.OH + rows - 1) / rows <= 65535) L.wgrad_rows = rows;
    }
    const size_t wgrad_blocks = L.wgrad_rows ? (size_t)g.N * ((g.OH + L.wgrad_rows - 1) / L.wgrad_rows) : 0;
    L.part_b = L.wgrad_mfma && L.splits > 1 ? align256((size_t)L.splits * f_elems * 4) : align256(wgrad_blocks * f_elems * 4);
    L.bias_b = align256((size_t)L.bias_chunks * g.OC * 4);
    return L;
}

int conv_grad(float *inputG, float *filterG, float *biasG, const float *outputG, const float *input,
              const float *filter, const size_t *odims, const size_t *idims, const size_t *fdims,
              const size_t *kernels, const size_t *strides, const size_t *pads, size_t group) {
    const char *who = "swc_hip_conv2dGrad_f";
    if (!odims || !idims || !fdims || !kernels || !strides || !pads) return fail(SWC_HIP_EINVAL, "%s: null shape array", who);
    if (group == 0 || odims[3] % group || idims[3] % group)
        return fail(SWC_HIP_EINVAL, "%s: group = %zu does not divide oC = %zu and iC = %zu", who, group, odims[3], idims[3]);
    for (int i = 0; i < 4; ++i)
        if (odims[i] > 0x7fffffffu || idims[i] > 0x7fffffffu || fdims[i] > 0x7fffffffu)
            return fail(SWC_HIP_EINVAL, "%s: dimension too large", who);
    if (odims[0] != idims[0] || fdims[0] != odims[3] || fdims[3] != idims[3] || fdims[1] != kernels[0] ||
        fdims[2] != kernels[1])
        return fail(SWC_HIP_EINVAL, "%s: output, input and filter dims do not fit together", who);
    if (strides[0] == 0 || strides[1] == 0 || strides[0] > 4096 || strides[1] > 4096 || pads[0] > 4096 ||
        pads[1] > 4096 || kernels[0] == 0 || kernels[1] == 0)
        return fail(SWC_HIP_EINVAL, "%s: bad kernel/stride/pad", who);
    const size_t M = odims[0] * odims[1] * odims[2];
    const size_t Kf = fdims[1] * fdims[2] * fdims[3];
    const size_t in_elems = idims[0] * idims[1] * idims[2] * idims[3], f_elems = fdims[0] * Kf;
    if (M > 0x7fffffffu || Kf > 0x7fffffffu || in_elems * 4 >= kMaxDmaBytes || M * odims[3] * 4 >= kMaxDmaBytes ||
        f_elems * 4 >= kMaxDmaBytes)
        return fail(SWC_HIP_EUNSUPPORTED, "%s: tensors of 2 GiB and more are not supported", who);
    if (!inputG || !filterG || !biasG || !outputG || !input || !filter) return fail(SWC_HIP_EINVAL, "%s: null pointer", who);
    ConvGeom g{(int)idims[0], (int)idims[1], (int)idims[2], (int)idims[3], (int)odims[1], (int)odims[2],
               (int)odims[3], (int)kernels[0], (int)kernels[1], (int)strides[0], (int)strides[1], (int)pads[0],
               (int)pads[1], (int)M, (int)Kf};
    if (in_elems == 0 && f_elems == 0 && g.OC == 0) return SWC_HIP_OK;
    if (M == 0 || g.OC == 0 || in_elems == 0 || f_elems == 0) {   // no products: the gradients are zero
        int rc = SWC_HIP_OK;   // fill kernels, not memset nodes: this may be recorded into a graph
        if (in_elems) rc = swc_hip_fill_f(inputG, 0.f, in_elems);
        if (rc == SWC_HIP_OK && f_elems) rc = swc_hip_fill_f(filterG, 0.f, f_elems);
        if (rc == SWC_HIP_OK && g.OC) rc = swc_hip_fill_f(biasG, 0.f, (size_t)g.OC);
        return rc;
    }

    const GradLayout L = grad_layout(g, odims, idims, fdims, kernels, aligned16(input), aligned16(outputG), aligned16(filterG));
    const bool dgrad_conv = L.dgrad_conv, wgrad_mfma = L.wgrad_mfma, narrow = L.narrow, narrow128 = L.narrow128;
    const int lda = L.lda, bias_chunks = L.bias_chunks, splits = L.splits, sps = L.sps, wgrad_rows = L.wgrad_rows;
    const size_t ocp = L.ocp, turned_b = L.turned_b, ogp_b = L.ogp_b, dgrad_b = L.dgrad_b, ogt_b = L.ogt_b,
                 part_b = L.part_b, bias_b = L.bias_b;
    const size_t *t_odims = L.t_odims, *t_idims = L.t_idims, *t_fdims = L.t_fdims, *t_strides = L.t_strides,
                 *t_pads = L.t_pads;
    // More than one group, as the reference indexes it (kernels.h:245-319: output channel co of group gr pairs
    // with channels [gr*iC/group, (gr+1)*iC/group) only): the gradients of the one-group layer whose filter has the
    // other channels zeroed — inputG then holds exactly the group's terms (plus products with zero), biasG does not
    // depend on groups, and filterG is right inside the groups and gets its cross-group elements zeroed at the end,
    // which is what the reference's zero fill leaves there.
    const size_t mask_b = group > 1 ? align256(f_elems * 4) : 0;
    char *ws0 = static_cast<char *>(workspace(mask_b + L.total(), who));
    if (!ws0) return fail_code();
    char *ws = ws0 + mask_b;
    const unsigned mask_blocks = ceil_div(f_elems, 256) > 16384 ? 16384 : ceil_div(f_elems, 256);
    if (group > 1) {
        float *masked = reinterpret_cast<float *>(ws0);
        mask_filter_groups<<<mask_blocks, 256, 0, stream()>>>(masked, filter, g.OC, g.kh * g.kw, g.C, (int)group);
        SWC_LAUNCH_CHECK();
        filter = masked;
    }
    float *turned = reinterpret_cast<float *>(ws);
    float *ogT = reinterpret_cast<float *>(ws + turned_b);
    float *part = reinterpret_cast<float *>(ws + turned_b + ogt_b);
    float *bias_part = reinterpret_cast<float *>(ws + turned_b + ogt_b + part_b);
    float *dgrad_pieces = reinterpret_cast<float *>(ws + turned_b + ogt_b + part_b + bias_b);
    float *og_padded = reinterpret_cast<float *>(ws + turned_b + ogt_b + part_b + bias_b + dgrad_b);

    // ---- bias gradient (with the filter gradient's transposed outputG in the same pass where that is needed)
    if (wgrad_mfma) {
        // the 128-bit loads of the last k chunk reach into the row padding: it must hold zeros, not stale bits
        if ((size_t)lda != M) {
            const int rc0 = swc_hip_fill_f(ogT, 0.f, (size_t)g.OC * lda);
            if (rc0 != SWC_HIP_OK) return rc0;
        }
        // (with the input gradient's filter turned by a few extra workgroups of the same launch)
        const unsigned turn_x = dgrad_conv ? ceil_div(ceil_div(idims[3] * fdims[1] * fdims[2] * ocp, 256), (g.OC + 31) / 32) : 0;
        trans_bias_partials<<<dim3(bias_chunks + (turn_x > 64 ? 64 : turn_x), (g.OC + 31) / 32), 256, 0, stream()>>>(
            ogT, (size_t)lda, bias_part, outputG, g, bias_chunks, TurnJob{filter, turned, g.OC, (int)ocp, g.kh, g.kw, g.C});
    } else {
        const bool vec4 = g.OC % 4 == 0 && aligned16(outputG);
        const int quads = vec4 ? g.OC / 4 : g.OC;
        int colsq = 1;
        while (colsq < quads && colsq < 256) colsq <<= 1;   // power of two, so that 256 % colsq == 0
        const dim3 grid((quads + colsq - 1) / colsq, bias_chunks);
        if (vec4) bias_partials<4><<<grid, 256, 0, stream()>>>(bias_part, outputG, g, colsq, 256 / colsq);
        else bias_partials<1><<<grid, 256, 0, stream()>>>(bias_part, outputG, g, colsq, 256 / colsq);
    }
    SWC_LAUNCH_CHECK();
    // the partial sums of the bias gradient are added up in the launch that adds up the filter gradient's, if there is one
    const bool sums_together = wgrad_mfma && splits > 1;
    const SumJob bias_sum{biasG, bias_part, (size_t)g.OC, bias_chunks};
    if (!sums_together)
        if (int rc = launch_sum_splits(biasG, bias_part, (size_t)g.OC, bias_chunks)) return rc;

    // ---- input gradient
    if (dgrad_conv) {
        unsigned blocks = ceil_div(idims[3] * fdims[1] * fdims[2] * ocp, 256);
        if (!wgrad_mfma) {   // (otherwise the launch above has turned the filter)
            turn_filter<<<blocks > 1024 ? 1024 : blocks, 256, 0, stream()>>>(TurnJob{filter, turned, g.OC, (int)ocp, g.kh, g.kw, g.C});
            SWC_LAUNCH_CHECK();
        }
        const float *og_in = outputG;
        if (ogp_b) {
            blocks = ceil_div(M * ocp, 256);
            pad_channels<<<blocks > 16384 ? 16384 : blocks, 256, 0, stream()>>>(og_padded, outputG, M, g.OC, (int)ocp);
            SWC_LAUNCH_CHECK();
            og_in = og_padded;
        }
        const Epilogue ep{nullptr, nullptr, nullptr, nullptr, nullptr, 0.f, 0};
        // its shared-tile pieces go into this call's own region: the library workspace is in use here
        const int rc = conv_dispatch(who, inputG, og_in, turned, nullptr, t_odims, t_idims, t_fdims, kernels, t_strides,
                                     t_pads, 1, ep, /*bias_optional=*/true, ConvScratch{dgrad_pieces, dgrad_b});
        if (rc != SWC_HIP_OK) return rc;
    } else if (g.C <= 4 && (size_t)g.kh * g.kw * g.C * ocp * 4 <= 48 * 1024) {
        unsigned blocks = ceil_div(in_elems / g.C, 256);
        blocks = blocks > 65536 ? 65536 : blocks;
        const size_t lds = (size_t)g.kh * g.kw * g.C * ocp * 4;
        const bool vec = g.OC % 4 == 0 && aligned16(outputG);
        auto launch = [&]<int CI>() {
            if (vec) dgrad_few_channels<CI, true><<<blocks, 256, lds, stream()>>>(inputG, outputG, filter, g, (int)ocp);
            else dgrad_few_channels<CI, false><<<blocks, 256, lds, stream()>>>(inputG, outputG, filter, g, (int)ocp);
        };
        switch (g.C) {
        case 1: launch.template operator()<1>(); break;
        case 2: launch.template operator()<2>(); break;
        case 3: launch.template operator()<3>(); break;
        default: launch.template operator()<4>(); break;
        }
        SWC_LAUNCH_CHECK();
    } else {
        unsigned blocks = ceil_div(in_elems, 256);
        dgrad_direct<<<blocks > 65536 ? 65536 : blocks, 256, 0, stream()>>>(inputG, outputG, filter, g);
        SWC_LAUNCH_CHECK();
    }

    // ---- filter gradient
    if (wgrad_mfma) {
        const Im2colB bsrc = Im2colB::of(input, in_elems * 4, g);
        float *dst = splits > 1 ? part : filterG;
        const size_t a_bytes = ((size_t)(g.OC - 1) * lda + M) * 4;
        const int rc2 = narrow128 ? launch_wgrad<1, 2, 2, 2, false, 4>(ogT, a_bytes, lda, bsrc, dst, g.OC, (int)Kf, (int)M, splits, sps)
                        : narrow  ? launch_wgrad<1, 4, 2, 2, false, 4>(ogT, a_bytes, lda, bsrc, dst, g.OC, (int)Kf, (int)M, splits, sps)
                                  : launch_wgrad<1, 4, 4, 2, false, 4>(ogT, a_bytes, lda, bsrc, dst, g.OC, (int)Kf, (int)M, splits, sps);
        if (rc2 != SWC_HIP_OK) return rc2;
        if (splits > 1) {
            if (int rc3 = launch_sum_splits(filterG, part, f_elems, splits, &bias_sum)) return rc3;
        }
    } else if (wgrad_rows) {
        const dim3 grid((unsigned)g.N, (unsigned)((g.OH + wgrad_rows - 1) / wgrad_rows));
        wgrad_small<<<grid, (unsigned)((f_elems + 63) / 64 * 64), wgrad_small_lds(g, wgrad_rows), stream()>>>(
            part, outputG, input, g, wgrad_rows);
        SWC_LAUNCH_CHECK();
        if (int rc3 = launch_sum_splits(filterG, part, f_elems, (int)(grid.x * grid.y))) return rc3;
    } else {
        wgrad_direct<<<(unsigned)f_elems, 256, 0, stream()>>>(filterG, outputG, input, g);
        SWC_LAUNCH_CHECK();
    }
    if (group > 1) {   // element-wise, in place
        mask_filter_groups<<<mask_blocks, 256, 0, stream()>>>(filterG, filterG, g.OC, g.kh * g.kw, g.C, (int)group);
        SWC_LAUNCH_CHECK();
    }
    return SWC_HIP_OK;
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

int swc_hip_conv2dFusedAdd_f(float *output, const float *input, const float *filter, const float *bias,
                             const size_t *odims, const size_t *idims, const size_t *fdims, const size_t *bdims,
                             const size_t *kernels, const size_t *strides, const size_t *pads, size_t group,
                             const float *bn_mean, const float *bn_var, const float *bn_scale, const float *bn_bias,
                             float epsilon, const float *residual, int relu) {
    SWC_REQUIRE_INIT();
    (void)bdims;
    if (bn_mean || bn_var || bn_scale || bn_bias)
        SWC_ARG(bn_mean && bn_var && bn_scale && bn_bias);
    Epilogue ep{nullptr, bn_mean, bn_var, bn_scale, bn_bias, epsilon, relu, residual};
    return conv_dispatch("swc_hip_conv2dFusedAdd_f", output, input, filter, bias, odims, idims, fdims, kernels, strides,
                         pads, group, ep);
}

// ---- convolution (+ batchnorm) (+ ReLU) + max-pooling in one call
namespace {

// The pooling the tile kernels can do in their epilogue: 2 x 2 windows, stride 2, no padding, over an output with
// whole windows only.
bool pool_is_2x2(const size_t *cdims, const size_t *pdims, const size_t *pk, const size_t *ps, const size_t *pp) {
    return pk[0] == 2 && pk[1] == 2 && ps[0] == 2 && ps[1] == 2 && pp[0] == 0 && pp[1] == 0 && cdims[1] % 2 == 0 &&
           cdims[2] % 2 == 0 && pdims[1] == cdims[1] / 2 && pdims[2] == cdims[2] / 2;
}

int check_pool_after_conv(const char *who, const size_t *cdims, const size_t *pdims, const size_t *pk, const size_t *ps,
                          const size_t *pp) {
    if (!pdims || !pk || !ps || !pp) return fail(SWC_HIP_EINVAL, "%s: null shape array", who);
    if (pdims[0] != cdims[0] || pdims[3] != cdims[3])
        return fail(SWC_HIP_EINVAL, "%s: pooled batch/channels differ from the convolution's", who);
    return SWC_HIP_OK;
}

} // namespace

size_t swc_hip_conv2dFusedMaxpool_workspace_bytes(const size_t *cdims, const size_t *idims, const size_t *fdims,
                                                  const size_t *kernels, const size_t *strides, const size_t *pads,
                                                  size_t group, const size_t *pdims, const size_t *pool_kernels,
                                                  const size_t *pool_strides, const size_t *pool_pads) {
    const char *who = "swc_hip_conv2dFusedMaxpool_workspace_bytes";
    if (!ready() || check_conv_dims(who, cdims, idims, fdims, kernels, strides, pads, group, true) ||
        check_pool_after_conv(who, cdims, pdims, pool_kernels, pool_strides, pool_pads))
        return 0;
    const size_t conv = swc_hip_conv2d_workspace_bytes(cdims, idims, fdims, kernels, strides, pads, group);
    const ConvGeom g = make_geom(cdims, idims, fdims, kernels, strides, pads);
    if (g.M == 0 || g.OC == 0) return 0;
    // Where the tile kernels pool in their epilogue they do so only for operands on 16-byte boundaries; otherwise the
    // convolution's own output goes through the workspace and maxpool_f's kernel pools it.  The query does not see the
    // pointers: it answers for the alignment that needs more (the direct kernel of first layers, and layers computed on
    // padded copies, pool whatever the alignment).
    const void *off_grid = reinterpret_cast<const void *>(4);
    if (pool_is_2x2(cdims, pdims, pool_kernels, pool_strides, pool_pads) && conv_pool_fusable(g, nullptr, nullptr, nullptr) &&
        conv_pool_fusable(g, off_grid, off_grid, off_grid))
        return conv;
    return align256((size_t)g.M * g.OC * 4) + conv;
}

int swc_hip_conv2dFusedMaxpool_f(float *output, const float *input, const float *filter, const float *bias,
                                 const size_t *cdims, const size_t *idims, const size_t *fdims, const size_t *bdims,
                                 const size_t *kernels, const size_t *strides, const size_t *pads, size_t group,
                                 const float *bn_mean, const float *bn_var, const float *bn_scale, const float *bn_bias,
                                 float epsilon, int relu, const size_t *pdims, const size_t *pool_kernels,
                                 const size_t *pool_strides, const size_t *pool_pads) {
    SWC_REQUIRE_INIT();
    (void)bdims;
    const char *who = "swc_hip_conv2dFusedMaxpool_f";
    if (bn_mean || bn_var || bn_scale || bn_bias)
        SWC_ARG(bn_mean && bn_var && bn_scale && bn_bias);
    if (int rc = check_conv_dims(who, cdims, idims, fdims, kernels, strides, pads, group, true)) return rc;
    if (int rc = check_pool_after_conv(who, cdims, pdims, pool_kernels, pool_strides, pool_pads)) return rc;
    Epilogue ep{nullptr, bn_mean, bn_var, bn_scale, bn_bias, epsilon, relu};
    const ConvGeom g = make_geom(cdims, idims, fdims, kernels, strides, pads);
    if (g.M == 0 || g.OC == 0) return SWC_HIP_OK;
    if (pool_is_2x2(cdims, pdims, pool_kernels, pool_strides, pool_pads) && conv_pool_fusable(g, input, filter, output))
        return conv_dispatch(who, output, input, filter, bias, cdims, idims, fdims, kernels, strides, pads, group, ep, false,
                             ConvScratch{nullptr, 0}, true);
    // any other pooling, or a layer for another kernel: the two steps, the convolution's output in the workspace
    const size_t inter = align256((size_t)g.M * g.OC * 4);
    const size_t need = inter + swc_hip_conv2d_workspace_bytes(cdims, idims, fdims, kernels, strides, pads, group);
    char *base = static_cast<char *>(workspace(need, who));
    if (!base) return fail_code();
    float *conv_out = reinterpret_cast<float *>(base);
    if (int rc = conv_dispatch(who, conv_out, input, filter, bias, cdims, idims, fdims, kernels, strides, pads, group, ep,
                               false, ConvScratch{reinterpret_cast<float *>(base + inter), need - inter}))
        return rc;
    return swc_hip_maxpool_f(conv_out, output, cdims, pdims, pool_kernels, pool_strides, pool_pads);
}

size_t swc_hip_conv2d_workspace_bytes(const size_t *odims, const size_t *idims, const size_t *fdims,
                                      const size_t *kernels, const size_t *strides, const size_t *pads, size_t group) {
    if (!ready() ||
        check_conv_dims("swc_hip_conv2d_workspace_bytes", odims, idims, fdims, kernels, strides, pads, group, true))
        return 0;
    const ConvGeom g = make_geom(odims, idims, fdims, kernels, strides, pads);
    if (g.M == 0 || g.OC == 0) return 0;
    const size_t masked = group > 1 ? align256((size_t)g.OC * g.K * 4) : 0;
    if (g.K <= kDirectMaxK && g.OC <= kDirectMaxOC && g.C % 4 != 0) return masked;
    return masked + conv_total_scratch(g, nullptr, nullptr);   // (tensors of a generated program are 256-byte aligned)
}

size_t swc_hip_conv2dGrad_workspace_bytes(const size_t *odims, const size_t *idims, const size_t *fdims,
                                          const size_t *kernels, const size_t *strides, const size_t *pads, size_t group) {
    if (!ready() ||
        check_conv_dims("swc_hip_conv2dGrad_workspace_bytes", odims, idims, fdims, kernels, strides, pads, group, true))
        return 0;
    const ConvGeom g = make_geom(odims, idims, fdims, kernels, strides, pads);
    const size_t f_elems = fdims[0] * fdims[1] * fdims[2] * fdims[3];
    if (g.M == 0 || g.OC == 0 || f_elems == 0 || idims[0] * idims[1] * idims[2] * idims[3] == 0) return 0;
    // each of the three alignment tests of the call (16-byte boundaries or not) picks kernels with their own needs, and
    // the query does not see the pointers: the largest of the eight layouts
    size_t most = 0;
    for (int c = 0; c < 8; ++c) {
        const size_t t = grad_layout(g, odims, idims, fdims, kernels, c & 1, c & 2, c & 4).total();
        most = t > most ? t : most;
    }
    return (group > 1 ? align256(f_elems * 4) : 0) + most;
}

int swc_hip_conv2dGrad_f(float *inputG, float *filterG, float *biasG, const float *outputG, const float *input,
                         const float *filter, const size_t *odims, const size_t *idims, const size_t *fdims,
                         const size_t *bdims, const size_t *kernels, const size_t *strides, const size_t *pads,
                         size_t group) {
    SWC_REQUIRE_INIT();
    (void)bdims;
    return conv_grad(inputG, filterG, biasG, outputG, input, filter, odims, idims, fdims, kernels, strides, pads, group);
}

} // extern "C"
