// Row-strip forward convolution on fp32 MFMA: the kernel.  Tile geometry, LDS
// layout, swizzles and the lane -> address maps are in conv_strip_index.hpp
// (shared with the host-side emulation that checks them).
//
// Synchronisation.  K is walked chunk by chunk (16 channels x all taps).  At
// the top of chunk c every wavefront waits for its own outstanding loads
// (s_waitcnt vmcnt(0)) and the workgroup meets at a barrier: the patch and the
// filter part of chunk c, requested one chunk earlier, are then in LDS for
// everyone, and nobody reads the other pair of buffers any more — into which
// the wavefronts at once request chunk c + 1, which has the whole of chunk c's
// MFMAs (tens of thousands of cycles) to arrive.  Between barriers the
// wavefronts run free.
#pragma once
#include "conv_strip_index.hpp"
#include "mfma_dma.hpp"
#include "mfma_tile.hpp"

namespace swc_hip {
namespace strip {

typedef float v4f __attribute__((ext_vector_type(4)));

// One v_mfma_f32_16x16x4_f32 with the accumulator in AGPRs (see mfma_acc in mfma_tile.hpp for why, and for the
// rule that the first ordinary read of the results is preceded by settle()).
__device__ __forceinline__ void mfma16(v4f &acc, float a, float b) {
#if __HIP_DEVICE_COMPILE__
    asm("v_mfma_f32_16x16x4_f32 %0, %1, %2, %0" : "+a"(acc) : "v"(a), "v"(b));
#endif
}

template <int TMW, int TNW>
__device__ __forceinline__ void settle(v4f (&acc)[TMW][TNW]) {
#if __HIP_DEVICE_COMPILE__
#pragma unroll
    for (int i = 0; i < TMW; ++i)
#pragma unroll
        for (int j = 0; j < TNW; ++j) asm volatile("" : "+a"(acc[i][j]));
    asm volatile("s_nop 7\n\ts_nop 7" : "+a"(acc[TMW - 1][TNW - 1]));   // an 8-pass MFMA needs 10 wait states
#endif
}

template <int TMW, int TNW>
__global__ __launch_bounds__(kThreads) void conv_strip(const float *__restrict__ in, const float *__restrict__ filt,
                                                       float *__restrict__ out, ConvGeom g, Plan p, unsigned in_bytes,
                                                       unsigned filt_bytes, mfma::Epilogue ep) {
#if __HIP_DEVICE_COMPILE__
    using mfma::lds_void_t;
    extern __shared__ __align__(16) float lds[];
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int j = lane & 15, q = lane >> 4;
    const TileOrigin t = tile_origin(p, blockIdx.x);
    const WaveBlocks wb = wave_blocks(p, wave);

    const __amdgpu_buffer_rsrc_t rsrc_in = mfma::make_rsrc(in, in_bytes);
    const __amdgpu_buffer_rsrc_t rsrc_f = mfma::make_rsrc(filt, filt_bytes);

    // fragment addresses that do not change over the K loop
    int px0[TMW];      // patch pixel under tap (0,0) of this lane's pixel in each of its blocks
#pragma unroll
    for (int m = 0; m < TMW; ++m) px0[m] = lane_patch_px0(g, p, wb.blk0 + (m < wb.cnt ? m : 0), j);
    int fbyte[TNW];    // byte offset of this lane's filter fragment inside tap 0 of a filter buffer
#pragma unroll
    for (int n = 0; n < TNW; ++n) fbyte[n] = lane_filter_byte(wb.cb0 + n, j, q);

    char *const lds_b = reinterpret_cast<char *>(lds);

    // This wavefront's share of a chunk's loads: block i*8 + wave of the patch (i < PW) and of the filter part
    // (i < FW).  The per-lane byte offsets do not depend on the chunk (a chunk adds 64 bytes as a scalar), so they
    // are formed once; what is left per chunk is the load instructions themselves.
    int pbyte[kMaxPW], fbyte_g[kMaxFW];
#pragma unroll
    for (int i = 0; i < kMaxPW; ++i) pbyte[i] = i < p.PW ? patch_lane_byte(g, p, t, i * kWaves + wave, lane) : kNoByte;
#pragma unroll
    for (int i = 0; i < kMaxFW; ++i) fbyte_g[i] = i < p.FW ? filter_lane_byte(g, p, t, i * kWaves + wave, lane) : kNoByte;
    auto request_chunk = [&](int chunk, int buf) {
        float *pdst = lds + lds_patch(p, buf) + wave * kLoadFloats, *fdst = lds + lds_filter(p, buf) + wave * kLoadFloats;
#pragma unroll
        for (int i = 0; i < kMaxPW; ++i)
            if (i < p.PW)
                __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrc_in, (lds_void_t *)(pdst + i * kWaves * kLoadFloats), 16, pbyte[i],
                                                         chunk * kPxBytes, 0, 0);
#pragma unroll
        for (int i = 0; i < kMaxFW; ++i)
            if (i < p.FW)
                __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrc_f, (lds_void_t *)(fdst + i * kWaves * kLoadFloats), 16, fbyte_g[i],
                                                         chunk * kPxBytes, 0, 0);
    };

    v4f acc[TMW][TNW];
#pragma unroll
    for (int m = 0; m < TMW; ++m)
#pragma unroll
        for (int n = 0; n < TNW; ++n) acc[m][n] = v4f{0.f, 0.f, 0.f, 0.f};

    // Fragments of one tap: TNW of the filter, TMW of the pixels.  Those of tap t + 1 are read while tap t is
    // multiplied — one read behind each block's MFMAs, pinned there by scheduling fences — so an LDS read has a
    // whole tap (hundreds of MFMA cycles) to return; only the first tap after a barrier waits for its reads.
    struct Frags {
        v4f a[TNW], b[TMW];
    };
    auto read_a = [&](Frags &f, const char *tap_b) {
#pragma unroll
        for (int n = 0; n < TNW; ++n) f.a[n] = *reinterpret_cast<const v4f *>(tap_b + fbyte[n]);
    };
    auto read_b = [&](Frags &f, const char *patch_b, int tap_px, int m) {
        const int pp = px0[m] + tap_px;
        f.b[m] = *reinterpret_cast<const v4f *>(patch_b + swz_byte(pp, q));
    };
    const int taps = p.taps;

    request_chunk(0, 0);
    for (int chunk = 0; chunk < p.chunks; ++chunk) {
        mfma::ring_sync<0>();   // chunk `chunk` is in LDS for everyone; the other buffer pair is free
        if (chunk + 1 < p.chunks) request_chunk(chunk + 1, (chunk + 1) & 1);
        const char *patch_b = lds_b + lds_patch(p, chunk & 1) * 4;
        const char *tap_b = lds_b + lds_filter(p, chunk & 1) * 4;
        Frags cur, nxt;
        read_a(cur, tap_b);
#pragma unroll
        for (int m = 0; m < TMW; ++m) read_b(cur, patch_b, 0, m);
        int ky = 0, kx = 0;   // of the tap being multiplied
        for (int tap = 0; tap < taps; ++tap) {
            // the next tap's coordinates (the last tap of a chunk re-reads itself: harmless, never used)
            int nky = ky, nkx = kx;
            const bool more = tap + 1 < taps;
            if (more) {
                if (++nkx == g.kw) nkx = 0, ++nky;
                tap_b += p.BN * kPxBytes;
            }
            const int next_px = nky * p.Wp + nkx;
            read_a(nxt, tap_b);
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int m = 0; m < TMW; ++m) {
                read_b(nxt, patch_b, next_px, m);
                if (m < wb.cnt) {
#pragma unroll
                    for (int s = 0; s < 4; ++s)
#pragma unroll
                        for (int n = 0; n < TNW; ++n) mfma16(acc[m][n], cur.a[n][s], cur.b[m][s]);
                }
                __builtin_amdgcn_sched_barrier(0);
            }
            cur = nxt;
            ky = nky, kx = nkx;
        }
    }
    settle<TMW, TNW>(acc);

    // ---- epilogue: lane (j, q) holds output channels 4q .. 4q+3 of pixel j of each of its blocks
    const bool bn = ep.bn_mean != nullptr;
    float bias[TNW][4], mean[TNW][4], slope[TNW][4], beta[TNW][4];
#pragma unroll
    for (int n = 0; n < TNW; ++n) {
        const int oc = t.n0 + (wb.cb0 + n) * 16 + 4 * q;
#pragma unroll
        for (int v = 0; v < 4; ++v) {
            bias[n][v] = ep.bias ? ep.bias[oc + v] : 0.f;
            mean[n][v] = 0.f, slope[n][v] = 1.f, beta[n][v] = 0.f;
            if (bn) {   // one fp32 multiply-add per element, the slope formed in double (as the other conv kernels)
                mean[n][v] = ep.bn_mean[oc + v];
                slope[n][v] = (float)((double)ep.bn_scale[oc + v] / sqrt((double)(ep.bn_var[oc + v] + ep.eps)));
                beta[n][v] = ep.bn_bias[oc + v];
            }
        }
    }
#pragma unroll
    for (int m = 0; m < TMW; ++m) {
        const int px = (wb.blk0 + m) * 16 + j;
        if (m < wb.cnt && px < p.P) {
            const size_t row = (size_t)(t.m0 + px) * g.OC;
#pragma unroll
            for (int n = 0; n < TNW; ++n) {
                const int oc = t.n0 + (wb.cb0 + n) * 16 + 4 * q;
                float x[4];
#pragma unroll
                for (int v = 0; v < 4; ++v) {
                    x[v] = acc[m][n][v] + bias[n][v];
                    if (bn) x[v] = fmaf(x[v] - mean[n][v], slope[n][v], beta[n][v]);
                }
                if (ep.residual) {
                    const float4 r = *reinterpret_cast<const float4 *>(ep.residual + row + oc);
                    x[0] += r.x, x[1] += r.y, x[2] += r.z, x[3] += r.w;
                }
                if (ep.relu) {
#pragma unroll
                    for (int v = 0; v < 4; ++v) x[v] = (x[v] > 0.f) ? x[v] : 0.f;
                }
                *reinterpret_cast<float4 *>(out + row + oc) = make_float4(x[0], x[1], x[2], x[3]);
            }
        }
    }
#endif
}

} // namespace strip
} // namespace swc_hip
