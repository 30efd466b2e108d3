// Row-strip forward convolution on fp32 MFMA: the kernel.  Tile geometry, LDS
// layout, swizzles and the lane -> address maps are in conv_strip_index.hpp
// (shared with the host-side emulation that checks them).
//
// Ring discipline.  A "slice" is one tap of one 16-channel chunk: 16 k.  Every
// wavefront issues exactly LP + 1 direct-to-LDS loads per slice — LP blocks of
// the NEXT chunk's patch (into the other patch buffer) and its block of the
// filter slice kDepth slices ahead (into the stage read one slice ago) — a load
// that has nothing to carry is issued all the same with an out-of-range offset,
// into a per-wavefront dump block, so that the pending-load counter advances
// identically in every slice.  Loads land in order, hence at the top of slice s
//     s_waitcnt vmcnt((kDepth-1) * (LP+1));  s_barrier
// certifies, for the wavefront and then for the workgroup, that everything
// issued up to slice s - kDepth is in LDS — the filter slice s, and, at a chunk
// boundary, the whole patch of the new chunk (the planner makes sure its last
// real block is issued kDepth slices before the chunk ends) — and that nobody
// still reads the stage and the patch buffer that this slice's loads overwrite.
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

template <int TMW, int TNW, int LP>
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
    int fbyte[TNW];    // byte offset of this lane's filter fragment inside a stage
#pragma unroll
    for (int n = 0; n < TNW; ++n) fbyte[n] = lane_filter_byte(wb.cb0 + n, j, q);
    const int f_lane = filter_lane_byte(g, p, t, wave, lane);   // this wavefront's block of a filter slice

    char *const lds_b = reinterpret_cast<char *>(lds);
    float *const dump = lds + lds_dump(p, wave);

    // patch block `i` (of PW per wavefront) of channel chunk `chunk` into patch buffer `buf`; a block beyond PW
    // or a chunk beyond the last goes to the dump block as an empty load
    auto load_patch = [&](int i, int chunk, int buf) {
        const bool real = i < p.PW && chunk < p.chunks;   // wavefront-uniform
        const int blk = i * kWaves + wave;
        const int v = real ? patch_lane_byte(g, p, t, blk, lane) : kNoByte;
        float *dst = real ? lds + lds_patch(p, buf) + blk * kLoadFloats : dump;
        __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrc_in, (lds_void_t *)dst, 16, v, chunk * kPxBytes, 0, 0);
    };
    // this wavefront's block of filter slice (tap, chunk) into ring stage `stage`
    auto load_filter = [&](int tap, int chunk, int stage, bool exists) {
        const bool real = exists && wave * kLoadPx < p.BN;
        float *dst = real ? lds + lds_bstage(p, stage) + wave * kLoadFloats : dump;
        __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrc_f, (lds_void_t *)dst, 16, real ? f_lane : kNoByte,
                                                 (tap * g.C + chunk * kChunk) * 4, 0, 0);
    };

    v4f acc[TMW][TNW];
#pragma unroll
    for (int m = 0; m < TMW; ++m)
#pragma unroll
        for (int n = 0; n < TNW; ++n) acc[m][n] = v4f{0.f, 0.f, 0.f, 0.f};

    // ---- prologue: the whole patch of chunk 0, then the loads of the kDepth slices "before" slice 0
    for (int i = 0; i < p.PW; ++i) load_patch(i, 0, 0);
    // (tap, chunk) of the filter slice to request next; slices run tap-fastest within a chunk
    int ld_tap = 0, ld_chunk = 0, ld_stage = 0;
    auto next_filter = [&]() {
        load_filter(ld_tap, ld_chunk, ld_stage, ld_chunk < p.chunks);
        if (++ld_tap == p.taps) ld_tap = 0, ++ld_chunk;
        ld_stage = ld_stage + 1 == kBStages ? 0 : ld_stage + 1;
    };
#pragma unroll
    for (int d = 0; d < kDepth; ++d) {
#pragma unroll
        for (int l = 0; l < LP; ++l) load_patch(p.PW, 0, 0);   // empty: keeps the count per slice
        next_filter();
    }

    int rd_stage = 0;
    for (int chunk = 0; chunk < p.chunks; ++chunk) {
        const char *patch_b = lds_b + lds_patch(p, chunk & 1) * 4;
        int tap = 0;
        for (int ky = 0; ky < g.kh; ++ky)
            for (int kx = 0; kx < g.kw; ++kx, ++tap) {
                mfma::ring_sync<(kDepth - 1) * (LP + 1)>();
                // this slice's loads: LP blocks of the next chunk's patch, one block of the filter slice kDepth ahead
#pragma unroll
                for (int l = 0; l < LP; ++l) load_patch(tap * LP + l, chunk + 1, (chunk + 1) & 1);
                next_filter();

                const char *stage_b = lds_b + lds_bstage(p, rd_stage) * 4;
                v4f fa[TNW];   // filter fragments: four consecutive channels of this lane's output channel
#pragma unroll
                for (int n = 0; n < TNW; ++n) fa[n] = *reinterpret_cast<const v4f *>(stage_b + fbyte[n]);
                const int tap_px = ky * p.Wp + kx;
                auto pixel_frag = [&](int m) {
                    const int pp = px0[m] + tap_px;
                    return *reinterpret_cast<const v4f *>(patch_b + swz_byte(pp, q));
                };
                v4f fb = pixel_frag(0);
#pragma unroll
                for (int m = 0; m < TMW; ++m) {
                    v4f fb_next = fb;
                    if (m + 1 < TMW) fb_next = pixel_frag(m + 1);   // in flight behind this block's MFMAs
                    if (m < wb.cnt) {
#pragma unroll
                        for (int s = 0; s < 4; ++s)
#pragma unroll
                            for (int n = 0; n < TNW; ++n) mfma16(acc[m][n], fa[n][s], fb[s]);
                    }
                    fb = fb_next;
                }
                rd_stage = rd_stage + 1 == kBStages ? 0 : rd_stage + 1;
            }
    }
    mfma::wait_vmcnt<0>();   // the trailing empty loads still target this workgroup's LDS
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
