// Host-side emulation of the data movement of the row-strip convolution kernel
// (swcompiler_amd/csrc/conv_strip.hpp), built from the same index header the
// kernel uses.  It runs the kernel's steps lane by lane on the CPU — the
// direct-to-LDS loads (lane l of a load lands at byte 16*l of its 1-KiB block,
// zeros for an out-of-range offset), the swizzled 128-bit fragment reads, the
// operand and result layout of v_mfma_f32_16x16x4_f32, the epilogue's pixel /
// channel mapping — so that a wrong swizzle, tap offset or block assignment
// shows up in a CPU test before the kernel ever runs on a GPU.  Ring timing and
// barriers are not emulated: every slice's data is simply loaded before it is
// multiplied.  Test infrastructure only.
#include <cstdint>
#include <cstring>
#include <vector>

#include "conv_strip_index.hpp"

using namespace swc_hip;
using namespace swc_hip::strip;

namespace {

// lane l's 16 bytes of a wavefront load: from `base + byte` (zeros if out of range) to lds[dst + 4*l ..]
void dma_lane(std::vector<float> &lds, int dst_float, int lane, const float *base, size_t bytes, long byte) {
    float v[4] = {0.f, 0.f, 0.f, 0.f};
    if (byte >= 0 && (size_t)byte + 16 <= bytes) std::memcpy(v, reinterpret_cast<const char *>(base) + byte, 16);
    for (int e = 0; e < 4; ++e) lds[dst_float + 4 * lane + e] = v[e];
}

} // namespace

extern "C" {

// Fills `plan_out` (R, BN, WM, WN, TMW, TNW, FW, PW, lds_bytes, tiles, eff*1000) and returns 1 if the kernel
// applies to the layer on `cus` compute units, else 0.
int strip_emu_plan(const int *geom, int cus, int *plan_out) {
    ConvGeom g{geom[0], geom[1], geom[2], geom[3], geom[4], geom[5], geom[6], geom[7], geom[8], geom[9], geom[10],
               geom[11], geom[12], geom[0] * geom[4] * geom[5], geom[7] * geom[8] * geom[3]};
    Plan p;
    if (!plan(g, cus, p)) return 0;
    const int v[11] = {p.R, p.BN, p.WM, p.WN, p.TMW, p.TNW, p.FW, p.PW, p.lds_bytes, p.tiles_m * p.tiles_n, (int)(p.eff * 1000)};
    std::memcpy(plan_out, v, sizeof(v));
    return 1;
}

// out = bias + conv(in, filt) through the emulated kernel.  geom = {N,H,W,C, OH,OW,OC, kh,kw, sh,sw, pt,pl}.
// force = {R, BN, WM} to emulate one particular plan, or null for the planner's choice.  Returns 1, or 0 if no plan.
int strip_emu_conv(const float *in, const float *filt, const float *bias, float *out, const int *geom, int cus,
                   const int *force) {
    ConvGeom g{geom[0], geom[1], geom[2], geom[3], geom[4], geom[5], geom[6], geom[7], geom[8], geom[9], geom[10],
               geom[11], geom[12], geom[0] * geom[4] * geom[5], geom[7] * geom[8] * geom[3]};
    Plan p;
    if (force) {
        if (g.C % kChunk || g.OC % 16 || !make_plan(g, cus, force[0], force[1], force[2], p)) return 0;
    } else if (!plan(g, cus, p)) {
        return 0;
    }
    const size_t in_bytes = (size_t)g.N * g.H * g.W * g.C * 4, filt_bytes = (size_t)g.OC * g.K * 4;
    std::vector<float> lds(lds_total_floats(p));
    for (int tile = 0; tile < p.tiles_m * p.tiles_n; ++tile) {
        const TileOrigin t = tile_origin(p, tile);
        // accumulators: [wave][m][n][lane][v]
        std::vector<float> acc((size_t)kWaves * p.TMW * p.TNW * 64 * 4, 0.f);
        auto A = [&](int w, int m, int n, int lane, int v) -> float & {
            return acc[((((size_t)w * p.TMW + m) * p.TNW + n) * 64 + lane) * 4 + v];
        };
        for (int chunk = 0; chunk < p.chunks; ++chunk) {
            // the chunk's patch and filter part: PW and FW loads per wavefront
            for (int w = 0; w < kWaves; ++w) {
                for (int i = 0; i < p.PW; ++i) {
                    const int blk = i * kWaves + w;
                    for (int lane = 0; lane < 64; ++lane) {
                        const int v = patch_lane_byte(g, p, t, blk, lane);
                        dma_lane(lds, lds_patch(p, chunk & 1) + blk * kLoadFloats, lane, in, in_bytes,
                                 v == kNoByte ? -1 : (long)v + chunk * kPxBytes);
                    }
                }
                for (int i = 0; i < p.FW; ++i) {
                    const int blk = i * kWaves + w;
                    for (int lane = 0; lane < 64; ++lane) {
                        const int v = filter_lane_byte(g, p, t, blk, lane);
                        dma_lane(lds, lds_filter(p, chunk & 1) + blk * kLoadFloats, lane, filt, filt_bytes,
                                 v == kNoByte ? -1 : (long)v + chunk * kPxBytes);
                    }
                }
            }
            int tap = 0;
            for (int ky = 0; ky < g.kh; ++ky)
                for (int kx = 0; kx < g.kw; ++kx, ++tap) {
                    const char *lds_b = reinterpret_cast<const char *>(lds.data());
                    const char *stage_b = lds_b + (size_t)lds_filter(p, chunk & 1) * 4 + (size_t)tap * p.BN * kPxBytes;
                    const char *patch_b = lds_b + (size_t)lds_patch(p, chunk & 1) * 4;
                    const int tap_px = ky * p.Wp + kx;
                    for (int w = 0; w < kWaves; ++w) {
                        const WaveBlocks wb = wave_blocks(p, w);
                        for (int m = 0; m < wb.cnt; ++m)
                            for (int n = 0; n < p.TNW; ++n) {
                                // fragments of all 64 lanes
                                float fa[64][4], fb[64][4];
                                for (int lane = 0; lane < 64; ++lane) {
                                    const int j = lane & 15, q = lane >> 4;
                                    std::memcpy(fa[lane], stage_b + lane_filter_byte(wb.cb0 + n, j, q), 16);
                                    const int pp = lane_patch_px0(g, p, wb.blk0 + m, j) + tap_px;
                                    std::memcpy(fb[lane], patch_b + swz_byte(pp, q), 16);
                                }
                                // four v_mfma_f32_16x16x4_f32: D[i][j] += sum_k A[i][k] B[k][j]; lane l gives A[l%16][l/16] and
                                // B[l/16][l%16]; D[i][j] sits in lane (j + 16*(i/4)), register i%4
                                for (int s = 0; s < 4; ++s)
                                    for (int i = 0; i < 16; ++i)
                                        for (int jj = 0; jj < 16; ++jj) {
                                            float sum = 0.f;
                                            for (int k = 0; k < 4; ++k) sum += fa[i + 16 * k][s] * fb[jj + 16 * k][s];
                                            A(w, m, n, jj + 16 * (i / 4), i % 4) += sum;
                                        }
                            }
                    }
                }
        }
        // epilogue: lane (j, q) holds output channels 4q .. 4q+3 of pixel j of each of its blocks
        for (int w = 0; w < kWaves; ++w) {
            const WaveBlocks wb = wave_blocks(p, w);
            for (int m = 0; m < wb.cnt; ++m)
                for (int lane = 0; lane < 64; ++lane) {
                    const int j = lane & 15, q = lane >> 4;
                    const int px = (wb.blk0 + m) * 16 + j;
                    if (px >= p.P) continue;
                    for (int n = 0; n < p.TNW; ++n) {
                        const int oc = t.n0 + (wb.cb0 + n) * 16 + 4 * q;
                        for (int v = 0; v < 4; ++v)
                            out[(size_t)(t.m0 + px) * g.OC + oc + v] = A(w, m, n, lane, v) + (bias ? bias[oc + v] : 0.f);
                    }
                }
        }
    }
    return 1;
}

} // extern "C"
