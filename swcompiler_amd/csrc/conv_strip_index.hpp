// Index arithmetic of the row-strip convolution kernel (conv_strip.hpp), in plain
// C++ so that the device kernel and a host-side emulation of its data movement
// (tests/host/strip_emu.cpp) use the very same formulas.
//
// The kernel computes conv2d_f (kernels.h:177-243) for stride-any, NHWC layers
// whose channel counts are multiples of 16.  A workgroup of eight wavefronts owns
// a tile of R whole output rows of one image (P = R*OW pixels) by BN output
// channels.  K = kh*kw*iC is walked as (channel chunk of 16) x (tap): for one
// chunk the input pixels the tile's taps touch — the "patch", Rp x Wp pixels of
// 16 channels = 64 bytes each, zeros where the image ends — stay in LDS for all
// kh*kw taps, so the input crosses from L2 into LDS once per chunk instead of
// once per tap, and no address arithmetic is left in the tap loop: a tap is a
// scalar offset into the patch.  The filter streams through a small ring, one
// slice (BN x 16 floats) per tap.
//
// Matrix blocks are 16 x 16 (v_mfma_f32_16x16x4_f32, the same flop rate as the
// 32 x 32 x 2 form): with blocks of 16 pixels a tile of 392 pixels is 24.5
// blocks, 2 % above its share, where blocks of 32 would waste 6 %.
// Lane l of a wavefront: j = l % 16, q = l / 16.  The filter is the A operand
// (row = output channel j of the block, k = q), the pixels the B operand
// (column = pixel j, k = q); each lane reads four consecutive channels
// 4q .. 4q+3 of its row with one 128-bit LDS read, which feed four MFMAs.  The
// result D[i][j] leaves lane l with output channels 4q .. 4q+3 of pixel j: one
// 128-bit store.
#pragma once

#ifndef SWC_HD
#if defined(__HIPCC__)
#define SWC_HD __host__ __device__ __forceinline__
#else
#define SWC_HD inline
#endif
#endif

namespace swc_hip {

struct ConvGeom {
    int N, H, W, C;      // input NHWC
    int OH, OW, OC;      // output
    int kh, kw, sh, sw, pt, pl;
    int M, K;            // GEMM view: output pixels, kh*kw*C
};

namespace strip {

constexpr int kWaves = 8;
constexpr int kThreads = 64 * kWaves;
constexpr int kChunk = 16;                 // channels per slice
constexpr int kPxFloats = kChunk;          // floats per patch pixel
constexpr int kPxBytes = kChunk * 4;       // 64
constexpr int kLoadFloats = 256;           // one wavefront load: 64 lanes x 16 bytes
constexpr int kLoadPx = kLoadFloats / kPxFloats;   // 16 patch pixels (or filter rows) per load
constexpr int kDepth = 3;                  // filter slices in flight ahead of the one being multiplied
constexpr int kBStages = kDepth + 1;
constexpr int kMaxLds = 160 * 1024;

// How one layer is cut into tiles; filled by plan() on the host, read by the kernel.
struct Plan {
    int R;            // output rows per tile (divides OH)
    int BN;           // output channels per tile (multiple of 16, divides OC)
    int WM, WN;       // wavefront grid: WM x WN = 8, rows split the pixel blocks, columns the channel blocks
    int TMW, TNW;     // pixel / channel blocks per wavefront (the kernel's template arguments)
    int LP;           // patch loads per wavefront per slice (template argument)
    int P;            // R * OW
    int nblk;         // ceil(P / 16)
    int Rp, Wp;       // patch rows, columns: (R-1)*sh + kh, (OW-1)*sw + kw
    int patch_px;     // Rp * Wp
    int PW;           // patch loads per wavefront per chunk: ceil(ceil(patch_px / 16) / 8)
    int patch_floats; // floats of one patch buffer: PW * 8 * 256
    int b_floats;     // floats of one filter stage: BN * 16
    int tiles_m, tiles_n, strips_per_img;
    int taps, chunks, slices;
    float inv_wp;     // 1.0f / Wp
    int lds_bytes;
    float eff;        // estimated share of the matrix cores' time that is useful work
};

// LDS layout in floats: patch[2], filter stages, then a dump block per wavefront for loads that carry nothing.
SWC_HD int lds_patch(const Plan &p, int buf) { return buf * p.patch_floats; }
SWC_HD int lds_bstage(const Plan &p, int stage) { return 2 * p.patch_floats + stage * p.b_floats; }
SWC_HD int lds_dump(const Plan &p, int wave) { return 2 * p.patch_floats + kBStages * p.b_floats + wave * kLoadFloats; }
SWC_HD int lds_total_floats(const Plan &p) { return 2 * p.patch_floats + kBStages * p.b_floats + kWaves * kLoadFloats; }

// Swizzle: a row of 64 bytes (a patch pixel or a filter row of one slice) holds four 16-byte chunks; logical
// chunk c of row r is stored at position c ^ key(r).  Sixteen lanes that read the same logical chunk of sixteen
// consecutive rows then touch all sixty-four banks once.
SWC_HD int swz_key(int row) { return (row >> 2) & 3; }
// byte offset, inside a buffer of 64-byte rows, of logical chunk `chunk` of row `row`
SWC_HD int swz_byte(int row, int chunk) { return row * kPxBytes + ((chunk ^ swz_key(row)) << 4); }

// pp / Wp for 0 <= pp < 2^20 without an integer division (inv_wp = 1.0f / Wp, one IEEE multiply)
SWC_HD int div_wp(int pp, float inv_wp) { return (int)(((float)pp + 0.5f) * inv_wp); }

// ---- which blocks a wavefront owns
struct WaveBlocks {
    int blk0, cnt;   // first pixel block and number of them (cnt <= TMW)
    int cb0;         // first channel block (TNW of them)
};
SWC_HD WaveBlocks wave_blocks(const Plan &p, int wave) {
    const int wrow = wave / p.WN, wcol = wave - wrow * p.WN;
    const int base = p.nblk / p.WM, rem = p.nblk - base * p.WM;
    WaveBlocks b;
    b.cnt = base + (wrow < rem ? 1 : 0);
    b.blk0 = wrow * base + (wrow < rem ? wrow : rem);
    b.cb0 = wcol * p.TNW;
    return b;
}

// ---- tile coordinates
struct TileOrigin {
    int img, oy0;   // image and first output row
    int m0;         // flattened index of the tile's first output pixel
    int n0;         // first output channel
};
SWC_HD TileOrigin tile_origin(const Plan &p, int tile) {
    const int tm = tile / p.tiles_n, tn = tile - tm * p.tiles_n;
    TileOrigin t;
    t.img = tm / p.strips_per_img;
    t.oy0 = (tm - t.img * p.strips_per_img) * p.R;
    t.m0 = tm * p.P;
    t.n0 = tn * p.BN;
    return t;
}

// ---- pixel fragments (B operand): patch pixel under tap (0,0) of the lane's pixel in block `blk`
SWC_HD int lane_patch_px0(const ConvGeom &g, const Plan &p, int blk, int j) {
    int px = blk * 16 + j;
    if (px > p.P - 1) px = p.P - 1;   // lanes past the tile read a valid pixel; their results are not stored
    const int r = px / g.OW, c = px - r * g.OW;
    return r * g.sh * p.Wp + c * g.sw;
}

// ---- filter fragments (A operand): byte offset inside a filter stage of the lane's four channels
SWC_HD int lane_filter_byte(int cb, int j, int q) { return swz_byte(cb * 16 + j, q); }

// ---- global -> LDS loads.  One wavefront load fills 1 KiB: lane l lands at byte 16*l of the block, i.e. row
// (l >> 2) of the block's sixteen rows, position (l & 3), which must hold logical chunk (l & 3) ^ key(row).
constexpr int kNoByte = 0x7fffffff;   // byte offset outside every buffer: the load returns zeros

// patch load `blk` (sixteen patch pixels 16*blk ..): byte offset of the lane's 16 bytes in the input, for channel
// chunk 0 (a later chunk adds 64 bytes per chunk as a scalar), or kNoByte outside the image or the patch
SWC_HD int patch_lane_byte(const ConvGeom &g, const Plan &p, const TileOrigin &t, int blk, int lane) {
    const int pp = blk * kLoadPx + (lane >> 2);
    const int chunk = (lane & 3) ^ swz_key(pp);
    const int pr = div_wp(pp, p.inv_wp), pc = pp - pr * p.Wp;
    const int iy = t.oy0 * g.sh - g.pt + pr, ix = pc - g.pl;
    const bool ok = pp < p.patch_px && (unsigned)iy < (unsigned)g.H && (unsigned)ix < (unsigned)g.W;
    return ok ? (((t.img * g.H + iy) * g.W + ix) * g.C + chunk * 4) * 4 : kNoByte;
}

// filter load of wavefront `wave` (filter rows 16*wave .. of the tile's BN): byte offset of the lane's 16 bytes
// in the filter for tap 0, chunk 0 (a slice adds (tap*C + 16*chunk)*4 bytes as a scalar), or kNoByte
SWC_HD int filter_lane_byte(const ConvGeom &g, const Plan &p, const TileOrigin &t, int wave, int lane) {
    const int r = wave * kLoadPx + (lane >> 2);
    const int chunk = (lane & 3) ^ swz_key(r);
    const bool ok = r < p.BN && t.n0 + r < g.OC;
    return ok ? ((t.n0 + r) * g.K + chunk * 4) * 4 : kNoByte;
}

// ---- host side: the plan
inline int ceil_div_i(int a, int b) { return (a + b - 1) / b; }

// Fills `p` for one choice of (R, BN, WM); false if the choice does not fit the kernel.
inline bool make_plan(const ConvGeom &g, int cus, int R, int BN, int WM, Plan &p) {
    if (R <= 0 || g.OH % R || BN <= 0 || BN % 16 || g.OC % BN || BN > 128 || kWaves % WM) return false;
    p.R = R, p.BN = BN, p.WM = WM, p.WN = kWaves / WM;
    const int cblk = BN / 16;
    if (cblk % p.WN) return false;
    p.TNW = cblk / p.WN;
    if (p.TNW != 1 && p.TNW != 2 && p.TNW != 4) return false;
    p.P = R * g.OW;
    p.nblk = ceil_div_i(p.P, 16);
    const int tmw = ceil_div_i(p.nblk, WM);
    p.TMW = tmw <= 7 ? 7 : 13;
    if (tmw > 13 || p.TMW * p.TNW > 28) return false;   // accumulators: 4 registers per block, at most 112 per lane
    p.Rp = (R - 1) * g.sh + g.kh, p.Wp = (g.OW - 1) * g.sw + g.kw;
    p.patch_px = p.Rp * p.Wp;
    if (p.patch_px >= (1 << 20)) return false;
    p.PW = ceil_div_i(ceil_div_i(p.patch_px, kLoadPx), kWaves);
    p.taps = g.kh * g.kw, p.chunks = g.C / kChunk, p.slices = p.taps * p.chunks;
    // the patch of the next chunk must be on its way kDepth slices before the chunk ends
    const int slots = p.taps - kDepth + 1;
    if (slots < 1) return false;
    p.LP = ceil_div_i(p.PW, slots);
    if (p.LP > 2) return false;
    p.patch_floats = p.PW * kWaves * kLoadFloats;
    p.b_floats = BN * kChunk;
    p.strips_per_img = g.OH / R;
    p.tiles_m = g.N * p.strips_per_img, p.tiles_n = g.OC / BN;
    p.inv_wp = 1.0f / (float)p.Wp;
    p.lds_bytes = lds_total_floats(p) * 4;
    if (p.lds_bytes > kMaxLds) return false;
    // estimate: blocks on the busiest SIMD (wavefronts w and w + 4 share one) against the tile's average, times
    // how evenly the tiles fill the compute units
    int simd[4] = {0, 0, 0, 0};
    for (int w = 0; w < kWaves; ++w) simd[w & 3] += wave_blocks(p, w).cnt * p.TNW;
    int crit = 0;
    for (int s = 0; s < 4; ++s) crit = simd[s] > crit ? simd[s] : crit;
    const long tiles = (long)p.tiles_m * p.tiles_n;
    const long rounds = (tiles + cus - 1) / cus;
    const double useful = (double)p.P / 16.0 * cblk / 4.0;
    p.eff = (float)(useful / crit * (double)tiles / (double)(rounds * cus));
    return true;
}

// The best plan for the layer on `cus` compute units; false if the kernel does not apply.
inline bool plan(const ConvGeom &g, int cus, Plan &best) {
    if (g.C % kChunk || g.OC % 16 || g.M <= 0 || g.kh * g.kw < kDepth) return false;
    bool found = false;
    for (int R = 1; R <= g.OH; ++R) {
        if (g.OH % R) continue;
        for (int BN = 16; BN <= 128 && BN <= g.OC; BN += 16) {
            for (int WM = 1; WM <= kWaves; WM *= 2) {
                Plan p;
                if (!make_plan(g, cus, R, BN, WM, p)) continue;
                // more useful matrix time first; on a tie (within 1 %) the plan with fewer LDS reads per MFMA:
                // more channel blocks per wavefront, then more pixel blocks
                const bool better = !found || p.eff > best.eff * 1.01f ||
                                    (p.eff > best.eff * 0.99f &&
                                     (p.TNW > best.TNW || (p.TNW == best.TNW && p.nblk > best.nblk)));
                if (better) best = p, found = true;
            }
        }
    }
    return found;
}

} // namespace strip
} // namespace swc_hip
