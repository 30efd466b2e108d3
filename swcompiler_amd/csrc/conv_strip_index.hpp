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
// scalar offset into the patch.  The filter's part for the chunk (kh*kw slices
// of BN x 16 floats) sits beside it.  Both are double-buffered: the workgroup
// meets at a barrier once per CHUNK — a barrier per tap left the matrix cores
// of all four SIMDs idle together at every tap boundary (measured: 1300-2200
// cycles per 3300-6400 cycles of MFMA work) — and between barriers its
// wavefronts run free, so the two wavefronts of a SIMD fill each other's waits.
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
    // Order in which the rows of the GEMM view walk the output pixels.  0: raster order (image, row, column).
    // 1: by 2 x 2 windows — row m is pixel (2py + d/2, 2px + d%2) of window m/4 = (image, py, px) in raster order
    // of the windows, d = m%4 — so that every aligned group of four rows is one window of a 2 x 2 / stride 2
    // pooling (even OH and OW only).
    int win = 0;
};

namespace strip {

constexpr int kWaves = 8;
constexpr int kThreads = 64 * kWaves;
constexpr int kChunk = 16;                 // channels per slice
constexpr int kPxFloats = kChunk;          // floats per patch pixel
constexpr int kPxBytes = kChunk * 4;       // 64
constexpr int kLoadFloats = 256;           // one wavefront load: 64 lanes x 16 bytes
constexpr int kLoadPx = kLoadFloats / kPxFloats;   // 16 patch pixels (or filter rows) per load
constexpr int kMaxLds = 160 * 1024;
constexpr int kMaxPW = 8;                  // patch loads per wavefront per chunk the kernel keeps offsets for
constexpr int kMaxFW = 10;                 // the same for the filter part

// How one layer is cut into tiles; filled by plan() on the host, read by the kernel.
struct Plan {
    int R;            // output rows per tile (divides OH)
    int BN;           // output channels per tile (multiple of 16, divides OC)
    int WM, WN;       // wavefront grid: WM x WN = 8, rows split the pixel blocks, columns the channel blocks
    int TMW, TNW;     // pixel / channel blocks per wavefront (the kernel's template arguments)
    int P;            // R * OW
    int nblk;         // ceil(P / 16)
    int Rp, Wp;       // patch rows, columns: (R-1)*sh + kh, (OW-1)*sw + kw
    int patch_px;     // Rp * Wp
    int PW;           // patch loads per wavefront per chunk: ceil(ceil(patch_px / 16) / 8)
    int patch_floats; // floats of one patch buffer: PW * 8 * 256
    int FW;           // filter loads per wavefront per chunk: ceil(taps * BN / 16 / 8)
    int b_floats;     // floats of one filter buffer: taps * BN * 16 (rounded up to whole rounds of loads)
    int tiles_m, tiles_n, strips_per_img;
    int taps, chunks, slices;
    float inv_wp;     // 1.0f / Wp
    int lds_bytes;
    float eff;        // estimated share of the matrix cores' time that is useful work
};

// LDS layout in floats: patch[2], then filter[2]; a filter buffer is [tap][BN rows][16 floats].
SWC_HD int lds_patch(const Plan &p, int buf) { return buf * p.patch_floats; }
SWC_HD int lds_filter(const Plan &p, int buf) { return 2 * p.patch_floats + buf * p.b_floats; }
SWC_HD int lds_total_floats(const Plan &p) { return 2 * p.patch_floats + 2 * p.b_floats; }

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

// ---- filter fragments (A operand): byte offset inside tap 0 of a filter buffer of the lane's four channels (a
// tap adds BN * 64 bytes; BN is a multiple of 16, so the swizzle key of a row does not depend on the tap)
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

// filter load `blk` (sixteen rows 16*blk .. of the buffer's taps*BN rows; row = tap*BN + output channel): byte
// offset of the lane's 16 bytes in the filter for channel chunk 0 (a later chunk adds 64 bytes per chunk as a
// scalar), or kNoByte past the last tap
SWC_HD int filter_lane_byte(const ConvGeom &g, const Plan &p, const TileOrigin &t, int blk, int lane) {
    const int nb = p.BN / kLoadPx;                   // loads per tap
    const int tap = blk / nb, r = (blk - tap * nb) * kLoadPx + (lane >> 2);
    const int chunk = (lane & 3) ^ swz_key(r);
    const bool ok = tap < p.taps && t.n0 + r < g.OC;
    return ok ? ((t.n0 + r) * g.K + tap * g.C + chunk * 4) * 4 : kNoByte;
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
    p.patch_floats = p.PW * kWaves * kLoadFloats;
    p.FW = ceil_div_i(p.taps * BN / kLoadPx, kWaves);
    p.b_floats = p.FW * kWaves * kLoadFloats;
    p.strips_per_img = g.OH / R;
    p.tiles_m = g.N * p.strips_per_img, p.tiles_n = g.OC / BN;
    p.inv_wp = 1.0f / (float)p.Wp;
    p.lds_bytes = lds_total_floats(p) * 4;
    if (p.lds_bytes > kMaxLds || p.PW > kMaxPW || p.FW > kMaxFW) return false;
    // estimate: blocks on the busiest SIMD (wavefronts w and w + 4 share one) against the tile's average, times
    // how evenly the tiles fill the compute units
    int simd[4] = {0, 0, 0, 0};
    for (int w = 0; w < kWaves; ++w) simd[w & 3] += wave_blocks(p, w).cnt * p.TNW;
    int crit = 0;
    for (int s = 0; s < 4; ++s) crit = simd[s] > crit ? simd[s] : crit;
    const long tiles = (long)p.tiles_m * p.tiles_n;
    const long rounds = (tiles + cus - 1) / cus;
    // in matrix-core cycles per SIMD: a block pair costs four MFMAs of 32 cycles per slice; a tile also pays for
    // its first chunk's loads, its stores and its launch slot before and after (about 8000 cycles, measured)
    const double per_block = 128.0 * p.slices, fixed = 8000.0;
    const double useful = (double)p.P / 16.0 * cblk / 4.0 * per_block;
    p.eff = (float)(useful * (double)tiles / ((double)rounds * cus * (crit * per_block + fixed)));
    return true;
}

// The best plan for the layer on `cus` compute units; false if the kernel does not apply.
inline bool plan(const ConvGeom &g, int cus, Plan &best) {
    if (g.C % kChunk || g.OC % 16 || g.M <= 0) return false;
    bool found = false;
    for (int R = 1; R <= g.OH; ++R) {
        if (g.OH % R) continue;
        for (int BN = 16; BN <= 128 && BN <= g.OC; BN += 16) {
            for (int WM = 1; WM <= kWaves; WM *= 2) {
                Plan p;
                if (!make_plan(g, cus, R, BN, WM, p)) continue;
                // A wavefront with one channel block reads a pixel fragment per four MFMAs, all four into the same
                // accumulator; with two or four it reads one per eight or sixteen.  Plans of at least two channel
                // blocks per wavefront come first unless they waste a tenth more of the matrix time; among equals
                // (within 1 %) the wider tile, whose input patch is fetched by fewer workgroups.
                const float score = p.eff * (p.TNW == 1 ? 0.9f : 1.0f);
                const float best_score = found ? best.eff * (best.TNW == 1 ? 0.9f : 1.0f) : 0.f;
                const bool better = !found || score > best_score * 1.01f ||
                                    (score > best_score * 0.99f && (p.BN > best.BN || (p.BN == best.BN && p.TNW > best.TNW)));
                if (better) best = p, found = true;
            }
        }
    }
    return found;
}

} // namespace strip
} // namespace swc_hip
