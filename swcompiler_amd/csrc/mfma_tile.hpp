// fp32 MFMA block-tile core shared by the FC GEMM and the implicit-GEMM conv.
//
// A workgroup of 256 threads (4 wavefronts as 2x2) computes a BM x BN tile of
// C = A*B, BM = 64*TM, BN = 64*TN; each wavefront owns a (32*TM) x (32*TN)
// sub-tile as TM x TN accumulators of v_mfma_f32_32x32x2_f32 (16 VGPRs each).
// K is consumed in slices of BK = 32 staged through LDS, double-buffered, with
// the next slice's global loads issued before the current slice's MFMAs.
//
// Operand layout of v_mfma_f32_32x32x2_f32 (lane l of 64):
//   A[i][kk]: i = l % 32, kk = l / 32        B[kk][j]: j = l % 32, kk = l / 32
//   D[i][j] in VGPR v (0..15): j = l % 32, i = 8*(v/4) + 4*(l/32) + v%4
// The sum over k is order-free, so within a group of 8 k's the half-wave
// h = l/32 takes k = 4h..4h+3: a lane then needs four CONSECUTIVE k's of one
// row of A, which is a single 128-bit LDS read when A is stored k-contiguous.
//
// LDS layouts (floats):
//   k-contiguous operand (A always; B when given as [n][k], i.e. conv filters):
//     rows of BK + 4 — the +4 shifts consecutive rows by 4 banks, so the eight
//     lanes served together by a 128-bit read touch disjoint bank quads.
//   n-contiguous B ([k][n], FC weights): rows of BN + 8 — the two half-waves
//     read rows 4 apart; 4*(BN+8) = 32 (mod 64) puts them on opposite halves
//     of the banks.
#pragma once
#include <hip/hip_runtime.h>

#include "devices/HipDevice.h"

namespace swc_hip {
namespace mfma {

typedef float v16f __attribute__((ext_vector_type(16)));

constexpr int kThreads = 256;
constexpr int BK = 32;
constexpr int kPadK = 4;
constexpr int kLdK = BK + kPadK;   // row length of a k-contiguous tile

template <int TM, int TN, bool B_NT>
struct Tile {
    static constexpr int BM = 64 * TM;
    static constexpr int BN = 64 * TN;
    static constexpr int kLdBn = BN + 8;                       // [k][n] layout of B
    static constexpr int kAFloats = BM * kLdK;
    static constexpr int kBFloats = B_NT ? BN * kLdK : BK * kLdBn;
    static constexpr int kStageFloats = kAFloats + kBFloats;
    static constexpr size_t kLdsBytes = 2u * kStageFloats * sizeof(float);
    // float4 per thread per k-slice
    static constexpr int kAVec = BM * BK / 4 / kThreads;       // = 2*TM
    static constexpr int kBVec = BN * BK / 4 / kThreads;       // = 2*TN
};

// One v_mfma_f32_32x32x2_f32 with the accumulator held in the AGPR half of the
// register file.  With accumulators in ordinary VGPRs every LDS or memory read
// that returns into VGPRs competes with the matrix core's accumulator traffic
// and stalls it (a 128-bit LDS read per four MFMAs costs ~10 % of the MFMA rate
// on MI355X, 3 % with AGPR accumulators); the compiler picks the VGPR form
// whenever registers are plentiful, so the choice is made here.  Written as
// inline assembly, the instruction is opaque to the compiler's hazard
// recogniser: the loop needs nothing (an accumulator is only ever read by the
// next MFMA that accumulates into it, which the hardware interlocks), but the
// first ordinary read of the results must be preceded by acc_settle().
__device__ __forceinline__ void mfma_acc(v16f &acc, float a, float b) {
#if __HIP_DEVICE_COMPILE__
    asm("v_mfma_f32_32x32x2_f32 %0, %1, %2, %0" : "+a"(acc) : "v"(a), "v"(b));
#endif
}

// Wait states between the last MFMA and the first read of its result (a
// 16-pass MFMA needs 18; the data dependences on acc keep this after the MFMAs).
template <int TM, int TN>
__device__ __forceinline__ void acc_settle(v16f (&acc)[TM][TN]) {
#if __HIP_DEVICE_COMPILE__
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j) asm volatile("" : "+a"(acc[i][j]));   // every accumulator's chain ends before the nops
    asm volatile("s_nop 7\n\ts_nop 7\n\ts_nop 7" : "+a"(acc[TM - 1][TN - 1]));
#endif
}

// Fragments of one group of 8 k's: a lane's four consecutive k's of each of its
// TM rows of A and TN columns of B.
template <int TM, int TN>
struct Frag {
    float a[TM][4];
    float b[TN][4];
};

template <int TM, int TN, bool B_NT>
__device__ __forceinline__ void load_frag(Frag<TM, TN> &f, const float *__restrict__ As, const float *__restrict__ Bs,
                                          int kb, int wave_m, int wave_n, int l32, int h) {
    using T = Tile<TM, TN, B_NT>;
#pragma unroll
    for (int tm = 0; tm < TM; ++tm) {
        const float4 v = *reinterpret_cast<const float4 *>(&As[(wave_m * 32 * TM + tm * 32 + l32) * kLdK + kb + 4 * h]);
        f.a[tm][0] = v.x; f.a[tm][1] = v.y; f.a[tm][2] = v.z; f.a[tm][3] = v.w;
    }
#pragma unroll
    for (int tn = 0; tn < TN; ++tn) {
        if (B_NT) {
            const float4 v =
                *reinterpret_cast<const float4 *>(&Bs[(wave_n * 32 * TN + tn * 32 + l32) * kLdK + kb + 4 * h]);
            f.b[tn][0] = v.x; f.b[tn][1] = v.y; f.b[tn][2] = v.z; f.b[tn][3] = v.w;
        } else {
#pragma unroll
            for (int s = 0; s < 4; ++s)
                f.b[tn][s] = Bs[(kb + 4 * h + s) * T::kLdBn + wave_n * 32 * TN + tn * 32 + l32];
        }
    }
}

// One k-slice of MFMAs for this wavefront.  As/Bs point at the current stage.
// The fragments of group g+1 are read from LDS before the MFMAs of group g are
// issued, so LDS latency hides behind 16*TM*TN/4 matrix instructions.
template <int TM, int TN, bool B_NT>
__device__ __forceinline__ void compute_slice(const float *__restrict__ As, const float *__restrict__ Bs,
                                              v16f (&acc)[TM][TN], int wave_m, int wave_n, int lane) {
    const int l32 = lane & 31;
    const int h = lane >> 5;
    Frag<TM, TN> frag[2];
    load_frag<TM, TN, B_NT>(frag[0], As, Bs, 0, wave_m, wave_n, l32, h);
#pragma unroll
    for (int g = 0; g < BK / 8; ++g) {
        if (g + 1 < BK / 8) load_frag<TM, TN, B_NT>(frag[(g + 1) & 1], As, Bs, (g + 1) * 8, wave_m, wave_n, l32, h);
        const Frag<TM, TN> &f = frag[g & 1];
#pragma unroll
        for (int s = 0; s < 4; ++s)
#pragma unroll
            for (int tm = 0; tm < TM; ++tm)
#pragma unroll
                for (int tn = 0; tn < TN; ++tn)
                    acc[tm][tn] = __builtin_amdgcn_mfma_f32_32x32x2f32(f.a[tm][s], f.b[tn][s], acc[tm][tn], 0, 0, 0);
    }
}

// Per-column epilogue constants: out = f(acc + bias[col]) with optional
// inference batchnorm, an optional second summand of the output's shape (the
// other branch of a residual block; read by the tile kernels of this header and
// by the convolution's own kernels) and optional ReLU, in that order.
struct Epilogue {
    const float *bias;      // may be null
    const float *bn_mean;   // null: no batchnorm
    const float *bn_var;
    const float *bn_scale;
    const float *bn_bias;
    float eps;
    int relu;
    const float *residual = nullptr;   // [M, ldc] like the output, or null; may be the output itself
};

// Writes this wavefront's accumulators to C (row-major, leading dimension ldc).
// One store instruction covers two rows of 32 consecutive floats (two full
// 128-byte lines).  GUARD = false is the path of a sub-tile that lies wholly
// inside the matrix: no per-row control flow, so the 16*TM*TN stores issue back
// to back.  (On this target stores and loads share one outstanding-operation
// counter; a branch per row makes the compiler wait for that counter — i.e. for
// the previous store to be acknowledged — before every store.)  The guarded
// path first waits for the per-column parameters explicitly, after which its
// row blocks have no load to wait for either.
template <int TM, int TN, bool GUARD, bool RES>
__device__ __forceinline__ void store_tile_impl(const v16f (&acc)[TM][TN], float *__restrict__ C, size_t ldc, int M,
                                                int N, int row0, int col0, int lane, const Epilogue &ep) {
    const int l32 = lane & 31;
    const int h = lane >> 5;
    const bool bn = ep.bn_mean != nullptr;
    float bias[TN], mean[TN], slope[TN], beta[TN];
#pragma unroll
    for (int tn = 0; tn < TN; ++tn) {
        const int col = col0 + tn * 32 + l32;
        const bool ok = !GUARD || col < N;
        bias[tn] = (ep.bias && ok) ? ep.bias[col] : 0.f;
        // batchnorm folded to one fp32 multiply-add per element: the slope
        // scale*(var+eps)^-1/2 is formed in double and rounded once; the result is
        // within 2 ulp of the reference's all-double evaluation
        mean[tn] = 0.f, slope[tn] = 1.f, beta[tn] = 0.f;
        if (bn && ok) {
            mean[tn] = ep.bn_mean[col];
            const float ve = ep.bn_var[col] + ep.eps;
            slope[tn] = (float)((double)ep.bn_scale[col] / sqrt((double)ve));
            beta[tn] = ep.bn_bias[col];
        }
    }
#if __HIP_DEVICE_COMPILE__
    if (GUARD) __builtin_amdgcn_s_waitcnt(0x0f70);   // vmcnt(0): the parameter loads above are complete
#endif
#pragma unroll
    for (int tn = 0; tn < TN; ++tn) {
        const int col = col0 + tn * 32 + l32;
        if (GUARD && col >= N) continue;
        float *__restrict__ p = C + (size_t)(row0 + 4 * h) * ldc + col;
        const float *res = RES ? ep.residual + (size_t)(row0 + 4 * h) * ldc + col : nullptr;
#pragma unroll
        for (int tm = 0; tm < TM; ++tm) {
            float add[16];   // the second summand of these 16 rows, all loads issued before the first store
            if (RES) {
#pragma unroll
                for (int v = 0; v < 16; ++v) {
                    const int r = tm * 32 + 8 * (v / 4) + (v % 4);   // row relative to row0 + 4*h
                    add[v] = (GUARD && row0 + 4 * h + r >= M) ? 0.f : res[(size_t)r * ldc];
                }
            }
#pragma unroll
            for (int v = 0; v < 16; ++v) {
                const int r = tm * 32 + 8 * (v / 4) + (v % 4);
                if (GUARD && row0 + 4 * h + r >= M) continue;
                float x = acc[tm][tn][v] + bias[tn];
                if (bn) x = fmaf(x - mean[tn], slope[tn], beta[tn]);
                if (RES) x += add[v];
                if (ep.relu) x = (x > 0.f) ? x : 0.f;
                p[(size_t)r * ldc] = x;
            }
        }
    }
}

template <int TM, int TN>
__device__ __forceinline__ void store_tile(const v16f (&acc)[TM][TN], float *__restrict__ C, size_t ldc, int M, int N,
                                           int row0, int col0, int lane, const Epilogue &ep) {
    const bool inside = row0 + 32 * TM <= M && col0 + 32 * TN <= N;   // all four choices are wavefront-uniform
    if (ep.residual) {
        if (inside) store_tile_impl<TM, TN, false, true>(acc, C, ldc, M, N, row0, col0, lane, ep);
        else store_tile_impl<TM, TN, true, true>(acc, C, ldc, M, N, row0, col0, lane, ep);
    } else {
        if (inside) store_tile_impl<TM, TN, false, false>(acc, C, ldc, M, N, row0, col0, lane, ep);
        else store_tile_impl<TM, TN, true, false>(acc, C, ldc, M, N, row0, col0, lane, ep);
    }
}

// Workgroup id -> tile coordinates.  Workgroups are dealt round-robin to the 8
// XCDs, each with its own L2; ids that land on one XCD are renumbered to be
// consecutive, and consecutive ids walk the tile grid in column strips 8 tiles
// tall, so the tiles resident on one XCD at a time share A rows and B columns.
__device__ __forceinline__ void tile_coords(int tiles_m, int tiles_n, int &tile_m, int &tile_n) {
    const int total = tiles_m * tiles_n;
    int pid = blockIdx.x;
    constexpr int kXcd = swc::devices::HipDevice::xcds;
    if (total % kXcd == 0) pid = (pid % kXcd) * (total / kXcd) + pid / kXcd;
    constexpr int kGroup = 8;
    const int per_group = kGroup * tiles_n;
    const int group = pid / per_group;
    const int first_m = group * kGroup;
    const int rows = (tiles_m - first_m < kGroup) ? (tiles_m - first_m) : kGroup;
    const int in_group = pid - group * per_group;
    tile_m = first_m + in_group % rows;
    tile_n = in_group / rows;
}

} // namespace mfma
} // namespace swc_hip
