// matrixMatrixMul_f (kernels.h:41-56) and the un-lowered MatrixMatrixFCBias
// (GEMM + bias + optional ReLU in the epilogue) on fp32 MFMA.
//
//   gemm_tiled   C[M,N] = A[M,K]*B[K,N], 64*TM x 64*TN workgroup tiles,
//                K slices of 32 through double-buffered LDS (mfma_tile.hpp).
//   gemm_skinny  N <= 16 (classifier heads): HBM-bound on A.  A workgroup owns
//                16 rows, its wavefronts split K, each feeds
//                v_mfma_f32_16x16x4_f32 straight from global memory (B is a few
//                KB and stays in cache) and the partial 16x16 tiles are summed
//                through LDS.
#include "common.hpp"
#include "mfma_dma.hpp"
#include "mfma_tile.hpp"

#include <cstdlib>
#include <cstring>

using namespace swc_hip;
using namespace swc_hip::mfma;

namespace {

// ---------------------------------------------------------------- tiled GEMM
// VEC: A and B rows may be read with aligned 128-bit loads (lda, ldb, K, N
// multiples of 4 and 16-byte aligned bases).  Otherwise 32-bit loads.
template <int TM, int TN, bool VEC>
__global__ __launch_bounds__(kThreads) void gemm_tiled(const float *__restrict__ A, const float *__restrict__ B,
                                                       float *__restrict__ C, int M, int N, int K, size_t lda,
                                                       size_t ldb, size_t ldc, Epilogue ep) {
    using T = Tile<TM, TN, false>;
    extern __shared__ __align__(16) float lds[];
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = tid >> 6;
    const int wave_m = wave >> 1, wave_n = wave & 1;

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

    constexpr int kAScalar = T::kAVec * 4, kBScalar = T::kBVec * 4;
    float4 ra[T::kAVec], rb[T::kBVec];
    float sa[VEC ? 1 : kAScalar], sb[VEC ? 1 : kBScalar];

    // guard == false: the whole slice lies inside A and B (interior tile, full
    // k slice), loads are unconditional and the compiler emits no branches.
    auto load_global = [&](int k0, bool guard) {
        if (VEC) {
#pragma unroll
            for (int i = 0; i < T::kAVec; ++i) {   // A: 8 threads per row of 32 k
                const int row = m0 + (tid >> 3) + 32 * i;
                const int k = k0 + (tid & 7) * 4;
                ra[i] = (!guard || (row < M && k < K)) ? *reinterpret_cast<const float4 *>(A + (size_t)row * lda + k)
                                                       : make_float4(0.f, 0.f, 0.f, 0.f);
            }
#pragma unroll
            for (int i = 0; i < T::kBVec; ++i) {   // B: BN/4 threads per k row
                constexpr int kPerRow = T::BN / 4;
                const int e = tid + kThreads * i;
                const int k = k0 + e / kPerRow;
                const int col = n0 + (e % kPerRow) * 4;
                rb[i] = (!guard || (k < K && col < N)) ? *reinterpret_cast<const float4 *>(B + (size_t)k * ldb + col)
                                                       : make_float4(0.f, 0.f, 0.f, 0.f);
            }
        } else {
#pragma unroll
            for (int i = 0; i < kAScalar; ++i) {
                const int e = tid + kThreads * i;
                const int row = m0 + e / BK, k = k0 + e % BK;
                sa[i] = (row < M && k < K) ? A[(size_t)row * lda + k] : 0.f;
            }
#pragma unroll
            for (int i = 0; i < kBScalar; ++i) {
                const int e = tid + kThreads * i;
                const int k = k0 + e / T::BN, col = n0 + e % T::BN;
                sb[i] = (k < K && col < N) ? B[(size_t)k * ldb + col] : 0.f;
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
            for (int i = 0; i < T::kBVec; ++i) {
                constexpr int kPerRow = T::BN / 4;
                const int e = tid + kThreads * i;
                *reinterpret_cast<float4 *>(&Bs[(e / kPerRow) * T::kLdBn + (e % kPerRow) * 4]) = rb[i];
            }
        } else {
#pragma unroll
            for (int i = 0; i < kAScalar; ++i) {
                const int e = tid + kThreads * i;
                As[(e / BK) * kLdK + e % BK] = sa[i];
            }
#pragma unroll
            for (int i = 0; i < kBScalar; ++i) {
                const int e = tid + kThreads * i;
                Bs[(e / T::BN) * T::kLdBn + e % T::BN] = sb[i];
            }
        }
    };

    const int nk = (K + BK - 1) / BK;
    const bool interior = VEC && m0 + T::BM <= M && n0 + T::BN <= N;   // workgroup-uniform
    const int full = interior ? K / BK : 0;                            // slices [0, full) need no guard
    if (full > 0) load_global(0, false);
    else load_global(0, true);
    store_lds(0);
    __syncthreads();
    for (int kt = 0; kt < nk; ++kt) {
        const int cur = kt & 1;
        if (kt + 1 < full) load_global((kt + 1) * BK, false);
        else if (kt + 1 < nk) load_global((kt + 1) * BK, true);
        const float *As = lds + cur * T::kStageFloats;
        compute_slice<TM, TN, false>(As, As + T::kAFloats, acc, wave_m, wave_n, lane);
        if (kt + 1 < nk) store_lds(cur ^ 1);
        __syncthreads();
    }
    store_tile<TM, TN>(acc, C, ldc, M, N, m0 + wave_m * 32 * TM, n0 + wave_n * 32 * TN, lane, ep);
}

// ------------------------------------------------- tiled GEMM, direct-to-LDS
// Same tiles, operands streamed by buffer_load ... lds into a STAGES-deep ring
// (mfma_dma.hpp).  Needs 16-byte-aligned rows (lda, ldb, K, N multiples of 4)
// and operands below 2 GiB (32-bit buffer offsets); gemm_tiled covers the rest.
template <int TM, int TN, int STAGES, bool MID = false>
__global__ __launch_bounds__(kThreads) void gemm_dma(const float *__restrict__ A, const float *__restrict__ B,
                                                     float *__restrict__ C, int M, int N, int K, int lda, int ldb,
                                                     size_t ldc, unsigned a_bytes, unsigned b_bytes, Epilogue ep) {
#if __HIP_DEVICE_COMPILE__   // the host pass only needs the launch stub; buffer-resource builtins are device-only
    using T = DmaTile<TM, TN, false, STAGES>;
    extern __shared__ __align__(16) float lds[];
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = tid >> 6;

    int tile_m, tile_n;
    tile_coords((M + T::BM - 1) / T::BM, (N + T::BN - 1) / T::BN, tile_m, tile_n);
    const int m0 = tile_m * T::BM, n0 = tile_n * T::BN;

    const __amdgpu_buffer_rsrc_t rsrc_a = make_rsrc(A, a_bytes);
    const __amdgpu_buffer_rsrc_t rsrc_b = make_rsrc(B, b_bytes);

    // byte offsets of this lane's 16 bytes in slice 0, per load
    const int a_k = kc_chunk(lane) * 4;           // k of the lane's chunk inside a slice
    int a_base[T::kALoads], b_base[T::kBLoads], b_k[T::kBLoads];
#pragma unroll
    for (int j = 0; j < T::kALoads; ++j) {
        const int row = m0 + (4 * j + wave) * 8 + kc_row_in_load(lane);
        a_base[j] = row < M ? (row * lda + a_k) * 4 : kOutOfRange;
    }
#pragma unroll
    for (int j = 0; j < T::kBLoads; ++j) {
        const int flat = (4 * j + wave) * 256 + lane * 4;       // float index inside the [32][BN] tile
        const int krow = flat / T::BN;
        const int pos = (flat % T::BN) >> 2;                    // chunk position in the LDS row
        const int col = n0 + ((pos ^ (((krow >> 2) & 1) << 3)) << 2);
        b_k[j] = krow;
        b_base[j] = col < N ? (krow * ldb + col) * 4 : kOutOfRange;
    }
    int va[T::kALoads], vb[T::kBLoads];
    auto offsets = [&](int kt) {
        const int k0 = kt * BK;
#pragma unroll
        for (int j = 0; j < T::kALoads; ++j)
            va[j] = (a_base[j] != kOutOfRange && k0 + a_k < K) ? a_base[j] + k0 * 4 : kOutOfRange;
#pragma unroll
        for (int j = 0; j < T::kBLoads; ++j)
            vb[j] = (b_base[j] != kOutOfRange && k0 + b_k[j] < K) ? b_base[j] + k0 * ldb * 4 : kOutOfRange;
    };

    v16f acc[TM][TN];
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j)
#pragma unroll
            for (int v = 0; v < 16; ++v) acc[i][j][v] = 0.f;

    // prologue: slices 0 .. STAGES-2 in flight
#pragma unroll
    for (int s = 0; s < STAGES - 1; ++s) {
        offsets(s);
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
    if constexpr (MID) {
        ring_sync<(STAGES - 2) * T::kLoads>();   // slice 0 has landed
        Frag<TM, TN> frag[2];
        load_frag_swz<TM, TN, false>(frag[0], lds, lds + T::kAFloats, 0, wave >> 1, wave & 1, lane & 31, lane >> 5);
        for (int kt = 0; kt < nk; ++kt) {
            offsets(kt + STAGES - 1);
            const int nx_stage = rd_stage + 1 == STAGES ? 0 : rd_stage + 1;
            dma_step_mid<TM, TN, false, STAGES>(lds + wr_stage * T::kStageFloats, lds + rd_stage * T::kStageFloats,
                                                lds + nx_stage * T::kStageFloats, rsrc_a, rsrc_b, va, vb, acc, frag,
                                                wave, lane);
            rd_stage = nx_stage;
            wr_stage = wr_stage + 1 == STAGES ? 0 : wr_stage + 1;
        }
    } else {
        for (int kt = 0; kt < nk; ++kt) {
            ring_sync<(STAGES - 2) * T::kLoads>();
            offsets(kt + STAGES - 1);
            dma_step<TM, TN, false, STAGES>(lds + wr_stage * T::kStageFloats, lds + rd_stage * T::kStageFloats, rsrc_a,
                                            rsrc_b, va, vb, acc, wave, lane);
            rd_stage = rd_stage + 1 == STAGES ? 0 : rd_stage + 1;
            wr_stage = wr_stage + 1 == STAGES ? 0 : wr_stage + 1;
        }
    }
    wait_vmcnt<0>();   // the trailing dummy loads still target this workgroup's LDS
    acc_settle(acc);
    store_tile<TM, TN>(acc, C, ldc, M, N, m0 + (wave >> 1) * 32 * TM, n0 + (wave & 1) * 32 * TN, lane, ep);
#endif
}

// -------------------------------------- tiled GEMM, column-interleaved B tile
// The [k][n] layout of B makes the fragment of the kernel above (four
// consecutive k of one column per lane) sixteen 32-bit LDS reads per group of 8
// k, and the matrix core stalls on every LDS instruction's register write-back
// far more than on the bytes it carries.  Here the columns are dealt to the
// MFMA column blocks round-robin instead: a wavefront owns 32*TN consecutive
// columns, and lane j of column block t computes column TN*j + t of them.  A
// lane's operands for the TN blocks at one k are then TN CONSECUTIVE floats of
// a B row — one LDS read of 32*TN bits, no swizzle needed (32 lanes read 128*TN
// contiguous bytes) — and in the epilogue the lane holds TN consecutive
// columns of each of its rows: one 32*TN-bit store.
// Wavefronts are arranged WM x (4/WM); the workgroup tile is
// (32*TM*WM) x (32*TN*4/WM); the A tile keeps the swizzled k-contiguous layout.
template <int TM, int TN, int WM, int STAGES, int NW = 4>
struct Dma2Tile {
    static constexpr int kWaves = NW;          // 4, or 8 (two wavefronts per SIMD from one workgroup)
    static constexpr int kThreadsWg = 64 * NW;
    static constexpr int WN = NW / WM;
    static constexpr int BM = 32 * TM * WM;
    static constexpr int BN = 32 * TN * WN;
    static constexpr int kAFloats = BM * BK;
    static constexpr int kBFloats = BN * BK;
    static constexpr int kStageFloats = kAFloats + kBFloats;
    static constexpr size_t kLdsBytes = (size_t)STAGES * kStageFloats * sizeof(float);
    static constexpr int kALoads = BM / 8 / NW;   // 1-KiB buffer loads per wavefront per slice
    static constexpr int kBLoads = BN / 8 / NW;
    static constexpr int kLoads = kALoads + kBLoads;
    static constexpr int kPieces = TM + 4;    // LDS reads per group of 8 k: TM of A, one per k of B
    static_assert(NW == 4 || NW == 8, "");
    static_assert(WM == 1 || WM == 2 || WM == 4 || WM == 8, "");
    static_assert(kALoads >= 1 && kBLoads >= 1 && kALoads * 8 * NW == BM && kBLoads * 8 * NW == BN, "");
    static_assert(TN == 2 || TN == 4, "a lane reads TN consecutive floats");
    static_assert(STAGES >= 2 && (STAGES - 1) * kLoads < 64, "pending loads must fit the vmcnt field");
};

#if __HIP_DEVICE_COMPILE__
template <int TM, int TN>
struct Frag2 {
    float a[TM][4];
    float b[4][TN];   // [k step][column block]
};

template <int TM, int TN, int BN>
__device__ __forceinline__ void load_frag2_piece(Frag2<TM, TN> &f, const float *__restrict__ As,
                                                 const float *__restrict__ Bs, int g, int piece, int row0, int col0,
                                                 int l32, int h) {
    if (piece < TM) {
        const int row = row0 + piece * 32 + l32;
        const float4 v = *reinterpret_cast<const float4 *>(&As[row * BK + (((2 * g + h) ^ (l32 & 7)) << 2)]);
        f.a[piece][0] = v.x; f.a[piece][1] = v.y; f.a[piece][2] = v.z; f.a[piece][3] = v.w;
    } else {
        const int s = piece - TM;
        const float *src = &Bs[(g * 8 + 4 * h + s) * BN + col0 + TN * l32];
        if (TN == 4) {
            const float4 v = *reinterpret_cast<const float4 *>(src);
            f.b[s][0] = v.x; f.b[s][1] = v.y; f.b[s][2] = v.z; f.b[s][3] = v.w;
        } else {
            const float2 v = *reinterpret_cast<const float2 *>(src);
            f.b[s][0] = v.x; f.b[s][1] = v.y;
        }
    }
}
#endif

#if __HIP_DEVICE_COMPILE__
// Epilogue of the column-interleaved kernels: lane (l32, h) holds, for each of
// its rows, the TN consecutive columns cbase + TN*l32 .. +TN-1 (cbase = first
// column of the wavefront), written with one 32*TN-bit store per row.
template <int TM, int TN>
__device__ __forceinline__ void store_tile2(const v16f (&acc)[TM][TN], float *__restrict__ C, size_t ldc, int M, int N,
                                            int rbase, int cbase, int lane, const Epilogue &ep) {
    const int l32 = lane & 31, h = lane >> 5;
    const int col = cbase + TN * l32;
    if (col >= N) return;   // N and col are multiples of TN: a lane's columns are all inside or all outside
    float bias[TN], mean[TN], slope[TN], beta[TN];
    const bool bn = ep.bn_mean != nullptr;
#pragma unroll
    for (int t = 0; t < TN; ++t) {
        bias[t] = ep.bias ? ep.bias[col + t] : 0.f;
        mean[t] = 0.f, slope[t] = 1.f, beta[t] = 0.f;
        if (bn) {
            mean[t] = ep.bn_mean[col + t];
            slope[t] = (float)((double)ep.bn_scale[col + t] / sqrt((double)(ep.bn_var[col + t] + ep.eps)));
            beta[t] = ep.bn_bias[col + t];
        }
    }
    __builtin_amdgcn_s_waitcnt(0x0f70);   // vmcnt(0): parameters are here; the stores below wait for nothing
    const int r0 = rbase + 4 * h;
    float *__restrict__ p = C + (size_t)r0 * ldc + col;
    const bool full = rbase + 32 * TM <= M;
#pragma unroll
    for (int tm = 0; tm < TM; ++tm)
#pragma unroll
        for (int v = 0; v < 16; ++v) {
            const int r = tm * 32 + 8 * (v / 4) + (v % 4);
            float x[TN];
#pragma unroll
            for (int t = 0; t < TN; ++t) {
                x[t] = acc[tm][t][v] + bias[t];
                if (bn) x[t] = fmaf(x[t] - mean[t], slope[t], beta[t]);
                if (ep.relu) x[t] = (x[t] > 0.f) ? x[t] : 0.f;
            }
            if (full || r0 + r < M) {
                if (TN == 4) *reinterpret_cast<float4 *>(p + (size_t)r * ldc) = make_float4(x[0], x[1], x[2], x[3]);
                else *reinterpret_cast<float2 *>(p + (size_t)r * ldc) = make_float2(x[0], x[1]);
            }
        }
}
#endif

// MID: ring hand-over after the first MFMA group of a slice (needs STAGES >= 3)
// instead of at its top; see dma_step_mid in mfma_dma.hpp.
template <int TM, int TN, int WM, int STAGES, bool MID, int NW>
__global__ __launch_bounds__(64 * NW) void gemm_dma2(const float *__restrict__ A, const float *__restrict__ B,
                                                      float *__restrict__ C, int M, int N, int K, int lda, int ldb,
                                                      size_t ldc, unsigned a_bytes, unsigned b_bytes, Epilogue ep) {
#if __HIP_DEVICE_COMPILE__
    using T = Dma2Tile<TM, TN, WM, STAGES, NW>;
    static_assert(!MID || STAGES >= 3, "");
    extern __shared__ __align__(16) float lds[];
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);   // scalar: LDS destinations of the loads stay in SGPRs
    const int l32 = lane & 31, h = lane >> 5;
    const int row0 = (wave / T::WN) * 32 * TM;   // of this wavefront inside the workgroup tile
    const int col0 = (wave % T::WN) * 32 * TN;

    int tile_m, tile_n;
    tile_coords((M + T::BM - 1) / T::BM, (N + T::BN - 1) / T::BN, tile_m, tile_n);
    const int m0 = tile_m * T::BM, n0 = tile_n * T::BN;

    // A wavefront's loads fill consecutive 1-KiB blocks of the tile, so up to four
    // of them share one LDS base (M0) and differ only in the instruction's
    // immediate offset — rewriting M0 before every load costs MFMA issue slots.
    // The immediate is also added to the memory address; the per-lane offsets
    // have it subtracted, and the descriptors start kImmSpan bytes below the
    // matrices so that no offset goes negative.
    constexpr int kImmSpan = 4096;
    const __amdgpu_buffer_rsrc_t rsrc_a = make_rsrc(reinterpret_cast<const char *>(A) - kImmSpan, a_bytes + kImmSpan);
    const __amdgpu_buffer_rsrc_t rsrc_b = make_rsrc(reinterpret_cast<const char *>(B) - kImmSpan, b_bytes + kImmSpan);

    // Per-lane byte offsets of slice 0 (out-of-range for rows/columns outside the
    // matrix); a slice adds a scalar: k0*4 bytes for A, k0*ldb*4 for B.  Only a
    // slice that reaches past K needs the per-lane k check.
    const int a_k = kc_chunk(lane) * 4;
    int a_base[T::kALoads], b_base[T::kBLoads], b_k[T::kBLoads];
#pragma unroll
    for (int j = 0; j < T::kALoads; ++j) {
        const int row = m0 + (wave * T::kALoads + j) * 8 + kc_row_in_load(lane);
        a_base[j] = row < M ? (row * lda + a_k) * 4 + kImmSpan - (j & 3) * 1024 : kOutOfRange;
    }
#pragma unroll
    for (int j = 0; j < T::kBLoads; ++j) {
        const int flat = (wave * T::kBLoads + j) * 256 + lane * 4;   // float index inside the [32][BN] tile
        const int col = n0 + flat % T::BN;
        b_k[j] = flat / T::BN;
        b_base[j] = col < N ? (b_k[j] * ldb + col) * 4 + kImmSpan - (j & 3) * 1024 : kOutOfRange;
    }
    int k0 = 0;   // first k of the slice whose loads are being issued
    auto issue = [&](float *__restrict__ wr, int j) {
        const bool whole = k0 + BK <= K;   // scalar
        if (j < T::kALoads) {
            const int v = whole ? a_base[j] : ((a_base[j] != kOutOfRange && k0 + a_k < K) ? a_base[j] : kOutOfRange);
            lds_void_t *dst = (lds_void_t *)(wr + (wave * T::kALoads + (j & ~3)) * 256);
            switch (j & 3) {   // the immediate must be a compile-time constant
            case 0: __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrc_a, dst, 16, v, k0 * 4, 0, 0); break;
            case 1: __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrc_a, dst, 16, v, k0 * 4, 1024, 0); break;
            case 2: __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrc_a, dst, 16, v, k0 * 4, 2048, 0); break;
            default: __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrc_a, dst, 16, v, k0 * 4, 3072, 0); break;
            }
        } else {
            const int jb = j - T::kALoads;
            const int v = whole ? b_base[jb] : ((b_base[jb] != kOutOfRange && k0 + b_k[jb] < K) ? b_base[jb] : kOutOfRange);
            lds_void_t *dst = (lds_void_t *)(wr + T::kAFloats + (wave * T::kBLoads + (jb & ~3)) * 256);
            switch (jb & 3) {
            case 0: __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrc_b, dst, 16, v, k0 * ldb * 4, 0, 0); break;
            case 1: __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrc_b, dst, 16, v, k0 * ldb * 4, 1024, 0); break;
            case 2: __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrc_b, dst, 16, v, k0 * ldb * 4, 2048, 0); break;
            default: __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrc_b, dst, 16, v, k0 * ldb * 4, 3072, 0); break;
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
#pragma unroll
        for (int j = 0; j < T::kLoads; ++j) issue(lds + s * T::kStageFloats, j);
        k0 += BK;
    }

    constexpr int kGroups = BK / 8;
    constexpr int kPerGroup = 4 * TM * TN;
    // Loads of a later slice go into the second halves of the MFMA groups: with the hand-over in
    // mid-slice, spread over groups 1..3; with the barrier at the top of the slice (where the stage
    // being filled is needed again one slice later) as early as they fit, from group 0 on.
    constexpr int kFirstLoadGroup = MID ? 1 : 0;
    constexpr int kSpread = (T::kLoads + kGroups - kFirstLoadGroup - 1) / (kGroups - kFirstLoadGroup);
    constexpr int kLoadsPerGroup = MID ? kSpread : (T::kLoads < kPerGroup / 2 ? T::kLoads : kPerGroup / 2);
    static_assert(kLoadsPerGroup <= kPerGroup / 2, "one load per MFMA slot at most");
    static_assert(kLoadsPerGroup * (kGroups - kFirstLoadGroup) >= T::kLoads, "every load has a slot");
    Frag2<TM, TN> frag[2];
    if constexpr (MID) {
        ring_sync<(STAGES - 2) * T::kLoads>();   // slice 0 has landed
#pragma unroll
        for (int p = 0; p < T::kPieces; ++p)
            load_frag2_piece<TM, TN, T::BN>(frag[0], lds, lds + T::kAFloats, 0, p, row0, col0, l32, h);
    }
    const int nk = (K + BK - 1) / BK;
    int rd_stage = 0, wr_stage = STAGES - 1;
    for (int kt = 0; kt < nk; ++kt) {
        const int nx_stage = rd_stage + 1 == STAGES ? 0 : rd_stage + 1;
        float *__restrict__ wr = lds + wr_stage * T::kStageFloats;
        const float *__restrict__ rd = lds + rd_stage * T::kStageFloats;
        const float *__restrict__ nx = lds + nx_stage * T::kStageFloats;
        if constexpr (!MID) {
            ring_sync<(STAGES - 2) * T::kLoads>();
#pragma unroll
            for (int p = 0; p < T::kPieces; ++p)
                load_frag2_piece<TM, TN, T::BN>(frag[0], rd, rd + T::kAFloats, 0, p, row0, col0, l32, h);
            __builtin_amdgcn_sched_barrier(0);
        }
        // Every MFMA is followed by at most one LDS read of the next group's
        // fragments (first half of a group) or one buffer load of a later slice
        // (second half); the fence after each pins that order, so the other work
        // issues in the shadow of a 64-cycle MFMA.
#pragma unroll
        for (int g = 0; g < kGroups; ++g) {
            if constexpr (MID) {
                if (g == 1) {
                    ring_sync<(STAGES - 3) * T::kLoads>();
                    __builtin_amdgcn_sched_barrier(0);
                }
            }
            const Frag2<TM, TN> &f = frag[g & 1];
            Frag2<TM, TN> &fn = frag[(g + 1) & 1];
            const bool last = g + 1 == kGroups;
            const float *__restrict__ src = last ? nx : rd;
            const int gn = last ? 0 : g + 1;
#pragma unroll
            for (int s = 0; s < 4; ++s)
#pragma unroll
                for (int tm = 0; tm < TM; ++tm)
#pragma unroll
                    for (int tn = 0; tn < TN; ++tn) {
                        const int i = (s * TM + tm) * TN + tn;
                        mfma_acc(acc[tm][tn], f.a[tm][s], f.b[s][tn]);
                        if (MID || !last) {
#pragma unroll
                            for (int p = 0; p < T::kPieces; ++p)
                                if (p * (kPerGroup / 2) / T::kPieces == i)
                                    load_frag2_piece<TM, TN, T::BN>(fn, src, src + T::kAFloats, gn, p, row0, col0, l32,
                                                                    h);
                        }
                        if (g >= kFirstLoadGroup) {
#pragma unroll
                            for (int q = 0; q < kLoadsPerGroup; ++q) {
                                const int j = (g - kFirstLoadGroup) * kLoadsPerGroup + q;
                                if (j < T::kLoads && kPerGroup / 2 + q * (kPerGroup / 2) / kLoadsPerGroup == i)
                                    issue(wr, j);
                            }
                        }
                        __builtin_amdgcn_sched_barrier(0);
                    }
        }
        k0 += BK;
        rd_stage = nx_stage;
        wr_stage = wr_stage + 1 == STAGES ? 0 : wr_stage + 1;
    }
    wait_vmcnt<0>();   // the trailing dummy loads still target this workgroup's LDS
    acc_settle(acc);
    store_tile2<TM, TN>(acc, C, ldc, M, N, m0 + row0, n0 + col0, lane, ep);
#endif
}

// --------------------------------------------------------------- skinny GEMM
typedef float v4f __attribute__((ext_vector_type(4)));
constexpr int kSkinnyMaxWaves = 16;
constexpr int kSkinnyUnroll = 4;

// v_mfma_f32_16x16x4_f32: A[i][kk] i = l%16, kk = l/16; B[kk][j] j = l%16, kk = l/16;
// D[i][j] in VGPR v: j = l%16, i = 4*(l/16) + v.
// K is walked in groups of 32: quarter-wave q = l/16 takes k = 8q..8q+7, so a
// lane reads 8 consecutive floats of one A row (two 128-bit loads when VEC).
template <bool VEC>
__global__ __launch_bounds__(64 * kSkinnyMaxWaves) void gemm_skinny(const float *__restrict__ A,
                                                                    const float *__restrict__ B,
                                                                    float *__restrict__ C, int M, int N, int K,
                                                                    size_t lda, size_t ldb, size_t ldc, Epilogue ep) {
    __shared__ float part[kSkinnyMaxWaves][16][17];
    const int tid = threadIdx.x;
    const int lane = tid & 63, wave = tid >> 6, waves = blockDim.x >> 6;
    const int i = lane & 15, q = lane >> 4;
    const int row = blockIdx.x * 16 + i;
    const bool row_ok = row < M;
    const bool col_ok = i < N;   // as B operand, lane's column j = i
    const float *arow = A + (size_t)(row_ok ? row : 0) * lda;
    v4f acc = {0.f, 0.f, 0.f, 0.f};
    // kSkinnyUnroll groups of 32 k per trip: all of a trip's loads are issued
    // before its first MFMA, so a wavefront keeps 8 KB of A in flight.
    for (int kbase = wave * 32; kbase < K; kbase += waves * 32 * kSkinnyUnroll) {
        float a[kSkinnyUnroll][8], b[kSkinnyUnroll][8];
#pragma unroll
        for (int u = 0; u < kSkinnyUnroll; ++u) {
            const int k = kbase + u * waves * 32 + q * 8;
            if (VEC) {   // K % 4 == 0: each float4 is wholly inside or outside
                const float4 z = make_float4(0.f, 0.f, 0.f, 0.f);
                const float4 lo = (row_ok && k < K) ? ld4<true>(reinterpret_cast<const float4 *>(arow + k)) : z;
                const float4 hi = (row_ok && k + 4 < K) ? ld4<true>(reinterpret_cast<const float4 *>(arow + k + 4)) : z;
                a[u][0] = lo.x; a[u][1] = lo.y; a[u][2] = lo.z; a[u][3] = lo.w;
                a[u][4] = hi.x; a[u][5] = hi.y; a[u][6] = hi.z; a[u][7] = hi.w;
            } else {
#pragma unroll
                for (int s = 0; s < 8; ++s) a[u][s] = (row_ok && k + s < K) ? arow[k + s] : 0.f;
            }
#pragma unroll
            for (int s = 0; s < 8; ++s) b[u][s] = (col_ok && k + s < K) ? B[(size_t)(k + s) * ldb + i] : 0.f;
        }
#pragma unroll
        for (int u = 0; u < kSkinnyUnroll; ++u)
#pragma unroll
            for (int s = 0; s < 8; ++s) acc = __builtin_amdgcn_mfma_f32_16x16x4f32(a[u][s], b[u][s], acc, 0, 0, 0);
    }
#pragma unroll
    for (int v = 0; v < 4; ++v) part[wave][4 * q + v][i] = acc[v];
    __syncthreads();
    if (tid < 256) {
        const int r = tid >> 4, c = tid & 15;
        float s = 0.f;
        for (int w = 0; w < waves; ++w) s += part[w][r][c];
        const int grow = blockIdx.x * 16 + r;
        if (grow < M && c < N) {
            float x = s + (ep.bias ? ep.bias[c] : 0.f);
            if (ep.relu) x = (x > 0.f) ? x : 0.f;
            C[(size_t)grow * ldc + c] = x;
        }
    }
}

template <int TM, int TN>
int launch_tiled(bool vec, const float *a, const float *b, float *c, int m, int n, int k, int lda, int ldb, int ldc,
                 const Epilogue &ep) {
    using T = Tile<TM, TN, false>;
    const long tiles = (long)((m + T::BM - 1) / T::BM) * ((n + T::BN - 1) / T::BN);
    if (tiles > 0x7fffffffL) return fail(SWC_HIP_EINVAL, "gemm: too many tiles");
    auto kern = vec ? gemm_tiled<TM, TN, true> : gemm_tiled<TM, TN, false>;
    static bool attr_set[2] = {false, false};
    if (!attr_set[vec]) {
        SWC_HIP_TRY(hipFuncSetAttribute(reinterpret_cast<const void *>(kern),
                                        hipFuncAttributeMaxDynamicSharedMemorySize, (int)T::kLdsBytes));
        attr_set[vec] = true;
    }
    kern<<<(unsigned)tiles, kThreads, T::kLdsBytes, stream()>>>(a, b, c, m, n, k, (size_t)lda, (size_t)ldb,
                                                                 (size_t)ldc, ep);
    SWC_LAUNCH_CHECK();
    return SWC_HIP_OK;
}

template <int TM, int TN, int STAGES, bool MID = false>
int launch_dma(const float *a, const float *b, float *c, int m, int n, int k, int lda, int ldb, int ldc,
               const Epilogue &ep) {
    using T = DmaTile<TM, TN, false, STAGES>;
    const long tiles = (long)((m + T::BM - 1) / T::BM) * ((n + T::BN - 1) / T::BN);
    if (tiles > 0x7fffffffL) return fail(SWC_HIP_EINVAL, "gemm: too many tiles");
    auto kern = gemm_dma<TM, TN, STAGES, MID>;
    static bool attr_set = false;
    if (!attr_set) {
        SWC_HIP_TRY(hipFuncSetAttribute(reinterpret_cast<const void *>(kern),
                                        hipFuncAttributeMaxDynamicSharedMemorySize, (int)T::kLdsBytes));
        attr_set = true;
    }
    const unsigned a_bytes = (unsigned)(((size_t)(m - 1) * lda + k) * 4);
    const unsigned b_bytes = (unsigned)(((size_t)(k - 1) * ldb + n) * 4);
    kern<<<(unsigned)tiles, kThreads, T::kLdsBytes, stream()>>>(a, b, c, m, n, k, lda, ldb, (size_t)ldc, a_bytes,
                                                                 b_bytes, ep);
    SWC_LAUNCH_CHECK();
    return SWC_HIP_OK;
}

template <int TM, int TN, int WM, int STAGES, bool MID, int NW = 4>
int launch_dma2(const float *a, const float *b, float *c, int m, int n, int k, int lda, int ldb, int ldc,
                const Epilogue &ep) {
    using T = Dma2Tile<TM, TN, WM, STAGES, NW>;
    const long tiles = (long)((m + T::BM - 1) / T::BM) * ((n + T::BN - 1) / T::BN);
    if (tiles > 0x7fffffffL) return fail(SWC_HIP_EINVAL, "gemm: too many tiles");
    auto kern = gemm_dma2<TM, TN, WM, STAGES, MID, NW>;
    static bool attr_set = false;
    if (!attr_set) {
        SWC_HIP_TRY(hipFuncSetAttribute(reinterpret_cast<const void *>(kern),
                                        hipFuncAttributeMaxDynamicSharedMemorySize, (int)T::kLdsBytes));
        attr_set = true;
    }
    const unsigned a_bytes = (unsigned)(((size_t)(m - 1) * lda + k) * 4);
    const unsigned b_bytes = (unsigned)(((size_t)(k - 1) * ldb + n) * 4);
    kern<<<(unsigned)tiles, T::kThreadsWg, T::kLdsBytes, stream()>>>(a, b, c, m, n, k, lda, ldb, (size_t)ldc, a_bytes,
                                                                 b_bytes, ep);
    SWC_LAUNCH_CHECK();
    return SWC_HIP_OK;
}

int gemm_dispatch(const char *who, int m, int n, int k, const float *a, int lda, const float *b, int ldb,
                  const float *bias, float *c, int ldc, int relu) {
    if (m < 0 || n < 0 || k < 0) return fail(SWC_HIP_EINVAL, "%s: negative dimension", who);
    if (m == 0 || n == 0) return SWC_HIP_OK;
    if (!a || !b || !c) return fail(SWC_HIP_EINVAL, "%s: null pointer", who);
    if (lda < k || ldb < n || ldc < n) return fail(SWC_HIP_EINVAL, "%s: leading dimension smaller than row length", who);
    Epilogue ep{bias, nullptr, nullptr, nullptr, nullptr, 0.f, relu};
    if (n <= 16) {
        const bool vec = (k % 4 == 0) && (lda % 4 == 0) && aligned16(a);
        int waves = (k + 31) / 32;
        waves = waves < 1 ? 1 : (waves > kSkinnyMaxWaves ? kSkinnyMaxWaves : waves);
        if (waves < 4) waves = 4;   // the reduction step needs 256 threads
        const unsigned blocks = ceil_div(m, 16);
        if (vec) gemm_skinny<true><<<blocks, 64 * waves, 0, stream()>>>(a, b, c, m, n, k, lda, ldb, ldc, ep);
        else gemm_skinny<false><<<blocks, 64 * waves, 0, stream()>>>(a, b, c, m, n, k, lda, ldb, ldc, ep);
        SWC_LAUNCH_CHECK();
        return SWC_HIP_OK;
    }
    const bool vec = (k % 4 == 0) && (n % 4 == 0) && (lda % 4 == 0) && (ldb % 4 == 0) && aligned16(a) && aligned16(b);
    const long big_tiles = (long)((m + 127) / 128) * ((n + 127) / 128);
    const bool dma_ok = vec && k > 0 && ((size_t)(m - 1) * lda + k) * 4 < kMaxDmaBytes &&
                        ((size_t)(k - 1) * ldb + n) * 4 < kMaxDmaBytes;
    // the column-interleaved kernels also write C with 128-bit stores and start their descriptors 4 KiB early
    const bool dma2_ok = dma_ok && (ldc % 4 == 0) && aligned16(c) && ((size_t)(m - 1) * lda + k) * 4 < 0x7fff0000u &&
                         ((size_t)(k - 1) * ldb + n) * 4 < 0x7fff0000u;
    const long huge_tiles = (long)((m + 255) / 256) * ((n + 255) / 256);
    // Forces a kernel variant (tests, tuning).  reg: register-staged.  <TM><TN>_<STAGES>[m]: gemm_dma, m = ring
    // hand-over in mid-slice.  <TM><TN>w<WM>_<STAGES>[m][x8]: gemm_dma2, x8 = eight wavefronts per workgroup.
    const char *force = getenv("SWC_HIP_GEMM");
    if (dma_ok && !(force && !strcmp(force, "reg"))) {
        if (force) {
            if (!strcmp(force, "22_2")) return launch_dma<2, 2, 2>(a, b, c, m, n, k, lda, ldb, ldc, ep);
            if (!strcmp(force, "22_3")) return launch_dma<2, 2, 3>(a, b, c, m, n, k, lda, ldb, ldc, ep);
            if (!strcmp(force, "21_3")) return launch_dma<2, 1, 3>(a, b, c, m, n, k, lda, ldb, ldc, ep);
            if (!strcmp(force, "12_3")) return launch_dma<1, 2, 3>(a, b, c, m, n, k, lda, ldb, ldc, ep);
            if (!strcmp(force, "11_3")) return launch_dma<1, 1, 3>(a, b, c, m, n, k, lda, ldb, ldc, ep);
            if (!strcmp(force, "11_4")) return launch_dma<1, 1, 4>(a, b, c, m, n, k, lda, ldb, ldc, ep);
            if (!strcmp(force, "11_3m")) return launch_dma<1, 1, 3, true>(a, b, c, m, n, k, lda, ldb, ldc, ep);
            if (!strcmp(force, "21_3m")) return launch_dma<2, 1, 3, true>(a, b, c, m, n, k, lda, ldb, ldc, ep);
            if (dma2_ok) {
                if (!strcmp(force, "24w4_2x8")) return launch_dma2<2, 4, 4, 2, false, 8>(a, b, c, m, n, k, lda, ldb, ldc, ep);
                if (!strcmp(force, "14w4_2")) return launch_dma2<1, 4, 4, 2, false>(a, b, c, m, n, k, lda, ldb, ldc, ep);
                if (!strcmp(force, "14w4_3m")) return launch_dma2<1, 4, 4, 3, true>(a, b, c, m, n, k, lda, ldb, ldc, ep);
                if (!strcmp(force, "24w2_3m")) return launch_dma2<2, 4, 2, 3, true>(a, b, c, m, n, k, lda, ldb, ldc, ep);
                if (!strcmp(force, "22w2_2")) return launch_dma2<2, 2, 2, 2, false>(a, b, c, m, n, k, lda, ldb, ldc, ep);
            }
        }
        // 256x256 tiles with eight wavefronts once they fill the chip (least operand traffic per flop: 146
        // TFLOP/s at 4096^3 against 134 for 128x128 tiles of four wavefronts), 128x128 tiles next, and 64x64
        // tiles for everything smaller, where the number of workgroups matters more than their efficiency
        if (dma2_ok && huge_tiles >= num_cus()) return launch_dma2<2, 4, 4, 2, false, 8>(a, b, c, m, n, k, lda, ldb, ldc, ep);
        if (dma2_ok && big_tiles >= num_cus()) return launch_dma2<1, 4, 4, 2, false>(a, b, c, m, n, k, lda, ldb, ldc, ep);
        if (big_tiles >= num_cus()) return launch_dma<2, 2, 2>(a, b, c, m, n, k, lda, ldb, ldc, ep);
        return launch_dma<1, 1, 3, true>(a, b, c, m, n, k, lda, ldb, ldc, ep);
    }
    if (big_tiles >= num_cus()) return launch_tiled<2, 2>(vec, a, b, c, m, n, k, lda, ldb, ldc, ep);
    return launch_tiled<1, 1>(vec, a, b, c, m, n, k, lda, ldb, ldc, ep);
}

} // namespace

extern "C" {

int swc_hip_matrixMatrixMul_f(int m, int n, int k, const float *a, int lda, const float *b, int ldb, float *c,
                              int ldc) {
    SWC_REQUIRE_INIT();
    return gemm_dispatch("swc_hip_matrixMatrixMul_f", m, n, k, a, lda, b, ldb, nullptr, c, ldc, 0);
}

int swc_hip_matrixMatrixFCBias_f(int m, int n, int k, const float *a, int lda, const float *b, int ldb,
                                 const float *bias, float *c, int ldc, int relu) {
    SWC_REQUIRE_INIT();
    return gemm_dispatch("swc_hip_matrixMatrixFCBias_f", m, n, k, a, lda, b, ldb, bias, c, ldc, relu);
}

} // extern "C"
