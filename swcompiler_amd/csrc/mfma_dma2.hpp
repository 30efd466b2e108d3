// Column-interleaved fp32 MFMA tile kernel body with direct global->LDS loads,
// shared by the FC GEMM (gemm.hip) and the filter gradient of the convolution
// (conv.hip).  See the comment above Dma2Tile for the layout.
#pragma once
#include "mfma_dma.hpp"

namespace swc_hip {
namespace mfma {

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
    static_assert(kLdsBytes <= swc::devices::HipDevice::ldsBytesPerCU, "the ring must fit one CU's LDS");
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
        const float4 v = *reinterpret_cast<const float4 *>(&As[row * BK + (((2 * g + h) ^ ((l32 >> 1) & 7)) << 2)]);
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
// Where the B tile comes from is a policy (BSrc): per load and lane it keeps a
// small state (Lane), gives the byte offset of the lane's 16 bytes for the slice
// starting at k0 (or kOutOfRange) plus a scalar offset common to the wavefront,
// and advances the state by one slice.  DenseB is a row-major [K][N] matrix.
//
// The body computes C[m0.., n0..] = A[:, k_begin:k_end] * B[k_begin:k_end, :] for
// the workgroup's tile (k_begin a multiple of BK); split-K callers give every
// split its own C.
constexpr int kImmSpan = 4096;

struct DenseB {
    const float *base;
    unsigned bytes;
    int ldb;
    struct Lane {
        int v, krow;
    };
#if __HIP_DEVICE_COMPILE__
    __device__ __forceinline__ __amdgpu_buffer_rsrc_t rsrc() const {
        return make_rsrc(reinterpret_cast<const char *>(base) - kImmSpan, bytes + kImmSpan);
    }
    __device__ __forceinline__ Lane init(int krow, int col, bool col_ok, int imm, int /*k_begin*/) const {
        return Lane{col_ok ? (krow * ldb + col) * 4 + kImmSpan - imm : kOutOfRange, krow};
    }
    __device__ __forceinline__ int voffset(const Lane &s, int k0, int k_end) const {
        return (k0 + BK <= k_end || (s.v != kOutOfRange && k0 + s.krow < k_end)) ? s.v : kOutOfRange;
    }
    __device__ __forceinline__ int soffset(int k0) const { return k0 * ldb * 4; }
    __device__ __forceinline__ void advance(Lane &) const {}
#endif
};

#if __HIP_DEVICE_COMPILE__
// SKIP: a wavefront whose columns all lie outside the matrix (the last column tile of an N that is no multiple of the
// tile width) takes part in the loads and barriers but issues no MFMA and reads no fragment.
template <int TM, int TN, int WM, int STAGES, bool MID, int NW, class BSrc, bool SKIP = false>
__device__ __forceinline__ void dma2_tile_body(const float *__restrict__ A, unsigned a_bytes, int lda, const BSrc &bsrc,
                                               float *__restrict__ C, size_t ldc, int M, int N, int k_begin, int k_end,
                                               const Epilogue &ep) {
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
    const __amdgpu_buffer_rsrc_t rsrc_a = make_rsrc(reinterpret_cast<const char *>(A) - kImmSpan, a_bytes + kImmSpan);
    const __amdgpu_buffer_rsrc_t rsrc_b = bsrc.rsrc();

    // Per-lane byte offsets of slice 0 (out-of-range for rows/columns outside the
    // matrix); a slice adds a scalar: k0*4 bytes for A, k0*ldb*4 for B.  Only a
    // slice that reaches past K needs the per-lane k check.
    int a_k[T::kALoads];   // k of the lane's chunk inside a slice, per load (the swizzle key depends on the row block)
    int a_base[T::kALoads];
    typename BSrc::Lane bl[T::kBLoads];
#pragma unroll
    for (int j = 0; j < T::kALoads; ++j) {
        const int row = m0 + (wave * T::kALoads + j) * 8 + kc_row_in_load(lane);
        a_k[j] = kc_chunk(lane, wave * T::kALoads + j) * 4;
        a_base[j] = row < M ? (row * lda + a_k[j]) * 4 + kImmSpan - (j & 3) * 1024 : kOutOfRange;
    }
#pragma unroll
    for (int j = 0; j < T::kBLoads; ++j) {
        const int flat = (wave * T::kBLoads + j) * 256 + lane * 4;   // float index inside the [32][BN] tile
        const int col = n0 + flat % T::BN;
        bl[j] = bsrc.init(flat / T::BN, col, col < N, (j & 3) * 1024, k_begin);
    }
    int k0 = k_begin;   // first k of the slice whose loads are being issued
    auto issue = [&](float *__restrict__ wr, int j) {
        const bool whole = k0 + BK <= k_end;   // scalar
        if (j < T::kALoads) {
            const int v = whole ? a_base[j] : ((a_base[j] != kOutOfRange && k0 + a_k[j] < k_end) ? a_base[j] : kOutOfRange);
            lds_void_t *dst = (lds_void_t *)(wr + (wave * T::kALoads + (j & ~3)) * 256);
            switch (j & 3) {   // the immediate must be a compile-time constant
            case 0: __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrc_a, dst, 16, v, k0 * 4, 0, 0); break;
            case 1: __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrc_a, dst, 16, v, k0 * 4, 1024, 0); break;
            case 2: __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrc_a, dst, 16, v, k0 * 4, 2048, 0); break;
            default: __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrc_a, dst, 16, v, k0 * 4, 3072, 0); break;
            }
        } else {
            const int jb = j - T::kALoads;
            const int v = bsrc.voffset(bl[jb], k0, k_end);
            const int so = bsrc.soffset(k0);
            bsrc.advance(bl[jb]);
            lds_void_t *dst = (lds_void_t *)(wr + T::kAFloats + (wave * T::kBLoads + (jb & ~3)) * 256);
            switch (jb & 3) {
            case 0: __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrc_b, dst, 16, v, so, 0, 0); break;
            case 1: __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrc_b, dst, 16, v, so, 1024, 0); break;
            case 2: __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrc_b, dst, 16, v, so, 2048, 0); break;
            default: __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrc_b, dst, 16, v, so, 3072, 0); break;
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
    const int nk = (k_end - k_begin + BK - 1) / BK;
    int rd_stage = 0, wr_stage = STAGES - 1;
    const bool computes = !SKIP || n0 + col0 < N;   // (wavefront-uniform)
    if (SKIP && !computes) {
        // The slices' barriers and this wavefront's share of the loads, nothing else.  (A loop of its own: as a branch
        // inside the loop below it made the compiler carry the accumulators through the loop in VGPRs and copy them
        // into the AGPRs in every slice.)
        for (int kt = 0; kt < nk; ++kt) {
            float *__restrict__ wr = lds + wr_stage * T::kStageFloats;
            ring_sync<MID ? (STAGES - 3) * T::kLoads : (STAGES - 2) * T::kLoads>();
#pragma unroll
            for (int j = 0; j < T::kLoads; ++j) issue(wr, j);
            k0 += BK;
            wr_stage = wr_stage + 1 == STAGES ? 0 : wr_stage + 1;
        }
        wait_vmcnt<0>();
        return;   // (nothing of this wavefront's tile lies inside the matrix)
    }
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
}
#endif  // __HIP_DEVICE_COMPILE__

} // namespace mfma
} // namespace swc_hip
