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
#include "mfma_tile.hpp"

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

    auto load_global = [&](int k0) {
        if (VEC) {
#pragma unroll
            for (int i = 0; i < T::kAVec; ++i) {   // A: 8 threads per row of 32 k
                const int row = m0 + (tid >> 3) + 32 * i;
                const int k = k0 + (tid & 7) * 4;
                ra[i] = (row < M && k < K) ? *reinterpret_cast<const float4 *>(A + (size_t)row * lda + k)
                                           : make_float4(0.f, 0.f, 0.f, 0.f);
            }
#pragma unroll
            for (int i = 0; i < T::kBVec; ++i) {   // B: BN/4 threads per k row
                constexpr int kPerRow = T::BN / 4;
                const int e = tid + kThreads * i;
                const int k = k0 + e / kPerRow;
                const int col = n0 + (e % kPerRow) * 4;
                rb[i] = (k < K && col < N) ? *reinterpret_cast<const float4 *>(B + (size_t)k * ldb + col)
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
    load_global(0);
    store_lds(0);
    __syncthreads();
    for (int kt = 0; kt < nk; ++kt) {
        const int cur = kt & 1;
        if (kt + 1 < nk) load_global((kt + 1) * BK);
        const float *As = lds + cur * T::kStageFloats;
        compute_slice<TM, TN, false>(As, As + T::kAFloats, acc, wave_m, wave_n, lane);
        if (kt + 1 < nk) store_lds(cur ^ 1);
        __syncthreads();
    }
    store_tile<TM, TN>(acc, C, ldc, M, N, m0 + wave_m * 32 * TM, n0 + wave_n * 32 * TN, lane, ep);
}

// --------------------------------------------------------------- skinny GEMM
typedef float v4f __attribute__((ext_vector_type(4)));
constexpr int kSkinnyMaxWaves = 16;

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
    for (int k0 = wave * 32; k0 < K; k0 += waves * 32) {
        const int k = k0 + q * 8;
        float a[8], b[8];
        if (VEC) {   // K % 4 == 0: each float4 is wholly inside or outside
            const float4 z = make_float4(0.f, 0.f, 0.f, 0.f);
            const float4 lo = (row_ok && k < K) ? *reinterpret_cast<const float4 *>(arow + k) : z;
            const float4 hi = (row_ok && k + 4 < K) ? *reinterpret_cast<const float4 *>(arow + k + 4) : z;
            a[0] = lo.x; a[1] = lo.y; a[2] = lo.z; a[3] = lo.w;
            a[4] = hi.x; a[5] = hi.y; a[6] = hi.z; a[7] = hi.w;
        } else {
#pragma unroll
            for (int s = 0; s < 8; ++s) a[s] = (row_ok && k + s < K) ? arow[k + s] : 0.f;
        }
#pragma unroll
        for (int s = 0; s < 8; ++s) b[s] = (col_ok && k + s < K) ? B[(size_t)(k + s) * ldb + i] : 0.f;
#pragma unroll
        for (int s = 0; s < 8; ++s) acc = __builtin_amdgcn_mfma_f32_16x16x4f32(a[s], b[s], acc, 0, 0, 0);
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
