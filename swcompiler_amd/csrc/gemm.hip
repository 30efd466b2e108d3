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
//   gemm_skinny_stream  the same product for K above 1024: A and B by LDS-DMA
//                into rings private to each wavefront, no barrier in the K loop.
#include "common.hpp"
#include "mfma_dma.hpp"
#include "mfma_dma2.hpp"
#include "mfma_tile.hpp"

#include <cstdlib>
#include <cstring>

using namespace swc_hip;
using namespace swc_hip::mfma;

// Scratch memory of swc_hip_matrixMatrixFCBias_noalloc_f, the one entry point that never allocates: the partial
// tiles of a product cut along K live in this fixed array instead of the workspace.  Every GPU the library runs
// on holds its own copy at its own address until the process ends.  In host code the array's name is only a
// handle for hipGetSymbolAddress, never a device address: kernels are given g_scratch_ptr[device].
static __device__ __align__(256) float scratch[SWC_HIP_NOALLOC_SCRATCH_BYTES / sizeof(float)];

namespace {

constexpr int kMaxDevices = 64;
float *g_scratch_ptr[kMaxDevices] = {};   // per device: address of `scratch` there (swc_hip::gemm_noalloc_setup)
int g_scratch_device = -1;                // the device swc_hip_init selected

// Where a product cut along K keeps its partial tiles: a fixed region (the call fails if it is too small), or,
// with ptr == nullptr, the workspace.
struct PartialStore {
    float *ptr = nullptr;
    size_t bytes = 0;
};

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
    const int a_k = kc_chunk(lane, wave) * 4;           // k of the lane's chunk inside a slice
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
// Kernel body, tile geometry and epilogue: mfma_dma2.hpp.
template <int TM, int TN, int WM, int STAGES, bool MID, int NW>
__global__ __launch_bounds__(64 * NW) void gemm_dma2(const float *__restrict__ A, const float *__restrict__ B,
                                                      float *__restrict__ C, int M, int N, int K, int lda, int ldb,
                                                      size_t ldc, unsigned a_bytes, unsigned b_bytes, Epilogue ep) {
#if __HIP_DEVICE_COMPILE__
    dma2_tile_body<TM, TN, WM, STAGES, MID, NW>(A, a_bytes, lda, DenseB{B, b_bytes, ldb}, C, ldc, M, N, 0, K, ep);
#endif
}

// Split-K form for shapes with few output tiles (batch-8 MLP, LeNet's FC layers: a handful of tiles,
// K of hundreds): blockIdx.y takes a range of K slices and writes its partial tile to the workspace;
// splitk_finish adds the partial results in split order and applies bias and ReLU.
template <int TM, int TN, int WM, int STAGES, bool MID, int NW>
__global__ __launch_bounds__(64 * NW) void gemm_dma2_splitk(const float *__restrict__ A, const float *__restrict__ B,
                                                             float *__restrict__ part, int M, int N, int K, int lda,
                                                             int ldb, unsigned a_bytes, unsigned b_bytes,
                                                             int slices_per_split) {
#if __HIP_DEVICE_COMPILE__
    const int k_begin = blockIdx.y * slices_per_split * BK;
    const int k_stop = k_begin + slices_per_split * BK;
    const Epilogue ep{nullptr, nullptr, nullptr, nullptr, nullptr, 0.f, 0};
    dma2_tile_body<TM, TN, WM, STAGES, MID, NW>(A, a_bytes, lda, DenseB{B, b_bytes, ldb},
                                                part + (size_t)blockIdx.y * M * N, (size_t)N, M, N, k_begin,
                                                k_stop < K ? k_stop : K, ep);
#endif
}

// c[r][j] = f(sum over splits of part[split][r][j] + bias[j]); four threads share an element (four chains)
__global__ __launch_bounds__(256) void splitk_finish(float *__restrict__ c, size_t ldc, const float *__restrict__ part,
                                                     int M, int N, int splits, Epilogue ep) {
    __shared__ float red[4][65];
    const int e = threadIdx.x & 63, p = threadIdx.x >> 6;
    const size_t n = (size_t)M * N;
    for (size_t base = (size_t)blockIdx.x * 64; base < n; base += (size_t)gridDim.x * 64) {
        const size_t i = base + e;
        float s = 0.f;
        if (i < n)
            for (int k = p; k < splits; k += 4) s += part[(size_t)k * n + i];
        red[p][e] = s;
        __syncthreads();
        if (p == 0 && i < n) {
            const size_t r = i / N, j = i - r * N;
            float x = (red[0][e] + red[1][e]) + (red[2][e] + red[3][e]);
            if (ep.bias) x += ep.bias[j];
            if (ep.relu) x = (x > 0.f) ? x : 0.f;
            c[r * ldc + j] = x;
        }
        __syncthreads();
    }
}

// --------------------------------------------------------------- skinny GEMM
typedef float v4f __attribute__((ext_vector_type(4)));
constexpr int kSkinnyMaxWaves = 16;
constexpr int kSkinnyUnroll = 4;

// The end of both skinny kernels, entered by every thread of the workgroup behind the barrier after which the
// partial 16x16 tile of wavefront w lies at part + w * wave_stride as [row][17]: thread 16 * row + column adds the
// tiles in wavefront order and applies bias and ReLU (the wavefronts past the fourth have nothing left to do).
// softmax != 0: the workgroup holds whole rows, so the row softmax of matrixSoftmax_f is stored instead, with the
// arithmetic of the stand-alone kernel for short rows (row maximum; exp(x - max) summed over the columns in
// ascending order; exp(x - max) times the reciprocal of that sum).  The sixteen lanes of a row work together:
// the maximum by lane exchange (any order gives the same maximum), each lane the exponential of its own column,
// the sum by every lane over the row's values in LDS.  No further barrier: a thread overwrites only the element
// of the first tile that it alone has read, and a row's sixteen lanes are in one wavefront, whose LDS accesses
// are served in program order.
__device__ inline float skinny_bias(const Epilogue &ep, int tid, int N) {   // asked for at kernel entry: a cold load
    return (ep.bias && tid < 256 && (tid & 15) < N) ? ep.bias[tid & 15] : 0.f;
}

__device__ inline void skinny_finish(float *part, int wave_stride, int waves, int tid, size_t row0, int rows, int N,
                                     float *C, size_t ldc, const Epilogue &ep, float bias, int softmax) {
    if (tid >= 256) return;
    const int r = tid >> 4, c = tid & 15;
    const bool live = r < rows && c < N;
    float *mine = part + r * 17 + c;
    float x = 0.f;
    for (int w = 0; w < waves; ++w) x += mine[w * wave_stride];
    x += bias;
    if (ep.relu) x = (x > 0.f) ? x : 0.f;
    if (!softmax) {
        if (live) C[(row0 + r) * ldc + c] = x;
        return;
    }
    float mx = live ? x : -__builtin_inff();
#pragma unroll
    for (int o = 8; o; o >>= 1) mx = fmaxf(mx, __shfl_xor(mx, o, 16));
    const float e = fast_exp(x - mx);
    *mine = e;
    __builtin_amdgcn_wave_barrier();
    float sum = 0.f;
    for (int j = 0; j < N; ++j) sum += part[r * 17 + j];
    const float inv = 1.f / sum;
    if (live) C[(row0 + r) * ldc + c] = e * inv;
}

// v_mfma_f32_16x16x4_f32: A[i][kk] i = l%16, kk = l/16; B[kk][j] j = l%16, kk = l/16;
// D[i][j] in VGPR v: j = l%16, i = 4*(l/16) + v.
// K is walked in groups of 32: quarter-wave q = l/16 takes k = 8q..8q+7, so a
// lane reads 8 consecutive floats of one A row (two 128-bit loads when VEC).
template <bool VEC>
__global__ __launch_bounds__(64 * kSkinnyMaxWaves) void gemm_skinny(const float *__restrict__ A,
                                                                    const float *__restrict__ B,
                                                                    float *__restrict__ C, int M, int N, int K,
                                                                    size_t lda, size_t ldb, size_t ldc, Epilogue ep,
                                                                    int softmax) {
    __shared__ float part[kSkinnyMaxWaves][16][17];
    const int tid = threadIdx.x;
    const int lane = tid & 63, wave = tid >> 6, waves = blockDim.x >> 6;
    const int i = lane & 15, q = lane >> 4;
    const int row = blockIdx.x * 16 + i;
    const bool row_ok = row < M;
    const bool col_ok = i < N;   // as B operand, lane's column j = i
    const float *arow = A + (size_t)(row_ok ? row : 0) * lda;
    const float bias = skinny_bias(ep, tid, N);
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
    const int rows = (M - (int)blockIdx.x * 16) < 16 ? (M - (int)blockIdx.x * 16) : 16;
    skinny_finish(&part[0][0][0], 16 * 17, waves, tid, (size_t)blockIdx.x * 16, rows, N, C, ldc, ep, bias, softmax);
}

// ------------------------------------------------- skinny GEMM, long K, streamed
// N <= 16 with K above 1024 (a classifier head behind a wide layer): one pass over A at close to the rate of a
// plain read.  What holds gemm_skinny back on such shapes is not the arithmetic but the loads: it fetches B with
// 32-bit gathers (four times as many load instructions as for A, each touching several cache lines) and its
// wavefronts alternate between "all loads of a trip" and "all MFMAs of a trip".  Here
//   * a workgroup still owns 16 rows and its sixteen wavefronts split K in groups of 32 (wavefront w takes groups
//     w, w + 16, ...), but every group travels by LDS-DMA into a ring that is private to the wavefront: the A tile
//     of the group (16 rows x 128 bytes: eight consecutive lanes fetch one whole cache line, streaming cache
//     policy) and the 32 rows of B that go with it (32 x N consecutive floats since ldb == N);
//   * no barrier inside the K loop: a wavefront waits for its own oldest group (s_waitcnt vmcnt), reads its
//     fragments out of the slot, and requests the group kRing steps ahead into the slot it has just read;
//   * workgroups start at different groups (rotated by the workgroup index), so that at any moment the chip
//     reads from many 2-KiB windows of the rows and not from the same one in every row;
//   * two MFMA chains (first and second 64 bytes of a row's line), added at the end.
// k of a group is dealt to the four k-lanes of v_mfma_f32_16x16x4_f32 as q, step s -> 4q + 16(s / 4) + s % 4, the
// same on the A and the B side.  The 16-byte pieces of a line are XOR-ed with the row inside a slot (bank spread).
// Partial tiles are summed through LDS in wavefront order, as in gemm_skinny, with the same epilogue.
// Where the time goes at 4096 x 4096 x 10 with the row softmax (13.3 us with A resident in the last-level cache,
// 14.1 us out of HBM, on a box where a plain read of the 64 MiB takes 8.5 / 11.0 us), measured by leaving parts out:
// the A loads alone 10.5 / 12.0 us; the B rows (every workgroup passes over all of B: 40 MB out of L2) +0.8 us;
// the MFMAs +1.0 us (what the last groups of a SIMD's four wavefronts still hold when the stream ends: N = 10 fills
// 10 of the 16 columns of every v_mfma_f32_16x16x4_f32, and every fp32 MFMA shape has the same rate); the reduction,
// the store of C and the end of the kernel behind it +1.0 us.  Tried and slower: each wavefront a contiguous range of
// K instead of every sixteenth group (+0.7 us), no rotation of the starting group (+1.0 us).
constexpr int kStreamWaves = 16;
constexpr int kStreamATile = 2048;   // bytes of a group's A tile in a slot; the B rows follow

__host__ __device__ inline int stream_slot_bytes(int ldb) { return kStreamATile + ((32 * ldb * 4 + 15) & ~15); }

template <int RING, bool B2>
__global__ __launch_bounds__(64 * kStreamWaves) void gemm_skinny_stream(const float *__restrict__ A,
                                                                         const float *__restrict__ B,
                                                                         float *__restrict__ C, int M, int N, int K,
                                                                         unsigned lda, int ldb, size_t ldc, Epilogue ep,
                                                                         int softmax) {
#if __HIP_DEVICE_COMPILE__
    extern __shared__ __align__(16) float lds[];
    constexpr int kNone = 0x7fffffff;   // byte offset outside every buffer: the load stores zeros
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int i = lane & 15, q = lane >> 4;
    const size_t row0 = (size_t)blockIdx.x * 16;
    const int rows = (M - (int)row0) < 16 ? (M - (int)row0) : 16;
    const float bias = skinny_bias(ep, tid, N);
    const __amdgpu_buffer_rsrc_t rs_a = make_rsrc(A + row0 * lda, (unsigned)(((size_t)(rows - 1) * lda + K) * 4));
    const __amdgpu_buffer_rsrc_t rs_b = make_rsrc(B, (unsigned)((size_t)K * ldb * 4));
    const int slot_bytes = stream_slot_bytes(ldb);
    char *const ring = reinterpret_cast<char *>(lds) + wave * (RING * slot_bytes);

    // loads: lane = 8 * (row % 8) + piece; load h of a group takes rows 8h .. 8h + 7
    const int r8 = lane >> 3, seg = (lane & 7) ^ r8;
    const int a_lane = (int)((r8 * lda + 4 * seg) * 4);
    const unsigned a_second = 8u * lda * 4u;
    const bool b1_lane = lane * 16 < 32 * ldb * 4, b2_lane = 1024 + lane * 16 < 32 * ldb * 4;
    // fragment reads: row i, pieces q and q + 4 of its line; B[4q + ..][column i]
    const int i8 = i & 7;
    const int rd0 = (i >> 3) * 1024 + (i8 * 8 + (q ^ i8)) * 16;
    const int rd1 = (i >> 3) * 1024 + (i8 * 8 + ((q + 4) ^ i8)) * 16;
    const bool col_ok = i < N;
    const int rdb = kStreamATile + (4 * q * ldb + (col_ok ? i : 0)) * 4;

    const int groups = (K + 31) / 32;
    const int T = (groups - wave + kStreamWaves - 1) / kStreamWaves;   // groups of this wavefront (may be 0)
    const int rot = T > 0 ? (int)(blockIdx.x % (unsigned)T) : 0;
    auto request = [&](int t, int r) {
        int tt = t + rot;
        if (tt >= T) tt -= T;
        const int k0 = (tt * kStreamWaves + wave) * 32;
        char *slot = ring + r * slot_bytes;
        if (b1_lane)   // (every lane for ldb >= 8; below that the rows of B end before the 1 KiB of a full load)
            __builtin_amdgcn_raw_ptr_buffer_load_lds(rs_b, (lds_void_t *)(slot + kStreamATile), 16, lane * 16, k0 * ldb * 4, 0, 0);
        if (B2) {
            if (b2_lane)
                __builtin_amdgcn_raw_ptr_buffer_load_lds(rs_b, (lds_void_t *)(slot + kStreamATile + 1024), 16, lane * 16,
                                                         k0 * ldb * 4 + 1024, 0, 0);
        }
        const int voff = (k0 + 4 * seg < K) ? a_lane : kNone;   // K % 4 == 0: a piece is wholly inside a row or not
        __builtin_amdgcn_raw_ptr_buffer_load_lds(rs_a, (lds_void_t *)(slot), 16, voff, k0 * 4, 0, 2);
        __builtin_amdgcn_raw_ptr_buffer_load_lds(rs_a, (lds_void_t *)(slot + 1024), 16, voff, k0 * 4 + a_second, 0, 2);
    };
    v4f acc0 = {0.f, 0.f, 0.f, 0.f}, acc1 = {0.f, 0.f, 0.f, 0.f};
    auto consume = [&](int r, bool refill, int t_next) {
        const char *slot = ring + r * slot_bytes;
        const v4f x0 = *reinterpret_cast<const v4f *>(slot + rd0);
        const v4f x1 = *reinterpret_cast<const v4f *>(slot + rd1);
        float b[8];
#pragma unroll
        for (int s = 0; s < 8; ++s) b[s] = *reinterpret_cast<const float *>(slot + rdb + (16 * (s >> 2) + (s & 3)) * ldb * 4);
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");   // the slot has been read: it may be written again
        if (refill) request(t_next, r);
#pragma unroll
        for (int s = 0; s < 8; ++s) b[s] = col_ok ? b[s] : 0.f;
#pragma unroll
        for (int s = 0; s < 4; ++s) {
            acc0 = __builtin_amdgcn_mfma_f32_16x16x4f32(x0[s], b[s], acc0, 0, 0, 0);
            acc1 = __builtin_amdgcn_mfma_f32_16x16x4f32(x1[s], b[4 + s], acc1, 0, 0, 0);
        }
    };
    constexpr int kPer = B2 ? 4 : 3;   // loads per group
    const int first = T < RING ? T : RING;
    for (int t = 0; t < first; ++t) request(t, t);
    int r = 0;
    for (int t = 0; t + RING < T; ++t) {   // steady state: RING groups in flight, the oldest is waited for
        wait_vmcnt<(RING - 1) * kPer>();
        asm volatile("" ::: "memory");
        consume(r, true, t + RING);
        r = r + 1 == RING ? 0 : r + 1;
    }
    for (int left = first - 1; left >= 0; --left) {   // the last groups: nothing is requested any more
        if (left >= 2) wait_vmcnt<2 * kPer>();
        else if (left == 1) wait_vmcnt<kPer>();
        else wait_vmcnt<0>();
        asm volatile("" ::: "memory");
        consume(r, false, 0);
        r = r + 1 == RING ? 0 : r + 1;
    }
    acc0 += acc1;
    // a wavefront's partial tile goes over the start of its own ring, which no other wavefront touches
    float(*part)[17] = reinterpret_cast<float(*)[17]>(ring);
#pragma unroll
    for (int v = 0; v < 4; ++v) part[4 * q + v][i] = acc0[v];
    __syncthreads();
    skinny_finish(lds, RING * slot_bytes / 4, kStreamWaves, tid, row0, rows, N, C, ldc, ep, bias, softmax);
#endif
}

struct StreamArgs {
    const float *a, *b;
    float *c;
    int m, n, k;
    unsigned lda;
    int ldb;
    size_t ldc;
    Epilogue ep;
    int softmax;
    unsigned blocks;
    size_t lds;
};

template <int RING, bool B2> int launch_stream(const StreamArgs &x) {
    auto kern = gemm_skinny_stream<RING, B2>;
    static bool configured = false;
    if (!configured) {
        SWC_HIP_TRY(hipFuncSetAttribute(reinterpret_cast<const void *>(kern), hipFuncAttributeMaxDynamicSharedMemorySize,
                                        (int)Device::ldsBytesPerCU));
        configured = true;
    }
    note_kernel("gemm_skinny_stream<%d,%s>", RING, B2 ? "true" : "false");
    kern<<<x.blocks, 64 * kStreamWaves, x.lds, stream()>>>(x.a, x.b, x.c, x.m, x.n, x.k, x.lda, x.ldb, x.ldc, x.ep, x.softmax);
    SWC_LAUNCH_CHECK();
    return SWC_HIP_OK;
}

// ------------------------------------------------------------ few-rows GEMM
// M <= 16 (single-sample and small-batch inference) with a B of a few MB: the product is bound by the latency
// of one pass over B.  (Also up to 256 rows in blocks of 16 over blockIdx.y while K fits one trip and the blocks'
// passes over B stay within 32 MB of L2 traffic: one launch where the tiled kernels need a split-K pair.)
// A workgroup owns 16 columns of C; its sixteen wavefronts split K into contiguous ranges
// and feed v_mfma_f32_16x16x4_f32 straight from global memory (A is a few KB and stays in cache), all operands
// of a trip requested before its first MFMA — for K up to 1024 a single trip, i.e. one memory latency.  The
// sixteen partial 16x16 tiles are summed through LDS in wavefront order.  One launch where the tiled kernels
// need a split-K pair.
constexpr int kFewRowsWaves = 16;
constexpr int kFewRowsUnroll = 16;

__global__ __launch_bounds__(64 * kFewRowsWaves) void gemm_fewrows(const float *__restrict__ A,
                                                                   const float *__restrict__ B, float *__restrict__ C,
                                                                   int M, int N, int K, size_t lda, size_t ldb,
                                                                   size_t ldc, Epilogue ep) {
    __shared__ float part[kFewRowsWaves][16][17];
    const int tid = threadIdx.x;
    const int lane = tid & 63, wave = tid >> 6;
    const int j = lane & 15, kk = lane >> 4;   // as operand A the lane's row is j, as operand B its column
    const int col = blockIdx.x * 16 + j, row0 = blockIdx.y * 16;
    const bool col_ok = col < N, row_ok = row0 + j < M;
    const float *arow = A + (size_t)(row_ok ? row0 + j : 0) * lda;
    // this wavefront's range of K, a multiple of 4 long
    const int chunk = ((K + kFewRowsWaves - 1) / kFewRowsWaves + 3) & ~3;
    const int k_begin = wave * chunk, k_end = (k_begin + chunk < K) ? k_begin + chunk : K;
    v4f acc = {0.f, 0.f, 0.f, 0.f};
    // Which four k an MFMA adds up is free (a sum).  In blocks of 16 k, step s of a block gives lane (j, kk) the
    // element k = 16 t + 4 kk + s: the lane's four A operands of a block are then 16 contiguous bytes of its row
    // (one 128-bit load where the row allows it, a quarter of the load instructions), and B follows the same k.
    const bool a_vec = (lda % 4 == 0) && ((reinterpret_cast<size_t>(A) & 15) == 0) && (k_begin % 4 == 0);
    for (int kb = k_begin; kb < k_end; kb += 4 * kFewRowsUnroll) {
        float a[kFewRowsUnroll], b[kFewRowsUnroll];
#pragma unroll
        for (int t = 0; t < kFewRowsUnroll / 4; ++t) {
            const int k0 = kb + 16 * t + 4 * kk;   // this lane's four k of block t
            if (a_vec && row_ok && k0 + 3 < k_end) {
                const float4 q = *reinterpret_cast<const float4 *>(arow + k0);
                a[4 * t] = q.x, a[4 * t + 1] = q.y, a[4 * t + 2] = q.z, a[4 * t + 3] = q.w;
            } else {
#pragma unroll
                for (int s4 = 0; s4 < 4; ++s4) a[4 * t + s4] = (row_ok && k0 + s4 < k_end) ? arow[k0 + s4] : 0.f;
            }
#pragma unroll
            for (int s4 = 0; s4 < 4; ++s4) b[4 * t + s4] = (col_ok && k0 + s4 < k_end) ? B[(size_t)(k0 + s4) * ldb + col] : 0.f;
        }
#pragma unroll
        for (int u = 0; u < kFewRowsUnroll; ++u) acc = __builtin_amdgcn_mfma_f32_16x16x4f32(a[u], b[u], acc, 0, 0, 0);
    }
#pragma unroll
    for (int v = 0; v < 4; ++v) part[wave][4 * kk + v][j] = acc[v];   // D[i][j]: i = 4*(l/16) + v
    __syncthreads();
    if (tid < 256) {
        const int r = tid >> 4, c = tid & 15;
        float s = 0.f;
        for (int w = 0; w < kFewRowsWaves; ++w) s += part[w][r][c];
        const int gc = blockIdx.x * 16 + c;
        if (row0 + r < M && gc < N) {
            float x = s + (ep.bias ? ep.bias[gc] : 0.f);
            if (ep.relu) x = (x > 0.f) ? x : 0.f;
            C[(size_t)(row0 + r) * ldc + gc] = x;
        }
    }
}

template <int TM, int TN>
int launch_tiled(bool vec, const float *a, const float *b, float *c, int m, int n, int k, int lda, int ldb, int ldc,
                 const Epilogue &ep) {
    using T = Tile<TM, TN, false>;
    const long tiles = (long)((m + T::BM - 1) / T::BM) * ((n + T::BN - 1) / T::BN);
    if (tiles > 0x7fffffffL) return fail(SWC_HIP_EINVAL, "gemm: too many tiles");
    note_kernel("gemm_tiled<%d,%d,%s>", TM, TN, vec ? "true" : "false");
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
    note_kernel("gemm_dma<%d,%d,%d,%s>", TM, TN, STAGES, MID ? "true" : "false");
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
    note_kernel("gemm_dma2<%d,%d,%d,%d,%s,%d>", TM, TN, WM, STAGES, MID ? "true" : "false", NW);
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

template <int TM, int TN, int WM, int STAGES>
int launch_splitk(const float *a, const float *b, float *c, int m, int n, int k, int lda, int ldb, int ldc,
                  const Epilogue &ep, int splits, int sps, const PartialStore &fixed) {
    using T = Dma2Tile<TM, TN, WM, STAGES, 4>;
    const size_t need = (size_t)splits * m * n * sizeof(float);
    float *part = fixed.ptr;
    if (part) {   // (the entry point that allocates nothing: refused here, where the kernel is known, before any launch)
        if (need > fixed.bytes)
            return fail(SWC_HIP_EINVAL, "swc_hip_matrixMatrixFCBias_noalloc_f: a %d x %d x %d product is cut into %d ranges of K "
                        "whose partial tiles take %zu bytes, more than the %zu bytes of fixed scratch "
                        "(SWC_HIP_NOALLOC_SCRATCH_BYTES); use swc_hip_matrixMatrixFCBias_f with a workspace", m, n, k, splits,
                        need, fixed.bytes);
    } else {
        part = static_cast<float *>(workspace(need, "gemm (split-K)"));
        if (!part) return fail_code();   // (no workspace, one too small, or the allocation failed)
    }
    note_kernel("gemm_dma2_splitk<%d,%d,%d,%d,false,4> x%d", TM, TN, WM, STAGES, splits);
    auto kern = gemm_dma2_splitk<TM, TN, WM, STAGES, false, 4>;
    static bool attr_set = false;
    if (!attr_set) {
        SWC_HIP_TRY(hipFuncSetAttribute(reinterpret_cast<const void *>(kern),
                                        hipFuncAttributeMaxDynamicSharedMemorySize, (int)T::kLdsBytes));
        attr_set = true;
    }
    const unsigned tiles = (unsigned)(((m + T::BM - 1) / T::BM) * ((n + T::BN - 1) / T::BN));
    const unsigned a_bytes = (unsigned)(((size_t)(m - 1) * lda + k) * 4);
    const unsigned b_bytes = (unsigned)(((size_t)(k - 1) * ldb + n) * 4);
    kern<<<dim3(tiles, splits), T::kThreadsWg, T::kLdsBytes, stream()>>>(a, b, part, m, n, k, lda, ldb, a_bytes, b_bytes,
                                                                         sps);
    SWC_LAUNCH_CHECK();
    unsigned blocks = ceil_div((size_t)m * n, 64);
    splitk_finish<<<blocks > 8192 ? 8192 : blocks, 256, 0, stream()>>>(c, (size_t)ldc, part, m, n, splits, ep);
    SWC_LAUNCH_CHECK();
    return SWC_HIP_OK;
}

// Split-K plan of an m x n x k product on this device: true with the number of splits and the K slices per
// split when the shape has too few output tiles to fill the chip.
bool takes_fewrows(int m, int n, int k) {
    if (k <= 0) return false;
    if (m <= 16) return (size_t)k * n <= ((size_t)2 << 20);
    // blocks of 16 rows: K in one trip of the sixteen wavefronts (and long enough to give each of them work), the
    // blocks' passes over B within 32 MB.  Between events, against the split-K pair: 32 x 784 x 512 7.6 against 12.8 us,
    // 64 x 1024 x 1024 8.8 against 15.9, 128 x 512 x 256 7.3 against 12.0, 256 x 800 x 500 13.1 against 17.7,
    // 256 x 1024 x 512 12.6 against 17.9; 200 x 300 x 1000 is better off on the tiled kernel (14.3 against 12.5)
    return m <= 256 && k >= 512 && k <= 64 * kFewRowsWaves && (size_t)((m + 15) / 16) * k * n <= ((size_t)8 << 20);
}

// Up to 64 rows (small-batch inference: the product streams B once and is bound by that): tiles of 32 x 256
// or 64 x 256 instead of 128 x 128, so that no matrix-core work goes into rows that do not exist — with
// 128-row tiles the MFMAs of the empty rows hold a 25088 x 4096 layer at 2.1 TB/s of B (32 rows: 5.1 TB/s
// with the thin tiles).  Always cut along K so that at least two workgroups per CU stream.
constexpr int kThinRows = 64;
constexpr int kThinCols = 256;   // Dma2Tile<1, 2, 1, ...>::BN
bool takes_thin(int m, int n, int k) {
    return m <= kThinRows && n > 16 && (size_t)k * n >= ((size_t)1 << 20) && !takes_fewrows(m, n, k);
}

bool splitk_plan(int m, int n, int k, int &splits, int &sps, bool forced = false) {
    if (!forced && takes_fewrows(m, n, k)) return false;
    const int nk = (k + BK - 1) / BK;
    long tiles;
    if (takes_thin(m, n, k)) {
        tiles = (n + kThinCols - 1) / kThinCols;
    } else {
        tiles = (long)((m + 127) / 128) * ((n + 127) / 128);
        if (n <= 16 || nk < 2 || (!forced && (tiles * 4 > num_cus() || nk < 8))) return false;
    }
    splits = (int)((2L * num_cus() + tiles - 1) / tiles);
    splits = splits > nk ? nk : splits;
    if (takes_thin(m, n, k) && splits > 1 && nk / splits < 4) splits = nk / 4 > 0 ? nk / 4 : 1;   // four slices a share at least
    sps = (nk + splits - 1) / splits;
    splits = (nk + sps - 1) / sps;
    if (takes_thin(m, n, k)) return (size_t)splits * m * n * 4 <= ((size_t)64 << 20);   // (one split: the finish adds the bias)
    return splits > 1 && (size_t)splits * m * n * 4 <= ((size_t)64 << 20);
}

// The one decision function for "is this product cut along K, and how": the dispatch, swc_hip_gemm_workspace_bytes
// and the entry point with fixed scratch all ask it, so a size query always matches what the call then does.
// SWC_HIP_GEMM is a test-only variable (it forces a kernel variant; read once at swc_hip_init, see Switches): "splitk" forces the cut for shapes the plan would leave whole, any other value rules it out.
bool splitk_decision(int m, int n, int k, int &splits, int &sps) {
    const char *force = switches().gemm;
    if (force && strcmp(force, "splitk")) return false;
    return splitk_plan(m, n, k, splits, sps, force != nullptr);
}

// softmax != 0: the row softmax of the result is stored instead of the result (n <= 16 only: the caller checks)
int gemm_dispatch(const char *who, int m, int n, int k, const float *a, int lda, const float *b, int ldb,
                  const float *bias, float *c, int ldc, int relu, int softmax = 0, const PartialStore &fixed = {}) {
    if (m < 0 || n < 0 || k < 0) return fail(SWC_HIP_EINVAL, "%s: negative dimension", who);
    if (m == 0 || n == 0) return SWC_HIP_OK;
    if (!a || !b || !c) return fail(SWC_HIP_EINVAL, "%s: null pointer", who);
    if (lda < k || ldb < n || ldc < n) return fail(SWC_HIP_EINVAL, "%s: leading dimension smaller than row length", who);
    Epilogue ep{bias, nullptr, nullptr, nullptr, nullptr, 0.f, relu};
    if (n <= 16) {
        const bool vec = (k % 4 == 0) && (lda % 4 == 0) && aligned16(a);
        // K is split over the wavefronts of a workgroup: four (the reduction step needs 256 threads) take K up
        // to 1024 in one or two trips each — more only lengthen the reduction (8x512x10: 6.0 us with sixteen,
        // 4.5 with four; 65536x1024x16: 116 against 79 us); sixteen for longer K (4096x4096x10 inside the MLP:
        // 19.6 us against 22.0 with eight).
        const int waves = k <= 1024 ? 4 : kSkinnyMaxWaves;
        const unsigned blocks = ceil_div(m, 16);
        // Long K: the streamed kernel.  It wants whole 16-byte pieces (the vec conditions and a contiguous,
        // aligned B) and 32-bit byte offsets inside the 16 rows of a workgroup and inside B.
        const bool stream_ok = vec && k > 1024 && ldb == n && aligned16(b) && (size_t)lda * 64 < 0x7fff0000u &&
                               (size_t)k * ldb * 4 < 0x7fff0000u && !switches().skinny_plain;   // (test-only switch: gemm_skinny for every shape)
        if (stream_ok) {
            const int slot = stream_slot_bytes(ldb);
            const int ring = (size_t)kStreamWaves * 3 * slot <= Device::ldsBytesPerCU ? 3 : 2;
            const bool b2 = 32 * ldb * 4 > 1024;
            const size_t lds = (size_t)kStreamWaves * ring * slot;
            const StreamArgs sa{a, b, c, m, n, k, (unsigned)lda, ldb, (size_t)ldc, ep, softmax, blocks, lds};
            if (ring == 3) return b2 ? launch_stream<3, true>(sa) : launch_stream<3, false>(sa);
            return b2 ? launch_stream<2, true>(sa) : launch_stream<2, false>(sa);
        }
        note_kernel("gemm_skinny<%s>", vec ? "true" : "false");
        if (vec) gemm_skinny<true><<<blocks, 64 * waves, 0, stream()>>>(a, b, c, m, n, k, lda, ldb, ldc, ep, softmax);
        else gemm_skinny<false><<<blocks, 64 * waves, 0, stream()>>>(a, b, c, m, n, k, lda, ldb, ldc, ep, softmax);
        SWC_LAUNCH_CHECK();
        return SWC_HIP_OK;
    }
    const char *force = switches().gemm;
    // a handful of rows and a B of a few MB: one latency-bound pass over B (see gemm_fewrows)
    if (takes_fewrows(m, n, k) && (!force || !strcmp(force, "fewrows"))) {
        note_kernel("gemm_fewrows");
        gemm_fewrows<<<dim3(ceil_div(n, 16), ceil_div(m, 16)), 64 * kFewRowsWaves, 0, stream()>>>(a, b, c, m, n, k, lda, ldb, ldc, ep);
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
    // hand-over in mid-slice.  <TM><TN>w<WM>_<STAGES>[m][x8]: gemm_dma2, x8 = eight wavefronts per workgroup.  splitk: K split
    // over blockIdx.y with partial tiles in the workspace.  fewrows: gemm_fewrows where it applies.
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
        // Few output tiles and a K of hundreds: K is split over the chip (needs the workspace; while a graph is
        // being recorded only if that is already large enough — an eager warm-up run or swc_hip_set_workspace
        // sees to it).  Otherwise 256x256 tiles with eight wavefronts once they fill the chip (least operand
        // traffic per flop: 146 TFLOP/s at 4096^3 against 134 for 128x128 tiles of four wavefronts), 128x128
        // tiles next, and 64x64 tiles for everything smaller, where the number of workgroups matters more than
        // their efficiency.
        int splits = 0, sps = 0;
        if (dma2_ok && splitk_decision(m, n, k, splits, sps))
            return !takes_thin(m, n, k) ? launch_splitk<1, 4, 4, 2>(a, b, c, m, n, k, lda, ldb, ldc, ep, splits, sps, fixed)
                   : m <= 32            ? launch_splitk<1, 2, 1, 3>(a, b, c, m, n, k, lda, ldb, ldc, ep, splits, sps, fixed)
                                        : launch_splitk<2, 2, 1, 3>(a, b, c, m, n, k, lda, ldb, ldc, ep, splits, sps, fixed);
        if (dma2_ok && huge_tiles >= num_cus()) return launch_dma2<2, 4, 4, 2, false, 8>(a, b, c, m, n, k, lda, ldb, ldc, ep);
        if (dma2_ok && big_tiles >= num_cus()) return launch_dma2<1, 4, 4, 2, false>(a, b, c, m, n, k, lda, ldb, ldc, ep);
        if (big_tiles >= num_cus()) return launch_dma<2, 2, 2>(a, b, c, m, n, k, lda, ldb, ldc, ep);
        return launch_dma<1, 1, 3, true>(a, b, c, m, n, k, lda, ldb, ldc, ep);
    }
    if (big_tiles >= num_cus()) return launch_tiled<2, 2>(vec, a, b, c, m, n, k, lda, ldb, ldc, ep);
    return launch_tiled<1, 1>(vec, a, b, c, m, n, k, lda, ldb, ldc, ep);
}

} // namespace

// Once per device, with that device current (swc_hip_init calls this): the address `scratch` has there.
int swc_hip::gemm_noalloc_setup(int device) {
    if (device < 0 || device >= kMaxDevices)
        return fail(SWC_HIP_EINVAL, "swc_hip_init: device %d is beyond the %d devices the library keeps scratch for", device,
                    kMaxDevices);
    g_scratch_device = device;
    if (g_scratch_ptr[device]) return SWC_HIP_OK;
    void *p = nullptr;
    const hipError_t e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
    if (e != hipSuccess || !p) {
        (void)hipGetLastError();
        return fail(SWC_HIP_ERUNTIME, "swc_hip_init: hipGetSymbolAddress(scratch) on device %d -> %s", device,
                    hipGetErrorString(e));
    }
    g_scratch_ptr[device] = static_cast<float *>(p);
    return SWC_HIP_OK;
}

extern "C" {

int swc_hip_matrixMatrixMul_f(int m, int n, int k, const float *a, int lda, const float *b, int ldb, float *c,
                              int ldc) {
    SWC_REQUIRE_INIT();
    return gemm_dispatch("swc_hip_matrixMatrixMul_f", m, n, k, a, lda, b, ldb, nullptr, c, ldc, 0);
}

size_t swc_hip_gemm_workspace_bytes(int m, int n, int k) {
    if (!ready() || m <= 0 || n <= 0 || k <= 0) return 0;
    int splits = 0, sps = 0;
    return splitk_decision(m, n, k, splits, sps) ? (size_t)splits * m * n * sizeof(float) : 0;
}

int swc_hip_matrixMatrixFCBias_f(int m, int n, int k, const float *a, int lda, const float *b, int ldb,
                                 const float *bias, float *c, int ldc, int relu) {
    SWC_REQUIRE_INIT();
    return gemm_dispatch("swc_hip_matrixMatrixFCBias_f", m, n, k, a, lda, b, ldb, bias, c, ldc, relu);
}

int swc_hip_matrixMatrixFCBias_noalloc_f(int m, int n, int k, const float *a, int lda, const float *b, int ldb,
                                         const float *bias, float *c, int ldc, int relu) {
    SWC_REQUIRE_INIT();
    const char *who = "swc_hip_matrixMatrixFCBias_noalloc_f";
    float *fixed = (g_scratch_device >= 0 && g_scratch_device < kMaxDevices) ? g_scratch_ptr[g_scratch_device] : nullptr;
    if (!fixed) return fail(SWC_HIP_ERUNTIME, "%s: the fixed scratch array was not located at swc_hip_init", who);
    // (a product whose partial tiles exceed the array is refused by the dispatch, at the one place that knows which
    // kernel the shape and the operands' alignment select, before anything is launched)
    return gemm_dispatch(who, m, n, k, a, lda, b, ldb, bias, c, ldc, relu, 0,
                         PartialStore{fixed, (size_t)SWC_HIP_NOALLOC_SCRATCH_BYTES});
}

int swc_hip_matrixMatrixFCBiasSoftmax_f(int m, int n, int k, const float *a, int lda, const float *b, int ldb,
                                        const float *bias, float *c, int ldc) {
    SWC_REQUIRE_INIT();
    const char *who = "swc_hip_matrixMatrixFCBiasSoftmax_f";
    if (n > 0 && n <= 16) return gemm_dispatch(who, m, n, k, a, lda, b, ldb, bias, c, ldc, 0, 1);
    // wider rows: the two kernels in sequence (every softmax kernel reads an element before it overwrites it)
    if (int rc = gemm_dispatch(who, m, n, k, a, lda, b, ldb, bias, c, ldc, 0)) return rc;
    return swc_hip_matrixSoftmax_f(m, n, c, ldc, c, ldc);
}

} // extern "C"
