// fp32 MFMA block-tile core with direct global->LDS loads (gfx950
// `buffer_load_dwordx4 ... lds`) and a multi-stage LDS ring.
//
// Same tile geometry as mfma_tile.hpp — 256 threads = 4 wavefronts as 2x2, each
// owning TM x TN accumulators of v_mfma_f32_32x32x2_f32, K in slices of 32 — but
// operand tiles never pass through registers: each wavefront issues 16-byte-per-
// lane buffer loads whose data the memory pipeline writes straight into LDS
// (lane l of an instruction lands at LDS base + 16*l).  That removes the staging
// VGPRs, the ds_write instructions and their wait, and lets STAGES-1 slices be
// in flight behind the one being multiplied.
//
// Out-of-range handling is the buffer resource's: a lane whose element lies
// outside the matrix (row >= M, k >= K, or a padding tap of a convolution) is
// given a byte offset beyond num_records, for which the load returns zeros —
// which is exactly the value the tile needs there.
//
// LDS layout of one stage (no padding is possible: the hardware places lanes
// contiguously), conflict-free by XOR swizzles chosen on the GLOBAL-address side:
//   k-contiguous operand (A; B given as [n][k]): row r = 32 floats = 8 chunks of
//     16 B; logical chunk q is stored at position q ^ ((r >> 1) & 7).  A 128-bit fragment read is served
//     sixteen lanes at a time (16 x 16 B = all 64 banks once): the sixteen consecutive rows of such a group,
//     same q, then touch 8 distinct positions in their even rows (the lower 32 banks) and 8 in their odd rows
//     (the upper 32).  (A key of r & 7 repeats after 8 rows: two-way conflicts on every read.)
//   n-contiguous B ([k][n]): row k = BN floats; column c of a row with
//     (k >> 2) & 1 == 1 is stored at c ^ 32, so the two half-waves of a fragment
//     read (rows 4 apart) use opposite halves of the banks.
//
// Synchronisation is explicit: the compiler is kept from serialising the ring
// (it cannot see which stage a load targets) by giving the stage being written
// and the stage being read to dma_step() as __restrict__ pointers, and the real
// ordering is enforced here with s_waitcnt vmcnt(n) + s_barrier:
//   top of slice kt:  wait until at most (STAGES-2) slices of loads are pending
//                     -> this wave's part of slice kt has landed;
//                     barrier -> everyone's part has, and everyone is done
//                     reading slice kt-1, whose stage is overwritten next.
// Loads are issued for slice indices past the end as all-out-of-range dummies so
// that the pending-load count is the same in every iteration.
#pragma once
#include <hip/hip_runtime.h>

#include "mfma_tile.hpp"

namespace swc_hip {
namespace mfma {

constexpr int kOutOfRange = 0x7fffffff;   // byte offset no buffer here reaches (operands are < 2 GiB)
constexpr unsigned kMaxDmaBytes = 0x7fffff00u;

template <int TM, int TN, bool B_NT, int STAGES>
struct DmaTile {
    static constexpr int BM = 64 * TM;
    static constexpr int BN = 64 * TN;
    static constexpr int kAFloats = BM * BK;
    static constexpr int kBFloats = BN * BK;
    static constexpr int kStageFloats = kAFloats + kBFloats;
    static constexpr size_t kLdsBytes = (size_t)STAGES * kStageFloats * sizeof(float);
    static constexpr int kALoads = BM / 32;   // buffer loads per wavefront per slice (1 KiB each)
    static constexpr int kBLoads = BN / 32;
    static constexpr int kLoads = kALoads + kBLoads;
    static_assert(STAGES >= 2 && (STAGES - 2) * kLoads < 64, "pending loads must fit the vmcnt field");
    static_assert(kLdsBytes <= swc::devices::HipDevice::ldsBytesPerCU, "the ring must fit one CU's LDS");
};

#if __HIP_DEVICE_COMPILE__   // buffer-resource types and LDS-DMA builtins exist in the device pass only
typedef __attribute__((address_space(3))) void lds_void_t;

__device__ __forceinline__ __amdgpu_buffer_rsrc_t make_rsrc(const void *base, unsigned bytes) {
    // raw buffer (stride 0), 32-bit data format, range checking on
    return __builtin_amdgcn_make_buffer_rsrc(const_cast<void *>(base), 0, (int)bytes, 0x00020000);
}

// s_waitcnt vmcnt(n) only (expcnt/lgkmcnt fields left at "no wait"), gfx9 encoding:
// vmcnt = bits [3:0] and [15:14].
template <int N> __device__ __forceinline__ void wait_vmcnt() {
    static_assert(N >= 0 && N < 64, "");
    __builtin_amdgcn_s_waitcnt(0x0f70 | (N & 15) | ((N >> 4) << 14));
}

// Position of a lane inside one 1-KiB load of a k-contiguous tile: the load
// covers 8 rows; lane l writes row (l >> 3), chunk position (l & 7), which holds
// logical chunk (l & 7) ^ key of its row, key = (row >> 1) & 7.
__device__ __forceinline__ int kc_row_in_load(int lane) { return lane >> 3; }
// `block` = which 8-row block of the tile the load fills (its parity is all that matters)
__device__ __forceinline__ int kc_chunk(int lane, int block) { return (lane & 7) ^ (((block & 1) << 2) | (lane >> 4)); }

template <int TM, int TN, bool B_NT>
__device__ __forceinline__ void load_frag_swz(Frag<TM, TN> &f, const float *__restrict__ As,
                                              const float *__restrict__ Bs, int g, int wave_m, int wave_n, int l32,
                                              int h) {
    constexpr int BN = 64 * TN;
    const int swz = (l32 >> 1) & 7;
#pragma unroll
    for (int tm = 0; tm < TM; ++tm) {
        const int row = wave_m * 32 * TM + tm * 32 + l32;
        const float4 v = *reinterpret_cast<const float4 *>(&As[row * BK + (((2 * g + h) ^ swz) << 2)]);
        f.a[tm][0] = v.x; f.a[tm][1] = v.y; f.a[tm][2] = v.z; f.a[tm][3] = v.w;
    }
#pragma unroll
    for (int tn = 0; tn < TN; ++tn) {
        if (B_NT) {
            const int row = wave_n * 32 * TN + tn * 32 + l32;
            const float4 v = *reinterpret_cast<const float4 *>(&Bs[row * BK + (((2 * g + h) ^ swz) << 2)]);
            f.b[tn][0] = v.x; f.b[tn][1] = v.y; f.b[tn][2] = v.z; f.b[tn][3] = v.w;
        } else {
            const int col = ((wave_n * 32 * TN + tn * 32) ^ (h << 5)) + l32;
#pragma unroll
            for (int s = 0; s < 4; ++s) f.b[tn][s] = Bs[(g * 8 + 4 * h + s) * BN + col];
        }
    }
}

template <int TM, int TN, bool B_NT>
__device__ __forceinline__ void compute_slice_swz(const float *__restrict__ As, const float *__restrict__ Bs,
                                                  v16f (&acc)[TM][TN], int wave_m, int wave_n, int lane) {
    const int l32 = lane & 31;
    const int h = lane >> 5;
    Frag<TM, TN> frag[2];
    load_frag_swz<TM, TN, B_NT>(frag[0], As, Bs, 0, wave_m, wave_n, l32, h);
#pragma unroll
    for (int g = 0; g < BK / 8; ++g) {
        if (g + 1 < BK / 8) load_frag_swz<TM, TN, B_NT>(frag[(g + 1) & 1], As, Bs, g + 1, wave_m, wave_n, l32, h);
        // Without this fence the scheduler sinks each LDS read to just before its
        // first use (one or two MFMAs of cover, then a wait); with it the reads of
        // group g+1 have the whole of group g's MFMAs to complete.
        __builtin_amdgcn_sched_barrier(0);
        const Frag<TM, TN> &f = frag[g & 1];
#pragma unroll
        for (int s = 0; s < 4; ++s)
#pragma unroll
            for (int tm = 0; tm < TM; ++tm)
#pragma unroll
                for (int tn = 0; tn < TN; ++tn)
                    mfma_acc(acc[tm][tn], f.a[tm][s], f.b[tn][s]);
        __builtin_amdgcn_sched_barrier(0);
    }
}

// One ring step: start the loads of a later slice into `wr`, multiply the slice
// held in `rd`.  `wr` and `rd` are different stages (STAGES >= 2), which is what
// the __restrict__ qualifiers state.  voff_a/voff_b give the per-lane byte
// offsets (or kOutOfRange) of the slice being loaded.
template <int TM, int TN, bool B_NT, int STAGES>
__device__ __forceinline__ void dma_step(float *__restrict__ wr, const float *__restrict__ rd,
                                         __amdgpu_buffer_rsrc_t rsrc_a, __amdgpu_buffer_rsrc_t rsrc_b,
                                         const int (&voff_a)[DmaTile<TM, TN, B_NT, STAGES>::kALoads],
                                         const int (&voff_b)[DmaTile<TM, TN, B_NT, STAGES>::kBLoads],
                                         v16f (&acc)[TM][TN], int wave, int lane) {
    using T = DmaTile<TM, TN, B_NT, STAGES>;
    // load j of wavefront w fills the 1-KiB block (4*j + w) of the operand's tile
#pragma unroll
    for (int j = 0; j < T::kALoads; ++j)
        __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrc_a, (lds_void_t *)(wr + (4 * j + wave) * 256), 16, voff_a[j], 0, 0,
                                                 0);
#pragma unroll
    for (int j = 0; j < T::kBLoads; ++j)
        __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrc_b, (lds_void_t *)(wr + T::kAFloats + (4 * j + wave) * 256), 16,
                                                 voff_b[j], 0, 0, 0);
    __builtin_amdgcn_sched_barrier(0);   // keep the loads ahead of the MFMAs
    compute_slice_swz<TM, TN, B_NT>(rd, rd + T::kAFloats, acc, wave >> 1, wave & 1, lane);
}

// Orders the ring: this wave's loads of the slice about to be read are complete
// (at most PENDING newer loads outstanding), then all waves meet.
template <int PENDING> __device__ __forceinline__ void ring_sync() {
    wait_vmcnt<PENDING>();
    asm volatile("" ::: "memory");
    __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");
}

// ---- ring with the hand-over in the middle of a slice (STAGES >= 3) ----
// The step above stops the matrix pipe at every slice boundary: barrier, issue
// loads, read the first fragments, and only then the next MFMA — and the
// wavefronts that share a SIMD reach their boundaries together, so nothing
// fills the gap.  Here the barrier sits after the first group of MFMAs of a
// slice instead: it certifies that slice kt+1 has landed (every wave waited for
// its own part) and that slice kt-1 is no longer read by anyone, whose stage
// then receives slice kt+STAGES-1.  The boundary itself needs no
// synchronisation any more, so the first fragments of slice kt+1 are fetched
// before the last MFMA group of slice kt, like any other group.
// frag[0] holds group 0 of `rd` on entry and group 0 of `nx` on exit.
template <int TM, int TN, bool B_NT, int STAGES>
__device__ __forceinline__ void dma_step_mid(float *__restrict__ wr, const float *__restrict__ rd,
                                             const float *__restrict__ nx, __amdgpu_buffer_rsrc_t rsrc_a,
                                             __amdgpu_buffer_rsrc_t rsrc_b,
                                             const int (&voff_a)[DmaTile<TM, TN, B_NT, STAGES>::kALoads],
                                             const int (&voff_b)[DmaTile<TM, TN, B_NT, STAGES>::kBLoads],
                                             v16f (&acc)[TM][TN], Frag<TM, TN> (&frag)[2], int wave, int lane) {
    using T = DmaTile<TM, TN, B_NT, STAGES>;
    static_assert(STAGES >= 3, "the slice being loaded, the one being read and the next must be distinct stages");
    const int l32 = lane & 31;
    const int h = lane >> 5;
    const int wave_m = wave >> 1, wave_n = wave & 1;
#pragma unroll
    for (int g = 0; g < BK / 8; ++g) {
        if (g == 1) {
            ring_sync<(STAGES - 3) * T::kLoads>();
#pragma unroll
            for (int j = 0; j < T::kALoads; ++j)
                __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrc_a, (lds_void_t *)(wr + (4 * j + wave) * 256), 16,
                                                         voff_a[j], 0, 0, 0);
#pragma unroll
            for (int j = 0; j < T::kBLoads; ++j)
                __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrc_b, (lds_void_t *)(wr + T::kAFloats + (4 * j + wave) * 256),
                                                         16, voff_b[j], 0, 0, 0);
        }
        if (g + 1 < BK / 8)
            load_frag_swz<TM, TN, B_NT>(frag[(g + 1) & 1], rd, rd + T::kAFloats, g + 1, wave_m, wave_n, l32, h);
        else
            load_frag_swz<TM, TN, B_NT>(frag[0], nx, nx + T::kAFloats, 0, wave_m, wave_n, l32, h);
        __builtin_amdgcn_sched_barrier(0);   // reads stay ahead of this group's MFMAs (see compute_slice_swz)
        const Frag<TM, TN> &f = frag[g & 1];
#pragma unroll
        for (int s = 0; s < 4; ++s)
#pragma unroll
            for (int tm = 0; tm < TM; ++tm)
#pragma unroll
                for (int tn = 0; tn < TN; ++tn)
                    mfma_acc(acc[tm][tn], f.a[tm][s], f.b[tn][s]);
        __builtin_amdgcn_sched_barrier(0);
    }
}

#endif  // __HIP_DEVICE_COMPILE__

} // namespace mfma
} // namespace swc_hip
