// Shared plumbing of libswc_hip: error record, stream access, launch checks.
#pragma once
#include <hip/hip_runtime.h>

#include <cstdarg>
#include <cstddef>
#include <cstdint>
#include <cstdio>

#include "devices/HipDevice.h"
#include "swc_hip.h"

namespace swc_hip {

// The device the kernels are written for (shared with the code generator).
using Device = swc::devices::HipDevice;

// Records a printf-style message for swc_hip_last_error() and returns `code`.
int fail(int code, const char *fmt, ...) __attribute__((format(printf, 2, 3)));
void clear_error();
int fail_code();   // the code of this thread's last fail() (for callers of helpers that return null on failure)

// The stream every op launches on; nullptr until swc_hip_init succeeded.
hipStream_t stream();
bool ready();
// Records which kernel variant an op dispatched to (printf-style), for swc_hip_last_kernel().
void note_kernel(const char *fmt, ...) __attribute__((format(printf, 1, 2)));
int num_cus();   // of the initialised device (Device::computeUnits on a whole MI355X)
// Scratch device memory for the current op (see runtime.hip); nullptr with the error recorded on failure.
void *workspace(size_t bytes, const char *who);
// Looks up, for `device` (which must be current), the address of the fixed scratch array of the entry point
// that allocates nothing (gemm.hip); called once per device by swc_hip_init.
int gemm_noalloc_setup(int device);

// Test and tuning switches (the SWC_HIP_* environment variables; none is part of the contract).  swc_hip_init reads
// them ONCE into this record (swc_hip_reload_switches reads them again, for a test process that changes them): no
// op touches the environment, so a size query, a warm-up run and a recorded graph all see the same choice.
struct Switches {
    const char *gemm = nullptr;   // SWC_HIP_GEMM: forces a GEMM kernel variant ("splitk", "fewrows", "reg", "22_2", ...)
    const char *conv = nullptr;   // SWC_HIP_CONV: forces a convolution kernel variant ("reg22", "11_3m", ...)
    bool skinny_plain = false;    // SWC_HIP_SKINNY=plain: gemm_skinny for every classifier head
    bool conv_share = true;       // SWC_HIP_CONV_SHARE=0: every convolution tile computed whole
    bool conv_raster = false;     // SWC_HIP_CONV_ORDER=raster: rows of the GEMM view in raster order
    bool conv_lean = true;        // SWC_HIP_CONV_LEAN=0: the general tile kernel where the lean one would run
    int conv_share_all = 0;       // SWC_HIP_CONV_SHARE_ALL=n: slices per tile from which a short layer is cut (unset 0: default; "0" -> -1: never)
    int conv_slots = 0;           // SWC_HIP_CONV_SLOTS=n: pretend the chip holds n workgroups at a time (0: ask the device)
    int conv_piece_min = 0;       // SWC_HIP_CONV_PIECE_MIN=n: least K slices per piece of a tile cut along K (0: default)
    int conv_min_idle = -1;       // SWC_HIP_CONV_MIN_IDLE=n: tiles are cut along K only if whole tiles would leave the average CU idle for n slices + 1/16 per cut tile (0: no such test; -1: default)
    bool conv_fair = true;        // SWC_HIP_CONV_FAIR=0: the last round's workgroups keep one priority (see conv_win)
    int wgrad_bn = 0;             // SWC_HIP_WGRAD_BN=128|256: tile width of the filter gradient (0: planner's choice)
};
const Switches &switches();

inline bool aligned16(const void *p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

inline unsigned ceil_div(size_t a, size_t b) { return (unsigned)((a + b - 1) / b); }

// Tensors at least this large are streamed with non-temporal loads and stores:
// they cannot stay in the 4 MB-per-XCD L2 / 256 MB infinity cache anyway, and
// marking the traffic as streaming measured ~10 % more HBM bandwidth on MI355X.
// Smaller tensors keep normal caching so the next kernel finds them on chip.
constexpr size_t kStreamingBytes = (size_t)64 << 20;

typedef float swc_f4 __attribute__((ext_vector_type(4)));
typedef int swc_i4 __attribute__((ext_vector_type(4)));
template <bool NT> __device__ __forceinline__ float4 ld4(const float4 *p) {
    if (NT) {
        const swc_f4 v = __builtin_nontemporal_load(reinterpret_cast<const swc_f4 *>(p));
        return make_float4(v.x, v.y, v.z, v.w);
    }
    return *p;
}
template <bool NT> __device__ __forceinline__ void st4(float4 *p, float4 r) {
    if (NT) {
        const swc_f4 v = {r.x, r.y, r.z, r.w};
        __builtin_nontemporal_store(v, reinterpret_cast<swc_f4 *>(p));
    } else {
        *p = r;
    }
}
template <bool NT> __device__ __forceinline__ void st4i(int4 *p, int4 r) {
    if (NT) {
        const swc_i4 v = {r.x, r.y, r.z, r.w};
        __builtin_nontemporal_store(v, reinterpret_cast<swc_i4 *>(p));
    } else {
        *p = r;
    }
}

// exp(x) for x <= 0 through the hardware exp2; relative error ~2e-6 at x = -30,
// far inside the 1e-4 contract of the softmax kernels.
__device__ __forceinline__ float fast_exp(float x) { return __builtin_amdgcn_exp2f(x * 1.44269504088896340736f); }

} // namespace swc_hip

#define SWC_REQUIRE_INIT()                                                              \
    do {                                                                                \
        if (!swc_hip::ready())                                                          \
            return swc_hip::fail(SWC_HIP_ENOTINIT, "%s: swc_hip_init has not been called", __func__); \
    } while (0)

#define SWC_ARG(cond)                                                                   \
    do {                                                                                \
        if (!(cond)) return swc_hip::fail(SWC_HIP_EINVAL, "%s: argument check failed: %s", __func__, #cond); \
    } while (0)

#define SWC_HIP_TRY(expr)                                                               \
    do {                                                                                \
        hipError_t e__ = (expr);                                                        \
        if (e__ != hipSuccess)                                                          \
            return swc_hip::fail(SWC_HIP_ERUNTIME, "%s: %s -> %s", __func__, #expr, hipGetErrorString(e__)); \
    } while (0)

// after a kernel launch
#define SWC_LAUNCH_CHECK() SWC_HIP_TRY(hipGetLastError())
