// Runtime half of libswc_hip: device selection, the single in-order stream,
// arena allocation and host<->device copies.  Replaces the cudaSetDevice /
// cudaMalloc / cudaMemcpy / cudaStreamCreate lines the reference's code
// generator prints (src/codegen/Codegen.cpp:154-172, 504-521, 1134-1169).
#include "common.hpp"

#include <cstdlib>
#include <cstring>
#include <mutex>

namespace swc_hip {
namespace {

thread_local char g_err[768] = "";
thread_local int g_err_code = SWC_HIP_OK;
constexpr int kEventSlots = 4096;
constexpr int kGraphSlots = 256;

struct State {
    std::mutex mu;
    bool ready = false;
    int device = -1;
    int cus = 0;
    hipStream_t own = nullptr;   // created by init
    hipStream_t cur = nullptr;   // where ops launch (own or caller's)
    bool cur_is_own = true;
    hipStream_t copy = nullptr;  // uploads that overlap the ops (created on first use)
    hipEvent_t ev_ops = nullptr, ev_copy = nullptr;
    hipEvent_t t0 = nullptr, t1 = nullptr;
    float last_ms = -1.f;
    hipEvent_t slots[kEventSlots] = {};
    bool capturing = false;
    char arch[64] = "";
    // scratch memory of the ops that need some (products and convolutions cut along K, padded or masked operand
    // copies, conv2dGrad_f, matrixSoftmaxWithLoss_f): the caller's (swc_hip_set_workspace) or the library's own
    void *ws = nullptr;
    size_t ws_bytes = 0;
    bool ws_owned = false;
    bool ws_auto = false;   // the library may allocate and grow a buffer of its own (swc_hip_enable_auto_workspace)
    // executable graphs recorded while the library's own buffer was the workspace: their kernels keep its
    // address, so it is neither freed nor replaced before the last of them is destroyed
    void *graphs_on_own_ws[kGraphSlots] = {};
    int n_graphs_on_own_ws = 0;
} g;

Switches g_switches;
char g_switch_gemm[32], g_switch_conv[32];

// Reads the SWC_HIP_* variables into g_switches (see Switches).
void load_switches() {
    auto text = [](const char *name, char (&buf)[32]) -> const char * {
        const char *e = getenv(name);
        if (!e || !e[0]) return nullptr;
        snprintf(buf, sizeof(buf), "%s", e);
        return buf;
    };
    auto number = [](const char *name) {
        const char *e = getenv(name);
        const int v = e ? atoi(e) : 0;
        return v > 0 ? v : 0;
    };
    auto is = [](const char *name, const char *value) {
        const char *e = getenv(name);
        return e && !strcmp(e, value);
    };
    Switches s;
    s.gemm = text("SWC_HIP_GEMM", g_switch_gemm);
    s.conv = text("SWC_HIP_CONV", g_switch_conv);
    s.skinny_plain = is("SWC_HIP_SKINNY", "plain");
    s.conv_share = !is("SWC_HIP_CONV_SHARE", "0");
    s.conv_raster = is("SWC_HIP_CONV_ORDER", "raster");
    s.conv_lean = !is("SWC_HIP_CONV_LEAN", "0");
    s.conv_share_all = getenv("SWC_HIP_CONV_SHARE_ALL") ? (number("SWC_HIP_CONV_SHARE_ALL") ? number("SWC_HIP_CONV_SHARE_ALL") : -1) : 0;
    s.conv_slots = number("SWC_HIP_CONV_SLOTS");
    s.conv_piece_min = number("SWC_HIP_CONV_PIECE_MIN");
    s.conv_min_idle = getenv("SWC_HIP_CONV_MIN_IDLE") ? number("SWC_HIP_CONV_MIN_IDLE") : -1;
    s.conv_fair = !is("SWC_HIP_CONV_FAIR", "0");
    s.wgrad_bn = number("SWC_HIP_WGRAD_BN");
    g_switches = s;
}

template <typename T> __global__ void fill_kernel(T *__restrict__ dst, T v, size_t n) {
    size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    const size_t step = (size_t)gridDim.x * blockDim.x;
    for (; i < n; i += step) dst[i] = v;
}

} // namespace

int fail(int code, const char *fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_err, sizeof(g_err), fmt, ap);
    va_end(ap);
    g_err_code = code;
    return code;
}
thread_local char g_kernel[96] = "";
void note_kernel(const char *fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_kernel, sizeof(g_kernel), fmt, ap);
    va_end(ap);
}
void clear_error() { g_err[0] = 0, g_err_code = SWC_HIP_OK; }
int fail_code() { return g_err_code != SWC_HIP_OK ? g_err_code : SWC_HIP_ERUNTIME; }
const Switches &switches() { return g_switches; }
hipStream_t stream() { return g.cur; }
bool ready() { return g.ready; }
int num_cus() { return g.cus; }

// Device memory an op may use until it returns control to the stream's next op
// (all ops run on one in-order stream, so one buffer serves them all).  Ops never
// allocate: the buffer is the caller's (swc_hip_set_workspace), sized with the
// swc_hip_*_workspace_bytes queries.  Only a caller that opted in with
// swc_hip_enable_auto_workspace lets the library keep one of its own, grown on
// demand — never while a graph is being recorded, where allocating is not
// allowed, and never while a recorded graph still holds the old buffer's address.
void *workspace(size_t bytes, const char *who) {
    if (bytes <= g.ws_bytes && g.ws) return g.ws;
    if (g.ws && !g.ws_owned) {
        fail(SWC_HIP_EINVAL, "%s: the workspace given to swc_hip_set_workspace has %zu bytes, %zu are needed", who,
             g.ws_bytes, bytes);
        return nullptr;
    }
    if (!g.ws_auto) {
        fail(SWC_HIP_EINVAL, "%s: needs %zu bytes of scratch memory and no workspace is set: size one with "
             "swc_hip_gemm_workspace_bytes / swc_hip_conv2d_workspace_bytes / swc_hip_conv2dGrad_workspace_bytes / "
             "swc_hip_matrixSoftmaxWithLoss_workspace_bytes and pass it to swc_hip_set_workspace (ops do not allocate; "
             "swc_hip_enable_auto_workspace lets the library keep a buffer of its own)", who, bytes);
        return nullptr;
    }
    if (g.capturing) {
        fail(SWC_HIP_ERUNTIME, "%s: needs a %zu-byte workspace, which cannot be allocated while a graph is recorded; "
             "run the op once eagerly first or provide one with swc_hip_set_workspace", who, bytes);
        return nullptr;
    }
    if (g.ws && g.n_graphs_on_own_ws > 0) {
        fail(SWC_HIP_ERUNTIME, "%s: needs a %zu-byte workspace, but %d recorded graph(s) still use the library's "
             "%zu-byte buffer, which therefore cannot be replaced: destroy them first, or provide a workspace large "
             "enough for every op with swc_hip_set_workspace before recording", who, bytes, g.n_graphs_on_own_ws,
             g.ws_bytes);
        return nullptr;
    }
    if (g.ws) {
        (void)hipStreamSynchronize(g.cur);   // earlier ops may still be using it
        (void)hipFree(g.ws);
        g.ws = nullptr;
        g.ws_bytes = 0;
    }
    const size_t want = (bytes + ((size_t)1 << 20) - 1) & ~(((size_t)1 << 20) - 1);
    hipError_t e = hipMalloc(&g.ws, want);
    if (e != hipSuccess) {
        (void)hipGetLastError();
        g.ws = nullptr;
        fail(SWC_HIP_ERUNTIME, "%s: workspace of %zu bytes: %s", who, want, hipGetErrorString(e));
        return nullptr;
    }
    g.ws_bytes = want;
    g.ws_owned = true;
    return g.ws;
}

} // namespace swc_hip

using namespace swc_hip;

extern "C" {

int swc_hip_init(int device) {
    std::lock_guard<std::mutex> lk(g.mu);
    load_switches();
    if (g.ready) {
        if (device != g.device)
            return fail(SWC_HIP_EINVAL, "swc_hip_init: already initialised on device %d", g.device);
        return SWC_HIP_OK;
    }
    int count = 0;
    hipError_t e = hipGetDeviceCount(&count);
    if (e != hipSuccess || count <= 0)
        return fail(SWC_HIP_ERUNTIME, "swc_hip_init: no HIP device (%s)",
                    e == hipSuccess ? "device count is 0" : hipGetErrorString(e));
    if (device < 0 || device >= count)
        return fail(SWC_HIP_EINVAL, "swc_hip_init: device %d out of range [0,%d)", device, count);
    SWC_HIP_TRY(hipSetDevice(device));
    hipDeviceProp_t prop;
    SWC_HIP_TRY(hipGetDeviceProperties(&prop, device));
    snprintf(g.arch, sizeof(g.arch), "%s", prop.gcnArchName);
    if (std::strncmp(g.arch, Device::arch, std::strlen(Device::arch)) != 0)
        return fail(SWC_HIP_EUNSUPPORTED, "swc_hip_init: kernels are built for %s only, device is %s", Device::arch, g.arch);
    g.cus = prop.multiProcessorCount > 0 ? prop.multiProcessorCount : Device::computeUnits;
    if (int rc = gemm_noalloc_setup(device)) return rc;   // (the device is current here)
    SWC_HIP_TRY(hipStreamCreateWithFlags(&g.own, hipStreamNonBlocking));
    SWC_HIP_TRY(hipEventCreate(&g.t0));
    SWC_HIP_TRY(hipEventCreate(&g.t1));
    g.cur = g.own;
    g.cur_is_own = true;
    g.device = device;
    g.ready = true;
    clear_error();
    return SWC_HIP_OK;
}

int swc_hip_reload_switches(void) {
    std::lock_guard<std::mutex> lk(g.mu);
    if (g.capturing) return fail(SWC_HIP_EINVAL, "swc_hip_reload_switches: not while a graph is being recorded");
    load_switches();
    return SWC_HIP_OK;
}

int swc_hip_shutdown(void) {
    std::lock_guard<std::mutex> lk(g.mu);
    if (!g.ready) return SWC_HIP_OK;
    (void)hipStreamSynchronize(g.cur);
    if (g.ws && g.ws_owned) (void)hipFree(g.ws);
    g.ws = nullptr;
    g.ws_bytes = 0;
    g.ws_owned = false;
    g.ws_auto = false;
    g.n_graphs_on_own_ws = 0;
    for (void *&h : g.graphs_on_own_ws) h = nullptr;
    (void)hipEventDestroy(g.t0);
    (void)hipEventDestroy(g.t1);
    if (g.copy) {
        (void)hipStreamSynchronize(g.copy);
        (void)hipStreamDestroy(g.copy);
        (void)hipEventDestroy(g.ev_ops);
        (void)hipEventDestroy(g.ev_copy);
        g.copy = nullptr;
        g.ev_ops = g.ev_copy = nullptr;
    }
    for (hipEvent_t &e : g.slots)
        if (e) {
            (void)hipEventDestroy(e);
            e = nullptr;
        }
    g.capturing = false;
    g.last_ms = -1.f;
    (void)hipStreamDestroy(g.own);
    g.own = g.cur = nullptr;
    g.t0 = g.t1 = nullptr;
    g.ready = false;
    g.device = -1;
    return SWC_HIP_OK;
}

int swc_hip_set_workspace(void *dptr, size_t bytes) {
    SWC_REQUIRE_INIT();
    std::lock_guard<std::mutex> lk(g.mu);
    SWC_ARG((dptr == nullptr) == (bytes == 0));
    SWC_ARG(aligned16(dptr));
    if (g.capturing) return fail(SWC_HIP_EINVAL, "swc_hip_set_workspace: not while a graph is being recorded");
    if (g.ws && g.ws_owned) {
        if (g.n_graphs_on_own_ws > 0)
            return fail(SWC_HIP_ERUNTIME, "swc_hip_set_workspace: %d recorded graph(s) still use the library's own "
                        "buffer; destroy them before replacing it", g.n_graphs_on_own_ws);
        SWC_HIP_TRY(hipStreamSynchronize(g.cur));
        SWC_HIP_TRY(hipFree(g.ws));
    }
    g.ws = dptr;
    g.ws_bytes = bytes;
    g.ws_owned = false;
    return SWC_HIP_OK;
}

int swc_hip_enable_auto_workspace(int enable) {
    SWC_REQUIRE_INIT();
    std::lock_guard<std::mutex> lk(g.mu);
    g.ws_auto = enable != 0;
    return SWC_HIP_OK;
}

void *swc_hip_malloc(size_t bytes) {
    if (!ready()) {
        fail(SWC_HIP_ENOTINIT, "swc_hip_malloc: swc_hip_init has not been called");
        return nullptr;
    }
    void *p = nullptr;
    hipError_t e = hipMalloc(&p, bytes ? bytes : 1);
    if (e != hipSuccess) {
        fail(SWC_HIP_ERUNTIME, "swc_hip_malloc(%zu): %s", bytes, hipGetErrorString(e));
        (void)hipGetLastError();
        return nullptr;
    }
    return p;
}

int swc_hip_free(void *dptr) {
    SWC_REQUIRE_INIT();
    if (!dptr) return SWC_HIP_OK;
    SWC_HIP_TRY(hipStreamSynchronize(stream()));
    SWC_HIP_TRY(hipFree(dptr));
    return SWC_HIP_OK;
}

void *swc_hip_host_malloc(size_t bytes) {
    if (!ready()) {
        fail(SWC_HIP_ENOTINIT, "swc_hip_host_malloc: swc_hip_init has not been called");
        return nullptr;
    }
    void *p = nullptr;
    hipError_t e = hipHostMalloc(&p, bytes ? bytes : 1, hipHostMallocDefault);
    if (e != hipSuccess) {
        fail(SWC_HIP_ERUNTIME, "swc_hip_host_malloc(%zu): %s", bytes, hipGetErrorString(e));
        (void)hipGetLastError();
        return nullptr;
    }
    return p;
}

int swc_hip_host_free(void *p) {
    SWC_REQUIRE_INIT();
    if (!p) return SWC_HIP_OK;
    SWC_HIP_TRY(hipHostFree(p));
    return SWC_HIP_OK;
}

int swc_hip_h2d(void *dst, const void *src, size_t bytes) {
    SWC_REQUIRE_INIT();
    SWC_ARG(bytes == 0 || (dst && src));
    if (!bytes) return SWC_HIP_OK;
    SWC_HIP_TRY(hipMemcpyAsync(dst, src, bytes, hipMemcpyHostToDevice, stream()));
    SWC_HIP_TRY(hipStreamSynchronize(stream()));
    return SWC_HIP_OK;
}

int swc_hip_d2h(void *dst, const void *src, size_t bytes) {
    SWC_REQUIRE_INIT();
    SWC_ARG(bytes == 0 || (dst && src));
    if (!bytes) return SWC_HIP_OK;
    SWC_HIP_TRY(hipMemcpyAsync(dst, src, bytes, hipMemcpyDeviceToHost, stream()));
    SWC_HIP_TRY(hipStreamSynchronize(stream()));
    return SWC_HIP_OK;
}

int swc_hip_d2d(void *dst, const void *src, size_t bytes) {
    SWC_REQUIRE_INIT();
    SWC_ARG(bytes == 0 || (dst && src));
    if (!bytes) return SWC_HIP_OK;
    SWC_HIP_TRY(hipMemcpyAsync(dst, src, bytes, hipMemcpyDeviceToDevice, stream()));
    return SWC_HIP_OK;
}

// ---- uploads on a second stream, so that the next batch arrives while the ops work on this one ----
namespace {
int copy_stream_ready() {
    if (g.copy) return SWC_HIP_OK;
    std::lock_guard<std::mutex> lk(g.mu);
    if (g.copy) return SWC_HIP_OK;
    hipStream_t s = nullptr;
    SWC_HIP_TRY(hipStreamCreateWithFlags(&s, hipStreamNonBlocking));   // default priority, like the op stream
    SWC_HIP_TRY(hipEventCreateWithFlags(&g.ev_ops, hipEventDisableTiming));
    SWC_HIP_TRY(hipEventCreateWithFlags(&g.ev_copy, hipEventDisableTiming));
    g.copy = s;
    return SWC_HIP_OK;
}
} // namespace

int swc_hip_copy_h2d_async(void *dst, const void *src, size_t bytes) {
    SWC_REQUIRE_INIT();
    SWC_ARG(bytes == 0 || (dst && src));
    if (int rc = copy_stream_ready()) return rc;
    if (!bytes) return SWC_HIP_OK;
    SWC_HIP_TRY(hipMemcpyAsync(dst, src, bytes, hipMemcpyHostToDevice, g.copy));
    return SWC_HIP_OK;
}

int swc_hip_copy_wait_ops(void) {
    SWC_REQUIRE_INIT();
    if (g.capturing) return fail(SWC_HIP_EINVAL, "swc_hip_copy_wait_ops: not while a graph is being recorded");
    if (int rc = copy_stream_ready()) return rc;
    SWC_HIP_TRY(hipEventRecord(g.ev_ops, stream()));
    SWC_HIP_TRY(hipStreamWaitEvent(g.copy, g.ev_ops, 0));
    return SWC_HIP_OK;
}

int swc_hip_ops_wait_copies(void) {
    SWC_REQUIRE_INIT();
    if (g.capturing) return fail(SWC_HIP_EINVAL, "swc_hip_ops_wait_copies: not while a graph is being recorded");
    if (int rc = copy_stream_ready()) return rc;
    SWC_HIP_TRY(hipEventRecord(g.ev_copy, g.copy));
    SWC_HIP_TRY(hipStreamWaitEvent(stream(), g.ev_copy, 0));
    return SWC_HIP_OK;
}

int swc_hip_copy_sync(void) {
    SWC_REQUIRE_INIT();
    if (g.copy) SWC_HIP_TRY(hipStreamSynchronize(g.copy));
    return SWC_HIP_OK;
}

int swc_hip_fill_f(float *dst, float value, size_t count) {
    SWC_REQUIRE_INIT();
    SWC_ARG(count == 0 || dst);
    if (!count) return SWC_HIP_OK;
    unsigned blocks = ceil_div(count, 256);
    if (blocks > 4096u) blocks = 4096u;
    fill_kernel<<<blocks, 256, 0, stream()>>>(dst, value, count);
    SWC_LAUNCH_CHECK();
    return SWC_HIP_OK;
}

int swc_hip_fill_i(int *dst, int value, size_t count) {
    SWC_REQUIRE_INIT();
    SWC_ARG(count == 0 || dst);
    if (!count) return SWC_HIP_OK;
    unsigned blocks = ceil_div(count, 256);
    if (blocks > 4096u) blocks = 4096u;
    fill_kernel<<<blocks, 256, 0, stream()>>>(dst, value, count);
    SWC_LAUNCH_CHECK();
    return SWC_HIP_OK;
}

int swc_hip_device_cus(void) { return ready() ? g.cus : 0; }

int swc_hip_sync(void) {
    SWC_REQUIRE_INIT();
    SWC_HIP_TRY(hipStreamSynchronize(stream()));
    return SWC_HIP_OK;
}

const char *swc_hip_last_error(void) { return g_err; }

const char *swc_hip_last_kernel(void) { return g_kernel; }

void *swc_hip_stream(void) { return (void *)g.cur; }

int swc_hip_set_stream(void *s) {
    SWC_REQUIRE_INIT();
    std::lock_guard<std::mutex> lk(g.mu);
    if (s) {
        g.cur = (hipStream_t)s;
        g.cur_is_own = false;
    } else {
        g.cur = g.own;
        g.cur_is_own = true;
    }
    return SWC_HIP_OK;
}

const char *swc_hip_device_name(void) { return g.arch; }

int swc_hip_timer_begin(void) {
    SWC_REQUIRE_INIT();
    SWC_HIP_TRY(hipEventRecord(g.t0, stream()));
    return SWC_HIP_OK;
}

int swc_hip_timer_end(void) {
    SWC_REQUIRE_INIT();
    SWC_HIP_TRY(hipEventRecord(g.t1, stream()));
    SWC_HIP_TRY(hipEventSynchronize(g.t1));
    float ms = 0.f;
    SWC_HIP_TRY(hipEventElapsedTime(&ms, g.t0, g.t1));
    g.last_ms = ms;
    return SWC_HIP_OK;
}

float swc_hip_timer_elapsed_ms(void) { return g.last_ms; }

// ---- HIP graphs: capture the op sequence once, replay it with one launch ----
int swc_hip_graph_begin(void) {
    SWC_REQUIRE_INIT();
    if (g.capturing) return fail(SWC_HIP_EINVAL, "swc_hip_graph_begin: a capture is already open");
    SWC_HIP_TRY(hipStreamBeginCapture(stream(), hipStreamCaptureModeRelaxed));
    g.capturing = true;
    return SWC_HIP_OK;
}

int swc_hip_graph_end(void **graph_out) {
    SWC_REQUIRE_INIT();
    SWC_ARG(graph_out);
    if (!g.capturing) return fail(SWC_HIP_EINVAL, "swc_hip_graph_end: no capture is open");
    g.capturing = false;
    hipGraph_t graph = nullptr;
    SWC_HIP_TRY(hipStreamEndCapture(stream(), &graph));
    hipGraphExec_t exec = nullptr;
    hipError_t e = hipGraphInstantiate(&exec, graph, nullptr, nullptr, 0);
    (void)hipGraphDestroy(graph);
    if (e != hipSuccess) return fail(SWC_HIP_ERUNTIME, "swc_hip_graph_end: hipGraphInstantiate -> %s", hipGetErrorString(e));
    if (g.ws && g.ws_owned) {   // its kernels may hold the address of the library's own buffer
        int slot = 0;
        while (slot < kGraphSlots && g.graphs_on_own_ws[slot]) ++slot;
        if (slot == kGraphSlots) {
            (void)hipGraphExecDestroy(exec);
            return fail(SWC_HIP_ERUNTIME, "swc_hip_graph_end: more than %d graphs alive on the library's own workspace; "
                        "provide one with swc_hip_set_workspace", kGraphSlots);
        }
        g.graphs_on_own_ws[slot] = (void *)exec;
        ++g.n_graphs_on_own_ws;
    }
    *graph_out = (void *)exec;
    return SWC_HIP_OK;
}

int swc_hip_graph_launch(void *graph) {
    SWC_REQUIRE_INIT();
    SWC_ARG(graph);
    SWC_HIP_TRY(hipGraphLaunch((hipGraphExec_t)graph, stream()));
    return SWC_HIP_OK;
}

int swc_hip_graph_destroy(void *graph) {
    SWC_REQUIRE_INIT();
    if (!graph) return SWC_HIP_OK;
    SWC_HIP_TRY(hipStreamSynchronize(stream()));
    SWC_HIP_TRY(hipGraphExecDestroy((hipGraphExec_t)graph));
    for (void *&h : g.graphs_on_own_ws)
        if (h == graph) {
            h = nullptr;
            --g.n_graphs_on_own_ws;
        }
    return SWC_HIP_OK;
}

int swc_hip_event_record(int slot) {
    SWC_REQUIRE_INIT();
    SWC_ARG(slot >= 0 && slot < kEventSlots);
    if (!g.slots[slot]) SWC_HIP_TRY(hipEventCreate(&g.slots[slot]));
    SWC_HIP_TRY(hipEventRecord(g.slots[slot], stream()));
    return SWC_HIP_OK;
}

float swc_hip_event_elapsed_ms(int first, int second) {
    if (!ready() || first < 0 || second < 0 || first >= kEventSlots || second >= kEventSlots ||
        !g.slots[first] || !g.slots[second]) {
        fail(SWC_HIP_EINVAL, "swc_hip_event_elapsed_ms: slot not recorded");
        return -1.f;
    }
    if (hipEventSynchronize(g.slots[second]) != hipSuccess) return -1.f;
    float ms = -1.f;
    if (hipEventElapsedTime(&ms, g.slots[first], g.slots[second]) != hipSuccess) return -1.f;
    return ms;
}

} // extern "C"
