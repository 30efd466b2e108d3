"""ctypes binding of libswc_hip.so (C ABI declared in include/swc_hip.h).

Method names and argument order mirror the reference's CPU kernels
(src/codegen/utils/kernels.h) — the same correspondence the C ABI keeps — so a
parity test reads like a call sequence of the reference's generated program.
Data lives in DeviceArray objects (device memory + shape); numpy arrays cross
only through upload()/download().

No fallback: a missing library or device raises SwcHipError.
"""
import ctypes as C
import os

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))

EXPORTS = [
    "swc_hip_init", "swc_hip_shutdown", "swc_hip_malloc", "swc_hip_free", "swc_hip_h2d", "swc_hip_d2h",
    "swc_hip_d2d", "swc_hip_copy_h2d_async", "swc_hip_copy_wait_ops", "swc_hip_ops_wait_copies", "swc_hip_copy_sync", "swc_hip_fill_f", "swc_hip_sync", "swc_hip_last_error", "swc_hip_stream",
    "swc_hip_set_stream", "swc_hip_device_name", "swc_hip_timer_begin", "swc_hip_timer_end",
    "swc_hip_timer_elapsed_ms", "swc_hip_event_record", "swc_hip_event_elapsed_ms", "swc_hip_graph_begin",
    "swc_hip_graph_end", "swc_hip_graph_launch", "swc_hip_graph_destroy", "swc_hip_device_cus", "swc_hip_last_kernel", "swc_hip_reload_switches",
    "swc_hip_enable_auto_workspace", "swc_hip_conv2dGrad_workspace_bytes", "swc_hip_matrixSoftmaxWithLoss_workspace_bytes",
    "swc_hip_matrixMatrixFCBias_noalloc_f",
    "swc_hip_matrixMatrixMul_f", "swc_hip_batchedadd_f", "swc_hip_relu_f",
    "swc_hip_vecAdd_f", "swc_hip_conv2d_f", "swc_hip_batchnormalization_f", "swc_hip_maxpool_f",
    "swc_hip_maxpool_argmax_f", "swc_hip_avgpool_f", "swc_hip_transpose4d_f", "swc_hip_transpose2d_f",
    "swc_hip_matrixSoftmax_f", "swc_hip_matrixTanh_f", "swc_hip_argMax_i", "swc_hip_accuracy_i", "swc_hip_fill_i",
    "swc_hip_matrixMatrixFCBias_f", "swc_hip_vecAddRelu_f", "swc_hip_batchnormRelu_f",
    "swc_hip_batchnormReluMaxpool_f", "swc_hip_conv2dFused_f", "swc_hip_conv2dFusedAdd_f",
    "swc_hip_conv2dFusedMaxpool_f", "swc_hip_conv2dFusedMaxpool_workspace_bytes",
    "swc_hip_set_workspace", "swc_hip_matrixMatrixFCBiasSoftmax_f", "swc_hip_gemm_workspace_bytes", "swc_hip_conv2d_workspace_bytes", "swc_hip_host_malloc", "swc_hip_host_free", "swc_hip_matrixTrans_f", "swc_hip_matrixTanhGrad_f", "swc_hip_matrixSoftmaxWithLoss_f",
    "swc_hip_matrixSoftmaxGrad_f", "swc_hip_matrixSoftmaxWithLossGrad_f", "swc_hip_conv2dGrad_f",
    "swc_hip_maxpoolGrad_f", "swc_hip_batchedreduceadd_f", "swc_hip_sgd_f", "swc_hip_reluGrad_f",
]


class SwcHipError(RuntimeError):
    pass


def lib_path():
    return os.path.join(_HERE, "libswc_hip.so")


def load_library():
    """dlopen the in-tree library; raises if it has not been built."""
    path = lib_path()
    if not os.path.exists(path):
        raise SwcHipError(f"{path} is missing: build it with `python -m swcompiler_amd.build` "
                          "(there is no CPU fallback)")
    lib = C.CDLL(path)
    vp, sz, i32, f32 = C.c_void_p, C.c_size_t, C.c_int, C.c_float
    szp = C.POINTER(C.c_size_t)
    sig = {
        "swc_hip_init": (i32, [i32]),
        "swc_hip_shutdown": (i32, []),
        "swc_hip_reload_switches": (i32, []),
        "swc_hip_malloc": (vp, [sz]),
        "swc_hip_free": (i32, [vp]),
        "swc_hip_h2d": (i32, [vp, vp, sz]),
        "swc_hip_d2h": (i32, [vp, vp, sz]),
        "swc_hip_d2d": (i32, [vp, vp, sz]),
        "swc_hip_fill_f": (i32, [vp, f32, sz]),
        "swc_hip_copy_h2d_async": (i32, [vp, vp, sz]),
        "swc_hip_copy_wait_ops": (i32, []),
        "swc_hip_ops_wait_copies": (i32, []),
        "swc_hip_copy_sync": (i32, []),
        "swc_hip_sync": (i32, []),
        "swc_hip_last_error": (C.c_char_p, []),
        "swc_hip_stream": (vp, []),
        "swc_hip_set_stream": (i32, [vp]),
        "swc_hip_device_name": (C.c_char_p, []),
        "swc_hip_timer_begin": (i32, []),
        "swc_hip_timer_end": (i32, []),
        "swc_hip_timer_elapsed_ms": (f32, []),
        "swc_hip_event_record": (i32, [i32]),
        "swc_hip_event_elapsed_ms": (f32, [i32, i32]),
        "swc_hip_graph_begin": (i32, []),
        "swc_hip_graph_end": (i32, [C.POINTER(vp)]),
        "swc_hip_graph_launch": (i32, [vp]),
        "swc_hip_graph_destroy": (i32, [vp]),
        "swc_hip_device_cus": (i32, []),
        "swc_hip_last_kernel": (C.c_char_p, []),
        "swc_hip_enable_auto_workspace": (i32, [i32]),
        "swc_hip_conv2dGrad_workspace_bytes": (sz, [szp] * 6 + [sz]),
        "swc_hip_matrixSoftmaxWithLoss_workspace_bytes": (sz, [i32, i32]),
        "swc_hip_matrixMatrixFCBias_noalloc_f": (i32, [i32, i32, i32, vp, i32, vp, i32, vp, vp, i32, i32]),
        "swc_hip_matrixMatrixMul_f": (i32, [i32, i32, i32, vp, i32, vp, i32, vp, i32]),
        "swc_hip_batchedadd_f": (i32, [vp, vp, vp, sz, sz]),
        "swc_hip_relu_f": (i32, [vp, vp, sz]),
        "swc_hip_vecAdd_f": (i32, [i32, vp, vp, vp]),
        "swc_hip_conv2d_f": (i32, [vp, vp, vp, vp, szp, szp, szp, szp, szp, szp, szp, sz]),
        "swc_hip_batchnormalization_f": (i32, [vp, vp, vp, vp, vp, vp, szp, f32]),
        "swc_hip_maxpool_f": (i32, [vp, vp, szp, szp, szp, szp, szp]),
        "swc_hip_maxpool_argmax_f": (i32, [vp, vp, vp, szp, szp, szp, szp, szp]),
        "swc_hip_avgpool_f": (i32, [vp, vp, szp, szp, szp, szp, szp]),
        "swc_hip_transpose4d_f": (i32, [vp, vp, szp, szp, szp]),
        "swc_hip_transpose2d_f": (i32, [vp, vp, szp, szp, szp]),
        "swc_hip_matrixSoftmax_f": (i32, [i32, i32, vp, i32, vp, i32]),
        "swc_hip_matrixTanh_f": (i32, [i32, i32, vp, i32, vp, i32]),
        "swc_hip_argMax_i": (i32, [vp, vp, i32, i32, i32]),
        "swc_hip_accuracy_i": (i32, [vp, vp, vp, i32, i32]),
        "swc_hip_fill_i": (i32, [vp, i32, sz]),
        "swc_hip_matrixMatrixFCBias_f": (i32, [i32, i32, i32, vp, i32, vp, i32, vp, vp, i32, i32]),
        "swc_hip_matrixMatrixFCBiasSoftmax_f": (i32, [i32, i32, i32, vp, i32, vp, i32, vp, vp, i32]),
        "swc_hip_vecAddRelu_f": (i32, [i32, vp, vp, vp]),
        "swc_hip_batchnormRelu_f": (i32, [vp, vp, vp, vp, vp, vp, szp, f32]),
        "swc_hip_batchnormReluMaxpool_f": (i32, [vp, vp, vp, vp, vp, vp, szp, f32, szp, szp, szp, szp]),
        "swc_hip_conv2dFused_f": (i32, [vp, vp, vp, vp, szp, szp, szp, szp, szp, szp, szp, sz,
                                        vp, vp, vp, vp, f32, i32]),
        "swc_hip_conv2dFusedAdd_f": (i32, [vp, vp, vp, vp, szp, szp, szp, szp, szp, szp, szp, sz,
                                        vp, vp, vp, vp, f32, vp, i32]),
        "swc_hip_conv2dFusedMaxpool_f": (i32, [vp, vp, vp, vp, szp, szp, szp, szp, szp, szp, szp, sz,
                                            vp, vp, vp, vp, f32, i32, szp, szp, szp, szp]),
        "swc_hip_conv2dFusedMaxpool_workspace_bytes": (sz, [szp] * 6 + [sz] + [szp] * 4),
        "swc_hip_set_workspace": (i32, [vp, sz]),
        "swc_hip_host_malloc": (vp, [sz]),
        "swc_hip_host_free": (i32, [vp]),
        "swc_hip_gemm_workspace_bytes": (sz, [i32, i32, i32]),
        "swc_hip_conv2d_workspace_bytes": (sz, [szp] * 6 + [sz]),
        "swc_hip_matrixTrans_f": (i32, [i32, i32, vp, i32, vp, i32]),
        "swc_hip_matrixTanhGrad_f": (i32, [i32, i32, vp, i32, vp, i32, vp, i32]),
        "swc_hip_matrixSoftmaxWithLoss_f": (i32, [i32, i32, vp, i32, vp, i32, vp, vp]),
        "swc_hip_matrixSoftmaxGrad_f": (i32, [i32, i32, vp, i32, vp, i32, vp]),
        "swc_hip_matrixSoftmaxWithLossGrad_f": (i32, [i32, i32, vp, i32, vp, i32, vp]),
        "swc_hip_conv2dGrad_f": (i32, [vp, vp, vp, vp, vp, vp, szp, szp, szp, szp, szp, szp, szp, sz]),
        "swc_hip_maxpoolGrad_f": (i32, [vp, vp, vp, szp, szp, szp, szp, szp]),
        "swc_hip_batchedreduceadd_f": (i32, [vp, vp, sz, sz]),
        "swc_hip_sgd_f": (i32, [sz, vp, vp, vp, vp, f32, f32, f32, sz]),
        "swc_hip_reluGrad_f": (i32, [vp, vp, vp, sz]),
    }
    for name, (res, args) in sig.items():
        fn = getattr(lib, name)
        fn.restype, fn.argtypes = res, args
    return lib


def _dims(seq):
    return (C.c_size_t * len(seq))(*[int(v) for v in seq])


def pool_out_dims(idims, kernels, strides, pads):
    """src/op/dlOp/dlOp.cpp:195-196: o = (i + pad_begin + pad_end - k) / s + 1, pads = {t,l,b,r}."""
    n, h, w, c = idims
    return (n, (h + pads[0] + pads[2] - kernels[0]) // strides[0] + 1,
            (w + pads[1] + pads[3] - kernels[1]) // strides[1] + 1, c)


class DeviceArray:
    """A device allocation with a shape and dtype (float32 or int32)."""

    def __init__(self, rt, shape, dtype=np.float32):
        self.rt = rt
        self.shape = tuple(int(s) for s in shape)
        self.dtype = np.dtype(dtype)
        self.size = int(np.prod(self.shape)) if self.shape else 1
        self.nbytes = self.size * self.dtype.itemsize
        self.ptr = rt._malloc(self.nbytes)

    def reshape(self, *shape):
        view = object.__new__(DeviceArray)
        view.__dict__.update(self.__dict__)
        shape = tuple(shape[0]) if len(shape) == 1 and not np.isscalar(shape[0]) else tuple(shape)
        if -1 in shape:
            known = int(np.prod([s for s in shape if s != -1]))
            shape = tuple(self.size // known if s == -1 else s for s in shape)
        view.shape = tuple(int(s) for s in shape)
        assert int(np.prod(view.shape)) == self.size
        view._base = self  # keep the owner alive; views never free
        return view

    def numpy(self):
        return self.rt.download(self)

    def offset_view(self, first, shape):
        """A view starting `first` elements in (to exercise unaligned pointers)."""
        view = self.reshape(self.shape)
        view.shape = tuple(int(s) for s in shape)
        view.size = int(np.prod(view.shape))
        assert first + view.size <= self.size
        view.nbytes = view.size * self.dtype.itemsize
        view.ptr = self.ptr + first * self.dtype.itemsize
        return view

    def free(self):
        if getattr(self, "_base", None) is None and self.ptr:
            self.rt._free(self.ptr)
        self.ptr = None

    def __del__(self):
        try:
            self.free()
        except Exception:
            pass


class SwcHip:
    """One process-wide runtime: device 0 unless told otherwise."""

    def __init__(self, device=0, auto_workspace=True):
        """auto_workspace: let the library keep (and grow) a scratch buffer of its own, as a harness that calls
        ops of many shapes wants; False: ops that need scratch fail until set_workspace() provides it, as in a
        generated program."""
        self.lib = load_library()
        self._check(self.lib.swc_hip_init(device), "swc_hip_init")
        self._check(self.lib.swc_hip_enable_auto_workspace(int(auto_workspace)), "swc_hip_enable_auto_workspace")
        self._pinned = {}   # address of a pinned numpy array -> the pointer to free
        self._bench_lib = None

    def enable_auto_workspace(self, on):
        self._check(self.lib.swc_hip_enable_auto_workspace(int(on)), "swc_hip_enable_auto_workspace")

    def last_kernel(self):
        """the kernel variant the last FC/GEMM or convolution call dispatched to"""
        return self.lib.swc_hip_last_kernel().decode()

    def device_cus(self):
        return int(self.lib.swc_hip_device_cus())

    def reload_switches(self):
        """have the library read the SWC_HIP_* environment variables again (it reads them once, at init)"""
        self._check(self.lib.swc_hip_reload_switches(), "swc_hip_reload_switches")

    # -- plumbing --------------------------------------------------------
    def _check(self, rc, what):
        if rc != 0:
            raise SwcHipError(f"{what} failed ({rc}): {self.lib.swc_hip_last_error().decode()}")

    def _malloc(self, nbytes):
        p = self.lib.swc_hip_malloc(nbytes)
        if not p:
            raise SwcHipError(self.lib.swc_hip_last_error().decode())
        return p

    def _free(self, ptr):
        self.lib.swc_hip_free(ptr)

    def device_name(self):
        return self.lib.swc_hip_device_name().decode()

    def empty(self, shape, dtype=np.float32):
        return DeviceArray(self, shape, dtype)

    def upload(self, host):
        host = np.ascontiguousarray(host)
        assert host.dtype in (np.float32, np.int32)
        d = DeviceArray(self, host.shape, host.dtype)
        self._check(self.lib.swc_hip_h2d(d.ptr, host.ctypes.data, host.nbytes), "swc_hip_h2d")
        return d

    def download(self, d):
        host = np.empty(d.shape, d.dtype)
        self._check(self.lib.swc_hip_d2h(host.ctypes.data, d.ptr, d.nbytes), "swc_hip_d2h")
        return host

    def upload_into(self, d, host):
        """h2d into an existing allocation of the same size"""
        host = np.ascontiguousarray(host)
        assert host.nbytes == d.nbytes
        self._check(self.lib.swc_hip_h2d(d.ptr, host.ctypes.data, host.nbytes), "swc_hip_h2d")

    def download_into(self, host, d):
        assert host.nbytes == d.nbytes and host.flags.c_contiguous
        self._check(self.lib.swc_hip_d2h(host.ctypes.data, d.ptr, d.nbytes), "swc_hip_d2h")

    def d2d(self, dst, src):
        """device-to-device copy on the op stream (asynchronous)"""
        assert dst.nbytes == src.nbytes
        self._check(self.lib.swc_hip_d2d(dst.ptr, src.ptr, src.nbytes), "swc_hip_d2d")

    # uploads on the library's second stream (see include/swc_hip.h)
    def copy_h2d_async(self, d, pinned_host):
        assert pinned_host.nbytes == d.nbytes
        self._check(self.lib.swc_hip_copy_h2d_async(d.ptr, pinned_host.ctypes.data, d.nbytes), "swc_hip_copy_h2d_async")

    def copy_wait_ops(self):
        self._check(self.lib.swc_hip_copy_wait_ops(), "swc_hip_copy_wait_ops")

    def ops_wait_copies(self):
        self._check(self.lib.swc_hip_ops_wait_copies(), "swc_hip_ops_wait_copies")

    def copy_sync(self):
        self._check(self.lib.swc_hip_copy_sync(), "swc_hip_copy_sync")

    def _bench(self):
        """the bench-only helper library (include/swc_hip_bench.h), loaded on first use"""
        if self._bench_lib is None:
            path = os.path.join(_HERE, "libswc_hip_bench.so")
            if not os.path.exists(path):
                raise SwcHipError(f"{path} is missing: build it with `python -m swcompiler_amd.build`")
            self._bench_lib = C.CDLL(path)
            self._bench_lib.swc_hip_bench_probe_mfma_f32.restype = C.c_int
            self._bench_lib.swc_hip_bench_probe_mfma_f32.argtypes = [C.c_void_p, C.c_int, C.c_void_p, C.c_size_t, C.c_int,
                                                                     C.POINTER(C.c_float), C.POINTER(C.c_double)]
            self._bench_lib.swc_hip_bench_clock_watch_start.restype = C.c_int
            self._bench_lib.swc_hip_bench_clock_watch_start.argtypes = [C.c_void_p, C.c_int, C.c_int]
            self._bench_lib.swc_hip_bench_clock_watch_wait.restype = C.c_int
            self._bench_lib.swc_hip_bench_clock_watch_wait.argtypes = []
        return self._bench_lib

    def shader_clock_ghz(self, fn, op_ms, watch_ms=4.0):
        """The shader clock (GHz) while `fn` — which enqueues one op of about op_ms on the library's stream — runs
        back to back: a one-wavefront watcher of the bench-only library notes the 100 MHz wall clock and the shader
        clock counter every ~3.5 us on a stream of its own for watch_ms; fn is enqueued often enough to outlast it;
        the figure is the median over consecutive samples of the middle 80 % of the watch."""
        import numpy as np
        lib = self._bench()
        n = max(16, int(watch_ms * 1e3 / 3.6))
        samples = self.empty((4 * n,))          # 2 n 64-bit words
        self.sync()
        rc = lib.swc_hip_bench_clock_watch_start(samples.ptr, n, 1)
        if rc != 0:
            raise SwcHipError(f"swc_hip_bench_clock_watch_start failed (hipError {rc})")
        for _ in range(max(3, int(1.5 * watch_ms / max(op_ms, 1e-3)) + 2)):
            fn()
        rc = lib.swc_hip_bench_clock_watch_wait()
        self.sync()
        if rc != 0:
            raise SwcHipError(f"swc_hip_bench_clock_watch_wait failed (hipError {rc})")
        s = samples.numpy().view(np.uint64).reshape(n, 2).astype(np.float64)
        samples.free()
        s = s[n // 10: n - n // 10]
        d = np.diff(s, axis=0)
        return float(np.median(0.1 * d[:, 1] / d[:, 0]))

    def probe_mfma_tflops(self, iters=2000):
        """fp32 MFMA rate a register-only loop sustains (TFLOP/s) and its duration in ms; runs the bench-only
        helper library (include/swc_hip_bench.h) on the library's stream"""
        self._bench()
        self.sync()
        scratch = self.empty((512 * 512,))
        ms, flop = C.c_float(), C.c_double()
        rc = self._bench_lib.swc_hip_bench_probe_mfma_f32(self.lib.swc_hip_stream(), self.device_cus(), scratch.ptr,
                                                          scratch.size, iters, C.byref(ms), C.byref(flop))
        if rc != 0:
            raise SwcHipError(f"swc_hip_bench_probe_mfma_f32 failed (hipError {rc})")
        scratch.free()
        return flop.value / (ms.value * 1e-3) / 1e12, ms.value

    def sync(self):
        self._check(self.lib.swc_hip_sync(), "swc_hip_sync")

    def timer_begin(self):
        self._check(self.lib.swc_hip_timer_begin(), "swc_hip_timer_begin")

    def timer_end_ms(self):
        self._check(self.lib.swc_hip_timer_end(), "swc_hip_timer_end")
        return float(self.lib.swc_hip_timer_elapsed_ms())

    def event_record(self, slot):
        self._check(self.lib.swc_hip_event_record(slot), "swc_hip_event_record")

    def event_elapsed_ms(self, first, second):
        ms = float(self.lib.swc_hip_event_elapsed_ms(first, second))
        if ms < 0:
            raise SwcHipError("swc_hip_event_elapsed_ms failed: " + self.lib.swc_hip_last_error().decode())
        return ms

    def capture(self, fn):
        """Records the ops `fn()` issues into a HIP graph; returns a handle for graph_launch()."""
        self._check(self.lib.swc_hip_graph_begin(), "swc_hip_graph_begin")
        try:
            fn()
        finally:
            handle = C.c_void_p()
            rc = self.lib.swc_hip_graph_end(C.byref(handle))
        self._check(rc, "swc_hip_graph_end")
        return handle

    def graph_launch(self, handle):
        self._check(self.lib.swc_hip_graph_launch(handle), "swc_hip_graph_launch")

    def graph_destroy(self, handle):
        self._check(self.lib.swc_hip_graph_destroy(handle), "swc_hip_graph_destroy")

    # -- ops (device in, device out) -------------------------------------
    def matrixMatrixMul(self, a, b, out=None):
        m, k = a.shape
        k2, n = b.shape
        assert k == k2
        out = out if out is not None else self.empty((m, n))
        self._check(self.lib.swc_hip_matrixMatrixMul_f(m, n, k, a.ptr, k, b.ptr, n, out.ptr, n), "matrixMatrixMul_f")
        return out

    def batchedadd(self, batch, slice_, out=None):
        rows, cols = batch.shape
        out = out if out is not None else self.empty(batch.shape)
        self._check(self.lib.swc_hip_batchedadd_f(out.ptr, batch.ptr, slice_.ptr, rows, cols), "batchedadd_f")
        return out

    def fcbias(self, a, w, bias, relu=False, softmax=False, out=None):
        """a @ w + bias, then ReLU or the row softmax (the fused calls of the HIP target)"""
        m, k = a.shape
        k2, n = w.shape
        assert k == k2 and not (relu and softmax)
        out = out if out is not None else self.empty((m, n))
        bptr = bias.ptr if bias is not None else None
        if softmax:
            self._check(self.lib.swc_hip_matrixMatrixFCBiasSoftmax_f(m, n, k, a.ptr, k, w.ptr, n, bptr, out.ptr, n),
                        "matrixMatrixFCBiasSoftmax_f")
        else:
            self._check(self.lib.swc_hip_matrixMatrixFCBias_f(m, n, k, a.ptr, k, w.ptr, n, bptr, out.ptr, n, int(relu)),
                        "matrixMatrixFCBias_f")
        return out

    def fcbias_noalloc(self, a, w, bias, relu=False, out=None):
        """fcbias through the entry point that allocates nothing (fixed scratch inside the library)"""
        m, k = a.shape
        k2, n = w.shape
        assert k == k2
        out = out if out is not None else self.empty((m, n))
        bptr = bias.ptr if bias is not None else None
        self._check(self.lib.swc_hip_matrixMatrixFCBias_noalloc_f(m, n, k, a.ptr, k, w.ptr, n, bptr, out.ptr, n, int(relu)),
                    "matrixMatrixFCBias_noalloc_f")
        return out

    def relu(self, x, out=None):
        out = out if out is not None else self.empty(x.shape)
        self._check(self.lib.swc_hip_relu_f(x.ptr, out.ptr, x.size), "relu_f")
        return out

    def vecAdd(self, a, b, out=None, relu=False):
        assert a.shape == b.shape
        out = out if out is not None else self.empty(a.shape)
        fn = self.lib.swc_hip_vecAddRelu_f if relu else self.lib.swc_hip_vecAdd_f
        self._check(fn(a.size, a.ptr, b.ptr, out.ptr), "vecAdd_f")
        return out

    def matrixTanh(self, a, out=None):
        m, n = a.shape
        out = out if out is not None else self.empty(a.shape)
        self._check(self.lib.swc_hip_matrixTanh_f(m, n, a.ptr, n, out.ptr, n), "matrixTanh_f")
        return out

    def matrixSoftmax(self, a, out=None):
        m, n = a.shape
        out = out if out is not None else self.empty(a.shape)
        self._check(self.lib.swc_hip_matrixSoftmax_f(m, n, a.ptr, n, out.ptr, n), "matrixSoftmax_f")
        return out

    def argMax(self, x, top_k):
        m, n = x.shape
        out = self.empty((m, top_k), np.int32)
        self._check(self.lib.swc_hip_argMax_i(x.ptr, out.ptr, m, n, top_k), "argMax_i")
        return out

    def accuracy(self, pred, label, counters):
        """adds this batch to the device counters [hits, rows] (int32[2]) and returns them"""
        m, n = pred.shape
        self._check(self.lib.swc_hip_accuracy_i(pred.ptr, label.ptr, counters.ptr, m, n), "accuracy_i")
        return counters

    def fill_i(self, t, value):
        self._check(self.lib.swc_hip_fill_i(t.ptr, int(value), t.size), "fill_i")
        return t

    def conv2d(self, x, filt, bias, kernels=None, strides=(1, 1), pads=(0, 0, 0, 0), group=1, bn=None,
               eps=1e-5, relu=False, out=None, residual=None, pool=None):
        """bn = (mean, var, scale, bias) DeviceArrays to fuse inference batchnorm; pool = (kernels, strides[, pads])
        to max-pool the result in the same call (the result is then the pooled tensor)."""
        if kernels is None:
            kernels = filt.shape[1:3]
        n, oh, ow, _ = pool_out_dims(x.shape, kernels, strides, pads)
        odims = (n, oh, ow, filt.shape[0])
        if pool is not None:
            assert residual is None
            pk, ps = pool[0], pool[1]
            pp = pool[2] if len(pool) > 2 else (0, 0, 0, 0)
            pdims = pool_out_dims(odims, pk, ps, pp)
            out = out if out is not None else self.empty(pdims)
            ptrs = [p.ptr for p in bn] if bn is not None else [None] * 4
            self._check(self.lib.swc_hip_conv2dFusedMaxpool_f(
                out.ptr, x.ptr, filt.ptr, bias.ptr, _dims(odims), _dims(x.shape), _dims(filt.shape), _dims(bias.shape),
                _dims(kernels), _dims(strides), _dims(pads), group, *ptrs, eps, int(relu), _dims(pdims), _dims(pk),
                _dims(ps), _dims(pp)), "conv2dFusedMaxpool_f")
            return out
        out = out if out is not None else self.empty(odims)
        shp = (_dims(odims), _dims(x.shape), _dims(filt.shape), _dims(bias.shape), _dims(kernels),
               _dims(strides), _dims(pads))
        if residual is not None:
            assert tuple(residual.shape) == tuple(odims)
            ptrs = [p.ptr for p in bn] if bn is not None else [None] * 4
            rc = self.lib.swc_hip_conv2dFusedAdd_f(out.ptr, x.ptr, filt.ptr, bias.ptr, *shp, group, *ptrs,
                                                   eps, residual.ptr, int(relu))
        elif bn is None and not relu:
            rc = self.lib.swc_hip_conv2d_f(out.ptr, x.ptr, filt.ptr, bias.ptr, *shp, group)
        else:
            ptrs = [p.ptr for p in bn] if bn is not None else [None] * 4
            rc = self.lib.swc_hip_conv2dFused_f(out.ptr, x.ptr, filt.ptr, bias.ptr, *shp, group, *ptrs,
                                                eps, int(relu))
        self._check(rc, "conv2d_f")
        return out

    def batchnormalization(self, x, mean, var, scale, bias, eps, relu=False, out=None):
        out = out if out is not None else self.empty(x.shape)
        fn = self.lib.swc_hip_batchnormRelu_f if relu else self.lib.swc_hip_batchnormalization_f
        self._check(fn(out.ptr, x.ptr, mean.ptr, var.ptr, scale.ptr, bias.ptr, _dims(x.shape), eps),
                    "batchnormalization_f")
        return out

    def maxpool(self, x, kernels, strides, pads=(0, 0, 0, 0), out=None):
        odims = pool_out_dims(x.shape, kernels, strides, pads)
        out = out if out is not None else self.empty(odims)
        self._check(self.lib.swc_hip_maxpool_f(x.ptr, out.ptr, _dims(x.shape), _dims(odims), _dims(kernels),
                                               _dims(strides), _dims(pads)), "maxpool_f")
        return out

    def avgpool(self, x, kernels, strides, pads=(0, 0, 0, 0), out=None):
        odims = pool_out_dims(x.shape, kernels, strides, pads)
        out = out if out is not None else self.empty(odims)
        self._check(self.lib.swc_hip_avgpool_f(x.ptr, out.ptr, _dims(x.shape), _dims(odims), _dims(kernels),
                                               _dims(strides), _dims(pads)), "avgpool_f")
        return out

    def transpose(self, x, shuffle, out=None):
        """out axis a = in axis shuffle[a] (2-D or 4-D)."""
        odims = tuple(x.shape[s] for s in shuffle)
        out = out if out is not None else self.empty(odims)
        fn = self.lib.swc_hip_transpose4d_f if len(x.shape) == 4 else self.lib.swc_hip_transpose2d_f
        self._check(fn(x.ptr, out.ptr, _dims(x.shape), _dims(odims), _dims(shuffle)), "transpose_f")
        return out

    def maxpool_argmax(self, x, kernels, strides, pads=(0, 0, 0, 0)):
        odims = pool_out_dims(x.shape, kernels, strides, pads)
        out, idx = self.empty(odims), self.empty(odims, np.int32)
        self._check(self.lib.swc_hip_maxpool_argmax_f(x.ptr, out.ptr, idx.ptr, _dims(x.shape), _dims(odims),
                                                      _dims(kernels), _dims(strides), _dims(pads)),
                    "maxpool_argmax_f")
        return out, idx

    def batchnormReluMaxpool(self, x, mean, var, scale, bias, eps, kernels, strides, pads=(0, 0, 0, 0), out=None):
        odims = pool_out_dims(x.shape, kernels, strides, pads)
        out = out if out is not None else self.empty(odims)
        self._check(self.lib.swc_hip_batchnormReluMaxpool_f(out.ptr, x.ptr, mean.ptr, var.ptr, scale.ptr, bias.ptr,
                                                            _dims(x.shape), eps, _dims(odims), _dims(kernels),
                                                            _dims(strides), _dims(pads)), "batchnormReluMaxpool_f")
        return out


    # -- training kernels ------------------------------------------------
    def matrixTrans(self, a):
        m, n = a.shape
        out = self.empty((n, m))
        self._check(self.lib.swc_hip_matrixTrans_f(m, n, a.ptr, n, out.ptr, m), "matrixTrans_f")
        return out

    def matrixTanhGrad(self, out_, out_grad):
        m, n = out_.shape
        ig = self.empty(out_.shape)
        self._check(self.lib.swc_hip_matrixTanhGrad_f(m, n, ig.ptr, n, out_.ptr, n, out_grad.ptr, n), "matrixTanhGrad_f")
        return ig

    def matrixSoftmaxWithLoss(self, a, selected):
        """-> (probabilities DeviceArray, loss as a python float)"""
        m, n = a.shape
        out, loss = self.empty(a.shape), self.empty((1,))
        self._check(self.lib.swc_hip_matrixSoftmaxWithLoss_f(m, n, a.ptr, n, out.ptr, n, selected.ptr, loss.ptr),
                    "matrixSoftmaxWithLoss_f")
        return out, float(loss.numpy()[0])

    def matrixSoftmaxGrad(self, prob, selected, with_loss=False):
        m, n = prob.shape
        ig = self.empty(prob.shape)
        fn = self.lib.swc_hip_matrixSoftmaxWithLossGrad_f if with_loss else self.lib.swc_hip_matrixSoftmaxGrad_f
        self._check(fn(m, n, ig.ptr, n, prob.ptr, n, selected.ptr), "matrixSoftmaxGrad_f")
        return ig

    def conv2dGrad(self, x, filt, out_grad, kernels=None, strides=(1, 1), pads=(0, 0, 0, 0), group=1, out=None):
        if kernels is None:
            kernels = filt.shape[1:3]
        ig, fg, bg = out if out is not None else (self.empty(x.shape), self.empty(filt.shape), self.empty((filt.shape[0],)))
        self._check(self.lib.swc_hip_conv2dGrad_f(ig.ptr, fg.ptr, bg.ptr, out_grad.ptr, x.ptr, filt.ptr,
                                                  _dims(out_grad.shape), _dims(x.shape), _dims(filt.shape),
                                                  _dims(bg.shape), _dims(kernels), _dims(strides), _dims(pads), group),
                    "conv2dGrad_f")
        return ig, fg, bg

    def maxpoolGrad(self, x, out_grad, kernels, strides, pads=(0, 0, 0, 0), out=None):
        ig = out.reshape(x.shape) if out is not None else self.empty(x.shape)
        self._check(self.lib.swc_hip_maxpoolGrad_f(ig.ptr, out_grad.ptr, x.ptr, _dims(x.shape), _dims(out_grad.shape),
                                                   _dims(kernels), _dims(strides), _dims(pads)), "maxpoolGrad_f")
        return ig

    def batchedreduceadd(self, batch):
        ns, ss = batch.shape
        out = self.empty((ns,))
        self._check(self.lib.swc_hip_batchedreduceadd_f(out.ptr, batch.ptr, ns, ss), "batchedreduceadd_f")
        return out

    def sgd(self, w, dw, mom, lr, decay, momentum, batch, out=None):
        """updates out (default: w itself, as the generated call passes it) and mom in place"""
        out = w if out is None else out
        self._check(self.lib.swc_hip_sgd_f(w.size, out.ptr, w.ptr, dw.ptr, mom.ptr, lr, decay, momentum, batch), "sgd_f")
        return out, mom

    def reluGrad(self, src, dest_grad, out=None):
        out = out if out is not None else self.empty(src.shape)
        self._check(self.lib.swc_hip_reluGrad_f(out.ptr, src.ptr, dest_grad.ptr, src.size), "reluGrad_f")
        return out

    def pinned_empty(self, shape, dtype=np.float32):
        """a numpy array in page-locked host memory (kept alive by the returned array; freed with free_pinned)"""
        n = int(np.prod(shape)) * np.dtype(dtype).itemsize
        ptr = self.lib.swc_hip_host_malloc(max(n, 1))
        if not ptr:
            raise SwcHipError("swc_hip_host_malloc: " + self.lib.swc_hip_last_error().decode())
        buf = (C.c_char * max(n, 1)).from_address(ptr)
        arr = np.frombuffer(buf, dtype=dtype, count=int(np.prod(shape))).reshape(shape)
        self._pinned[arr.ctypes.data] = ptr
        return arr

    def free_pinned(self, arr):
        self._check(self.lib.swc_hip_host_free(self._pinned.pop(arr.ctypes.data)), "swc_hip_host_free")

    def gemm_workspace_bytes(self, m, n, k):
        """scratch bytes an m x n x k FC/GEMM call uses on this device (0 unless it is split over K)"""
        return int(self.lib.swc_hip_gemm_workspace_bytes(m, n, k))

    def conv2d_maxpool_workspace_bytes(self, xshape, fshape, strides, pads, pool, group=1):
        n, oh, ow, _ = pool_out_dims(xshape, fshape[1:3], strides, pads)
        odims = (n, oh, ow, fshape[0])
        pk, ps = pool[0], pool[1]
        pp = pool[2] if len(pool) > 2 else (0, 0, 0, 0)
        pdims = pool_out_dims(odims, pk, ps, pp)
        return int(self.lib.swc_hip_conv2dFusedMaxpool_workspace_bytes(
            _dims(odims), _dims(xshape), _dims(fshape), _dims(fshape[1:3]), _dims(strides), _dims(pads), group, _dims(pdims),
            _dims(pk), _dims(ps), _dims(pp)))

    def conv2d_workspace_bytes(self, xshape, fshape, strides=(1, 1), pads=(0, 0, 0, 0), group=1):
        """scratch bytes a conv2d call of these shapes uses on this device (0 if every tile is computed whole)"""
        odims = pool_out_dims(xshape, fshape[1:3], strides, pads)[:3] + (fshape[0],)
        return int(self.lib.swc_hip_conv2d_workspace_bytes(_dims(odims), _dims(xshape), _dims(fshape), _dims(fshape[1:3]),
                                                           _dims(strides), _dims(pads), group))

    def conv2dGrad_workspace_bytes(self, xshape, fshape, strides=(1, 1), pads=(0, 0, 0, 0), group=1):
        odims = pool_out_dims(xshape, fshape[1:3], strides, pads)[:3] + (fshape[0],)
        return int(self.lib.swc_hip_conv2dGrad_workspace_bytes(_dims(odims), _dims(xshape), _dims(fshape),
                                                               _dims(fshape[1:3]), _dims(strides), _dims(pads), group))

    def set_workspace(self, arr):
        """give the library a DeviceArray to use as scratch (None: its own buffer again)"""
        if arr is None:
            self._check(self.lib.swc_hip_set_workspace(None, 0), "swc_hip_set_workspace")
        else:
            self._check(self.lib.swc_hip_set_workspace(arr.ptr, arr.nbytes), "swc_hip_set_workspace")


_RT = None


def runtime():
    """The process-wide SwcHip instance (created on first use)."""
    global _RT
    if _RT is None:
        _RT = SwcHip(0)
    return _RT
