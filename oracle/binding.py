"""numpy-level access to the CPU checker libraries (test infrastructure only).

`load_oracle()` binds oracle/liboracle.so (the restatement, symbols `oracle_*`);
`load_ref()` binds oracle/_ref/libswc_ref.so (the reference's own kernels.h,
symbols `ref_*`) when that has been built.  Both expose the same methods, whose
names and argument meaning follow the reference's kernels
(src/codegen/utils/kernels.h): arrays in, freshly allocated arrays out.

Nothing in the shipped package may import this module.
"""
import ctypes as C
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_f32p = C.POINTER(C.c_float)
_i32p = C.POINTER(C.c_int32)
_szp = C.POINTER(C.c_size_t)


def _fp(a):
    return a.ctypes.data_as(_f32p)


def _dims(seq):
    return (C.c_size_t * len(seq))(*[int(v) for v in seq])


def pool_out_dims(idims, kernels, strides, pads):
    """Output NHWC dims of conv/pool windows, src/op/dlOp/dlOp.cpp:195-196:
    o = (i + pad_begin + pad_end - k) / s + 1 with pads = {t, l, b, r}."""
    n, h, w, c = idims
    oh = (h + pads[0] + pads[2] - kernels[0]) // strides[0] + 1
    ow = (w + pads[1] + pads[3] - kernels[1]) // strides[1] + 1
    return (n, oh, ow, c)


class CpuKernels:
    def __init__(self, path, prefix):
        self.path = path
        self.prefix = prefix
        self.lib = C.CDLL(path)

    def _fn(self, name):
        f = getattr(self.lib, self.prefix + name)
        f.restype = None
        return f

    def has(self, name):
        return hasattr(self.lib, self.prefix + name)

    # ---- kernels -------------------------------------------------------
    def matrixMatrixMul(self, a, b):
        a = np.ascontiguousarray(a, np.float32)
        b = np.ascontiguousarray(b, np.float32)
        m, k = a.shape
        k2, n = b.shape
        assert k == k2
        c = np.empty((m, n), np.float32)
        self._fn("matrixMatrixMul_f")(C.c_int(m), C.c_int(n), C.c_int(k), _fp(a),
                                      C.c_int(k), _fp(b), C.c_int(n), _fp(c),
                                      C.c_int(n))
        return c

    def batchedadd(self, batch, slice_):
        batch = np.ascontiguousarray(batch, np.float32)
        slice_ = np.ascontiguousarray(slice_, np.float32)
        rows, cols = batch.shape
        out = np.empty_like(batch)
        self._fn("batchedadd_f")(_fp(out), _fp(batch), _fp(slice_),
                                 C.c_size_t(rows), C.c_size_t(cols))
        return out

    def fcbias(self, a, w, bias, relu=False):
        """The reference lowers FC+bias to matrixMatrixMul then batchedadd
        (src/op/dlOp/dlOpEinsum.cpp:154-237)."""
        y = self.batchedadd(self.matrixMatrixMul(a, w), bias)
        return self.relu(y) if relu else y

    def matrixTanh(self, a):
        a = np.ascontiguousarray(a, np.float32)
        m, n = a.shape
        out = np.empty_like(a)
        self._fn("matrixTanh_f")(C.c_int(m), C.c_int(n), _fp(a), C.c_int(n),
                                 _fp(out), C.c_int(n))
        return out

    def matrixSoftmax(self, a):
        a = np.ascontiguousarray(a, np.float32)
        m, n = a.shape
        out = np.empty_like(a)
        self._fn("matrixSoftmax_f")(C.c_int(m), C.c_int(n), _fp(a), C.c_int(n),
                                    _fp(out), C.c_int(n))
        return out

    def relu(self, x):
        x = np.ascontiguousarray(x, np.float32)
        out = np.empty_like(x)
        self._fn("relu_f")(_fp(x), _fp(out), C.c_size_t(x.size))
        return out

    def vecAdd(self, a, b):
        a = np.ascontiguousarray(a, np.float32)
        b = np.ascontiguousarray(b, np.float32)
        assert a.shape == b.shape
        out = np.empty_like(a)
        self._fn("vecAdd_f")(C.c_int(a.size), _fp(a), _fp(b), _fp(out))
        return out

    def conv2d(self, x, filt, bias, kernels=None, strides=(1, 1),
               pads=(0, 0, 0, 0), group=1):
        x = np.ascontiguousarray(x, np.float32)
        filt = np.ascontiguousarray(filt, np.float32)
        bias = np.ascontiguousarray(bias, np.float32)
        if kernels is None:
            kernels = filt.shape[1:3]
        n, oh, ow, _ = pool_out_dims(x.shape, kernels, strides, pads)
        odims = (n, oh, ow, filt.shape[0])
        out = np.empty(odims, np.float32)
        self._fn("conv2d_f")(_fp(out), _fp(x), _fp(filt), _fp(bias), _dims(odims),
                             _dims(x.shape), _dims(filt.shape),
                             _dims(bias.shape), _dims(kernels), _dims(strides),
                             _dims(pads), C.c_size_t(group))
        return out

    def maxpool(self, x, kernels, strides, pads=(0, 0, 0, 0)):
        x = np.ascontiguousarray(x, np.float32)
        odims = pool_out_dims(x.shape, kernels, strides, pads)
        out = np.empty(odims, np.float32)
        self._fn("maxpool_f")(_fp(x), _fp(out), _dims(x.shape), _dims(odims),
                              _dims(kernels), _dims(strides), _dims(pads))
        return out

    def avgpool(self, x, kernels, strides, pads=(0, 0, 0, 0)):
        x = np.ascontiguousarray(x, np.float32)
        odims = pool_out_dims(x.shape, kernels, strides, pads)
        out = np.empty(odims, np.float32)
        self._fn("avgpool_f")(_fp(x), _fp(out), _dims(x.shape), _dims(odims),
                              _dims(kernels), _dims(strides), _dims(pads))
        return out

    def transpose(self, x, shuffle):
        """out axis a = in axis shuffle[a] (2-D or 4-D)."""
        x = np.ascontiguousarray(x, np.float32)
        odims = tuple(x.shape[s] for s in shuffle)
        out = np.empty(odims, np.float32)
        fn = self._fn("transpose4d_f" if x.ndim == 4 else "transpose2d_f")
        fn(_fp(x), _fp(out), _dims(x.shape), _dims(odims), _dims(shuffle))
        return out

    def maxpool_argmax(self, x, kernels, strides, pads=(0, 0, 0, 0)):
        """values + flat NHWC input index of the first maximum (oracle only)."""
        x = np.ascontiguousarray(x, np.float32)
        odims = pool_out_dims(x.shape, kernels, strides, pads)
        out = np.empty(odims, np.float32)
        idx = np.empty(odims, np.int32)
        self._fn("maxpool_argmax_f")(_fp(x), _fp(out), idx.ctypes.data_as(_i32p),
                                     _dims(x.shape), _dims(odims), _dims(kernels),
                                     _dims(strides), _dims(pads))
        return out, idx

    def maxpoolGrad(self, x, out_grad, kernels, strides, pads=(0, 0, 0, 0)):
        """scatter out_grad to the taps the windows selected (kernels.h:380-442)"""
        x = np.ascontiguousarray(x, np.float32)
        out_grad = np.ascontiguousarray(out_grad, np.float32)
        ig = np.empty_like(x)
        self._fn("maxpoolGrad_f")(_fp(ig), _fp(out_grad), _fp(x), _dims(x.shape),
                                  _dims(out_grad.shape), _dims(kernels),
                                  _dims(strides), _dims(pads))
        return ig

    def batchnormalization(self, x, mean, var, scale, bias, eps):
        x = np.ascontiguousarray(x, np.float32)
        args = [np.ascontiguousarray(v, np.float32) for v in (mean, var, scale, bias)]
        out = np.empty_like(x)
        self._fn("batchnormalization_f")(_fp(out), _fp(x), _fp(args[0]),
                                         _fp(args[1]), _fp(args[2]), _fp(args[3]),
                                         _dims(x.shape), C.c_float(eps))
        return out

    def argMax(self, x, top_k):
        x = np.ascontiguousarray(x, np.float32)
        m, n = x.shape
        idx = np.empty((m, top_k), np.int32)
        self._fn("argMax_i")(_fp(x), idx.ctypes.data_as(_i32p), C.c_int(m),
                             C.c_int(n), C.c_int(top_k))
        return idx

    def accuracy(self, pred, label, counters):
        """adds this batch to counters = [hits, rows] (int32[2]) in place and returns it"""
        pred = np.ascontiguousarray(pred, np.int32)
        label = np.ascontiguousarray(label, np.int32)
        m, n = pred.shape
        assert counters.dtype == np.int32 and counters.size == 2 and counters.flags.c_contiguous
        self._fn("accuracy_i")(pred.ctypes.data_as(_i32p), label.ctypes.data_as(_i32p),
                               counters.ctypes.data_as(_i32p), C.c_int(m), C.c_int(n))
        return counters

    # ---- training kernels ---------------------------------------------
    def matrixTrans(self, a):
        a = np.ascontiguousarray(a, np.float32)
        m, n = a.shape
        out = np.empty((n, m), np.float32)
        self._fn("matrixTrans_f")(C.c_int(m), C.c_int(n), _fp(a), C.c_int(n), _fp(out), C.c_int(m))
        return out

    def matrixTanhGrad(self, out, out_grad):
        """(tanh output, gradient of it) -> gradient of the tanh input"""
        out = np.ascontiguousarray(out, np.float32)
        out_grad = np.ascontiguousarray(out_grad, np.float32)
        m, n = out.shape
        ig = np.empty_like(out)
        self._fn("matrixTanhGrad_f")(C.c_int(m), C.c_int(n), _fp(ig), C.c_int(n), _fp(out), C.c_int(n),
                                     _fp(out_grad), C.c_int(n))
        return ig

    def matrixSoftmaxWithLoss(self, a, selected):
        a = np.ascontiguousarray(a, np.float32)
        selected = np.ascontiguousarray(selected, np.int32)
        m, n = a.shape
        out = np.empty_like(a)
        loss = np.zeros(1, np.float32)
        self._fn("matrixSoftmaxWithLoss_f")(C.c_int(m), C.c_int(n), _fp(a), C.c_int(n), _fp(out), C.c_int(n),
                                            selected.ctypes.data_as(_i32p), _fp(loss))
        return out, loss[0]

    def matrixSoftmaxGrad(self, prob, selected, with_loss=False):
        prob = np.ascontiguousarray(prob, np.float32)
        selected = np.ascontiguousarray(selected, np.int32)
        m, n = prob.shape
        ig = np.empty_like(prob)
        name = "matrixSoftmaxWithLossGrad_f" if with_loss and self.has("matrixSoftmaxWithLossGrad_f") else "matrixSoftmaxGrad_f"
        self._fn(name)(C.c_int(m), C.c_int(n), _fp(ig), C.c_int(n), _fp(prob), C.c_int(n),
                       selected.ctypes.data_as(_i32p))
        return ig

    def conv2dGrad(self, x, filt, out_grad, kernels=None, strides=(1, 1), pads=(0, 0, 0, 0), group=1):
        """-> (input gradient, filter gradient, bias gradient)"""
        x = np.ascontiguousarray(x, np.float32)
        filt = np.ascontiguousarray(filt, np.float32)
        out_grad = np.ascontiguousarray(out_grad, np.float32)
        if kernels is None:
            kernels = filt.shape[1:3]
        ig, fg, bg = np.empty_like(x), np.empty_like(filt), np.empty(filt.shape[0], np.float32)
        self._fn("conv2dGrad_f")(_fp(ig), _fp(fg), _fp(bg), _fp(out_grad), _fp(x), _fp(filt), _dims(out_grad.shape),
                                 _dims(x.shape), _dims(filt.shape), _dims(bg.shape), _dims(kernels), _dims(strides),
                                 _dims(pads), C.c_size_t(group))
        return ig, fg, bg

    def batchedreduceadd(self, batch):
        """one sum per row (slice) of a 2-D array"""
        batch = np.ascontiguousarray(batch, np.float32)
        ns, ss = batch.shape
        out = np.empty(ns, np.float32)
        self._fn("batchedreduceadd_f")(_fp(out), _fp(batch), C.c_size_t(ns), C.c_size_t(ss))
        return out

    def sgd(self, w, dw, mom, lr, decay, momentum, batch):
        """-> (updated weights, updated momentum buffer); inputs are not modified"""
        w = np.array(w, np.float32, copy=True, order="C")
        mom = np.array(mom, np.float32, copy=True, order="C")
        dw = np.ascontiguousarray(dw, np.float32)
        self._fn("sgd_f")(C.c_size_t(w.size), _fp(w), _fp(w), _fp(dw), _fp(mom), C.c_float(lr), C.c_float(decay),
                          C.c_float(momentum), C.c_size_t(batch))
        return w, mom

    def reluGrad(self, src, dest_grad):
        src = np.ascontiguousarray(src, np.float32)
        dest_grad = np.ascontiguousarray(dest_grad, np.float32)
        out = np.empty_like(src)
        self._fn("reluGrad_f")(_fp(out), _fp(src), _fp(dest_grad), C.c_size_t(src.size))
        return out


def build(force=False):
    """Compile liboracle.so (and _ref when the reference tree is present)."""
    so = os.path.join(_HERE, "liboracle.so")
    if force or not os.path.exists(so) or \
            os.path.getmtime(so) < os.path.getmtime(os.path.join(_HERE, "swc_oracle.cpp")):
        subprocess.check_call(["make", "-C", _HERE, "-B", "all"],
                              stdout=subprocess.DEVNULL)
    return so


def load_oracle():
    so = os.path.join(_HERE, "liboracle.so")
    if not os.path.exists(so):
        build()
    return CpuKernels(so, "oracle_")


def ref_available():
    return os.path.exists(os.path.join(_HERE, "_ref", "libswc_ref.so"))


def load_ref():
    so = os.path.join(_HERE, "_ref", "libswc_ref.so")
    if not os.path.exists(so):
        raise FileNotFoundError(so)
    return CpuKernels(so, "ref_")
