"""The five benchmark graphs as op sequences, backend-agnostic.

A "backend" is any object with the reference's kernel vocabulary as methods
(matrixMatrixMul, batchedadd, relu, vecAdd, conv2d, batchnormalization,
maxpool, matrixSoftmax): swcompiler_amd.hip.SwcHip on device arrays, or a CPU
checker on numpy arrays.  `unfused` sequences are call-for-call what the
reference's code generator emits for the graph (FCBias lowered to
matrixMatrixMul + batchedadd, src/op/dlOp/dlOpEinsum.cpp:154-237; one call per
op node in topological order, src/codegen/Codegen.cpp:1035-1060).  `fused`
sequences are what the HIP target emits: bias/BN/ReLU (and a 2x2 max-pooling
behind them) folded into the GEMM or conv epilogue and BN+ReLU(+pool) into one
pass.

Activations are NHWC and conv filters [oC,kH,kW,iC] (the reference's layout,
src/tensor/tensor.h:96-98); the "NCHW" shapes quoted for the configurations
are the logical shapes the inputs are drawn in before being permuted.
"""
import numpy as np

EPS = 1e-5  # src/importer/Caffe2Importer.cpp:259 default
F = np.float32


def _rng(cfg):
    return np.random.default_rng(0x5C0DE + cfg)


def _bn_params(rng, c):
    # order of the reference's BatchNormalization parents after the input:
    # scale, bias, mean, var (Codegen.cpp:1833-1837); kept here as a dict
    return dict(scale=rng.uniform(0.5, 1.5, c).astype(F), bias=(rng.standard_normal(c) * 0.1).astype(F),
                mean=(rng.standard_normal(c) * 0.1).astype(F), var=rng.uniform(0.5, 2.0, c).astype(F))


def make_inputs(cfg, batch=None):
    """Seeded synthetic inputs and parameters of configuration `cfg` (1..5) as numpy arrays."""
    rng = _rng(cfg)
    t = {}
    if cfg == 1:
        b = batch or 8
        t["x"] = rng.uniform(0, 1, (b, 784)).astype(F)
        t["w1"] = (rng.standard_normal((784, 512)) * 0.05).astype(F)
        t["w2"] = (rng.standard_normal((512, 10)) * 0.05).astype(F)
        t["b1"], t["b2"] = np.zeros(512, F), np.zeros(10, F)
    elif cfg == 2:
        b = batch or 4096
        t["x"] = rng.uniform(0, 1, (b, 784)).astype(F)
        for i, (k, n) in enumerate([(784, 4096), (4096, 4096), (4096, 10)], 1):
            t[f"w{i}"] = (rng.standard_normal((k, n)) / np.sqrt(k)).astype(F)
            t[f"b{i}"] = rng.uniform(-0.01, 0.01, n).astype(F)
    elif cfg == 3:
        b = batch or 256
        # drawn as NCHW [b,1,28,28], fed as NHWC
        t["x"] = np.ascontiguousarray(rng.uniform(0, 1, (b, 1, 28, 28)).astype(F).transpose(0, 2, 3, 1))
        t["f1"] = (rng.standard_normal((20, 5, 5, 1)) / np.sqrt(25)).astype(F)
        t["f2"] = (rng.standard_normal((50, 5, 5, 20)) / np.sqrt(500)).astype(F)
        t["cb1"], t["cb2"] = np.zeros(20, F), np.zeros(50, F)
        t["w1"] = (rng.standard_normal((800, 500)) / np.sqrt(800)).astype(F)
        t["w2"] = (rng.standard_normal((500, 10)) / np.sqrt(500)).astype(F)
        t["b1"], t["b2"] = np.zeros(500, F), np.zeros(10, F)
    elif cfg == 4:
        b = batch or 32
        t["x"] = np.ascontiguousarray(rng.standard_normal((b, 64, 56, 56)).astype(F).transpose(0, 2, 3, 1))
        for i, (ci, co) in enumerate([(64, 64), (64, 128), (128, 128), (128, 128)], 1):
            t[f"f{i}"] = (rng.standard_normal((co, 3, 3, ci)) / np.sqrt(9 * ci)).astype(F)
            t[f"cb{i}"] = np.zeros(co, F)
            for k, v in _bn_params(rng, co).items():
                t[f"bn{i}_{k}"] = v
    elif cfg == 5:
        b = batch or 256
        rows = (batch * 256) if batch else 65536
        t["logits"] = (rng.standard_normal((rows, 1000)) * 3).astype(F)
        t["p"] = rng.standard_normal((b, 32, 32, 256)).astype(F)
        t["q"] = rng.standard_normal((b, 32, 32, 256)).astype(F)
        for k, v in _bn_params(rng, 256).items():
            t[f"bn_{k}"] = v
    else:
        raise ValueError(cfg)
    return t


def batch_of(cfg, t):
    return t["logits"].shape[0] if cfg == 5 else t["x"].shape[0]


class _Ws:
    """Reuses output buffers between runs when the backend takes `out=` (device backend)."""

    def __init__(self, store):
        self.store = store

    def __call__(self, key, fn, *a, **kw):
        if self.store is None:
            return fn(*a, **kw)
        res = fn(*a, out=self.store.get(key), **kw)
        self.store[key] = res
        return res


def _fc(be, ws, key, x, w, b, relu, fused, softmax=False):
    """FC + bias, then ReLU or the row softmax; fused: as the single calls the HIP target emits"""
    if fused:
        return ws(key, be.fcbias, x, w, b, softmax=True) if softmax else ws(key, be.fcbias, x, w, b, relu=relu)
    y = ws(key + ".mm", be.matrixMatrixMul, x, w)
    y = ws(key + ".add", be.batchedadd, y, b)
    if softmax:
        return ws("sm", be.matrixSoftmax, y)
    return ws(key + ".relu", be.relu, y) if relu else y


def _bn(t, pre):
    return (t[pre + "_mean"], t[pre + "_var"], t[pre + "_scale"], t[pre + "_bias"])


def run(cfg, be, t, fused=False, ws=None):
    """Runs configuration `cfg` on backend `be` over tensors `t` (as produced by
    make_inputs, already converted to the backend's array type).  Returns the
    graph output (a dict of the three outputs for cfg 5)."""
    w = _Ws(ws)
    if cfg == 1:
        h = _fc(be, w, "fc1", t["x"], t["w1"], t["b1"], True, fused)
        return _fc(be, w, "fc2", h, t["w2"], t["b2"], False, fused, softmax=True)
    if cfg == 2:
        h = _fc(be, w, "fc1", t["x"], t["w1"], t["b1"], True, fused)
        h = _fc(be, w, "fc2", h, t["w2"], t["b2"], True, fused)
        return _fc(be, w, "fc3", h, t["w3"], t["b3"], False, fused, softmax=True)
    if cfg == 3:
        h = t["x"]
        for i in (1, 2):
            if fused:   # ReLU and the 2x2 pooling in the convolution's epilogue (the direct kernel's and the tile kernels')
                h = w(f"c{i}", be.conv2d, h, t[f"f{i}"], t[f"cb{i}"], relu=True, pool=((2, 2), (2, 2)))
                continue
            h = w(f"c{i}", be.conv2d, h, t[f"f{i}"], t[f"cb{i}"])
            h = w(f"r{i}", be.relu, h)
            h = w(f"p{i}", be.maxpool, h, (2, 2), (2, 2))
        h = h.reshape(h.shape[0], -1)  # ReshapeOp alias, (h,w,c) order
        h = _fc(be, w, "fc1", h, t["w1"], t["b1"], True, fused)
        return _fc(be, w, "fc2", h, t["w2"], t["b2"], False, fused, softmax=True)
    if cfg == 4:
        h = t["x"]
        for i in (1, 2, 3, 4):
            bn = _bn(t, f"bn{i}")
            if fused and i in (2, 4):   # the pooling in the convolution's epilogue
                h = w(f"c{i}", be.conv2d, h, t[f"f{i}"], t[f"cb{i}"], pads=(1, 1, 1, 1), bn=bn, eps=EPS, relu=True,
                      pool=((2, 2), (2, 2)))
                continue
            if fused:
                h = w(f"c{i}", be.conv2d, h, t[f"f{i}"], t[f"cb{i}"], pads=(1, 1, 1, 1), bn=bn, eps=EPS, relu=True)
            else:
                h = w(f"c{i}", be.conv2d, h, t[f"f{i}"], t[f"cb{i}"], pads=(1, 1, 1, 1))
                h = w(f"b{i}", be.batchnormalization, h, *bn, EPS)
                h = w(f"r{i}", be.relu, h)
            if i in (2, 4):
                h = w(f"p{i}", be.maxpool, h, (2, 2), (2, 2))
        return h
    if cfg == 5:
        out = {"a": w("a", be.matrixSoftmax, t["logits"])}
        bn = _bn(t, "bn")
        if fused:
            out["b"] = w("b", be.vecAdd, t["p"], t["q"], relu=True)
            out["c"] = w("c", be.batchnormReluMaxpool, t["p"], *bn, EPS, (2, 2), (2, 2))
            return out
        else:
            out["b"] = w("b.relu", be.relu, w("b.add", be.vecAdd, t["p"], t["q"]))
            h = w("c.relu", be.relu, w("c.bn", be.batchnormalization, t["p"], *bn, EPS))
        out["c"] = w("c.pool", be.maxpool, h, (2, 2), (2, 2))
        return out
    raise ValueError(cfg)


def flops(cfg, batch):
    """Dense algorithmic flop count of one batch (GEMM 2mnk; conv 2*M*oC*kh*kw*iC, padding taps counted)."""
    if cfg == 1:
        return 2.0 * batch * (784 * 512 + 512 * 10)
    if cfg == 2:
        return 2.0 * batch * (784 * 4096 + 4096 * 4096 + 4096 * 10)
    if cfg == 3:
        return 2.0 * batch * (24 * 24 * 20 * 25 + 8 * 8 * 50 * 500 + 800 * 500 + 500 * 10)
    if cfg == 4:
        return 2.0 * batch * (56 * 56 * 64 * 576 + 56 * 56 * 128 * 576 + 2 * 28 * 28 * 128 * 1152)
    return 0.0
