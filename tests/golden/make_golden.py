"""Writes tests/golden/kernels_golden.npz by running the reference's own CPU
kernels (oracle/_ref/libswc_ref.so = src/codegen/utils/kernels.h of the
reference, compiled by oracle/Makefile) on small seeded inputs.

Run in a container that has the reference tree:
    make -C oracle && python tests/golden/make_golden.py
The .npz holds every input next to the expected output, so checking it needs
neither the reference nor this script's random stream.  tests/golden/mnist8/
holds the reference's own test inputs (test/input/*.bin, raw little-endian
fp32) and label file, copied as data.
"""
import os
import sys

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)
from oracle.binding import load_ref  # noqa: E402

OUT = os.path.join(os.path.dirname(os.path.abspath(__file__)), "kernels_golden.npz")
F = np.float32


def training(ref, g):
    """fixtures of the training kernels (their own random stream, so the arrays above never change)"""
    rng = np.random.default_rng(0x7EA1)
    convs = {
        "p1": ((2, 9, 9, 4), (5, 3, 3, 4), (1, 1), (1, 1, 1, 1)),
        "s2": ((2, 11, 10, 6), (7, 3, 3, 6), (2, 2), (1, 1, 1, 1)),
        "k5": ((1, 12, 12, 1), (5, 5, 5, 1), (1, 1), (0, 0, 0, 0)),
        "asym": ((1, 8, 7, 4), (3, 3, 2, 4), (1, 2), (2, 0, 1, 1)),
        "c32": ((2, 6, 6, 32), (16, 3, 3, 32), (1, 1), (1, 1, 1, 1)),
    }
    for tag, (idims, fdims, strides, pads) in convs.items():
        x = rng.standard_normal(idims).astype(F)
        f = (rng.standard_normal(fdims) / np.sqrt(fdims[1] * fdims[2] * fdims[3])).astype(F)
        y = ref.conv2d(x, f, np.zeros(fdims[0], F), fdims[1:3], strides, pads)
        og = rng.standard_normal(y.shape).astype(F)
        g[f"cgrad_{tag}_x"], g[f"cgrad_{tag}_f"], g[f"cgrad_{tag}_og"] = x, f, og
        g[f"cgrad_{tag}_sp"] = np.array(list(strides) + list(pads), np.int64)
        g[f"cgrad_{tag}_ig"], g[f"cgrad_{tag}_fg"], g[f"cgrad_{tag}_bg"] = ref.conv2dGrad(x, f, og, fdims[1:3], strides, pads)
    # maxpool gradient with real-valued gradients; overlapping windows accumulate (k3s1, k3s2p1)
    pools = {"k2": ((2, 8, 8, 5), (2, 2), (2, 2), (0, 0, 0, 0)), "k3s2p1": ((2, 7, 9, 4), (3, 3), (2, 2), (1, 1, 1, 1)),
             "k3s1": ((1, 6, 6, 3), (3, 3), (1, 1), (1, 1, 1, 1))}
    for tag, (idims, kernels, strides, pads) in pools.items():
        x = np.round(rng.standard_normal(idims) * 2).astype(F) / F(2)
        y = ref.maxpool(x, kernels, strides, pads)
        og = rng.standard_normal(y.shape).astype(F)
        g[f"pgrad_{tag}_x"], g[f"pgrad_{tag}_og"] = x, og
        g[f"pgrad_{tag}_ksp"] = np.array(list(kernels) + list(strides) + list(pads), np.int64)
        g[f"pgrad_{tag}_ig"] = ref.maxpoolGrad(x, og, kernels, strides, pads)
    # softmax with loss, its gradient
    for tag, (m, n, sigma) in {"a": (8, 10, 1.0), "b": (5, 1000, 3.0), "c": (33, 67, 10.0)}.items():
        x = (rng.standard_normal((m, n)) * sigma).astype(F)
        sel = rng.integers(0, n, m).astype(np.int32)
        p, loss = ref.matrixSoftmaxWithLoss(x, sel)
        g[f"swl_{tag}_x"], g[f"swl_{tag}_sel"], g[f"swl_{tag}_p"], g[f"swl_{tag}_loss"] = x, sel, p, np.array([loss], F)
        g[f"swl_{tag}_grad"] = ref.matrixSoftmaxGrad(p, sel, with_loss=True)
    # tanh gradient, transpose, relu gradient (with specials), row sums, sgd
    t = ref.matrixTanh((rng.standard_normal((6, 40)) * 2).astype(F))
    og = rng.standard_normal(t.shape).astype(F)
    g["tanhgrad_y"], g["tanhgrad_og"], g["tanhgrad_ig"] = t, og, ref.matrixTanhGrad(t, og)
    a = rng.standard_normal((37, 53)).astype(F)
    g["mtrans_x"], g["mtrans_y"] = a, ref.matrixTrans(a)
    x = rng.standard_normal(1031).astype(F)
    x[:8] = [0.0, -0.0, np.nan, np.inf, -np.inf, 1e-45, -1e-45, 3.0]
    dg = rng.standard_normal(1031).astype(F)
    dg[8:12] = [np.nan, np.inf, -0.0, 0.0]
    g["relugrad_x"], g["relugrad_dg"], g["relugrad_sg"] = x, dg, ref.reluGrad(x, dg)
    b = rng.standard_normal((19, 300)).astype(F)
    g["rowsum_x"], g["rowsum_y"] = b, ref.batchedreduceadd(b)
    w, dw, mom = (rng.standard_normal(777).astype(F) for _ in range(3))
    g["sgd_w"], g["sgd_dw"], g["sgd_mom"] = w, dw, mom
    g["sgd_params"] = np.array([0.01, 0.0005, 0.9, 16], np.float64)
    g["sgd_w1"], g["sgd_mom1"] = ref.sgd(w, dw, mom, 0.01, 0.0005, 0.9, 16)


def main():
    ref = load_ref()
    rng = np.random.default_rng(0x5C0DE)
    g = {}

    # GEMM: ragged shapes, fp32 order-sensitive values
    for tag, (m, k, n) in {"a": (7, 13, 5), "b": (33, 100, 17), "c": (8, 257, 10),
                           "d": (1, 1, 1), "e": (64, 96, 130)}.items():
        a = rng.standard_normal((m, k)).astype(F)
        b = (rng.standard_normal((k, n)) / np.sqrt(k)).astype(F)
        bias = rng.uniform(-0.01, 0.01, n).astype(F)
        g[f"gemm_{tag}_a"], g[f"gemm_{tag}_b"], g[f"gemm_{tag}_bias"] = a, b, bias
        c = ref.matrixMatrixMul(a, b)
        g[f"gemm_{tag}_c"] = c
        g[f"gemm_{tag}_cb"] = ref.batchedadd(c, bias)

    # conv: (idims, fdims(oC,kh,kw,iC), strides, pads)
    convs = {
        "p1": ((2, 9, 9, 3), (4, 3, 3, 3), (1, 1), (1, 1, 1, 1)),
        "k5": ((1, 12, 12, 1), (5, 5, 5, 1), (1, 1), (0, 0, 0, 0)),
        "s2": ((2, 11, 10, 6), (7, 3, 3, 6), (2, 2), (1, 1, 1, 1)),
        "asym": ((1, 8, 7, 4), (3, 3, 2, 4), (1, 2), (2, 0, 1, 1)),
        "k1": ((3, 5, 5, 16), (8, 1, 1, 16), (1, 1), (0, 0, 0, 0)),
        "c64": ((1, 6, 6, 64), (32, 3, 3, 64), (1, 1), (1, 1, 1, 1)),
    }
    for tag, (idims, fdims, strides, pads) in convs.items():
        x = rng.standard_normal(idims).astype(F)
        fan = fdims[1] * fdims[2] * fdims[3]
        f = (rng.standard_normal(fdims) / np.sqrt(fan)).astype(F)
        b = rng.standard_normal(fdims[0]).astype(F) * F(0.1)
        g[f"conv_{tag}_x"], g[f"conv_{tag}_f"], g[f"conv_{tag}_b"] = x, f, b
        g[f"conv_{tag}_sp"] = np.array(list(strides) + list(pads), np.int64)
        g[f"conv_{tag}_y"] = ref.conv2d(x, f, b, fdims[1:3], strides, pads)

    # maxpool: (idims, kernels, strides, pads); quantised values force ties
    pools = {
        "k2": ((2, 8, 8, 5), (2, 2), (2, 2), (0, 0, 0, 0)),
        "k3s3": ((1, 9, 9, 3), (3, 3), (3, 3), (0, 0, 0, 0)),
        "k3s2p1": ((2, 7, 9, 4), (3, 3), (2, 2), (1, 1, 1, 1)),
        "odd": ((1, 7, 7, 2), (2, 2), (2, 2), (0, 0, 0, 0)),
    }
    for tag, (idims, kernels, strides, pads) in pools.items():
        x = np.round(rng.standard_normal(idims) * 2).astype(F) / F(2)
        x.flat[::17] = F(-0.0)
        x.flat[5::29] = np.nan
        x.flat[7::31] = -np.inf
        g[f"pool_{tag}_x"] = x
        g[f"pool_{tag}_ksp"] = np.array(list(kernels) + list(strides) + list(pads), np.int64)
        y = ref.maxpool(x, kernels, strides, pads)
        g[f"pool_{tag}_y"] = y
        # chosen taps, as the reference's gradient kernel records them
        og = np.arange(1, y.size + 1, dtype=F).reshape(y.shape)
        g[f"pool_{tag}_scatter"] = ref.maxpoolGrad(x, og, kernels, strides, pads)

    # avgpool / transpose (reuse the pool inputs without the non-finite values)
    for tag, (idims, kernels, strides, pads) in pools.items():
        x = rng.standard_normal(idims).astype(F)
        g[f"avg_{tag}_x"] = x
        g[f"avg_{tag}_y"] = ref.avgpool(x, kernels, strides, pads)
    x = rng.standard_normal((2, 3, 5, 7)).astype(F)
    g["tr4_x"] = x
    for tag, sh in {"nchw2nhwc": (0, 2, 3, 1), "nhwc2nchw": (0, 3, 1, 2), "rev": (3, 2, 1, 0)}.items():
        g[f"tr4_{tag}_y"] = ref.transpose(x, sh)
    g["tr2_x"] = rng.standard_normal((5, 9)).astype(F)
    g["tr2_y"] = ref.transpose(g["tr2_x"], (1, 0))

    # batchnorm
    for tag, idims in {"a": (2, 5, 5, 8), "b": (1, 3, 4, 130)}.items():
        c = idims[3]
        x = rng.standard_normal(idims).astype(F)
        p = dict(mean=rng.standard_normal(c).astype(F) * F(0.1),
                 var=rng.uniform(0.5, 2, c).astype(F),
                 scale=rng.uniform(0.5, 1.5, c).astype(F),
                 bias=rng.standard_normal(c).astype(F) * F(0.1))
        g[f"bn_{tag}_x"] = x
        for k, v in p.items():
            g[f"bn_{tag}_{k}"] = v
        g[f"bn_{tag}_y"] = ref.batchnormalization(x, p["mean"], p["var"], p["scale"],
                                                  p["bias"], 1e-5)

    # softmax / tanh
    for tag, (m, n, sigma) in {"a": (8, 10, 1.0), "b": (5, 1000, 3.0), "c": (3, 1, 1.0),
                               "d": (4, 67, 30.0)}.items():
        x = (rng.standard_normal((m, n)) * sigma).astype(F)
        g[f"softmax_{tag}_x"] = x
        g[f"softmax_{tag}_y"] = ref.matrixSoftmax(x)
    x = (rng.standard_normal((6, 40)) * 2).astype(F)
    g["tanh_x"], g["tanh_y"] = x, ref.matrixTanh(x)

    # relu / add with specials
    x = rng.standard_normal(1031).astype(F)
    x[:8] = [0.0, -0.0, np.nan, np.inf, -np.inf, 1e-45, -1e-45, 3.0]
    y = rng.standard_normal(1031).astype(F)
    y[:8] = [-0.0, -0.0, 1.0, -np.inf, -np.inf, 1e-45, 1e-45, -3.0]
    g["elt_x"], g["elt_y"] = x, y
    g["relu_y"] = ref.relu(x)
    g["add_y"] = ref.vecAdd(x, y)

    # argmax with ties
    x = np.round(rng.standard_normal((6, 10)) * 2).astype(F)
    g["argmax_x"] = x
    g["argmax_top3"] = ref.argMax(x, 3)

    # MNIST-8 MLP of the reference's own test inputs
    d = os.path.join(os.path.dirname(OUT), "mnist8")
    img = np.fromfile(os.path.join(d, "mnist_images_8.bin"), F).reshape(8, 784)
    w0 = np.fromfile(os.path.join(d, "mlp_weight0.bin"), F).reshape(784, 512)
    b0 = np.fromfile(os.path.join(d, "mlp_bias0.bin"), F)
    w1 = np.fromfile(os.path.join(d, "mlp_weight1.bin"), F).reshape(512, 10)
    b1 = np.fromfile(os.path.join(d, "mlp_bias1.bin"), F)
    h = ref.matrixTanh(ref.fcbias(img, w0, b0))
    g["mnist8_prob"] = ref.matrixSoftmax(ref.fcbias(h, w1, b1))
    g["mnist8_top3"] = ref.argMax(g["mnist8_prob"], 3)

    training(ref, g)

    np.savez_compressed(OUT, **g)
    print("wrote", OUT, os.path.getsize(OUT), "bytes,", len(g), "arrays")


if __name__ == "__main__":
    main()
