"""The oracle restatement against outputs of the reference's own kernels.h
(committed in tests/golden/kernels_golden.npz by tests/golden/make_golden.py).

Bit-exact everywhere except where glibc's expf takes part (softmax, tanh):
glibc picks an FMA or a non-FMA expf at load time depending on the CPU, so
those are held to 1 ulp instead."""
import os

import numpy as np
import pytest

from tests.util import assert_bit_exact, ulp_distance

HERE = os.path.dirname(os.path.abspath(__file__))


@pytest.mark.parametrize("tag", ["a", "b", "c", "d", "e"])
def test_gemm_and_bias(oracle, golden, tag):
    a, b, bias = golden[f"gemm_{tag}_a"], golden[f"gemm_{tag}_b"], golden[f"gemm_{tag}_bias"]
    c = oracle.matrixMatrixMul(a, b)
    assert_bit_exact(c, golden[f"gemm_{tag}_c"], "matrixMatrixMul")
    assert_bit_exact(oracle.batchedadd(c, bias), golden[f"gemm_{tag}_cb"], "batchedadd")


@pytest.mark.parametrize("tag", ["p1", "k5", "s2", "asym", "k1", "c64"])
def test_conv2d(oracle, golden, tag):
    x, f, b = golden[f"conv_{tag}_x"], golden[f"conv_{tag}_f"], golden[f"conv_{tag}_b"]
    sp = golden[f"conv_{tag}_sp"]
    y = oracle.conv2d(x, f, b, f.shape[1:3], tuple(sp[:2]), tuple(sp[2:]))
    assert_bit_exact(y, golden[f"conv_{tag}_y"], "conv2d")


@pytest.mark.parametrize("tag", ["k2", "k3s3", "k3s2p1", "odd"])
def test_maxpool_values_and_chosen_tap(oracle, golden, tag):
    x = golden[f"pool_{tag}_x"]
    ksp = [int(v) for v in golden[f"pool_{tag}_ksp"]]
    k, s, p = ksp[:2], ksp[2:4], ksp[4:]
    y, idx = oracle.maxpool_argmax(x, k, s, p)
    assert_bit_exact(y, golden[f"pool_{tag}_y"], "maxpool")
    assert_bit_exact(oracle.maxpool(x, k, s, p), golden[f"pool_{tag}_y"], "maxpool")
    # the reference exposes the chosen tap only through maxpoolGrad_f's scatter
    og = np.arange(1, y.size + 1, dtype=np.float32)
    scat = np.zeros(x.size, np.float32)
    assert (idx >= 0).all()
    np.add.at(scat, idx.ravel(), og)
    assert_bit_exact(scat.reshape(x.shape), golden[f"pool_{tag}_scatter"], "argmax scatter")


@pytest.mark.parametrize("tag", ["k2", "k3s3", "k3s2p1", "odd"])
def test_avgpool(oracle, golden, tag):
    ksp = [int(v) for v in golden[f"pool_{tag}_ksp"]]
    y = oracle.avgpool(golden[f"avg_{tag}_x"], ksp[:2], ksp[2:4], ksp[4:])
    assert_bit_exact(y, golden[f"avg_{tag}_y"], "avgpool")


def test_transpose(oracle, golden):
    x = golden["tr4_x"]
    for tag, sh in {"nchw2nhwc": (0, 2, 3, 1), "nhwc2nchw": (0, 3, 1, 2), "rev": (3, 2, 1, 0)}.items():
        assert_bit_exact(oracle.transpose(x, sh), golden[f"tr4_{tag}_y"], tag)
        assert_bit_exact(oracle.transpose(x, sh), np.transpose(x, sh), tag + " vs numpy")
    assert_bit_exact(oracle.transpose(golden["tr2_x"], (1, 0)), golden["tr2_y"], "2d")


@pytest.mark.parametrize("tag", ["a", "b"])
def test_batchnorm(oracle, golden, tag):
    g = lambda k: golden[f"bn_{tag}_{k}"]
    y = oracle.batchnormalization(g("x"), g("mean"), g("var"), g("scale"), g("bias"), 1e-5)
    assert_bit_exact(y, g("y"), "batchnormalization")


@pytest.mark.parametrize("tag", ["a", "b", "c", "d"])
def test_softmax(oracle, golden, tag):
    y = oracle.matrixSoftmax(golden[f"softmax_{tag}_x"])
    assert ulp_distance(y, golden[f"softmax_{tag}_y"]).max() <= 1


def test_tanh(oracle, golden):
    assert ulp_distance(oracle.matrixTanh(golden["tanh_x"]), golden["tanh_y"]).max() <= 1


def test_relu_add_specials(oracle, golden):
    assert_bit_exact(oracle.relu(golden["elt_x"]), golden["relu_y"], "relu")
    assert_bit_exact(oracle.vecAdd(golden["elt_x"], golden["elt_y"]), golden["add_y"], "vecAdd")


def test_argmax_ties(oracle, golden):
    assert_bit_exact(oracle.argMax(golden["argmax_x"], 3), golden["argmax_top3"], "argMax")


def test_mnist8_known_answer(oracle, golden):
    """test/input/mnist_images_8.meta.txt of the reference: 5 0 4 1 9 2 1 3."""
    d = os.path.join(HERE, "golden", "mnist8")
    ld = lambda n, shape: np.fromfile(os.path.join(d, n), np.float32).reshape(shape)
    img, w0, b0 = ld("mnist_images_8.bin", (8, 784)), ld("mlp_weight0.bin", (784, 512)), ld("mlp_bias0.bin", (512,))
    w1, b1 = ld("mlp_weight1.bin", (512, 10)), ld("mlp_bias1.bin", (10,))
    labels = [int(t) for t in open(os.path.join(d, "mnist_images_8.meta.txt")).read().split()]
    assert labels == [5, 0, 4, 1, 9, 2, 1, 3]
    h = oracle.matrixTanh(oracle.fcbias(img, w0, b0))
    prob = oracle.matrixSoftmax(oracle.fcbias(h, w1, b1))
    assert oracle.argMax(prob, 1).ravel().tolist() == labels
    assert_bit_exact(oracle.argMax(prob, 3), golden["mnist8_top3"], "top3")
    assert ulp_distance(prob, golden["mnist8_prob"]).max() <= 4
