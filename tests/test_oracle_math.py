"""What the mathematics fixes, independent of any build of the reference:
closed forms, invariants and brute force on tiny inputs, chosen so that a
dropped term, wrong index or transposed operand in the oracle fails."""
import itertools

import numpy as np

from tests.util import assert_bit_exact


def test_gemm_integer_valued_is_exact_and_not_transposed(oracle):
    rng = np.random.default_rng(0)
    a = rng.integers(-8, 9, (9, 23)).astype(np.float32)
    b = rng.integers(-8, 9, (23, 14)).astype(np.float32)
    want = (a.astype(np.int64) @ b.astype(np.int64)).astype(np.float32)
    assert_bit_exact(oracle.matrixMatrixMul(a, b), want, "integer gemm")
    eye = np.eye(23, dtype=np.float32)
    assert_bit_exact(oracle.matrixMatrixMul(a, eye), a, "A*I")


def test_gemm_sequential_fp32_sum_order(oracle):
    # 1 + 2^-24 + 2^-24 ... summed left to right in fp32 stays 1; any pairwise
    # or double accumulation would give 1 + 2^-23
    k = 3
    a = np.array([[1.0, 2.0 ** -24, 2.0 ** -24]], np.float32)
    b = np.ones((k, 1), np.float32)
    assert oracle.matrixMatrixMul(a, b)[0, 0] == np.float32(1.0)
    a2 = a[:, ::-1].copy()
    assert oracle.matrixMatrixMul(a2, b)[0, 0] == np.float32(1.0 + 2.0 ** -23)


def test_conv_1x1_is_gemm_and_constant_counts_taps(oracle):
    rng = np.random.default_rng(1)
    x = rng.integers(-4, 5, (2, 5, 6, 7)).astype(np.float32)
    f = rng.integers(-4, 5, (3, 1, 1, 7)).astype(np.float32)
    b = rng.integers(-4, 5, 3).astype(np.float32)
    y = oracle.conv2d(x, f, b)
    want = x.reshape(-1, 7) @ f.reshape(3, 7).T + b
    assert_bit_exact(y, want.reshape(2, 5, 6, 3).astype(np.float32), "1x1 conv")
    ones = np.ones((1, 5, 5, 2), np.float32)
    f = np.full((1, 3, 3, 2), 0.5, np.float32)
    y = oracle.conv2d(ones, f, np.array([0.25], np.float32), pads=(1, 1, 1, 1))[0, :, :, 0]
    taps = np.array([[4, 6, 6, 6, 4], [6, 9, 9, 9, 6], [6, 9, 9, 9, 6], [6, 9, 9, 9, 6], [4, 6, 6, 6, 4]])
    assert_bit_exact(y, (taps * 2 * 0.5 + 0.25).astype(np.float32), "tap count")


def test_conv_brute_force_integer(oracle):
    rng = np.random.default_rng(2)
    n, h, w, ci, co, kh, kw, sh, sw, pt, pl, pb, pr = 2, 6, 7, 3, 4, 3, 2, 2, 1, 1, 0, 1, 1
    x = rng.integers(-3, 4, (n, h, w, ci)).astype(np.float32)
    f = rng.integers(-3, 4, (co, kh, kw, ci)).astype(np.float32)
    b = rng.integers(-3, 4, co).astype(np.float32)
    oh, ow = (h + pt + pb - kh) // sh + 1, (w + pl + pr - kw) // sw + 1
    want = np.zeros((n, oh, ow, co), np.float32)
    for nn, ox, oy, c in itertools.product(range(n), range(oh), range(ow), range(co)):
        acc = float(b[c])
        for kx, ky in itertools.product(range(kh), range(kw)):
            ix, iy = ox * sh - pt + kx, oy * sw - pl + ky
            if 0 <= ix < h and 0 <= iy < w:
                acc += float(np.dot(x[nn, ix, iy], f[c, kx, ky]))
        want[nn, ox, oy, c] = acc
    assert_bit_exact(oracle.conv2d(x, f, b, (kh, kw), (sh, sw), (pt, pl, pb, pr)), want, "conv brute")


def test_maxpool_brute_force_and_first_max(oracle):
    rng = np.random.default_rng(3)
    x = rng.integers(-2, 3, (2, 7, 6, 3)).astype(np.float32)
    k, s, p = (3, 2), (2, 2), (1, 0, 1, 0)
    y, idx = oracle.maxpool_argmax(x, k, s, p)
    n, h, w, c = x.shape
    for nn, ox, oy, cc in itertools.product(range(n), range(y.shape[1]), range(y.shape[2]), range(c)):
        taps = [(x[nn, ix, iy, cc], ((nn * h + ix) * w + iy) * c + cc)
                for kx in range(3) for ky in range(2)
                for ix, iy in [(ox * 2 - 1 + kx, oy * 2 + ky)] if 0 <= ix < h and 0 <= iy < w]
        best = max(v for v, _ in taps)
        first = next(i for v, i in taps if v == best)
        assert y[nn, ox, oy, cc] == best and idx[nn, ox, oy, cc] == first
    const = np.full((1, 4, 4, 2), 3.5, np.float32)
    y, idx = oracle.maxpool_argmax(const, (2, 2), (2, 2))
    assert (y == 3.5).all()
    assert idx[0, 0, 0, 0] == 0 and idx[0, 1, 1, 1] == ((2 * 4) + 2) * 2 + 1


def test_softmax_invariants(oracle):
    rng = np.random.default_rng(4)
    x = (rng.standard_normal((16, 37)) * 3).astype(np.float32)
    y = oracle.matrixSoftmax(x)
    assert np.allclose(y.sum(1, dtype=np.float64), 1, atol=1e-5) and (y > 0).all()
    want = np.exp(x.astype(np.float64) - x.max(1, keepdims=True))
    want /= want.sum(1, keepdims=True)
    assert np.max(np.abs(y - want) / want) < 1e-5
    assert_bit_exact(oracle.matrixSoftmax(np.zeros((2, 10), np.float32)), np.full((2, 10), np.float32(1) / np.float32(10)), "uniform")
    two = oracle.matrixSoftmax(np.array([[0.0, np.log(3.0)]], np.float32))
    assert np.allclose(two, [[0.25, 0.75]], rtol=1e-6)
    assert np.array_equal(np.argmax(y, 1), np.argmax(x, 1))


def test_batchnorm_is_double_closed_form(oracle):
    rng = np.random.default_rng(5)
    x = rng.standard_normal((2, 3, 3, 5)).astype(np.float32)
    mean, beta = rng.standard_normal(5).astype(np.float32), rng.standard_normal(5).astype(np.float32)
    var, gamma = rng.uniform(0.5, 2, 5).astype(np.float32), rng.uniform(0.5, 1.5, 5).astype(np.float32)
    eps = np.float32(1e-5)
    ve = (var + eps).astype(np.float32).astype(np.float64)
    want = ((x - mean).astype(np.float32).astype(np.float64) * ve ** -0.5 * gamma.astype(np.float64)
            + beta.astype(np.float64)).astype(np.float32)
    got = oracle.batchnormalization(x, mean, var, gamma, beta, 1e-5)
    assert np.max(np.abs(got.view(np.int32).astype(np.int64) - want.view(np.int32))) <= 1
    # identity statistics: y == x up to the double round trip
    one, zero = np.ones(5, np.float32), np.zeros(5, np.float32)
    assert_bit_exact(oracle.batchnormalization(x, zero, one, one, zero, 0.0), x, "identity bn")


def test_relu_add_bias_specials(oracle):
    x = np.array([0.0, -0.0, np.nan, np.inf, -np.inf, 1e-45, -1e-45, 2.5, -2.5], np.float32)
    want = np.array([0.0, 0.0, 0.0, np.inf, 0.0, 1e-45, 0.0, 2.5, 0.0], np.float32)
    assert_bit_exact(oracle.relu(x), want, "relu")
    assert_bit_exact(oracle.vecAdd(x, x), (x + x).astype(np.float32), "vecAdd")
    m = np.arange(12, dtype=np.float32).reshape(3, 4)
    assert_bit_exact(oracle.batchedadd(m, np.array([1, 2, 3, 4], np.float32)), m + np.array([1, 2, 3, 4], np.float32), "batchedadd")


def test_conv_groups_are_independent_convolutions(oracle):
    """A convolution in G groups equals G separate one-group convolutions over the channel slices, each with the
    filter's slice of the same channels (the filter keeps all iC channels per tap: kernels.h:208-211)."""
    rng = np.random.default_rng(12)
    idims, fdims, group = (2, 7, 6, 6), (4, 3, 3, 6), 2
    x = rng.standard_normal(idims).astype(np.float32)
    f = rng.standard_normal(fdims).astype(np.float32)
    b = rng.standard_normal(fdims[0]).astype(np.float32)
    got = oracle.conv2d(x, f, b, (3, 3), (1, 1), (1, 1, 1, 1), group)
    cg, ocg = idims[3] // group, fdims[0] // group
    for g in range(group):
        cs, os_ = slice(g * cg, (g + 1) * cg), slice(g * ocg, (g + 1) * ocg)
        part = oracle.conv2d(x[..., cs], f[os_][..., cs], b[os_], (3, 3), (1, 1), (1, 1, 1, 1))
        assert_bit_exact(got[..., os_], part, f"group {g}")


def test_accuracy_counts(oracle):
    """kernels.h:615-627: hits and rows accumulate over calls; a label listed twice in a row counts once."""
    pred = np.array([[3, 1], [2, 2], [0, 4], [7, 7]], np.int32)
    label = np.array([1, 2, 5, 7], np.int32)
    cnt = np.array([10, 100], np.int32)
    assert oracle.accuracy(pred, label, cnt).tolist() == [13, 104]
    assert oracle.accuracy(pred[:, :1], label, cnt).tolist() == [15, 108]   # first column only: rows 1 and 3 hit
    rng = np.random.default_rng(3)
    pred, label = rng.integers(0, 10, (500, 3)).astype(np.int32), rng.integers(0, 10, 500).astype(np.int32)
    want = int((pred == label[:, None]).any(axis=1).sum())
    assert oracle.accuracy(pred, label, np.zeros(2, np.int32)).tolist() == [want, 500]


def test_argmax_order(oracle):
    x = np.array([[1, 3, 3, 2, 0]], np.float32)
    assert oracle.argMax(x, 3).tolist() == [[2, 1, 3]]
