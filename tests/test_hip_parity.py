"""Parity of the HIP kernels (through the C ABI) against the CPU oracle.

Bit-exact: relu, vecAdd, batchedadd, maxpool (values and chosen tap).
Within 1e-4 relative: GEMM/FC, conv, batchnorm, softmax, tanh.  For batchnorm,
softmax and tanh that is the strict element-wise |g-w|/|w|.  For the
contractions (GEMM, conv) the HIP kernels add the k products in a different
order than the oracle's sequential fp32 loop, and two fp32 orders of one dot
product differ by ~k*eps*sum|a||b| however small the cancelled result is; so
  * on non-negative operands (no cancellation) the strict element-wise relative
    error is asserted, and
  * on signed operands the error is taken relative to sum_k|a_ik||b_kj| (+|bias|)
    (tests/util.py scaled_err),
both against 1e-4, and integer-valued operands (exact in any order) are asserted
bit-exact.
"""
import ctypes
import itertools
import os

import numpy as np
import pytest

from tests.util import assert_bit_exact, rel_err, scaled_err, strict_rel_err

pytestmark = pytest.mark.gpu
TOL = 1e-4
HERE = os.path.dirname(os.path.abspath(__file__))


@pytest.fixture(scope="module")
def rt():
    from swcompiler_amd.hip import runtime
    return runtime()


def up(rt, *arrays):
    return [rt.upload(a) for a in arrays]


# ------------------------------------------------------------ elementwise
@pytest.mark.parametrize("n", [0, 1, 3, 4, 1031, 4096, (1 << 20) + 5])
def test_relu_add_bit_exact(rt, oracle, n):
    print("case relu/add n =", n, flush=True)
    rng = np.random.default_rng(n)
    x = rng.standard_normal(n).astype(np.float32)
    y = rng.standard_normal(n).astype(np.float32)
    if n >= 8:
        x[:8] = [0.0, -0.0, np.nan, np.inf, -np.inf, 1e-45, -1e-45, 3.0]
        y[:8] = [-0.0, -0.0, 1.0, -np.inf, -np.inf, 1e-45, 1e-45, -3.0]
    dx, dy = up(rt, x, y)
    assert_bit_exact(rt.relu(dx).numpy(), oracle.relu(x), "relu")
    assert_bit_exact(rt.vecAdd(dx, dy).numpy(), oracle.vecAdd(x, y), "vecAdd")
    assert_bit_exact(rt.vecAdd(dx, dy, relu=True).numpy(), oracle.relu(oracle.vecAdd(x, y)), "vecAddRelu")


def test_relu_unaligned_and_in_place(rt, oracle):
    x = np.random.default_rng(0).standard_normal(5000).astype(np.float32)
    d = rt.upload(x)
    v = d.offset_view(1, (4099,))
    out = rt.empty((5000,))
    o = out.offset_view(3, (4099,))
    rt.relu(v, out=o)
    assert_bit_exact(o.numpy(), oracle.relu(x[1:4100]), "unaligned relu")
    rt.relu(d, out=d)
    assert_bit_exact(d.numpy(), oracle.relu(x), "in-place relu")


@pytest.mark.parametrize("rows,cols", [(1, 1), (8, 512), (33, 10), (256, 500), (7, 4096)])
def test_batchedadd_bit_exact(rt, oracle, rows, cols):
    rng = np.random.default_rng(rows * cols)
    a = rng.standard_normal((rows, cols)).astype(np.float32)
    b = rng.standard_normal(cols).astype(np.float32)
    da, db = up(rt, a, b)
    assert_bit_exact(rt.batchedadd(da, db).numpy(), oracle.batchedadd(a, b), "batchedadd")


def test_tanh(rt, oracle, golden):
    x = golden["tanh_x"]
    got = rt.matrixTanh(rt.upload(x)).numpy()
    assert np.max(np.abs(got - golden["tanh_y"])) < 1e-6
    assert rel_err(got, oracle.matrixTanh(x)) < TOL


# ------------------------------------------------------------------ GEMM
GEMM_SHAPES = [(1, 1, 1), (7, 13, 5), (33, 100, 17), (8, 784, 512), (64, 96, 130), (130, 70, 257),
               (256, 800, 500), (200, 512, 128), (129, 33, 129), (64, 300, 10), (8, 512, 10),
               (256, 500, 10), (100, 4096, 10), (17, 37, 16), (300, 64, 20)]


@pytest.mark.parametrize("m,k,n", GEMM_SHAPES)
def test_gemm_vs_oracle(rt, oracle, m, k, n):
    print(f"case gemm {m}x{k}x{n}", flush=True)
    rng = np.random.default_rng(m * 1000003 + k * 1009 + n)
    a = rng.uniform(0, 1, (m, k)).astype(np.float32)
    b = (rng.standard_normal((k, n)) / np.sqrt(k)).astype(np.float32)
    bias = rng.uniform(-0.01, 0.01, n).astype(np.float32)
    da, db, dbias = up(rt, a, b, bias)
    want = oracle.matrixMatrixMul(a, b)
    mag = np.abs(a).astype(np.float64) @ np.abs(b).astype(np.float64) + np.abs(bias)
    assert scaled_err(rt.matrixMatrixMul(da, db).numpy(), want, mag) < TOL
    assert scaled_err(rt.fcbias(da, db, dbias).numpy(), oracle.batchedadd(want, bias), mag) < TOL
    assert scaled_err(rt.fcbias(da, db, dbias, relu=True).numpy(), oracle.relu(oracle.batchedadd(want, bias)), mag) < TOL
    # no cancellation: strict element-wise relative error
    bp = np.abs(b)
    assert strict_rel_err(rt.matrixMatrixMul(da, rt.upload(bp)).numpy(), oracle.matrixMatrixMul(a, bp)) < TOL


@pytest.mark.parametrize("m,k,n", [(70, 45, 90), (130, 260, 136), (40, 64, 12), (128, 128, 128)])
def test_gemm_integer_valued_is_exact(rt, m, k, n):
    """Small integers make every partial sum exact in fp32, so any summation
    order must give the same bits; catches a wrong fragment/lane mapping."""
    rng = np.random.default_rng(m + k + n)
    a = rng.integers(-8, 9, (m, k)).astype(np.float32)
    b = rng.integers(-8, 9, (k, n)).astype(np.float32)
    want = (a.astype(np.int64) @ b.astype(np.int64)).astype(np.float32)
    da, db = up(rt, a, b)
    assert_bit_exact(rt.matrixMatrixMul(da, db).numpy(), want, "integer gemm")


def _random_gemm_cases(count, seed):
    rng = np.random.default_rng(seed)
    ms = [1, 3, 8, 16, 40, 64, 100, 128, 256, 300, 513, 1024]
    ks = [1, 4, 30, 64, 100, 500, 800, 1024, 1500, 2048, 4100]
    ns = [1, 3, 10, 16, 20, 64, 100, 128, 256, 500, 1000]
    return [(int(rng.choice(ms)), int(rng.choice(ks)), int(rng.choice(ns))) for _ in range(count)]


@pytest.mark.parametrize("m,k,n", _random_gemm_cases(40, 99))
def test_gemm_random_shapes_integer_exact(rt, m, k, n):
    """Random (rows, K, columns) across every FC kernel's territory (few rows, heads of up to 16 columns streamed or
    not, K split over the chip, ragged tiles): small integers make every order of summation exact, so the product,
    with bias and ReLU in the epilogue, must equal integer arithmetic bit for bit."""
    print("case random gemm", m, k, n, flush=True)
    rng = np.random.default_rng(m * 7 + k * 3 + n)
    a = rng.integers(-4, 5, (m, k)).astype(np.float32)
    b = rng.integers(-4, 5, (k, n)).astype(np.float32)
    bias = rng.integers(-4, 5, n).astype(np.float32)
    want = a.astype(np.int64) @ b.astype(np.int64)
    da, db, dbias = up(rt, a, b, bias)
    assert_bit_exact(rt.matrixMatrixMul(da, db).numpy(), want.astype(np.float32), f"integer gemm [{rt.last_kernel()}]")
    got = rt.fcbias(da, db, dbias, relu=True).numpy()
    assert_bit_exact(got, np.maximum(want + bias.astype(np.int64), 0).astype(np.float32), f"integer FC + bias + ReLU [{rt.last_kernel()}]")


@pytest.mark.parametrize("tag", ["a", "b", "c", "d", "e"])
def test_gemm_golden(rt, golden, tag):
    da, db, dbias = up(rt, golden[f"gemm_{tag}_a"], golden[f"gemm_{tag}_b"], golden[f"gemm_{tag}_bias"])
    a, b = golden[f"gemm_{tag}_a"], golden[f"gemm_{tag}_b"]
    mag = np.abs(a).astype(np.float64) @ np.abs(b) + np.abs(golden[f"gemm_{tag}_bias"])
    assert scaled_err(rt.matrixMatrixMul(da, db).numpy(), golden[f"gemm_{tag}_c"], mag) < TOL
    assert scaled_err(rt.fcbias(da, db, dbias).numpy(), golden[f"gemm_{tag}_cb"], mag) < TOL


def test_gemm_full_size_rows(rt, oracle):
    """4096x4096x4096 (the GEMM-bound layer of the wide MLP): the oracle is run
    on 12 sampled rows of A, which fixes those rows of C exactly."""
    rng = np.random.default_rng(42)
    m = k = n = 4096
    a = rng.uniform(0, 1, (m, k)).astype(np.float32)
    b = (rng.standard_normal((k, n)) / np.sqrt(k)).astype(np.float32)
    bias = rng.uniform(-0.01, 0.01, n).astype(np.float32)
    da, db, dbias = up(rt, a, b, bias)
    got = rt.fcbias(da, db, dbias, relu=True).numpy()
    rows = np.array([0, 1, 31, 32, 63, 64, 127, 128, 2047, 2048, 4094, 4095])
    want = oracle.relu(oracle.batchedadd(oracle.matrixMatrixMul(a[rows], b), bias))
    mag = a[rows].astype(np.float64) @ np.abs(b) + np.abs(bias)
    assert scaled_err(got[rows], want, mag) < TOL
    bp = np.abs(b)
    assert strict_rel_err(rt.matrixMatrixMul(da, rt.upload(bp)).numpy()[rows], oracle.matrixMatrixMul(a[rows], bp)) < TOL
    # linearity in A over the whole output: (2A)B == 2(AB) exactly in fp32
    got2 = rt.matrixMatrixMul(rt.upload(a * np.float32(2)), db).numpy()
    assert_bit_exact(got2, rt.matrixMatrixMul(da, db).numpy() * np.float32(2), "scaling by 2")


# ------------------------------------------------------------------ conv
CONVS = [((2, 9, 9, 3), (4, 3, 3, 3), (1, 1), (1, 1, 1, 1)),
         ((2, 28, 28, 1), (20, 5, 5, 1), (1, 1), (0, 0, 0, 0)),
         ((2, 12, 12, 20), (50, 5, 5, 20), (1, 1), (0, 0, 0, 0)),
         ((1, 14, 14, 64), (64, 3, 3, 64), (1, 1), (1, 1, 1, 1)),
         ((1, 14, 14, 64), (128, 3, 3, 64), (1, 1), (1, 1, 1, 1)),
         ((2, 15, 13, 8), (6, 3, 5, 8), (2, 3), (1, 2, 1, 2)),
         ((1, 10, 10, 3), (4, 7, 7, 3), (2, 2), (3, 3, 3, 3)),
         ((3, 5, 5, 16), (8, 1, 1, 16), (1, 1), (0, 0, 0, 0)),
         ((1, 8, 7, 4), (3, 3, 2, 4), (1, 2), (2, 0, 1, 1)),
         ((4, 28, 28, 128), (128, 3, 3, 128), (1, 1), (1, 1, 1, 1)),
         ((2, 56, 56, 64), (64, 3, 3, 64), (1, 1), (1, 1, 1, 1))]


@pytest.mark.parametrize("idims,fdims,strides,pads", CONVS)
def test_conv_vs_oracle(rt, oracle, idims, fdims, strides, pads):
    print("case conv", idims, fdims, strides, pads, flush=True)
    rng = np.random.default_rng(sum(idims) * 131 + sum(fdims))
    x = rng.standard_normal(idims).astype(np.float32)
    f = (rng.standard_normal(fdims) / np.sqrt(np.prod(fdims[1:]))).astype(np.float32)
    b = (rng.standard_normal(fdims[0]) * 0.1).astype(np.float32)
    c = fdims[0]
    mean, beta = (rng.standard_normal(c) * 0.1).astype(np.float32), (rng.standard_normal(c) * 0.1).astype(np.float32)
    var, gamma = rng.uniform(0.5, 2, c).astype(np.float32), rng.uniform(0.5, 1.5, c).astype(np.float32)
    dx, df, db, dm, dv, dg, dbe = up(rt, x, f, b, mean, var, gamma, beta)
    want = oracle.conv2d(x, f, b, fdims[1:3], strides, pads)
    mag = oracle.conv2d(np.abs(x), np.abs(f), np.abs(b), fdims[1:3], strides, pads)   # sum of |terms|
    got = rt.conv2d(dx, df, db, fdims[1:3], strides, pads).numpy()
    assert got.shape == want.shape
    assert scaled_err(got, want, mag) < TOL
    assert scaled_err(rt.conv2d(dx, df, db, fdims[1:3], strides, pads, relu=True).numpy(), oracle.relu(want), mag) < TOL
    want_bn = oracle.relu(oracle.batchnormalization(want, mean, var, gamma, beta, 1e-5))
    got_bn = rt.conv2d(dx, df, db, fdims[1:3], strides, pads, bn=(dm, dv, dg, dbe), eps=1e-5, relu=True).numpy()
    mag_bn = (mag + np.abs(mean)) * (gamma / np.sqrt(var + 1e-5)) + np.abs(beta)
    assert scaled_err(got_bn, want_bn, mag_bn) < TOL
    # no cancellation: strict element-wise relative error
    xp, fp = np.abs(x), np.abs(f)
    assert strict_rel_err(rt.conv2d(rt.upload(xp), rt.upload(fp), db, fdims[1:3], strides, pads, relu=True).numpy(),
                          oracle.relu(oracle.conv2d(xp, fp, b, fdims[1:3], strides, pads))) < TOL


def _random_conv_cases(count, seed):
    rng = np.random.default_rng(seed)
    cases = []
    while len(cases) < count:
        c = int(rng.choice([1, 3, 4, 8, 20, 32, 36, 64, 96, 128]))
        kh, kw = (int(v) for v in rng.choice([1, 2, 3, 5], 2))
        sh, sw = (int(v) for v in rng.choice([1, 1, 2], 2))
        pads = tuple(int(v) for v in rng.integers(0, 3, 4))      # top, left, bottom, right
        n, h, w = int(rng.integers(1, 4)), int(rng.integers(4, 23)), int(rng.integers(4, 23))
        oc = int(rng.choice([3, 16, 40, 64, 70, 128, 136]))
        if h + pads[0] + pads[2] < kh or w + pads[1] + pads[3] < kw:
            continue
        cases.append(((n, h, w, c), (oc, kh, kw, c), (sh, sw), pads, [None, "7", "3"][len(cases) % 3]))
    return cases


@pytest.mark.parametrize("idims,fdims,strides,pads,slots", _random_conv_cases(48, 2024))
def test_conv_random_shapes_integer_exact(rt, oracle, idims, fdims, strides, pads, slots, switch_env):
    """Random layer shapes (channel counts for every kernel form, ragged tiles, strides, uneven padding), on a chip
    pretended to hold 7 or 3 workgroups for two thirds of them so that tiles are cut along K: small-integer operands
    make every order of summation exact, so the result must equal the oracle's bit for bit — plain, with ReLU and a
    second summand, and with the 2x2 pooling where the output allows it."""
    print("case random conv", idims, fdims, strides, pads, slots, flush=True)
    if slots:
        switch_env.setenv("SWC_HIP_CONV_SLOTS", slots)
        switch_env.setenv("SWC_HIP_CONV_MIN_IDLE", "0")   # cut tiles however little that saves
    rng = np.random.default_rng(sum(idims) * 7 + sum(fdims) * 3 + sum(pads))
    x = rng.integers(-3, 4, idims).astype(np.float32)
    f = rng.integers(-3, 4, fdims).astype(np.float32)
    b = rng.integers(-3, 4, fdims[0]).astype(np.float32)
    dx, df, db = up(rt, x, f, b)
    want = oracle.conv2d(x, f, b, fdims[1:3], strides, pads)
    got = rt.conv2d(dx, df, db, fdims[1:3], strides, pads).numpy()
    kernel = rt.last_kernel()
    assert_bit_exact(got, want, f"conv on integers [{kernel}]")
    res = rng.integers(-3, 4, want.shape).astype(np.float32)
    got = rt.conv2d(dx, df, db, fdims[1:3], strides, pads, relu=True, residual=rt.upload(res)).numpy()
    assert_bit_exact(got, oracle.relu(want + res), f"conv + summand + ReLU on integers [{rt.last_kernel()}]")
    if want.shape[1] % 2 == 0 and want.shape[2] % 2 == 0:
        pool = ((2, 2), (2, 2))
        got = rt.conv2d(dx, df, db, fdims[1:3], strides, pads, relu=True, pool=pool).numpy()
        assert_bit_exact(got, oracle.maxpool(oracle.relu(want), *pool), f"conv + ReLU + pool on integers [{rt.last_kernel()}]")


def _random_window_order_cases(count, seed):
    """layers for conv_win: channel counts that are multiples of 32, outputs with whole 2x2 windows of every size
    (one window per row up to wide images), any stride, kernel and padding, ragged tiles in both directions"""
    rng = np.random.default_rng(seed)
    cases = []
    while len(cases) < count:
        c, oc = int(rng.choice([32, 64, 96])), int(rng.choice([8, 64, 70, 128, 136]))
        kh, kw = int(rng.choice([1, 3, 5])), int(rng.choice([1, 3, 3]))
        sh, sw = int(rng.choice([1, 1, 2])), int(rng.choice([1, 1, 2, 3]))
        pads = tuple(int(v) for v in rng.integers(0, 3, 4))
        small = len(cases) % 2 == 0
        n = int(rng.integers(1, 6))
        h, w = (int(rng.integers(2, 14)), int(rng.integers(2, 14))) if small else (int(rng.integers(8, 40)), int(rng.integers(16, 70)))
        if h + pads[0] + pads[2] < kh or w + pads[1] + pads[3] < kw:
            continue
        oh, ow = (h + pads[0] + pads[2] - kh) // sh + 1, (w + pads[1] + pads[3] - kw) // sw + 1
        if oh % 2 or ow % 2 or oh < 2 or ow < 2:
            continue
        cases.append(((n, h, w, c), (oc, kh, kw, c), (sh, sw), pads, [None, "7", "20"][len(cases) % 3]))
    return cases


@pytest.mark.parametrize("idims,fdims,strides,pads,slots", _random_window_order_cases(36, 31))
def test_conv_win_integer_exact(rt, oracle, idims, fdims, strides, pads, slots, switch_env):
    """conv_win (rows in 2x2 window order, channel counts that are multiples of 32) over random layer shapes — from one
    window per output row to wide images, ragged last tiles, strides, uneven padding, tiles cut along K on a chip
    pretended to hold 7 or 20 workgroups: integer operands, the oracle's bits, plain, with a second summand and ReLU,
    and with the pooled epilogue."""
    print("case conv_win", idims, fdims, strides, pads, slots, flush=True)
    if slots:
        switch_env.setenv("SWC_HIP_CONV_SLOTS", slots)
        switch_env.setenv("SWC_HIP_CONV_MIN_IDLE", "0")   # cut tiles however little that saves
    rng = np.random.default_rng(sum(idims) * 13 + sum(fdims))
    x = rng.integers(-3, 4, idims).astype(np.float32)
    f = rng.integers(-3, 4, fdims).astype(np.float32)
    b = rng.integers(-3, 4, fdims[0]).astype(np.float32)
    dx, df, db = up(rt, x, f, b)
    want = oracle.conv2d(x, f, b, fdims[1:3], strides, pads)
    got = rt.conv2d(dx, df, db, fdims[1:3], strides, pads).numpy()
    assert rt.last_kernel().startswith("conv_win"), rt.last_kernel()
    assert_bit_exact(got, want, f"conv on integers [{rt.last_kernel()}]")
    res = rng.integers(-3, 4, want.shape).astype(np.float32)
    got = rt.conv2d(dx, df, db, fdims[1:3], strides, pads, relu=True, residual=rt.upload(res)).numpy()
    assert rt.last_kernel().startswith("conv_win"), rt.last_kernel()
    assert_bit_exact(got, oracle.relu(want + res), f"conv + summand + ReLU on integers [{rt.last_kernel()}]")
    pool = ((2, 2), (2, 2))
    got = rt.conv2d(dx, df, db, fdims[1:3], strides, pads, relu=True, pool=pool).numpy()
    assert rt.last_kernel().startswith("conv_win") and rt.last_kernel().endswith("(pooled)"), rt.last_kernel()
    assert_bit_exact(got, oracle.maxpool(oracle.relu(want), *pool), f"conv + ReLU + pool on integers [{rt.last_kernel()}]")


def test_conv_integer_valued_is_exact(rt):
    rng = np.random.default_rng(9)
    for idims, fdims, pads in [((2, 9, 10, 8), (40, 3, 3, 8), (1, 1, 1, 1)), ((1, 12, 12, 3), (70, 5, 5, 3), (2, 2, 2, 2))]:
        x = rng.integers(-4, 5, idims).astype(np.float32)
        f = rng.integers(-4, 5, fdims).astype(np.float32)
        b = rng.integers(-4, 5, fdims[0]).astype(np.float32)
        n, h, w, ci = idims
        co, kh, kw, _ = fdims
        xp = np.zeros((n, h + 2 * pads[0], w + 2 * pads[1], ci), np.int64)
        xp[:, pads[0]:pads[0] + h, pads[1]:pads[1] + w] = x
        oh, ow = h + 2 * pads[0] - kh + 1, w + 2 * pads[1] - kw + 1
        want = np.zeros((n, oh, ow, co), np.int64) + b.astype(np.int64)
        for ky, kx in itertools.product(range(kh), range(kw)):
            want += xp[:, ky:ky + oh, kx:kx + ow] @ f[:, ky, kx].astype(np.int64).T
        got = rt.conv2d(*up(rt, x, f, b), fdims[1:3], (1, 1), pads).numpy()
        assert_bit_exact(got, want.astype(np.float32), "integer conv")


@pytest.mark.parametrize("tag", ["p1", "k5", "s2", "asym", "k1", "c64"])
def test_conv_golden(rt, golden, tag):
    x, f, b, sp = (golden[f"conv_{tag}_{k}"] for k in ("x", "f", "b", "sp"))
    st, pd = tuple(int(v) for v in sp[:2]), tuple(int(v) for v in sp[2:])
    got = rt.conv2d(*up(rt, x, f, b), f.shape[1:3], st, pd).numpy()
    from oracle.binding import load_oracle
    mag = load_oracle().conv2d(np.abs(x), np.abs(f), np.abs(b), f.shape[1:3], st, pd)
    assert scaled_err(got, golden[f"conv_{tag}_y"], mag) < TOL


GROUPED_CONV_CASES = [((2, 9, 9, 8), (8, 3, 3, 8), (1, 1), (1, 1, 1, 1), 2),          # few channels, MFMA path
                      ((3, 14, 14, 64), (96, 3, 3, 64), (1, 1), (1, 1, 1, 1), 4),     # direct-to-LDS path
                      ((2, 7, 7, 16), (16, 3, 3, 16), (2, 2), (1, 1, 1, 1), 16),      # one channel per group
                      ((2, 10, 10, 6), (9, 3, 3, 6), (1, 1), (0, 0, 0, 0), 3),        # padded-channel path
                      ((4, 12, 12, 2), (4, 5, 5, 2), (1, 1), (2, 2, 2, 2), 2)]        # the direct kernel


@pytest.mark.parametrize("idims,fdims,strides,pads,group", GROUPED_CONV_CASES)
def test_conv_with_groups(rt, oracle, idims, fdims, strides, pads, group):
    """group > 1 as conv2d_f indexes it (kernels.h:196-238): the filter keeps all iC channels per tap and output
    channel co reads the channels of its group only."""
    rng = np.random.default_rng(sum(idims) + sum(fdims) + group)
    b = rng.integers(-4, 5, fdims[0]).astype(np.float32)
    x = rng.integers(-4, 5, idims).astype(np.float32)
    f = rng.integers(-4, 5, fdims).astype(np.float32)
    got = rt.conv2d(*up(rt, x, f, b), fdims[1:3], strides, pads, group=group).numpy()
    assert_bit_exact(got, oracle.conv2d(x, f, b, fdims[1:3], strides, pads, group), "grouped conv, integer-valued")
    xr = rng.standard_normal(idims).astype(np.float32)
    fr = rng.standard_normal(fdims).astype(np.float32)
    got = rt.conv2d(*up(rt, xr, fr, b), fdims[1:3], strides, pads, group=group, relu=True).numpy()
    want = oracle.relu(oracle.conv2d(xr, fr, b, fdims[1:3], strides, pads, group))
    scale = oracle.conv2d(np.abs(xr), np.abs(fr), np.abs(b), fdims[1:3], strides, pads, group)
    assert np.max(np.abs(got - want) / scale) < TOL
    # the result does not depend on the filter channels outside the group
    f2 = f.copy()
    cg, ocg = idims[3] // group, fdims[0] // group
    for co in range(fdims[0]):
        g = co // ocg
        f2[co, :, :, :g * cg] = 99
        f2[co, :, :, (g + 1) * cg:] = -99
    assert_bit_exact(rt.conv2d(*up(rt, x, f2, b), fdims[1:3], strides, pads, group=group).numpy(),
                     oracle.conv2d(x, f, b, fdims[1:3], strides, pads, group), "channels outside the group")


def test_conv_groups_in_a_caller_workspace_and_error_paths(rt, oracle):
    from swcompiler_amd.hip import SwcHipError
    idims, fdims, strides, pads, group = GROUPED_CONV_CASES[1]
    need = rt.conv2d_workspace_bytes(idims, fdims, strides, pads, group)
    assert need >= int(np.prod(fdims)) * 4 and need >= rt.conv2d_workspace_bytes(idims, fdims, strides, pads)
    rng = np.random.default_rng(77)
    x = rng.integers(-4, 5, idims).astype(np.float32)
    f = rng.integers(-4, 5, fdims).astype(np.float32)
    b = rng.integers(-4, 5, fdims[0]).astype(np.float32)
    ws = rt.empty((need // 4,))
    try:
        rt.set_workspace(ws)
        assert_bit_exact(rt.conv2d(*up(rt, x, f, b), fdims[1:3], strides, pads, group=group).numpy(),
                         oracle.conv2d(x, f, b, fdims[1:3], strides, pads, group), "groups, caller workspace")
    finally:
        rt.sync()
        rt.set_workspace(None)
    z = up(rt, np.zeros((1, 4, 4, 4), np.float32), np.zeros((4, 1, 1, 4), np.float32), np.zeros(4, np.float32))
    with pytest.raises(SwcHipError, match="group"):
        rt.conv2d(*z, group=3)          # divides neither channel count
    with pytest.raises(SwcHipError, match="group"):
        rt.conv2dGrad(z[0], z[1], rt.upload(np.zeros((1, 4, 4, 4), np.float32)), group=3)   # the gradients likewise


# ------------------------------------------------------- batchnorm / pool
@pytest.mark.parametrize("idims", [(2, 5, 5, 8), (1, 3, 4, 130), (3, 7, 7, 20), (2, 4, 4, 3), (4, 28, 28, 128), (1, 1, 1, 1)])
def test_batchnorm(rt, oracle, idims):
    rng = np.random.default_rng(sum(idims))
    c = idims[3]
    x = rng.standard_normal(idims).astype(np.float32)
    mean, beta = (rng.standard_normal(c) * 0.1).astype(np.float32), (rng.standard_normal(c) * 0.1).astype(np.float32)
    var, gamma = rng.uniform(0.5, 2, c).astype(np.float32), rng.uniform(0.5, 1.5, c).astype(np.float32)
    dx, dm, dv, dg, db = up(rt, x, mean, var, gamma, beta)
    want = oracle.batchnormalization(x, mean, var, gamma, beta, 1e-5)
    got = rt.batchnormalization(dx, dm, dv, dg, db, 1e-5).numpy()
    # double arithmetic on both sides: at most the last bit may differ (pow vs 1/sqrt)
    assert np.max(np.abs(got.view(np.int32).astype(np.int64) - want.view(np.int32))) <= 1
    assert strict_rel_err(got, want) < TOL
    got_r = rt.batchnormalization(dx, dm, dv, dg, db, 1e-5, relu=True).numpy()
    assert_bit_exact(got_r, oracle.relu(got), "fused relu of the same bn values")


POOLS = [((2, 8, 8, 5), (2, 2), (2, 2), (0, 0, 0, 0)), ((1, 9, 9, 3), (3, 3), (3, 3), (0, 0, 0, 0)),
         ((2, 7, 9, 4), (3, 3), (2, 2), (1, 1, 1, 1)), ((1, 7, 7, 2), (2, 2), (2, 2), (0, 0, 0, 0)),
         ((3, 24, 24, 20), (2, 2), (2, 2), (0, 0, 0, 0)), ((2, 8, 8, 50), (2, 2), (2, 2), (0, 0, 0, 0)),
         ((2, 28, 28, 128), (2, 2), (2, 2), (0, 0, 0, 0)), ((1, 9, 9, 8), (3, 2), (1, 3), (0, 1, 0, 1)),
         ((2, 9, 12, 8), (3, 3), (3, 3), (0, 0, 0, 0)), ((1, 10, 9, 4), (2, 2), (2, 2), (0, 0, 0, 0))]


@pytest.mark.parametrize("idims,k,s,p", POOLS)
def test_maxpool_bit_exact_with_first_max(rt, oracle, idims, k, s, p):
    print("case pool", idims, k, s, p, flush=True)
    rng = np.random.default_rng(sum(idims) + k[0])
    x = (np.round(rng.standard_normal(idims) * 2) / 2).astype(np.float32)  # many ties
    x.flat[::17] = np.float32(-0.0)
    x.flat[5::29] = np.nan
    x.flat[7::31] = -np.inf
    want, want_idx = oracle.maxpool_argmax(x, k, s, p)
    dx = rt.upload(x)
    assert_bit_exact(rt.maxpool(dx, k, s, p).numpy(), want, "maxpool")
    got, idx = rt.maxpool_argmax(dx, k, s, p)
    assert_bit_exact(got.numpy(), want, "maxpool(argmax variant)")
    assert_bit_exact(idx.numpy(), want_idx, "argmax")


@pytest.mark.parametrize("tag", ["k2", "k3s3", "k3s2p1", "odd"])
def test_maxpool_golden(rt, golden, tag):
    x = golden[f"pool_{tag}_x"]
    ksp = [int(v) for v in golden[f"pool_{tag}_ksp"]]
    got, idx = rt.maxpool_argmax(rt.upload(x), ksp[:2], ksp[2:4], ksp[4:])
    assert_bit_exact(got.numpy(), golden[f"pool_{tag}_y"], "maxpool golden")
    scat = np.zeros(x.size, np.float32)
    np.add.at(scat, idx.numpy().ravel(), np.arange(1, got.size + 1, dtype=np.float32))
    assert_bit_exact(scat.reshape(x.shape), golden[f"pool_{tag}_scatter"], "chosen tap golden")


@pytest.mark.parametrize("idims,k,s,p", POOLS + [((2, 7, 7, 2048), (7, 7), (1, 1), (0, 0, 0, 0)),        # global pooling
                                                 ((1, 13, 19, 8), (11, 9), (3, 2), (5, 4, 5, 4)),           # windows wider than 8
                                                 ((2, 9, 9, 6), (9, 9), (1, 1), (4, 4, 4, 4))])
def test_avgpool_bit_exact(rt, oracle, idims, k, s, p):
    x = np.random.default_rng(sum(idims)).standard_normal(idims).astype(np.float32)
    x.flat[::7] = -0.0
    assert_bit_exact(rt.avgpool(rt.upload(x), k, s, p).numpy(), oracle.avgpool(x, k, s, p), "avgpool")
    z = np.full(idims, -0.0, np.float32)      # all taps -0: the sum starts from +0 either way
    assert_bit_exact(rt.avgpool(rt.upload(z), k, s, p).numpy(), oracle.avgpool(z, k, s, p), "avgpool of -0")


@pytest.mark.parametrize("shape,shuffle", [((2, 3, 5, 7), (0, 2, 3, 1)), ((2, 3, 5, 7), (0, 3, 1, 2)),
                                           ((2, 3, 5, 7), (3, 2, 1, 0)), ((4, 64, 33, 35), (0, 2, 3, 1)),
                                           ((4, 33, 35, 64), (0, 3, 1, 2)), ((3, 4, 5, 6), (1, 0, 2, 3)),
                                           ((2, 40, 3, 50), (2, 3, 0, 1)), ((5, 9), (1, 0)), ((130, 257), (1, 0)),
                                           ((7, 11), (0, 1)), ((1, 224, 224, 3), (0, 3, 1, 2))])
def test_transpose_bit_exact(rt, oracle, shape, shuffle):
    print("case transpose", shape, shuffle, flush=True)
    x = np.random.default_rng(len(shape)).standard_normal(shape).astype(np.float32)
    got = rt.transpose(rt.upload(x), shuffle).numpy()
    assert_bit_exact(got, oracle.transpose(x, shuffle), "transpose vs oracle")
    assert_bit_exact(got, np.ascontiguousarray(np.transpose(x, shuffle)), "transpose vs numpy")


def test_transpose_golden(rt, golden):
    x = rt.upload(golden["tr4_x"])
    for tag, sh in {"nchw2nhwc": (0, 2, 3, 1), "nhwc2nchw": (0, 3, 1, 2), "rev": (3, 2, 1, 0)}.items():
        assert_bit_exact(rt.transpose(x, sh).numpy(), golden[f"tr4_{tag}_y"], tag)
    assert_bit_exact(rt.transpose(rt.upload(golden["tr2_x"]), (1, 0)).numpy(), golden["tr2_y"], "2d")
    for tag in ("k2", "k3s3", "k3s2p1", "odd"):
        ksp = [int(v) for v in golden[f"pool_{tag}_ksp"]]
        got = rt.avgpool(rt.upload(golden[f"avg_{tag}_x"]), ksp[:2], ksp[2:4], ksp[4:]).numpy()
        assert_bit_exact(got, golden[f"avg_{tag}_y"], "avgpool golden " + tag)


@pytest.mark.parametrize("idims,k", [((2, 16, 16, 64), (2, 2)), ((1, 9, 12, 8), (3, 3)), ((2, 7, 9, 12), (2, 2)),
                                     ((1, 6, 6, 5), (2, 2))])
def test_bn_relu_maxpool_fused_equals_sequence(rt, oracle, idims, k):
    rng = np.random.default_rng(77)
    x = rng.standard_normal(idims).astype(np.float32)
    c = idims[3]
    mean, beta = (rng.standard_normal(c) * 0.1).astype(np.float32), (rng.standard_normal(c) * 0.1).astype(np.float32)
    var, gamma = rng.uniform(0.5, 2, c).astype(np.float32), rng.uniform(0.5, 1.5, c).astype(np.float32)
    dx, dm, dv, dg, db = up(rt, x, mean, var, gamma, beta)
    seq = rt.maxpool(rt.batchnormalization(dx, dm, dv, dg, db, 1e-5, relu=True), k, k).numpy()
    fused = rt.batchnormReluMaxpool(dx, dm, dv, dg, db, 1e-5, k, k).numpy()
    assert_bit_exact(fused, seq, "bn+relu+pool fused vs sequence")
    want = oracle.maxpool(oracle.relu(oracle.batchnormalization(x, mean, var, gamma, beta, 1e-5)), k, k)
    assert rel_err(fused, want) < TOL


# --------------------------------------------------------------- softmax
@pytest.mark.parametrize("m,n,sigma", [(8, 10, 1.0), (5, 1000, 3.0), (3, 1, 1.0), (4, 67, 30.0), (64, 1000, 3.0),
                                       (9, 256, 3.0), (7, 2048, 3.0), (3, 5000, 3.0), (4096, 10, 2.0), (33, 36, 5.0)])
def test_softmax(rt, oracle, m, n, sigma):
    print(f"case softmax {m}x{n}", flush=True)
    x = (np.random.default_rng(m * n).standard_normal((m, n)) * sigma).astype(np.float32)
    want = oracle.matrixSoftmax(x)
    got = rt.matrixSoftmax(rt.upload(x)).numpy()
    nz = want > 1e-30  # exp underflow region: both sides are ~0, relative error is undefined there
    assert strict_rel_err(got[nz], want[nz]) < TOL
    assert np.all(got[~nz] < 1e-29)
    assert np.allclose(got.sum(1, dtype=np.float64), 1, atol=1e-5)


def test_softmax_golden_and_argmax(rt, oracle, golden):
    for tag in "abcd":
        got = rt.matrixSoftmax(rt.upload(golden[f"softmax_{tag}_x"])).numpy()
        want = golden[f"softmax_{tag}_y"]
        nz = want > 1e-30
        assert strict_rel_err(got[nz], want[nz]) < TOL
    x = golden["argmax_x"]
    assert_bit_exact(rt.argMax(rt.upload(x), 3).numpy(), golden["argmax_top3"], "argMax ties")
    z = np.round(np.random.default_rng(5).standard_normal((300, 10)) * 2).astype(np.float32)
    for k in (1, 3, 8):
        assert_bit_exact(rt.argMax(rt.upload(z), k).numpy(), oracle.argMax(z, k), f"argMax top{k}")


@pytest.mark.parametrize("m,n", [(32, 1000), (7, 128), (5, 129), (3, 4099), (130, 200)])
def test_argmax_of_long_rows(rt, oracle, m, n):
    """Rows of 128 columns and more take a wavefront each; same order as argMax_i (ties: the larger column first)."""
    rng = np.random.default_rng(m * n)
    z = np.round(rng.standard_normal((m, n)) * 1.5).astype(np.float32)     # many ties
    z[0, :] = 2.0                                                           # a constant row: the last columns win
    if m > 2:
        z[2, :] = -np.inf
        z[2, n // 2] = -1e30
    dz = rt.upload(z)
    for k in (1, 3, 5, 8):
        assert_bit_exact(rt.argMax(dz, k).numpy(), oracle.argMax(z, k), f"argMax top{k} of {m}x{n}")
    x = rng.standard_normal((m, n)).astype(np.float32)
    assert_bit_exact(rt.argMax(rt.upload(x), 5).numpy(), oracle.argMax(x, 5), "argMax top5, distinct values")


@pytest.mark.parametrize("m,n", [(8, 1), (300, 3), (4097, 5), (256, 8), (1, 1)])
def test_accuracy_counters(rt, oracle, m, n):
    """accuracy_i: the two counters accumulate over calls exactly as the host loop's."""
    rng = np.random.default_rng(m + n)
    want = np.array([5, 7], np.int32)
    counters = rt.upload(want.copy())
    for call in range(3):
        pred = rng.integers(0, 10, (m, n)).astype(np.int32)
        label = rng.integers(0, 10, m).astype(np.int32)
        rt.accuracy(rt.upload(pred), rt.upload(label), counters)
        oracle.accuracy(pred, label, want)
        assert_bit_exact(counters.numpy(), want, f"accuracy call {call}")
    assert want[1] == 7 + 3 * m
    # no rows: nothing changes; fill_i sets the counters
    rt._check(rt.lib.swc_hip_accuracy_i(None, None, counters.ptr, 0, n), "accuracy_i of no rows")
    assert_bit_exact(counters.numpy(), want, "accuracy of no rows")
    assert rt.fill_i(counters, 0).numpy().tolist() == [0, 0]
    assert rt.fill_i(counters, -3).numpy().tolist() == [-3, -3]


def test_mnist8_known_answer(rt, golden):
    """test/input of the reference: FCBias -> Tanh -> FCBias -> Softmax -> ArgMax = 5 0 4 1 9 2 1 3."""
    d = os.path.join(HERE, "golden", "mnist8")
    ld = lambda n, shape: np.fromfile(os.path.join(d, n), np.float32).reshape(shape)
    img, w0, b0 = ld("mnist_images_8.bin", (8, 784)), ld("mlp_weight0.bin", (784, 512)), ld("mlp_bias0.bin", (512,))
    w1, b1 = ld("mlp_weight1.bin", (512, 10)), ld("mlp_bias1.bin", (10,))
    dimg, dw0, db0, dw1, db1 = up(rt, img, w0, b0, w1, b1)
    h = rt.matrixTanh(rt.fcbias(dimg, dw0, db0))
    prob = rt.matrixSoftmax(rt.fcbias(h, dw1, db1))
    assert rt.argMax(prob, 1).numpy().ravel().tolist() == [5, 0, 4, 1, 9, 2, 1, 3]
    assert_bit_exact(rt.argMax(prob, 3).numpy(), golden["mnist8_top3"], "top3")
    assert strict_rel_err(prob.numpy(), golden["mnist8_prob"]) < TOL


def test_error_paths(rt):
    from swcompiler_amd.hip import SwcHipError
    a = rt.upload(np.zeros((4, 4), np.float32))
    with pytest.raises(SwcHipError):
        rt._check(rt.lib.swc_hip_matrixMatrixMul_f(4, 4, 4, None, 4, a.ptr, 4, a.ptr, 4), "null a")
    with pytest.raises(SwcHipError):
        rt._check(rt.lib.swc_hip_matrixMatrixMul_f(4, 4, 4, a.ptr, 2, a.ptr, 4, a.ptr, 4), "lda < k")
    with pytest.raises(SwcHipError):
        rt._check(rt.lib.swc_hip_relu_f(None, a.ptr, 16), "null src")
    assert rt.lib.swc_hip_relu_f(None, None, 0) == 0


# ------------------------------------------------- every kernel variant
# SWC_HIP_GEMM / SWC_HIP_CONV force a tile shape / pipeline variant; the library
# reads them on every call.  "reg*" = register-staged kernels (the path taken for
# unaligned shapes and for operands beyond the 2 GiB reach of 32-bit buffer
# offsets), "TMTN_S[m]" = direct-to-LDS kernels with an S-stage ring (m: ring hand-over in
# mid-slice), "TMTNwWM_S[m][x8]" = the column-interleaved kernels (x8: eight wavefronts).
GEMM_VARIANTS = ["reg", "22_2", "22_3", "21_3", "12_3", "11_3", "11_4", "11_3m", "21_3m",
                 "24w4_2x8", "14w4_2", "14w4_3m", "24w2_3m", "22w2_2", "splitk"]


@pytest.mark.parametrize("variant", GEMM_VARIANTS)
def test_gemm_every_variant(rt, oracle, variant, switch_env):
    print("case gemm variant", variant, flush=True)
    switch_env.setenv("SWC_HIP_GEMM", variant)
    rng = np.random.default_rng(11)
    for m, k, n in [(300, 200, 260), (128, 64, 128), (70, 36, 132), (64, 4, 64)]:
        a = rng.integers(-8, 9, (m, k)).astype(np.float32)
        b = rng.integers(-8, 9, (k, n)).astype(np.float32)
        bias = rng.integers(-8, 9, n).astype(np.float32)
        want = np.maximum((a.astype(np.int64) @ b.astype(np.int64) + bias.astype(np.int64)), 0).astype(np.float32)
        got = rt.fcbias(*up(rt, a, b, bias), relu=True).numpy()
        assert_bit_exact(got, want, f"integer gemm {m}x{k}x{n} variant {variant}")
    a = rng.uniform(0, 1, (257, 516)).astype(np.float32)
    b = rng.uniform(0, 1, (516, 260)).astype(np.float32)
    assert strict_rel_err(rt.matrixMatrixMul(*up(rt, a, b)).numpy(), oracle.matrixMatrixMul(a, b)) < TOL
    # tiles on every edge of a 256x256 grid, K not a multiple of the slice, bias without ReLU
    m, k, n = 520, 100, 776
    a = rng.integers(-8, 9, (m, k)).astype(np.float32)
    b = rng.integers(-8, 9, (k, n)).astype(np.float32)
    bias = rng.integers(-8, 9, n).astype(np.float32)
    want = (a.astype(np.int64) @ b.astype(np.int64) + bias.astype(np.int64)).astype(np.float32)
    assert_bit_exact(rt.fcbias(*up(rt, a, b, bias), relu=False).numpy(), want, f"integer gemm {m}x{k}x{n} variant {variant}")


@pytest.mark.parametrize("m,k,n", [(8, 512, 10), (256, 500, 10), (1000, 4096, 10), (33, 70, 16), (5, 12, 1), (17, 36, 3),
                                   (40, 64, 100), (17, 33, 1000), (300, 128, 17)])
def test_fcbias_softmax_fused(rt, oracle, m, k, n):
    """FC + bias + row softmax in one call: the reference's matrixMatrixMul_f, batchedadd_f, matrixSoftmax_f"""
    print("case fcbias+softmax", m, k, n, flush=True)
    rng = np.random.default_rng(m + k + n)
    a = rng.uniform(0, 1, (m, k)).astype(np.float32)
    w = (rng.standard_normal((k, n)) / np.sqrt(k)).astype(np.float32)
    b = rng.uniform(-0.01, 0.01, n).astype(np.float32)
    da, dw, db = up(rt, a, w, b)
    got = rt.fcbias(da, dw, db, softmax=True).numpy()
    want = oracle.matrixSoftmax(oracle.fcbias(a, w, b))
    nz = want > 1e-30
    assert strict_rel_err(got[nz], want[nz]) < TOL
    assert np.allclose(got.sum(axis=1), 1.0, atol=1e-5)
    # the same bits as the two calls in sequence on the device
    assert_bit_exact(got, rt.matrixSoftmax(rt.fcbias(da, dw, db)).numpy(), "fused vs sequence")
    # no bias
    assert_bit_exact(rt.fcbias(da, dw, None, softmax=True).numpy(), rt.matrixSoftmax(rt.fcbias(da, dw, None)).numpy(),
                     "fused vs sequence, no bias")


POOLED_CONVS = [
    # idims, fdims, pads: the two layers of the conv block that a pooling follows, at full size
    ((32, 56, 56, 64), (128, 3, 3, 64), (1, 1, 1, 1)),
    ((32, 28, 28, 128), (128, 3, 3, 128), (1, 1, 1, 1)),
    ((2, 8, 12, 8), (24, 3, 3, 8), (1, 1, 1, 1)),       # one partial tile, 24 of 64 columns
    ((3, 10, 6, 16), (70, 3, 3, 16), (1, 1, 1, 1)),     # columns over two tiles, rows end inside a tile
    ((5, 16, 16, 12), (64, 5, 5, 12), (2, 2, 2, 2)),
    ((1, 2, 2, 4), (4, 1, 1, 4), (0, 0, 0, 0)),         # a single window
    ((2, 18, 20, 32), (96, 3, 3, 32), (0, 0, 0, 0)),    # 16 x 18 output
]


@pytest.mark.parametrize("shift", [0, 1])
def test_pooled_conv_query_covers_unaligned_operands(rt, oracle, shift):
    """swc_hip_conv2dFusedMaxpool_workspace_bytes does not see the pointers: an input that is not on a 16-byte boundary
    takes the call off the pooling epilogue (the convolution's own output then goes through the workspace).  With
    auto-workspace off and a buffer of exactly the queried size the call must run either way."""
    print("case pooled conv query, shift", shift, flush=True)
    idims, fdims, pads, pool = (2, 12, 12, 32), (64, 3, 3, 32), (1, 1, 1, 1), ((2, 2), (2, 2))
    rng = np.random.default_rng(5)
    x = rng.integers(-3, 4, idims).astype(np.float32)
    f = rng.integers(-2, 3, fdims).astype(np.float32)
    b = rng.integers(-2, 3, fdims[0]).astype(np.float32)
    want = oracle.maxpool(oracle.relu(oracle.conv2d(x, f, b, pads=pads)), *pool)
    base = rt.empty((x.size + 4,))
    dx = base.offset_view(shift, idims)
    rt.upload_into(dx, x)
    df, db = up(rt, f, b)
    out = rt.empty(want.shape)
    need = rt.conv2d_maxpool_workspace_bytes(idims, fdims, (1, 1), pads, pool)
    ws = rt.empty((max(need, 4) // 4,))
    rt.sync()
    rt.set_workspace(ws)
    rt.enable_auto_workspace(False)
    try:
        rt.conv2d(dx, df, db, pads=pads, relu=True, pool=pool, out=out)
        name = rt.last_kernel()
        got = out.numpy()
    finally:
        rt.sync()
        rt.set_workspace(None)
        rt.enable_auto_workspace(True)
    assert name.endswith("(pooled)") == (shift == 0), name
    assert_bit_exact(got, want, f"pooled conv, input shifted by {shift} floats")   # integer-valued data: exact in any order


@pytest.mark.parametrize("idims,fdims,pads", POOLED_CONVS)
@pytest.mark.parametrize("slots", [None, "7"])
def test_conv_with_the_pooling_in_its_epilogue(rt, oracle, idims, fdims, pads, slots, switch_env):
    """conv (+BN) (+ReLU) + 2x2/2 max-pooling in one call is bit for bit the pooling of the separate convolution:
    both put a pixel into the same tile (rows in window order) and add its products in the same sequence, whole
    tiles and tiles cut along K alike (slots = 7 pretends a chip of seven workgroups, so that most tiles are cut)."""
    print("case pooled conv", idims, fdims, pads, slots, flush=True)
    if slots:
        switch_env.setenv("SWC_HIP_CONV_SLOTS", slots)
        switch_env.setenv("SWC_HIP_CONV_MIN_IDLE", "0")   # cut tiles however little that saves
    rng = np.random.default_rng(sum(idims) + sum(fdims))
    oc, c = fdims[0], fdims[3]
    x = rng.standard_normal(idims).astype(np.float32)
    f = (rng.standard_normal(fdims) / np.sqrt(fdims[1] * fdims[2] * c)).astype(np.float32)
    b = (rng.standard_normal(oc) * 0.1).astype(np.float32)
    bn = [rng.uniform(-0.1, 0.1, oc).astype(np.float32), rng.uniform(0.5, 2.0, oc).astype(np.float32),
          rng.uniform(0.5, 1.5, oc).astype(np.float32), rng.uniform(-0.1, 0.1, oc).astype(np.float32)]   # mean var scale bias
    dx, df, db = up(rt, x, f, b)
    dbn = up(rt, *bn)
    pool = ((2, 2), (2, 2))
    for with_bn, relu in [(True, True), (False, True), (False, False), (True, False)]:
        kw = dict(pads=pads, bn=dbn if with_bn else None, eps=1e-5, relu=relu)
        fused = rt.conv2d(dx, df, db, pool=pool, **kw)
        assert rt.last_kernel().startswith(("conv_dma", "conv_win")) and rt.last_kernel().endswith("(pooled)"), rt.last_kernel()
        plain = rt.conv2d(dx, df, db, **kw)
        assert rt.last_kernel().startswith(("conv_dma", "conv_win")), rt.last_kernel()
        want = rt.maxpool(plain, *pool).numpy()
        assert_bit_exact(fused.numpy(), want, f"pooled in the epilogue vs conv then maxpool (bn {with_bn}, relu {relu})")
    # against the oracle (full-size layers: the first image only)
    n = 1 if idims[0] * idims[1] * idims[2] * fdims[0] > (1 << 22) else idims[0]
    ref = oracle.conv2d(x[:n], f, b, pads=pads)
    ref = oracle.maxpool(oracle.relu(oracle.batchnormalization(ref, *bn, 1e-5)), *pool)
    got = rt.conv2d(dx, df, db, pads=pads, bn=dbn, eps=1e-5, relu=True, pool=pool).numpy()[:n]
    # (signed operands: the error of a sum is judged against the sum of the magnitudes of its terms, here carried
    # through the batchnorm's slope and the pooling)
    slope = np.abs(bn[2] / np.sqrt(bn[1] + np.float32(1e-5)))
    scale = oracle.maxpool(oracle.conv2d(np.abs(x[:n]), np.abs(f), np.abs(b), pads=pads) * slope + np.abs(bn[3]), *pool)
    assert scaled_err(got, ref, scale) < TOL
    # raster order of the rows gives the same values up to the order of summation of the tiles cut along K
    switch_env.setenv("SWC_HIP_CONV_ORDER", "raster")
    raster = rt.maxpool(rt.conv2d(dx, df, db, pads=pads, bn=dbn, eps=1e-5, relu=True), *pool).numpy()[:n]
    assert scaled_err(raster, ref, scale) < TOL
    if not slots and rt.last_kernel().find("conv_sk_finish") < 0:
        assert_bit_exact(raster, got, "window order vs raster order, every tile whole")


@pytest.mark.parametrize("idims,fdims,pads", [((32, 56, 56, 64), (128, 3, 3, 64), (1, 1, 1, 1)),
                                              ((32, 28, 28, 128), (128, 3, 3, 128), (1, 1, 1, 1)),
                                              ((3, 10, 6, 32), (70, 3, 3, 32), (1, 1, 1, 1)),
                                              ((2, 9, 11, 96), (64, 5, 5, 96), (2, 2, 2, 2)),     # odd output: raster order
                                              ((4, 16, 16, 64), (64, 1, 1, 64), (0, 0, 0, 0))])
@pytest.mark.parametrize("slots", [None, "11"])
def test_conv_kernel_forms_agree_bit_for_bit(rt, idims, fdims, pads, slots, switch_env):
    """The three forms of the 64x64-tile kernel — conv_dma (any channel count that is a multiple of 4), conv_dma_lean
    (multiples of 32: gather offsets per filter tap) and conv_win (rows in window order, no vector-ALU work in the K
    loop) — walk K in the same order and cut the same tiles: the same bits, whole and cut tiles, plain and pooled.
    (Eleven slots: every layer here then stays on the 64x64 tiles, and the two full-size ones have tiles cut along K.)"""
    print("case conv kernel forms", idims, fdims, pads, slots, flush=True)
    if slots:
        switch_env.setenv("SWC_HIP_CONV_SLOTS", slots)
        switch_env.setenv("SWC_HIP_CONV_MIN_IDLE", "0")   # cut tiles however little that saves
    rng = np.random.default_rng(sum(idims) * 3 + sum(fdims))
    oc = fdims[0]
    x = rng.standard_normal(idims).astype(np.float32)
    f = (rng.standard_normal(fdims) / np.sqrt(np.prod(fdims[1:]))).astype(np.float32)
    b = (rng.standard_normal(oc) * 0.1).astype(np.float32)
    bn = up(rt, rng.uniform(-0.1, 0.1, oc).astype(np.float32), rng.uniform(0.5, 2.0, oc).astype(np.float32),
            rng.uniform(0.5, 1.5, oc).astype(np.float32), rng.uniform(-0.1, 0.1, oc).astype(np.float32))
    dx, df, db = up(rt, x, f, b)
    kw = dict(pads=pads, bn=bn, eps=1e-5, relu=True)
    windows = idims[1] % 2 == 0 and idims[2] % 2 == 0 and fdims[1] != 5   # (the 5x5 layer's output is 9 x 11: raster order)
    default = rt.conv2d(dx, df, db, **kw).numpy()
    assert rt.last_kernel().startswith("conv_win" if windows else "conv_dma_lean"), rt.last_kernel()
    if slots and idims[0] >= 32:
        assert "conv_sk_finish" in rt.last_kernel(), rt.last_kernel()
    switch_env.setenv("SWC_HIP_CONV", "11_3m")
    lean = rt.conv2d(dx, df, db, **kw).numpy()
    assert rt.last_kernel().startswith("conv_dma_lean"), rt.last_kernel()
    assert_bit_exact(default, lean, "default vs conv_dma_lean")
    switch_env.setenv("SWC_HIP_CONV_LEAN", "0")
    plain = rt.conv2d(dx, df, db, **kw).numpy()
    assert rt.last_kernel().startswith("conv_dma<1,1,3,true>"), rt.last_kernel()
    assert_bit_exact(lean, plain, "conv_dma_lean vs conv_dma")
    if windows:
        pool = ((2, 2), (2, 2))
        plain_pooled = rt.conv2d(dx, df, db, pool=pool, **kw).numpy()
        switch_env.delenv("SWC_HIP_CONV_LEAN")
        lean_pooled = rt.conv2d(dx, df, db, pool=pool, **kw).numpy()
        assert rt.last_kernel().startswith("conv_dma_lean") and rt.last_kernel().endswith("(pooled)"), rt.last_kernel()
        switch_env.delenv("SWC_HIP_CONV")
        win_pooled = rt.conv2d(dx, df, db, pool=pool, **kw).numpy()
        assert rt.last_kernel().startswith("conv_win") and rt.last_kernel().endswith("(pooled)"), rt.last_kernel()
        assert_bit_exact(win_pooled, rt.maxpool(rt.upload(plain), *pool).numpy(), "pooled, conv_win")
        assert_bit_exact(lean_pooled, win_pooled, "pooled, conv_dma_lean")
        assert_bit_exact(plain_pooled, win_pooled, "pooled, general form")


@pytest.mark.parametrize("idims,fdims,pads", [((256, 28, 28, 1), (20, 5, 5, 1), (0, 0, 0, 0)),      # LeNet's first layer
                                              ((3, 10, 14, 3), (8, 3, 3, 3), (1, 1, 1, 1)),
                                              ((2, 6, 6, 1), (3, 3, 3, 1), (1, 1, 1, 1)),
                                              ((1, 8, 8, 2), (20, 3, 3, 2), (0, 0, 0, 0)),
                                              ((2, 12, 12, 3), (30, 3, 3, 3), (1, 1, 1, 1)),
                                              ((400, 28, 28, 3), (16, 3, 3, 3), (1, 1, 1, 1)),        # two pixels per thread
                                              ((700, 28, 28, 1), (20, 5, 5, 1), (2, 2, 2, 2))])        # four pixels per thread
def test_direct_conv_with_the_pooling_in_its_epilogue(rt, oracle, idims, fdims, pads):
    """first layers (the direct kernel: four neighbouring threads hold a window): bit-exact with the oracle's
    conv2d_f -> relu_f -> maxpool_f, with and without ReLU and batchnorm, and with the two calls in sequence"""
    print("case direct pooled conv", idims, fdims, pads, flush=True)
    rng = np.random.default_rng(sum(idims) + sum(fdims))
    oc = fdims[0]
    x = rng.standard_normal(idims).astype(np.float32)
    f = (rng.standard_normal(fdims) / 4).astype(np.float32)
    b = (rng.standard_normal(oc) * 0.1).astype(np.float32)
    dx, df, db = up(rt, x, f, b)
    pool = ((2, 2), (2, 2))
    n = min(idims[0], 8)
    want = oracle.conv2d(x[:n], f, b, pads=pads)
    got = rt.conv2d(dx, df, db, pads=pads, pool=pool)
    assert rt.last_kernel().startswith("conv_direct") and rt.last_kernel().endswith("(pooled)"), rt.last_kernel()
    per_thread = 4 if idims[0] >= 700 else 2 if idims[0] >= 400 else 1
    assert rt.last_kernel() == f"conv_direct<{(oc + 3) // 4},{per_thread}> (pooled)", rt.last_kernel()
    assert rt.conv2d_maxpool_workspace_bytes(idims, fdims, (1, 1), pads, pool) == 0
    assert_bit_exact(got.numpy()[:n], oracle.maxpool(want, *pool), "conv + pool")
    assert_bit_exact(got.numpy(), rt.maxpool(rt.conv2d(dx, df, db, pads=pads), *pool).numpy(), "one call vs two")
    got = rt.conv2d(dx, df, db, pads=pads, relu=True, pool=pool).numpy()
    assert_bit_exact(got[:n], oracle.maxpool(oracle.relu(want), *pool), "conv + ReLU + pool")
    bn = up(rt, rng.uniform(-0.1, 0.1, oc).astype(np.float32), rng.uniform(0.5, 2.0, oc).astype(np.float32),
            rng.uniform(0.5, 1.5, oc).astype(np.float32), rng.uniform(-0.1, 0.1, oc).astype(np.float32))
    kw = dict(pads=pads, bn=bn, eps=1e-5, relu=True)
    assert_bit_exact(rt.conv2d(dx, df, db, pool=pool, **kw).numpy(), rt.maxpool(rt.conv2d(dx, df, db, **kw), *pool).numpy(),
                     "conv + BN + ReLU + pool, one call vs two")


def test_conv_with_a_pooling_the_epilogue_cannot_do(rt, oracle):
    """odd output sizes, 3x3 windows, a layer for the direct kernel: conv into the workspace, then maxpool_f's kernel"""
    rng = np.random.default_rng(5)
    cases = [((2, 9, 9, 8), (16, 3, 3, 8), (1, 1, 1, 1), ((2, 2), (2, 2))),          # 9 x 9 output
             ((2, 12, 12, 8), (16, 3, 3, 8), (1, 1, 1, 1), ((3, 3), (2, 2))),        # 3 x 3 windows
             ((2, 12, 12, 8), (16, 3, 3, 8), (1, 1, 1, 1), ((2, 2), (2, 2), (1, 1, 1, 1))),   # padded pooling
             ((4, 27, 27, 1), (20, 5, 5, 1), (0, 0, 0, 0), ((2, 2), (2, 2), (0, 0, 1, 1)))]   # the direct kernel's layer, 23 x 23 output
    for idims, fdims, pads, pool in cases:
        print("case conv + other pooling", idims, fdims, pads, pool, flush=True)
        x = rng.standard_normal(idims).astype(np.float32)
        f = (rng.standard_normal(fdims) / 8).astype(np.float32)
        b = (rng.standard_normal(fdims[0]) * 0.1).astype(np.float32)
        dx, df, db = up(rt, x, f, b)
        assert rt.conv2d_maxpool_workspace_bytes(idims, fdims, (1, 1), pads, pool) >= 4 * np.prod(idims[:3]) * fdims[0] // 2
        fused = rt.conv2d(dx, df, db, pads=pads, relu=True, pool=pool).numpy()
        assert not rt.last_kernel().endswith("(pooled)"), rt.last_kernel()
        assert_bit_exact(fused, rt.maxpool(rt.conv2d(dx, df, db, pads=pads, relu=True), *pool).numpy(), "two steps")
        assert rel_err(fused, oracle.maxpool(oracle.relu(oracle.conv2d(x, f, b, pads=pads)), *pool)) < TOL
    # error paths
    dx, df, db = up(rt, np.zeros((1, 4, 4, 4), np.float32), np.zeros((4, 1, 1, 4), np.float32), np.zeros(4, np.float32))
    out = rt.empty((1, 2, 2, 8))
    d = lambda *v: (ctypes.c_size_t * len(v))(*v)
    rc = rt.lib.swc_hip_conv2dFusedMaxpool_f(out.ptr, dx.ptr, df.ptr, db.ptr, d(1, 4, 4, 4), d(1, 4, 4, 4), d(4, 1, 1, 4),
                                             d(4), d(1, 1), d(1, 1), d(0, 0, 0, 0), 1, None, None, None, None, 0.0, 1,
                                             d(1, 2, 2, 8), d(2, 2), d(2, 2), d(0, 0, 0, 0))
    assert rc != 0 and b"pooled batch/channels" in rt.lib.swc_hip_last_error()


STREAMED_HEADS = [(4096, 4096, 10), (1000, 4096, 10), (33, 1028, 7), (16, 2048, 16), (257, 1056, 1), (100, 1200, 3),
                  (17, 5000, 8), (50, 1444, 11), (1, 8192, 16), (130, 2052, 4), (48, 70000, 10)]


@pytest.mark.parametrize("m,k,n", STREAMED_HEADS)
def test_skinny_gemm_streamed_along_k(rt, oracle, m, k, n, switch_env):
    """N <= 16 behind a K above 1024: A and B by LDS-DMA through per-wavefront rings.  Integer-valued operands make the
    result exact whatever the order of summation, so every k, every row and every column is checked bit by bit (rows
    and k past the end must come in as zeros, not as whatever the ring held); then real-valued data against the
    oracle, and the fused softmax against the two calls in sequence, also with the plain kernel."""
    print("case streamed head", m, k, n, flush=True)
    rng = np.random.default_rng(m * 7 + k + n)
    a = rng.integers(-4, 5, (m, k)).astype(np.float32)
    b = rng.integers(-4, 5, (k, n)).astype(np.float32)
    bias = rng.integers(-8, 9, n).astype(np.float32)
    want = (a.astype(np.int64) @ b.astype(np.int64) + bias.astype(np.int64)).astype(np.float32)
    da, db, dbias = up(rt, a, b, bias)
    got = rt.fcbias(da, db, dbias, relu=False).numpy()
    assert rt.last_kernel().startswith("gemm_skinny_stream<"), rt.last_kernel()
    assert_bit_exact(got, want, f"integer head {m}x{k}x{n}")
    assert_bit_exact(rt.fcbias(da, db, dbias, relu=True).numpy(), np.maximum(want, 0), "with ReLU")
    assert_bit_exact(rt.matrixMatrixMul(da, db).numpy(), want - bias, "no bias")
    # a second call right after one on other data: nothing of the first may be left in the rings
    a2 = np.where(rng.uniform(size=(m, k)) < 0.5, np.float32(np.inf), np.float32(1)).astype(np.float32)
    rt.matrixMatrixMul(rt.upload(a2), db)
    assert_bit_exact(rt.fcbias(da, db, dbias, relu=False).numpy(), want, "after a call full of infinities")
    # real-valued
    x = rng.uniform(0, 1, (m, k)).astype(np.float32)
    w = (rng.standard_normal((k, n)) / np.sqrt(k)).astype(np.float32)
    c = rng.uniform(-0.01, 0.01, n).astype(np.float32)
    dx, dw, dc = up(rt, x, w, c)
    ref = oracle.fcbias(x, w, c) if m * k <= (1 << 23) else (x.astype(np.float64) @ w.astype(np.float64) + c).astype(np.float32)
    assert scaled_err(rt.fcbias(dx, dw, dc).numpy(), ref, np.abs(x) @ np.abs(w) + np.abs(c)) < TOL
    fused = rt.fcbias(dx, dw, dc, softmax=True).numpy()
    assert_bit_exact(fused, rt.matrixSoftmax(rt.fcbias(dx, dw, dc)).numpy(), "fused softmax vs sequence")
    assert np.allclose(fused.sum(axis=1), 1.0, atol=1e-5)
    # rows of a wider matrix (lda > k)
    wide = rng.integers(-4, 5, (m, k + 8)).astype(np.float32)
    dwide, out = rt.upload(wide), rt.empty((m, n))
    rt._check(rt.lib.swc_hip_matrixMatrixMul_f(m, n, k, dwide.ptr, k + 8, db.ptr, n, out.ptr, n), "matrixMatrixMul_f")
    assert rt.last_kernel().startswith("gemm_skinny_stream<"), rt.last_kernel()
    assert_bit_exact(out.numpy(), (wide[:, :k].astype(np.int64) @ b.astype(np.int64)).astype(np.float32), "lda > k")
    # the plain kernel gives the same integers
    switch_env.setenv("SWC_HIP_SKINNY", "plain")
    assert_bit_exact(rt.fcbias(da, db, dbias, relu=False).numpy(), want, "plain kernel")
    assert rt.last_kernel().startswith("gemm_skinny<"), rt.last_kernel()


@pytest.mark.parametrize("m,k,n", [(1, 4100, 600), (7, 4096, 1000), (32, 2048, 1000), (32, 1030, 1028), (17, 3000, 404),
                                   (8, 25088, 512), (33, 2048, 1000), (64, 4100, 300), (50, 1111, 1000)])
def test_gemm_of_up_to_64_rows_and_a_large_b(rt, oracle, m, k, n):
    """Small-batch FC layers stream B once: 32 x 256 or 64 x 256 tiles cut along K, partial sums in the workspace."""
    print("case thin gemm", m, k, n, flush=True)
    assert rt.gemm_workspace_bytes(m, n, k) >= 4 * m * n
    rng = np.random.default_rng(m * 7 + k + n)
    a = rng.integers(-8, 9, (m, k)).astype(np.float32)
    b = rng.integers(-8, 9, (k, n)).astype(np.float32)
    bias = rng.integers(-8, 9, n).astype(np.float32)
    exact = a.astype(np.int64) @ b.astype(np.int64)
    assert_bit_exact(rt.matrixMatrixMul(*up(rt, a, b)).numpy(), exact.astype(np.float32), "integer product")
    assert_bit_exact(rt.fcbias(*up(rt, a, b, bias), relu=True).numpy(),
                     np.maximum(exact + bias.astype(np.int64), 0).astype(np.float32), "integer product + bias + relu")
    ar = rng.standard_normal((m, k)).astype(np.float32)
    br = (rng.standard_normal((k, n)) / np.sqrt(k)).astype(np.float32)
    got = rt.fcbias(*up(rt, ar, br, bias)).numpy()
    want = ar.astype(np.float64) @ br.astype(np.float64) + bias
    mag = np.abs(ar).astype(np.float64) @ np.abs(br).astype(np.float64) + np.abs(bias)
    assert np.max(np.abs(got - want) / mag) < TOL
    if m * k * n <= 32 * 2048 * 1000:
        assert np.max(np.abs(got - oracle.fcbias(ar, br, bias)) / mag) < TOL


@pytest.mark.parametrize("m,k,n", [(8, 784, 512), (1, 784, 512), (16, 1000, 100), (3, 5, 17), (16, 1, 33), (7, 64, 520),
                                   (8, 4096, 512), (2, 130, 4099),
                                   (32, 784, 512), (40, 700, 300), (128, 512, 256), (100, 1000, 90), (17, 1024, 33), (256, 800, 500),
                                   (250, 513, 37)])   # blocks of 16 rows
def test_gemm_of_a_few_rows(rt, oracle, m, k, n):
    """M <= 16 with a small B (or up to 256 rows of a K of 512 to 1024, in blocks of 16 rows): one launch, K split
    over the wavefronts of a workgroup"""
    print("case few-rows gemm", m, k, n, flush=True)
    rng = np.random.default_rng(m * 7 + k + n)
    a = rng.integers(-8, 9, (m, k)).astype(np.float32)
    b = rng.integers(-8, 9, (k, n)).astype(np.float32)
    bias = rng.integers(-8, 9, n).astype(np.float32)
    exact = a.astype(np.int64) @ b.astype(np.int64)
    assert_bit_exact(rt.matrixMatrixMul(*up(rt, a, b)).numpy(), exact.astype(np.float32), "integer product")
    if m > 16 or k * n <= (2 << 20):
        assert rt.last_kernel() == "gemm_fewrows", rt.last_kernel()
    assert_bit_exact(rt.fcbias(*up(rt, a, b, bias), relu=True).numpy(),
                     np.maximum(exact + bias.astype(np.int64), 0).astype(np.float32), "integer product + bias + relu")
    a = rng.uniform(0, 1, (m, k)).astype(np.float32)
    b = rng.uniform(0, 1, (k, n)).astype(np.float32)
    assert strict_rel_err(rt.matrixMatrixMul(*up(rt, a, b)).numpy(), oracle.matrixMatrixMul(a, b)) < TOL
    a = rng.standard_normal((m, k)).astype(np.float32)
    b = rng.standard_normal((k, n)).astype(np.float32)
    assert scaled_err(rt.matrixMatrixMul(*up(rt, a, b)).numpy(), oracle.matrixMatrixMul(a, b),
                      np.abs(a).astype(np.float64) @ np.abs(b).astype(np.float64)) < TOL


def test_gemm_split_over_k_uses_exactly_the_size_it_reports(rt, oracle):
    from swcompiler_amd.hip import SwcHipError
    assert rt.gemm_workspace_bytes(4096, 4096, 784) == 0 and rt.gemm_workspace_bytes(8, 10, 512) == 0
    assert rt.gemm_workspace_bytes(8, 512, 784) == 0   # a handful of rows: the one-pass kernel, no scratch
    assert rt.gemm_workspace_bytes(32, 512, 784) == 0  # up to 256 rows of a K of up to 1024: the same kernel in blocks of 16 rows
    m, n, k = 32, 512, 1568
    need = rt.gemm_workspace_bytes(m, n, k)
    assert need > 0 and need % (m * n * 4) == 0
    rng = np.random.default_rng(21)
    a = rng.integers(-8, 9, (m, k)).astype(np.float32)
    b = rng.integers(-8, 9, (k, n)).astype(np.float32)
    bias = rng.integers(-8, 9, n).astype(np.float32)
    want = np.maximum(a.astype(np.int64) @ b.astype(np.int64) + bias.astype(np.int64), 0).astype(np.float32)
    exact, short = rt.empty((need // 4,)), rt.empty((need // 4 - 4,))
    try:
        rt.set_workspace(exact)
        assert_bit_exact(rt.fcbias(*up(rt, a, b, bias), relu=True).numpy(), want, "split-K in a caller workspace")
        rt.set_workspace(short)
        with pytest.raises(SwcHipError, match="workspace"):
            rt.fcbias(*up(rt, a, b, bias), relu=True)
    finally:
        rt.sync()
        rt.set_workspace(None)


@pytest.mark.parametrize("variant", ["reg22", "reg21", "reg12", "reg11", "22_2", "21_3", "12_3", "11_3", "11_4", "11_3m", "21_3m", "12_3m", "22_3m"])
def test_conv_every_variant(rt, oracle, variant, switch_env):
    print("case conv variant", variant, flush=True)
    switch_env.setenv("SWC_HIP_CONV", variant)
    rng = np.random.default_rng(12)
    for idims, fdims, strides, pads in [((2, 9, 10, 8), (40, 3, 3, 8), (1, 1), (1, 1, 1, 1)),
                                        ((1, 13, 11, 20), (70, 5, 5, 20), (2, 1), (2, 2, 2, 2)),
                                        ((3, 6, 6, 64), (130, 3, 3, 64), (1, 1), (1, 1, 1, 1))]:
        x = rng.integers(-4, 5, idims).astype(np.float32)
        f = rng.integers(-4, 5, fdims).astype(np.float32)
        b = rng.integers(-4, 5, fdims[0]).astype(np.float32)
        want = oracle.relu(oracle.conv2d(x, f, b, fdims[1:3], strides, pads))   # exact: integer-valued
        got = rt.conv2d(*up(rt, x, f, b), fdims[1:3], strides, pads, relu=True).numpy()
        assert_bit_exact(got, want, f"integer conv {idims} variant {variant}")


# Leftover output tiles (those beyond one full round over the chip's workgroup slots) are cut along K and
# their partial sums added by a second kernel.  SWC_HIP_CONV_SLOTS makes a small chip of the real one so that
# small shapes have a full round and leftovers.
SHARED_CONV_CASES = [((2, 20, 20, 32), (70, 3, 3, 32), (1, 1), (1, 1, 1, 1)),     # oC % 4 != 0: scalar stores
                     ((3, 17, 23, 32), (136, 3, 3, 32), (1, 1), (1, 1, 1, 1)),    # ragged rows and columns
                     ((1, 50, 50, 16), (64, 5, 5, 16), (2, 2), (2, 2, 2, 2))]


@pytest.mark.parametrize("variant", [None, "11_3m", "11_4", "21_3", "12_3m", "22_2", "22_3m"])
def test_conv_tiles_shared_along_k(rt, oracle, variant, switch_env):
    print("case conv shared tiles, variant", variant, flush=True)
    if variant:
        switch_env.setenv("SWC_HIP_CONV", variant)
    rng = np.random.default_rng(31)
    for idims, fdims, strides, pads in SHARED_CONV_CASES:
        oc = fdims[0]
        x = rng.integers(-4, 5, idims).astype(np.float32)
        f = rng.integers(-4, 5, fdims).astype(np.float32)
        b = rng.integers(-4, 5, oc).astype(np.float32)
        mean, beta = (rng.integers(-4, 5, oc).astype(np.float32) for _ in range(2))
        var = rng.uniform(0.5, 2.0, oc).astype(np.float32)
        gamma = rng.uniform(0.5, 1.5, oc).astype(np.float32)
        dx, df, db = up(rt, x, f, b)
        bn = up(rt, mean, var, gamma, beta)
        want = oracle.conv2d(x, f, b, fdims[1:3], strides, pads)
        switch_env.setenv("SWC_HIP_CONV_SHARE", "0")
        assert rt.conv2d_workspace_bytes(idims, fdims, strides, pads) == 0
        whole = rt.conv2d(dx, df, db, fdims[1:3], strides, pads, bn=bn, eps=1e-5, relu=True).numpy()
        switch_env.setenv("SWC_HIP_CONV_SHARE", "1")
        shared = 0
        for slots in (3, 4, 5, 6, 7, 9, 11, 13, 17, 19, 23, 29, 37, 47):
            switch_env.setenv("SWC_HIP_CONV_SLOTS", str(slots))
            switch_env.setenv("SWC_HIP_CONV_MIN_IDLE", "0")   # cut tiles however little that saves
            shared += rt.conv2d_workspace_bytes(idims, fdims, strides, pads) > 0
            plain = rt.conv2d(dx, df, db, fdims[1:3], strides, pads).numpy()
            fused = rt.conv2d(dx, df, db, fdims[1:3], strides, pads, bn=bn, eps=1e-5, relu=True).numpy()
            # integer-valued operands: every summation order is exact, so the sums agree bit for bit with the
            # reference's, and the fused epilogue sees the same sums whether a tile was cut or not
            assert_bit_exact(plain, want, f"shared tiles {idims} {variant} slots {slots}")
            assert_bit_exact(fused, whole, f"shared tiles, fused epilogue {idims} {variant} slots {slots}")
        switch_env.delenv("SWC_HIP_CONV_SLOTS")
        assert shared, f"{idims} {variant}: no slot count made this case share tiles"
    # real-valued operands: the usual tolerance
    idims, fdims, strides, pads = SHARED_CONV_CASES[1]
    switch_env.setenv("SWC_HIP_CONV_SLOTS", "4")
    switch_env.setenv("SWC_HIP_CONV_MIN_IDLE", "0")   # cut tiles however little that saves
    x = rng.standard_normal(idims).astype(np.float32)
    f = rng.standard_normal(fdims).astype(np.float32)
    b = rng.standard_normal(fdims[0]).astype(np.float32)
    got = rt.conv2d(*up(rt, x, f, b), fdims[1:3], strides, pads).numpy()
    want = oracle.conv2d(x, f, b, fdims[1:3], strides, pads)
    scale = oracle.conv2d(np.abs(x), np.abs(f), np.abs(b), fdims[1:3], strides, pads)
    assert np.max(np.abs(got - want) / scale) < TOL


@pytest.mark.parametrize("idims,fdims,strides,pads", [((2, 7, 7, 256), (130, 3, 3, 256), (1, 1), (1, 1, 1, 1)),    # 6 tiles of 72 slices
                                                      ((1, 9, 9, 2048), (64, 1, 1, 2048), (1, 1), (0, 0, 0, 0)),   # 1x1, 2 tiles of 64 slices
                                                      ((3, 14, 14, 96), (72, 3, 3, 96), (2, 2), (1, 1, 1, 1)),      # 6 tiles of 27 slices: few enough tiles
                                                      ((3, 14, 14, 32), (72, 3, 3, 32), (2, 2), (1, 1, 1, 1))])     # 9 slices: below the limit
def test_conv_layers_of_few_tiles_and_a_long_k_are_cut_throughout(rt, oracle, idims, fdims, strides, pads, switch_env):
    """Fewer tiles than the chip holds workgroups and K >= 2048 (K >= 512 for a twelfth of a round or less): every
    tile is cut along K (no whole tiles at all)."""
    print("case conv, all tiles shared", idims, fdims, flush=True)
    rng = np.random.default_rng(sum(idims) + sum(fdims))
    x = rng.integers(-4, 5, idims).astype(np.float32)
    f = rng.integers(-4, 5, fdims).astype(np.float32)
    b = rng.integers(-4, 5, fdims[0]).astype(np.float32)
    want = oracle.conv2d(x, f, b, fdims[1:3], strides, pads)
    long_k = int(np.prod(fdims[1:])) >= 512
    assert (rt.conv2d_workspace_bytes(idims, fdims, strides, pads) > 0) == long_k
    dx, df, db = up(rt, x, f, b)
    for slots in (None, 5, 9, 37, 100):
        if slots:
            switch_env.setenv("SWC_HIP_CONV_SLOTS", str(slots))
            switch_env.setenv("SWC_HIP_CONV_MIN_IDLE", "0")   # cut tiles however little that saves
        assert_bit_exact(rt.conv2d(dx, df, db, fdims[1:3], strides, pads).numpy(), want, f"all tiles shared, slots {slots}")
        assert_bit_exact(rt.conv2d(dx, df, db, fdims[1:3], strides, pads, relu=True).numpy(), oracle.relu(want),
                         f"all tiles shared + relu, slots {slots}")
    switch_env.delenv("SWC_HIP_CONV_SLOTS")
    switch_env.setenv("SWC_HIP_CONV_SHARE_ALL", "0")
    switch_env.setenv("SWC_HIP_CONV_MIN_IDLE", "0")   # cut tiles however little that saves
    assert rt.conv2d_workspace_bytes(idims, fdims, strides, pads) == 0
    assert_bit_exact(rt.conv2d(dx, df, db, fdims[1:3], strides, pads).numpy(), want, "whole tiles")
    switch_env.setenv("SWC_HIP_CONV_SHARE_ALL", "8")
    assert rt.conv2d_workspace_bytes(idims, fdims, strides, pads) > 0
    xr = rng.standard_normal(idims).astype(np.float32)
    fr = rng.standard_normal(fdims).astype(np.float32)
    got = rt.conv2d(*up(rt, xr, fr, b), fdims[1:3], strides, pads).numpy()
    scale = oracle.conv2d(np.abs(xr), np.abs(fr), np.abs(b), fdims[1:3], strides, pads)
    assert np.max(np.abs(got - oracle.conv2d(xr, fr, b, fdims[1:3], strides, pads)) / scale) < TOL


@pytest.mark.parametrize("idims,fdims,strides,pads", [((2, 9, 10, 6), (40, 3, 3, 6), (1, 1), (1, 1, 1, 1)),
                                                      ((1, 13, 11, 50), (20, 5, 5, 50), (1, 1), (0, 0, 0, 0)),
                                                      ((2, 15, 15, 3), (64, 7, 7, 3), (2, 2), (3, 3, 3, 3)),
                                                      ((3, 8, 8, 10), (33, 3, 3, 10), (1, 1), (1, 1, 1, 1))])
def test_conv_with_a_channel_count_that_is_no_multiple_of_4(rt, oracle, idims, fdims, strides, pads):
    """Too large for the direct kernel: computed on zero-padded copies of input and filter in the workspace."""
    from swcompiler_amd.hip import SwcHipError
    print("case conv, padded channels", idims, fdims, flush=True)
    rng = np.random.default_rng(sum(idims) + sum(fdims))
    x = rng.integers(-4, 5, idims).astype(np.float32)
    f = rng.integers(-4, 5, fdims).astype(np.float32)
    b = rng.integers(-4, 5, fdims[0]).astype(np.float32)
    want = oracle.conv2d(x, f, b, fdims[1:3], strides, pads)
    need = rt.conv2d_workspace_bytes(idims, fdims, strides, pads)
    cp = (idims[3] + 3) // 4 * 4
    assert need >= 4 * (idims[0] * idims[1] * idims[2] * cp + fdims[0] * fdims[1] * fdims[2] * cp)
    assert_bit_exact(rt.conv2d(*up(rt, x, f, b), fdims[1:3], strides, pads).numpy(), want, "padded channels")
    exact, short = rt.empty((need // 4,)), rt.empty((need // 4 - 4,))
    try:
        rt.set_workspace(exact)
        assert_bit_exact(rt.conv2d(*up(rt, x, f, b), fdims[1:3], strides, pads, relu=True).numpy(), oracle.relu(want),
                         "padded channels, caller workspace")
        rt.set_workspace(short)
        with pytest.raises(SwcHipError, match="workspace"):
            rt.conv2d(*up(rt, x, f, b), fdims[1:3], strides, pads)
    finally:
        rt.sync()
        rt.set_workspace(None)
    xr = rng.standard_normal(idims).astype(np.float32)
    fr = rng.standard_normal(fdims).astype(np.float32)
    got = rt.conv2d(*up(rt, xr, fr, b), fdims[1:3], strides, pads).numpy()
    scale = oracle.conv2d(np.abs(xr), np.abs(fr), np.abs(b), fdims[1:3], strides, pads)
    assert np.max(np.abs(got - oracle.conv2d(xr, fr, b, fdims[1:3], strides, pads)) / scale) < TOL


RESIDUAL_CONV_CASES = [((2, 14, 14, 64), (256, 1, 1, 64), (1, 1), (0, 0, 0, 0)),      # 1x1, whole tiles
                       ((3, 17, 23, 32), (136, 3, 3, 32), (1, 1), (1, 1, 1, 1)),     # ragged rows and columns
                       ((2, 7, 7, 256), (130, 3, 3, 256), (1, 1), (1, 1, 1, 1)),     # every tile cut along K
                       ((2, 9, 10, 6), (40, 3, 3, 6), (1, 1), (1, 1, 1, 1)),         # padded channels
                       ((4, 12, 12, 3), (16, 3, 3, 3), (1, 1), (1, 1, 1, 1))]        # the direct kernel


@pytest.mark.parametrize("idims,fdims,strides,pads", RESIDUAL_CONV_CASES)
@pytest.mark.parametrize("variant", [None, "reg11", "22_3m"])
def test_conv_with_a_second_summand(rt, oracle, idims, fdims, strides, pads, variant, switch_env):
    """conv2dFusedAdd_f = conv2d_f, batchnormalization_f, vecAdd_f with the other branch, relu_f."""
    print("case conv + residual", idims, fdims, variant, flush=True)
    if variant:
        switch_env.setenv("SWC_HIP_CONV", variant)
    rng = np.random.default_rng(sum(idims) + sum(fdims))
    oc = fdims[0]
    x = rng.integers(-4, 5, idims).astype(np.float32)
    f = rng.integers(-4, 5, fdims).astype(np.float32)
    b = rng.integers(-4, 5, oc).astype(np.float32)
    conv = oracle.conv2d(x, f, b, fdims[1:3], strides, pads)
    res = rng.integers(-40, 41, conv.shape).astype(np.float32)
    dx, df, db, dres = up(rt, x, f, b, res)
    add = lambda a, c: oracle.vecAdd(a.ravel(), c.ravel()).reshape(a.shape)
    # integer-valued, no batchnorm: exact
    assert_bit_exact(rt.conv2d(dx, df, db, fdims[1:3], strides, pads, residual=dres).numpy(), add(conv, res), "conv + residual")
    assert_bit_exact(rt.conv2d(dx, df, db, fdims[1:3], strides, pads, residual=dres, relu=True).numpy(),
                     oracle.relu(add(conv, res)), "conv + residual + relu")
    # the summand may be the output itself (a Sum that writes one of its operands)
    inplace = rt.upload(res)
    rt.conv2d(dx, df, db, fdims[1:3], strides, pads, residual=inplace, relu=True, out=inplace)
    assert_bit_exact(inplace.numpy(), oracle.relu(add(conv, res)), "conv + residual in place")
    # with batchnorm: the fused call equals the library's own conv+BN call followed by add and relu, bit for bit
    mean, beta = (rng.integers(-4, 5, oc).astype(np.float32) for _ in range(2))
    var = rng.uniform(0.5, 2.0, oc).astype(np.float32)
    gamma = rng.uniform(0.5, 1.5, oc).astype(np.float32)
    bn = up(rt, mean, var, gamma, beta)
    xr = rng.standard_normal(idims).astype(np.float32)
    fr = (rng.standard_normal(fdims) / np.sqrt(np.prod(fdims[1:]))).astype(np.float32)
    resr = rng.standard_normal(conv.shape).astype(np.float32)
    dxr, dfr, dresr = up(rt, xr, fr, resr)
    fused = rt.conv2d(dxr, dfr, db, fdims[1:3], strides, pads, bn=bn, eps=1e-5, relu=True, residual=dresr).numpy()
    steps = rt.vecAdd(rt.conv2d(dxr, dfr, db, fdims[1:3], strides, pads, bn=bn, eps=1e-5).reshape((-1,)), dresr.reshape((-1,)), relu=True)
    assert_bit_exact(fused.ravel(), steps.numpy(), "conv + bn + residual + relu against the separate calls")
    want = oracle.relu(add(oracle.batchnormalization(oracle.conv2d(xr, fr, b, fdims[1:3], strides, pads), mean, var, gamma, beta, 1e-5), resr))
    mag = np.abs(oracle.batchnormalization(oracle.conv2d(np.abs(xr), np.abs(fr), np.abs(b), fdims[1:3], strides, pads),
                                           -np.abs(mean), var, gamma, np.abs(beta), 1e-5)) + np.abs(resr)
    assert np.max(np.abs(fused - want) / mag) < TOL


def test_conv_shared_tiles_in_a_caller_workspace(rt, oracle, switch_env):
    from swcompiler_amd.hip import SwcHipError
    idims, fdims, strides, pads = SHARED_CONV_CASES[0]
    switch_env.setenv("SWC_HIP_CONV_SLOTS", "19")
    switch_env.setenv("SWC_HIP_CONV_MIN_IDLE", "0")   # cut tiles however little that saves
    need = rt.conv2d_workspace_bytes(idims, fdims, strides, pads)
    assert need > 0
    rng = np.random.default_rng(32)
    x = rng.integers(-4, 5, idims).astype(np.float32)
    f = rng.integers(-4, 5, fdims).astype(np.float32)
    b = rng.integers(-4, 5, fdims[0]).astype(np.float32)
    want = oracle.conv2d(x, f, b, fdims[1:3], strides, pads)
    exact, short = rt.empty((need // 4,)), rt.empty((need // 4 - 4,))
    try:
        rt.set_workspace(exact)
        assert_bit_exact(rt.conv2d(*up(rt, x, f, b), fdims[1:3], strides, pads).numpy(), want, "caller workspace")
        rt.set_workspace(short)
        with pytest.raises(SwcHipError, match="workspace"):
            rt.conv2d(*up(rt, x, f, b), fdims[1:3], strides, pads)
    finally:
        rt.sync()
        rt.set_workspace(None)


@pytest.mark.parametrize("idims,fdims,strides,pads", [((4, 28, 28, 1), (20, 5, 5, 1), (1, 1), (0, 0, 0, 0)),
                                                      ((2, 9, 9, 3), (4, 3, 3, 3), (1, 1), (1, 1, 1, 1)),
                                                      ((1, 17, 13, 3), (32, 5, 3, 3), (2, 1), (2, 1, 2, 1)),
                                                      ((3, 8, 8, 2), (7, 7, 7, 1 + 1), (3, 3), (3, 3, 3, 3))])
def test_small_direct_conv_is_bit_exact(rt, oracle, idims, fdims, strides, pads):
    """First-layer shapes (iC not a multiple of 4, K <= 128, oC <= 32) run the direct kernel, which
    performs the reference's own sequence of fp32 multiplies and adds per output."""
    rng = np.random.default_rng(sum(idims) + sum(fdims))
    x = rng.standard_normal(idims).astype(np.float32)
    f = rng.standard_normal(fdims).astype(np.float32)
    b = rng.standard_normal(fdims[0]).astype(np.float32)
    want = oracle.conv2d(x, f, b, fdims[1:3], strides, pads)
    dx, df, db = up(rt, x, f, b)
    assert_bit_exact(rt.conv2d(dx, df, db, fdims[1:3], strides, pads).numpy(), want, "direct conv")
    assert_bit_exact(rt.conv2d(dx, df, db, fdims[1:3], strides, pads, relu=True).numpy(), oracle.relu(want), "direct conv + relu")


@pytest.mark.parametrize("idims,oc", [((32, 56, 56, 64), 64), ((32, 56, 56, 64), 128), ((32, 28, 28, 128), 128)])
@pytest.mark.parametrize("variant", [None, "11_3m"])
def test_conv_block_layers_full_size(rt, oracle, idims, oc, variant, switch_env):
    """The convolutions of the ResNet-stage-like block at their full sizes, as the default dispatch runs them and
    on the general form of the tile kernel: integer-valued operands, three images through the oracle bit for bit
    and the exact sum over the whole output."""
    print("case conv block layer, full size", idims, oc, variant, flush=True)
    if variant:
        switch_env.setenv("SWC_HIP_CONV", variant)
    fdims = (oc, 3, 3, idims[3])
    rng = np.random.default_rng(oc + idims[1])
    x = rng.integers(-3, 4, idims).astype(np.float32)
    f = rng.integers(-3, 4, fdims).astype(np.float32)
    b = rng.integers(-3, 4, oc).astype(np.float32)
    got = rt.conv2d(*up(rt, x, f, b), (3, 3), (1, 1), (1, 1, 1, 1)).numpy()
    img = [0, 17, 31]
    assert_bit_exact(got[img], oracle.conv2d(x[img], f, b, (3, 3), (1, 1), (1, 1, 1, 1)), "sampled images")
    # sum over everything, exactly: each filter tap multiplies the sum of the input pixels it reaches
    xs = x.astype(np.int64)
    total = int(b.astype(np.int64).sum()) * idims[0] * idims[1] * idims[2]
    fsum = f.astype(np.int64).sum(axis=0)                      # [3,3,C]
    h, w = idims[1], idims[2]
    for ky in range(3):
        for kx in range(3):
            ys = slice(max(0, ky - 1), min(h, h + ky - 1))
            xs_ = slice(max(0, kx - 1), min(w, w + kx - 1))
            total += int((xs[:, ys, xs_, :].sum(axis=(0, 1, 2)) * fsum[ky, kx]).sum())
    assert int(got.astype(np.float64).sum()) == total
