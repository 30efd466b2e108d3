"""The oracle restatement against the reference's kernels.h itself
(oracle/_ref/libswc_ref.so), on larger seeded inputs than the committed
fixtures.  Skipped where the reference build is absent."""
import numpy as np
import pytest

from oracle.binding import load_ref, ref_available
from tests.util import assert_bit_exact, ulp_distance

pytestmark = pytest.mark.skipif(not ref_available(), reason="oracle/_ref not built (no reference tree)")


@pytest.fixture(scope="module")
def ref():
    return load_ref()


def test_gemm(oracle, ref):
    rng = np.random.default_rng(1)
    for m, k, n in [(8, 784, 512), (64, 300, 10), (17, 1, 9), (40, 513, 70)]:
        a = rng.uniform(0, 1, (m, k)).astype(np.float32)
        b = (rng.standard_normal((k, n)) * 0.05).astype(np.float32)
        assert_bit_exact(oracle.matrixMatrixMul(a, b), ref.matrixMatrixMul(a, b), f"gemm {m}x{k}x{n}")


def test_conv(oracle, ref):
    rng = np.random.default_rng(2)
    cases = [((2, 28, 28, 1), (20, 5, 5, 1), (1, 1), (0, 0, 0, 0)),
             ((2, 12, 12, 20), (50, 5, 5, 20), (1, 1), (0, 0, 0, 0)),
             ((1, 14, 14, 64), (32, 3, 3, 64), (1, 1), (1, 1, 1, 1)),
             ((2, 15, 13, 8), (6, 3, 5, 8), (2, 3), (1, 2, 1, 2)),
             ((1, 10, 10, 3), (4, 7, 7, 3), (2, 2), (3, 3, 3, 3))]
    for idims, fdims, s, p in cases:
        x = rng.standard_normal(idims).astype(np.float32)
        f = rng.standard_normal(fdims).astype(np.float32)
        b = rng.standard_normal(fdims[0]).astype(np.float32)
        assert_bit_exact(oracle.conv2d(x, f, b, fdims[1:3], s, p),
                         ref.conv2d(x, f, b, fdims[1:3], s, p), f"conv {idims} {fdims}")
    # more than one group: the filter keeps all iC channels per tap, each output channel reads its group's
    for idims, fdims, s, p, group in [((2, 9, 9, 8), (6, 3, 3, 8), (1, 1), (1, 1, 1, 1), 2),
                                      ((1, 7, 8, 12), (12, 3, 2, 12), (2, 1), (0, 1, 0, 1), 12),
                                      ((2, 6, 6, 6), (9, 1, 1, 6), (1, 1), (0, 0, 0, 0), 3)]:
        x = rng.standard_normal(idims).astype(np.float32)
        f = rng.standard_normal(fdims).astype(np.float32)
        b = rng.standard_normal(fdims[0]).astype(np.float32)
        assert_bit_exact(oracle.conv2d(x, f, b, fdims[1:3], s, p, group),
                         ref.conv2d(x, f, b, fdims[1:3], s, p, group), f"conv {idims} {fdims} in {group} groups")


def test_maxpool(oracle, ref):
    rng = np.random.default_rng(3)
    for idims, k, s, p in [((3, 24, 24, 20), (2, 2), (2, 2), (0, 0, 0, 0)),
                           ((2, 13, 17, 7), (3, 3), (2, 2), (1, 1, 1, 1)),
                           ((1, 9, 9, 3), (3, 2), (1, 3), (0, 1, 0, 1))]:
        x = np.round(rng.standard_normal(idims) * 3).astype(np.float32)
        x.flat[3::37] = np.nan
        y, idx = oracle.maxpool_argmax(x, k, s, p)
        assert_bit_exact(y, ref.maxpool(x, k, s, p), "maxpool")
        og = rng.standard_normal(y.shape).astype(np.float32)
        want = ref.maxpoolGrad(x, og, k, s, p)
        # accumulate in the reference's (n, ox, oy, c) order so overlapping
        # windows add in the same sequence
        scat = np.zeros(x.size, np.float32)
        for o, i in zip(og.ravel(), idx.ravel()):
            scat[i] = np.float32(scat[i] + o)
        assert_bit_exact(scat.reshape(x.shape), want, "chosen taps")


def test_bn_softmax_tanh_elt(oracle, ref):
    rng = np.random.default_rng(4)
    x = rng.standard_normal((4, 14, 14, 128)).astype(np.float32)
    mean, beta = [rng.standard_normal(128).astype(np.float32) * np.float32(0.1) for _ in range(2)]
    var = rng.uniform(0.5, 2, 128).astype(np.float32)
    gamma = rng.uniform(0.5, 1.5, 128).astype(np.float32)
    assert_bit_exact(oracle.batchnormalization(x, mean, var, gamma, beta, 1e-5),
                     ref.batchnormalization(x, mean, var, gamma, beta, 1e-5), "bn")
    z = (rng.standard_normal((64, 1000)) * 3).astype(np.float32)
    assert ulp_distance(oracle.matrixSoftmax(z), ref.matrixSoftmax(z)).max() == 0
    assert ulp_distance(oracle.matrixTanh(z), ref.matrixTanh(z)).max() == 0
    v = x.ravel()
    assert_bit_exact(oracle.relu(v), ref.relu(v), "relu")
    assert_bit_exact(oracle.vecAdd(v, v[::-1].copy()), ref.vecAdd(v, v[::-1].copy()), "vecAdd")
    assert_bit_exact(oracle.argMax(np.round(z), 5), ref.argMax(np.round(z), 5), "argMax")
    pred = oracle.argMax(np.round(z), 2)
    label = np.random.default_rng(9).integers(0, z.shape[1], z.shape[0]).astype(np.int32)
    assert_bit_exact(oracle.accuracy(pred, label, np.array([3, 4], np.int32)),
                     ref.accuracy(pred, label, np.array([3, 4], np.int32)), "accuracy")
