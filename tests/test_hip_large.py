"""Operands beyond 2 GiB: the direct-to-LDS kernels address their operands with 32-bit byte offsets and hand such
calls to the register-staged kernels; element-wise kernels index with 64 bits.  Too large for the CPU checker in
seconds, so the results are checked on samples against numpy (float64 sums) and through exact integer-valued data."""
import numpy as np
import pytest

from tests.util import assert_bit_exact

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def rt():
    from swcompiler_amd.hip import runtime
    return runtime()


def test_eltwise_beyond_2_gib(rt):
    print("case eltwise > 2 GiB", flush=True)
    n = (1 << 29) + 12345          # 2.0 GiB + a ragged tail
    rng = np.random.default_rng(5)
    a = rng.integers(-100, 100, n).astype(np.float32)
    b = rng.integers(-100, 100, n).astype(np.float32)
    da, db = rt.upload(a), rt.upload(b)
    out = rt.vecAdd(da, db, relu=True)
    got = out.numpy()
    for lo in (0, n // 2 - 5000, n - 10000):      # head, the 2 GiB boundary region, tail
        hi = lo + 10000
        assert_bit_exact(got[lo:hi], np.maximum(a[lo:hi] + b[lo:hi], 0), f"add+relu at {lo}")
    assert float(got.astype(np.float64).sum()) == float(np.maximum(a + b, 0).astype(np.float64).sum())
    rt.relu(da, out=out)
    got = out.numpy()
    assert_bit_exact(got[-20000:], np.maximum(a[-20000:], 0), "relu tail")
    assert float(got.astype(np.float64).sum()) == float(np.maximum(a, 0).astype(np.float64).sum())
    for t in (da, db, out):
        t.free()


def test_gemm_with_an_operand_beyond_2_gib(rt):
    print("case gemm > 2 GiB", flush=True)
    m, k, n = 140000, 4096, 24          # A: 2.29 GB
    rng = np.random.default_rng(6)
    a = rng.integers(-3, 4, (m, k)).astype(np.float32)
    b = rng.integers(-3, 4, (k, n)).astype(np.float32)
    bias = rng.integers(-3, 4, n).astype(np.float32)
    da, dw, db = rt.upload(a), rt.upload(b), rt.upload(bias)
    got = rt.fcbias(da, dw, db, relu=True).numpy()
    rows = np.r_[0:64, m // 2 - 32:m // 2 + 32, m - 64:m]
    want = np.maximum(a[rows].astype(np.int64) @ b.astype(np.int64) + bias.astype(np.int64), 0).astype(np.float32)
    assert_bit_exact(got[rows], want, "sampled rows")
    # every row at once: column sums of the un-rectified product
    got = rt.matrixMatrixMul(da, dw).numpy()
    assert np.array_equal(got.astype(np.float64).sum(axis=0), a.astype(np.float64).sum(axis=0) @ b.astype(np.float64))
    for t in (da, dw, db):
        t.free()


def test_conv_with_an_input_beyond_2_gib(rt, oracle):
    print("case conv > 2 GiB", flush=True)
    idims, fdims = (8, 224, 224, 184), (8, 3, 3, 184)      # input 2.36 GB
    rng = np.random.default_rng(7)
    x = rng.integers(-3, 4, idims).astype(np.float32)
    f = rng.integers(-3, 4, fdims).astype(np.float32)
    bias = rng.integers(-3, 4, fdims[0]).astype(np.float32)
    dx, df, db = rt.upload(x), rt.upload(f), rt.upload(bias)
    got = rt.conv2d(dx, df, db, (3, 3), (1, 1), (1, 1, 1, 1), relu=True).numpy()
    # the first and the last image through the CPU checker, rows of the top, the middle and the bottom
    for img in (0, idims[0] - 1):
        for r0 in (0, 111, 221):
            sl = x[img:img + 1, max(r0 - 1, 0):r0 + 4]
            want = oracle.relu(oracle.conv2d(sl, f, bias, (3, 3), (1, 1), (1, 1, 1, 1)))
            off = r0 - max(r0 - 1, 0)
            assert_bit_exact(got[img, r0 + 1:r0 + 2], want[0, off + 1:off + 2], f"image {img} row {r0 + 1}")
    for t in (dx, df, db):
        t.free()
