"""The oracle's training kernels (kernels.h:68-86, 105-151, 245-319, 380-442, 554-590):
against the committed outputs of the reference's own build, against that build itself on
larger inputs (when present), and against what calculus fixes — each gradient kernel is the
derivative of the forward kernel it belongs to, checked by central differences in float64."""
import numpy as np
import pytest

from oracle.binding import load_ref, pool_out_dims, ref_available
from tests.util import assert_bit_exact, ulp_distance


def _sp(golden, key):
    v = [int(t) for t in golden[key]]
    return v


# ------------------------------------------------------------------ golden
@pytest.mark.parametrize("tag", ["p1", "s2", "k5", "asym", "c32"])
def test_conv2dGrad_golden(oracle, golden, tag):
    x, f, og = golden[f"cgrad_{tag}_x"], golden[f"cgrad_{tag}_f"], golden[f"cgrad_{tag}_og"]
    sp = _sp(golden, f"cgrad_{tag}_sp")
    ig, fg, bg = oracle.conv2dGrad(x, f, og, f.shape[1:3], sp[:2], sp[2:])
    assert_bit_exact(ig, golden[f"cgrad_{tag}_ig"], "inputG")
    assert_bit_exact(fg, golden[f"cgrad_{tag}_fg"], "filterG")
    assert_bit_exact(bg, golden[f"cgrad_{tag}_bg"], "biasG")


@pytest.mark.parametrize("tag", ["k2", "k3s2p1", "k3s1"])
def test_maxpoolGrad_golden(oracle, golden, tag):
    ksp = _sp(golden, f"pgrad_{tag}_ksp")
    ig = oracle.maxpoolGrad(golden[f"pgrad_{tag}_x"], golden[f"pgrad_{tag}_og"], ksp[:2], ksp[2:4], ksp[4:])
    assert_bit_exact(ig, golden[f"pgrad_{tag}_ig"], "maxpoolGrad")


@pytest.mark.parametrize("tag", ["a", "b", "c"])
def test_softmax_with_loss_golden(oracle, golden, tag):
    x, sel = golden[f"swl_{tag}_x"], golden[f"swl_{tag}_sel"]
    p, loss = oracle.matrixSoftmaxWithLoss(x, sel)
    # glibc selects an FMA or non-FMA expf/logf by CPU at load time: 1 ulp on the probabilities
    assert ulp_distance(p, golden[f"swl_{tag}_p"]).max() <= 1
    assert abs(loss - golden[f"swl_{tag}_loss"][0]) <= 4e-6 * abs(golden[f"swl_{tag}_loss"][0])
    assert_bit_exact(oracle.matrixSoftmaxGrad(golden[f"swl_{tag}_p"], sel), golden[f"swl_{tag}_grad"], "softmax grad")
    assert_bit_exact(oracle.matrixSoftmaxGrad(golden[f"swl_{tag}_p"], sel, with_loss=True), golden[f"swl_{tag}_grad"],
                     "softmax-with-loss grad")


def test_elementwise_training_golden(oracle, golden):
    assert_bit_exact(oracle.matrixTanhGrad(golden["tanhgrad_y"], golden["tanhgrad_og"]), golden["tanhgrad_ig"], "tanhGrad")
    assert_bit_exact(oracle.matrixTrans(golden["mtrans_x"]), golden["mtrans_y"], "matrixTrans")
    assert_bit_exact(oracle.reluGrad(golden["relugrad_x"], golden["relugrad_dg"]), golden["relugrad_sg"], "reluGrad")
    assert_bit_exact(oracle.batchedreduceadd(golden["rowsum_x"]), golden["rowsum_y"], "batchedreduceadd")
    lr, decay, mom, batch = golden["sgd_params"]
    w1, m1 = oracle.sgd(golden["sgd_w"], golden["sgd_dw"], golden["sgd_mom"], lr, decay, mom, int(batch))
    assert_bit_exact(w1, golden["sgd_w1"], "sgd weights")
    assert_bit_exact(m1, golden["sgd_mom1"], "sgd momentum")


# ------------------------------------------------------- the reference build itself
@pytest.mark.skipif(not ref_available(), reason="oracle/_ref not built (no reference tree)")
def test_training_kernels_vs_reference_build(oracle):
    ref = load_ref()
    rng = np.random.default_rng(21)
    for idims, fdims, st, pd in [((2, 14, 14, 8), (12, 3, 3, 8), (1, 1), (1, 1, 1, 1)),
                                 ((3, 12, 12, 20), (50, 5, 5, 20), (1, 1), (0, 0, 0, 0)),
                                 ((2, 13, 11, 4), (6, 3, 3, 4), (2, 2), (1, 1, 1, 1)),
                                 ((1, 9, 9, 6), (4, 2, 3, 6), (1, 2), (0, 1, 0, 1))]:
        x = rng.standard_normal(idims).astype(np.float32)
        f = rng.standard_normal(fdims).astype(np.float32)
        n, oh, ow, _ = pool_out_dims(idims, fdims[1:3], st, pd)
        og = rng.standard_normal((n, oh, ow, fdims[0])).astype(np.float32)
        for got, want, name in zip(oracle.conv2dGrad(x, f, og, fdims[1:3], st, pd), ref.conv2dGrad(x, f, og, fdims[1:3], st, pd),
                                   ("inputG", "filterG", "biasG")):
            assert_bit_exact(got, want, f"conv2dGrad {name} {idims} {fdims}")
    for idims, k, st, pd in [((2, 24, 24, 20), (2, 2), (2, 2), (0, 0, 0, 0)), ((2, 15, 13, 7), (3, 3), (2, 2), (1, 1, 1, 1)),
                             ((1, 8, 8, 5), (3, 3), (1, 1), (0, 0, 0, 0))]:
        x = np.round(rng.standard_normal(idims) * 2).astype(np.float32) / np.float32(2)
        og = rng.standard_normal(pool_out_dims(idims, k, st, pd)).astype(np.float32)
        assert_bit_exact(oracle.maxpoolGrad(x, og, k, st, pd), ref.maxpoolGrad(x, og, k, st, pd), f"maxpoolGrad {idims}")
    x = (rng.standard_normal((64, 1000)) * 3).astype(np.float32)
    sel = rng.integers(0, 1000, 64).astype(np.int32)
    (p, loss), (pr, lossr) = oracle.matrixSoftmaxWithLoss(x, sel), ref.matrixSoftmaxWithLoss(x, sel)
    assert_bit_exact(p, pr, "softmax with loss")   # same process, same libm
    assert loss == lossr
    b = rng.standard_normal((300, 4096)).astype(np.float32)
    assert_bit_exact(oracle.batchedreduceadd(b), ref.batchedreduceadd(b), "batchedreduceadd")
    w, dw, mom = (rng.standard_normal(50000).astype(np.float32) for _ in range(3))
    for got, want in zip(oracle.sgd(w, dw, mom, 0.05, 0.001, 0.9, 32), ref.sgd(w, dw, mom, 0.05, 0.001, 0.9, 32)):
        assert_bit_exact(got, want, "sgd")


# ------------------------------------------------------------- what calculus fixes
def _conv64(x, f, st, pd):
    """direct convolution in float64 (NHWC, filter [oC,kh,kw,iC], pads t,l,b,r)"""
    n, h, w, c = x.shape
    oc, kh, kw, _ = f.shape
    oh = (h + pd[0] + pd[2] - kh) // st[0] + 1
    ow = (w + pd[1] + pd[3] - kw) // st[1] + 1
    xp = np.zeros((n, h + pd[0] + pd[2], w + pd[1] + pd[3], c))
    xp[:, pd[0]:pd[0] + h, pd[1]:pd[1] + w] = x
    y = np.zeros((n, oh, ow, oc))
    for a in range(kh):
        for b in range(kw):
            patch = xp[:, a:a + oh * st[0]:st[0], b:b + ow * st[1]:st[1]]
            y += np.einsum("nhwc,oc->nhwo", patch, f[:, a, b])
    return y


@pytest.mark.parametrize("st,pd", [((1, 1), (1, 1, 1, 1)), ((2, 2), (1, 1, 1, 1)), ((1, 2), (2, 0, 1, 1)), ((1, 1), (0, 0, 0, 0))])
def test_conv2dGrad_is_the_derivative_of_conv2d(oracle, st, pd):
    """L = sum(conv(x, f) * G): dL/dx, dL/df by central differences (L is bilinear, so they are
    exact up to rounding) and dL/db = sum of G over pixels.  A swapped operand, a flipped tap
    index or a wrong stride/pad sign fails this."""
    rng = np.random.default_rng(3)
    x = rng.standard_normal((2, 6, 7, 3))
    f = rng.standard_normal((4, 3, 2, 3))
    y = _conv64(x, f, st, pd)
    G = rng.standard_normal(y.shape)
    ig, fg, bg = oracle.conv2dGrad(x.astype(np.float32), f.astype(np.float32), G.astype(np.float32), (3, 2), st, pd)
    num_ig = np.zeros_like(x)
    for i in np.ndindex(*x.shape):
        d = np.zeros_like(x)
        d[i] = 1.0
        num_ig[i] = (_conv64(d, f, st, pd) * G).sum()          # linear in x
    num_fg = np.zeros_like(f)
    for i in np.ndindex(*f.shape):
        d = np.zeros_like(f)
        d[i] = 1.0
        num_fg[i] = (_conv64(x, d, st, pd) * G).sum()          # linear in f
    assert np.abs(ig - num_ig).max() < 1e-4
    assert np.abs(fg - num_fg).max() < 1e-4
    # The reference adds outputG to biasG inside the tap loop, at tap (0,0), AFTER the bounds test:
    # output pixels whose first tap lies in the padding are left out (kernels.h:296-311).  With no
    # padding this is the true bias gradient.
    oh, ow = y.shape[1:3]
    keep = np.zeros((oh, ow), bool)
    for ox in range(oh):
        for oy in range(ow):
            keep[ox, oy] = 0 <= ox * st[0] - pd[0] < x.shape[1] and 0 <= oy * st[1] - pd[1] < x.shape[2]
    assert np.abs(bg - (G * keep[None, :, :, None]).sum(axis=(0, 1, 2))).max() < 1e-4
    if pd == (0, 0, 0, 0):
        assert keep.all()


def test_maxpoolGrad_routes_to_first_maximum_and_accumulates(oracle):
    x = np.zeros((1, 4, 4, 1), np.float32)
    x[0, :, :, 0] = [[1, 5, 5, 0], [2, 3, 4, 4], [7, 7, 1, 1], [7, 0, 1, 1]]
    og = np.array([[10, 20], [30, 40]], np.float32).reshape(1, 2, 2, 1)
    ig = oracle.maxpoolGrad(x, og, (2, 2), (2, 2))[0, :, :, 0]
    want = np.zeros((4, 4), np.float32)
    want[0, 1] = 10      # 5 at (0,1) comes first in scan order (kx,ky) = (0,1)
    want[0, 2] = 20      # window (0,2..3): 5 first
    want[2, 0] = 30      # 7 at (2,0) before (2,1) and (3,0)
    want[2, 2] = 40      # all ones: first tap
    assert_bit_exact(ig, want, "first maximum")
    # overlapping windows (3x3, stride 1): one peak receives the sum of every window that sees it
    x = np.zeros((1, 5, 5, 1), np.float32)
    x[0, 2, 2, 0] = 9
    og = np.ones((1, 3, 3, 1), np.float32)
    ig = oracle.maxpoolGrad(x, og, (3, 3), (1, 1))
    assert ig[0, 2, 2, 0] == 9 and ig.sum() == 9
    # gradient mass is conserved whatever the geometry
    rng = np.random.default_rng(5)
    x = rng.standard_normal((2, 9, 8, 3)).astype(np.float32)
    og = rng.integers(-8, 9, pool_out_dims(x.shape, (3, 3), (2, 2), (1, 1, 1, 1))).astype(np.float32)
    assert oracle.maxpoolGrad(x, og, (3, 3), (2, 2), (1, 1, 1, 1)).sum() == og.sum()


def test_softmax_loss_and_its_gradient(oracle):
    rng = np.random.default_rng(7)
    x = rng.standard_normal((6, 9)) * 2
    sel = rng.integers(0, 9, 6).astype(np.int32)

    def loss64(z):
        z = z - z.max(axis=1, keepdims=True)
        return (np.log(np.exp(z).sum(axis=1)) - z[np.arange(6), sel]).mean()
    p, loss = oracle.matrixSoftmaxWithLoss(x.astype(np.float32), sel)
    assert abs(loss - loss64(x)) < 1e-5
    assert np.abs(p.sum(axis=1) - 1).max() < 1e-6
    # the reference's gradient is that of the SUM over rows (no 1/m): m * d(mean loss)/dx
    g = oracle.matrixSoftmaxGrad(p, sel, with_loss=True)
    num = np.zeros_like(x)
    for i in np.ndindex(*x.shape):
        d = np.zeros_like(x)
        d[i] = 1e-5
        num[i] = (loss64(x + d) - loss64(x - d)) / 2e-5 * 6
    assert np.abs(g - num).max() < 1e-4


def test_tanhGrad_reluGrad_rowsum_sgd_closed_forms(oracle):
    rng = np.random.default_rng(9)
    z = rng.standard_normal((5, 7))
    t = np.tanh(z).astype(np.float32)
    og = rng.standard_normal((5, 7)).astype(np.float32)
    assert np.abs(oracle.matrixTanhGrad(t, og) - (1 - np.tanh(z) ** 2) * og).max() < 1e-6
    x = np.array([1.0, -1.0, 0.0, -0.0, np.nan, np.inf, -np.inf, 2.0], np.float32)
    dg = np.arange(1, 9, dtype=np.float32)
    assert_bit_exact(oracle.reluGrad(x, dg), np.array([1, 0, 0, 0, 0, 6, 0, 8], np.float32), "reluGrad")
    b = rng.integers(-8, 9, (11, 300)).astype(np.float32)
    assert_bit_exact(oracle.batchedreduceadd(b), b.sum(axis=1, dtype=np.float64).astype(np.float32), "row sums")
    # rows, not columns; sequential fp32 order
    b = np.array([[1e8, 1.0, -1e8, 1.0]], np.float32)
    assert oracle.batchedreduceadd(b)[0] == 1.0      # ((1e8 + 1) - 1e8) + 1 in fp32 = 0 + 1
    w = np.array([1.0, -2.0], np.float32)
    dw = np.array([0.5, 0.25], np.float32)
    mom = np.array([0.1, -0.2], np.float32)
    w1, m1 = oracle.sgd(w, dw, mom, lr=0.5, decay=0.0, momentum=0.5, batch=2)
    # negDelta = dw * (-lr/batch) + mom*momentum: all values exact in binary
    assert_bit_exact(m1, np.array([0.5 * -0.25 + np.float32(0.1) * np.float32(0.5), 0.25 * -0.25 + np.float32(-0.2) * np.float32(0.5)],
                                  np.float32), "momentum")
    assert_bit_exact(w1, w + m1, "weights")
    a = rng.standard_normal((4, 6)).astype(np.float32)
    assert_bit_exact(oracle.matrixTrans(a), a.T.copy(), "matrixTrans")
