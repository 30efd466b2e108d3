"""Parity of the HIP training kernels (through the C ABI) against the CPU oracle.

Bit-exact: reluGrad, matrixTanhGrad, matrixSoftmax[WithLoss]Grad, sgd, matrixTrans,
batchedreduceadd (row sums in the reference's order), maxpoolGrad (also with
overlapping windows: the gather adds in the reference's order).
Within 1e-4: matrixSoftmaxWithLoss (probabilities element-wise, loss relative) and
conv2dGrad.  The gradients of a convolution are contractions like the forward pass
and are judged the same way: bit-exact on integer-valued operands, error relative
to the sum of the magnitudes of the products on signed operands (see
test_hip_parity.py); the sums of magnitudes come from the oracle run on |operands|.
"""
import numpy as np
import pytest

from oracle.binding import pool_out_dims
from tests.util import assert_bit_exact, strict_rel_err

pytestmark = pytest.mark.gpu
TOL = 1e-4


@pytest.fixture(scope="module")
def rt():
    from swcompiler_amd.hip import runtime
    return runtime()


def up(rt, *arrays):
    return [rt.upload(a) for a in arrays]


# ------------------------------------------------------------ bit-exact kernels
@pytest.mark.parametrize("n", [1, 3, 4, 1031, 4096, (1 << 20) + 4])
def test_reluGrad_bit_exact(rt, oracle, n):
    print("case reluGrad n =", n, flush=True)
    rng = np.random.default_rng(n)
    x = rng.standard_normal(n).astype(np.float32)
    dg = rng.standard_normal(n).astype(np.float32)
    if n >= 12:
        x[:8] = [0.0, -0.0, np.nan, np.inf, -np.inf, 1e-45, -1e-45, 3.0]
        dg[8:12] = [np.nan, np.inf, -0.0, 0.0]
    assert_bit_exact(rt.reluGrad(*up(rt, x, dg)).numpy(), oracle.reluGrad(x, dg), "reluGrad")


def test_elementwise_training_golden(rt, golden):
    assert_bit_exact(rt.reluGrad(*up(rt, golden["relugrad_x"], golden["relugrad_dg"])).numpy(), golden["relugrad_sg"], "reluGrad")
    assert_bit_exact(rt.matrixTanhGrad(*up(rt, golden["tanhgrad_y"], golden["tanhgrad_og"])).numpy(), golden["tanhgrad_ig"],
                     "tanhGrad")
    assert_bit_exact(rt.matrixTrans(rt.upload(golden["mtrans_x"])).numpy(), golden["mtrans_y"], "matrixTrans")
    assert_bit_exact(rt.batchedreduceadd(rt.upload(golden["rowsum_x"])).numpy(), golden["rowsum_y"], "batchedreduceadd")
    lr, decay, mom, batch = golden["sgd_params"]
    w, m = rt.sgd(*up(rt, golden["sgd_w"], golden["sgd_dw"], golden["sgd_mom"]), lr, decay, mom, int(batch))
    assert_bit_exact(w.numpy(), golden["sgd_w1"], "sgd weights")
    assert_bit_exact(m.numpy(), golden["sgd_mom1"], "sgd momentum")
    for tag in "abc":
        p, sel = golden[f"swl_{tag}_p"], golden[f"swl_{tag}_sel"]
        for with_loss in (False, True):
            assert_bit_exact(rt.matrixSoftmaxGrad(rt.upload(p), rt.upload(sel), with_loss).numpy(), golden[f"swl_{tag}_grad"],
                             "softmax grad")


@pytest.mark.parametrize("m,n", [(1, 1), (7, 13), (64, 64), (300, 129), (33, 1000)])
def test_tanhGrad_trans_rowsum_bit_exact(rt, oracle, m, n):
    print("case tanhGrad/trans/rowsum", m, n, flush=True)
    rng = np.random.default_rng(m * 1000 + n)
    t = np.tanh(rng.standard_normal((m, n))).astype(np.float32)
    og = rng.standard_normal((m, n)).astype(np.float32)
    assert_bit_exact(rt.matrixTanhGrad(*up(rt, t, og)).numpy(), oracle.matrixTanhGrad(t, og), "tanhGrad")
    assert_bit_exact(rt.matrixTrans(rt.upload(og)).numpy(), oracle.matrixTrans(og), "matrixTrans")
    assert_bit_exact(rt.batchedreduceadd(rt.upload(og)).numpy(), oracle.batchedreduceadd(og), "row sums")


def test_rowsum_order_sensitive_values(rt, oracle):
    """values whose fp32 sum depends on the order: only the reference's order gives the reference's bits"""
    rng = np.random.default_rng(4)
    b = (rng.standard_normal((130, 3000)) * 10.0 ** rng.integers(-4, 5, (130, 3000))).astype(np.float32)
    assert_bit_exact(rt.batchedreduceadd(rt.upload(b)).numpy(), oracle.batchedreduceadd(b), "row sums")


@pytest.mark.parametrize("n", [1, 1000, 100003])
def test_sgd_bit_exact(rt, oracle, n):
    rng = np.random.default_rng(n)
    w, dw, mom = (rng.standard_normal(n).astype(np.float32) for _ in range(3))
    gw, gm = rt.sgd(*up(rt, w, dw, mom), 0.05, 0.001, 0.9, 32)
    ow, om = oracle.sgd(w, dw, mom, 0.05, 0.001, 0.9, 32)
    assert_bit_exact(gw.numpy(), ow, "sgd weights")
    assert_bit_exact(gm.numpy(), om, "sgd momentum")
    # two steps in a row: state carried on the device
    dwd = rt.upload(dw)
    gw2, gm2 = rt.sgd(gw, dwd, gm, 0.05, 0.001, 0.9, 32)
    ow2, om2 = oracle.sgd(ow, dw, om, 0.05, 0.001, 0.9, 32)
    assert_bit_exact(gw2.numpy(), ow2, "sgd weights, step 2")
    assert_bit_exact(gm2.numpy(), om2, "sgd momentum, step 2")


@pytest.mark.parametrize("n", [3, 4096, 100003])
def test_sgd_into_another_tensor(rt, oracle, n):
    """out != w: out receives out + the step computed from w (kernels.h:565-573)"""
    rng = np.random.default_rng(n + 1)
    w, dw, mom, out = (rng.standard_normal(n).astype(np.float32) for _ in range(4))
    _, om = oracle.sgd(w, dw, mom, 0.05, 0.001, 0.9, 32)
    dwv, ddw, dmom, dout = up(rt, w, dw, mom, out)
    gout, gm = rt.sgd(dwv, ddw, dmom, 0.05, 0.001, 0.9, 32, out=dout)
    assert_bit_exact(gm.numpy(), om, "sgd momentum")
    assert_bit_exact(gout.numpy(), out + om, "sgd out")
    assert_bit_exact(dwv.numpy(), w, "w untouched")


POOLS = [((2, 8, 8, 8), (2, 2), (2, 2), (0, 0, 0, 0)), ((2, 9, 12, 8), (3, 3), (3, 3), (0, 0, 0, 0)),
         ((1, 10, 9, 4), (2, 2), (2, 2), (0, 0, 0, 0)), ((2, 6, 8, 12), (3, 2), (3, 2), (0, 0, 0, 0)),
         ((2, 8, 8, 5), (2, 2), (2, 2), (0, 0, 0, 0)), ((2, 7, 9, 4), (3, 3), (2, 2), (1, 1, 1, 1)),
         ((1, 6, 6, 3), (3, 3), (1, 1), (1, 1, 1, 1)), ((3, 24, 24, 20), (2, 2), (2, 2), (0, 0, 0, 0)),
         ((2, 9, 11, 7), (3, 2), (2, 3), (1, 0, 0, 1)), ((2, 5, 5, 2), (2, 2), (1, 1), (2, 2, 2, 2))]


@pytest.mark.parametrize("idims,k,st,pd", POOLS)
def test_maxpoolGrad_bit_exact(rt, oracle, idims, k, st, pd):
    print("case maxpoolGrad", idims, k, st, pd, flush=True)
    rng = np.random.default_rng(sum(idims))
    x = np.round(rng.standard_normal(idims) * 2).astype(np.float32) / np.float32(2)     # ties
    og = rng.standard_normal(pool_out_dims(idims, k, st, pd)).astype(np.float32)
    assert_bit_exact(rt.maxpoolGrad(*up(rt, x, og), k, st, pd).numpy(), oracle.maxpoolGrad(x, og, k, st, pd), "maxpoolGrad")


@pytest.mark.parametrize("tag", ["k2", "k3s2p1", "k3s1"])
def test_maxpoolGrad_golden(rt, golden, tag):
    ksp = [int(v) for v in golden[f"pgrad_{tag}_ksp"]]
    got = rt.maxpoolGrad(*up(rt, golden[f"pgrad_{tag}_x"], golden[f"pgrad_{tag}_og"]), ksp[:2], ksp[2:4], ksp[4:]).numpy()
    assert_bit_exact(got, golden[f"pgrad_{tag}_ig"], "maxpoolGrad")


# ------------------------------------------------------------ softmax with loss
@pytest.mark.parametrize("m,n,sigma", [(8, 10, 1.0), (5, 1000, 3.0), (256, 10, 2.0), (4096, 10, 1.0), (33, 67, 10.0), (3000, 33, 1.0)])
def test_softmax_with_loss(rt, oracle, m, n, sigma):
    print("case softmaxWithLoss", m, n, flush=True)
    rng = np.random.default_rng(m + n)
    x = (rng.standard_normal((m, n)) * sigma).astype(np.float32)
    sel = rng.integers(0, n, m).astype(np.int32)
    want_p, want_loss = oracle.matrixSoftmaxWithLoss(x, sel)
    p, loss = rt.matrixSoftmaxWithLoss(*up(rt, x, sel))
    assert strict_rel_err(p.numpy(), want_p) < TOL
    assert abs(loss - want_loss) <= TOL * abs(want_loss)
    # the gradient of what the device produced, bit-exact from the same probabilities
    assert_bit_exact(rt.matrixSoftmaxGrad(p, rt.upload(sel), True).numpy(), oracle.matrixSoftmaxGrad(p.numpy(), sel), "grad")


@pytest.mark.parametrize("tag", ["a", "b", "c"])
def test_softmax_with_loss_golden(rt, golden, tag):
    p, loss = rt.matrixSoftmaxWithLoss(*up(rt, golden[f"swl_{tag}_x"], golden[f"swl_{tag}_sel"]))
    assert strict_rel_err(p.numpy(), golden[f"swl_{tag}_p"]) < TOL
    assert abs(loss - golden[f"swl_{tag}_loss"][0]) <= TOL * abs(golden[f"swl_{tag}_loss"][0])


# ------------------------------------------------------------ convolution gradient
def _scaled(got, want, mag):
    den = np.where(mag == 0, 1.0, mag).astype(np.float64)
    return float(np.max(np.abs(got.astype(np.float64) - want.astype(np.float64)) / den))


CONVS = [  # idims, fdims, strides, pads
    ((2, 9, 9, 4), (5, 3, 3, 4), (1, 1), (1, 1, 1, 1)),          # stride 1: forward kernels for inputG, MFMA for filterG
    ((2, 14, 14, 8), (12, 3, 3, 8), (1, 1), (1, 1, 1, 1)),
    ((3, 12, 12, 20), (50, 5, 5, 20), (1, 1), (0, 0, 0, 0)),     # LeNet conv2
    ((2, 28, 28, 1), (20, 5, 5, 1), (1, 1), (0, 0, 0, 0)),       # LeNet conv1: iC = 1, direct filter gradient
    ((2, 11, 10, 8), (7, 3, 3, 8), (2, 2), (1, 1, 1, 1)),        # stride 2: direct inputG
    ((1, 8, 7, 4), (3, 3, 2, 4), (1, 2), (2, 0, 1, 1)),          # asymmetric
    ((2, 6, 6, 64), (32, 3, 3, 64), (1, 1), (1, 1, 1, 1)),
    ((4, 16, 16, 64), (128, 3, 3, 64), (1, 1), (1, 1, 1, 1)),    # wide: 128x128 filter-gradient tiles
    ((1, 5, 7, 12), (9, 1, 1, 12), (1, 1), (0, 0, 0, 0)),        # 1x1; pixel count not a multiple of 4
    ((3, 10, 10, 3), (6, 3, 3, 3), (1, 1), (1, 1, 1, 1)),        # iC = 3
]


@pytest.mark.parametrize("idims,fdims,st,pd", CONVS)
def test_conv2dGrad_vs_oracle(rt, oracle, idims, fdims, st, pd):
    print("case conv2dGrad", idims, fdims, st, pd, flush=True)
    rng = np.random.default_rng(sum(idims) + sum(fdims))
    n, oh, ow, _ = pool_out_dims(idims, fdims[1:3], st, pd)
    odims = (n, oh, ow, fdims[0])
    x = rng.standard_normal(idims).astype(np.float32)
    f = (rng.standard_normal(fdims) / np.sqrt(fdims[1] * fdims[2] * fdims[3])).astype(np.float32)
    og = rng.standard_normal(odims).astype(np.float32)
    want = oracle.conv2dGrad(x, f, og, fdims[1:3], st, pd)
    mags = oracle.conv2dGrad(np.abs(x), np.abs(f), np.abs(og), fdims[1:3], st, pd)
    got = [t.numpy() for t in rt.conv2dGrad(*up(rt, x, f, og), fdims[1:3], st, pd)]
    for g, w, mag, name in zip(got, want, mags, ("inputG", "filterG", "biasG")):
        assert _scaled(g, w, mag) < TOL, name
    # integer-valued operands: every product and sum is exact, any order gives the same bits
    xi = rng.integers(-4, 5, idims).astype(np.float32)
    fi = rng.integers(-4, 5, fdims).astype(np.float32)
    ogi = rng.integers(-4, 5, odims).astype(np.float32)
    want = oracle.conv2dGrad(xi, fi, ogi, fdims[1:3], st, pd)
    got = [t.numpy() for t in rt.conv2dGrad(*up(rt, xi, fi, ogi), fdims[1:3], st, pd)]
    for g, w, name in zip(got, want, ("inputG", "filterG", "biasG")):
        assert_bit_exact(g, w, f"integer {name}")


def _random_grad_cases(count, seed):
    rng = np.random.default_rng(seed)
    cases = []
    while len(cases) < count:
        c = int(rng.choice([1, 3, 4, 8, 20, 32, 64, 96]))
        kh, kw = (int(v) for v in rng.choice([1, 2, 3, 5], 2))
        st = tuple(int(v) for v in rng.choice([1, 1, 2], 2))
        pd = tuple(int(v) for v in rng.integers(0, 3, 4))
        n, h, w = int(rng.integers(1, 4)), int(rng.integers(4, 20)), int(rng.integers(4, 20))
        oc = int(rng.choice([3, 16, 40, 64, 70, 128]))
        if h + pd[0] + pd[2] < kh or w + pd[1] + pd[3] < kw:
            continue
        cases.append(((n, h, w, c), (oc, kh, kw, c), st, pd, [None, "7"][len(cases) % 2]))
    return cases


@pytest.mark.gpu
@pytest.mark.parametrize("idims,fdims,st,pd,slots", _random_grad_cases(32, 777))
def test_conv2dGrad_random_shapes_integer_exact(rt, oracle, idims, fdims, st, pd, slots, switch_env):
    """Random layer shapes (strides, uneven padding, channel counts for every kernel form of the three gradients; on
    a chip pretended to hold seven workgroups for every other one): with small-integer operands any order of
    summation is exact, so inputG, filterG and biasG must equal the oracle's bit for bit."""
    print("case random conv2dGrad", idims, fdims, st, pd, slots, flush=True)
    if slots:
        switch_env.setenv("SWC_HIP_CONV_SLOTS", slots)
        switch_env.setenv("SWC_HIP_CONV_MIN_IDLE", "0")   # cut tiles however little that saves
    rng = np.random.default_rng(sum(idims) * 11 + sum(fdims) * 5 + sum(pd))
    n, oh, ow, _ = pool_out_dims(idims, fdims[1:3], st, pd)
    odims = (n, oh, ow, fdims[0])
    x = rng.integers(-3, 4, idims).astype(np.float32)
    f = rng.integers(-3, 4, fdims).astype(np.float32)
    og = rng.integers(-3, 4, odims).astype(np.float32)
    want = oracle.conv2dGrad(x, f, og, fdims[1:3], st, pd)
    got = [t.numpy() for t in rt.conv2dGrad(*up(rt, x, f, og), fdims[1:3], st, pd)]
    for g, w, name in zip(got, want, ("inputG", "filterG", "biasG")):
        assert_bit_exact(g, w, f"integer {name}")


@pytest.mark.parametrize("tag", ["p1", "s2", "k5", "asym", "c32"])
def test_conv2dGrad_golden(rt, oracle, golden, tag):
    x, f, og = golden[f"cgrad_{tag}_x"], golden[f"cgrad_{tag}_f"], golden[f"cgrad_{tag}_og"]
    sp = [int(v) for v in golden[f"cgrad_{tag}_sp"]]
    got = [t.numpy() for t in rt.conv2dGrad(*up(rt, x, f, og), f.shape[1:3], sp[:2], sp[2:])]
    mags = oracle.conv2dGrad(np.abs(x), np.abs(f), np.abs(og), f.shape[1:3], sp[:2], sp[2:])
    for g, key, mag in zip(got, ("ig", "fg", "bg"), mags):
        assert _scaled(g, golden[f"cgrad_{tag}_{key}"], mag) < TOL, key


def test_conv2dGrad_many_pixels_split_k(rt, oracle):
    """a pixel count that needs many K splits and leaves a ragged last slice (integer-valued: exact)"""
    rng = np.random.default_rng(77)
    idims, fdims = (7, 31, 29, 8), (16, 3, 3, 8)
    odims = pool_out_dims(idims, (3, 3), (1, 1), (1, 1, 1, 1))[:3] + (16,)
    x = rng.integers(-2, 3, idims).astype(np.float32)
    f = rng.integers(-2, 3, fdims).astype(np.float32)
    og = rng.integers(-2, 3, odims).astype(np.float32)
    want = oracle.conv2dGrad(x, f, og, (3, 3), (1, 1), (1, 1, 1, 1))
    got = [t.numpy() for t in rt.conv2dGrad(*up(rt, x, f, og), (3, 3), (1, 1), (1, 1, 1, 1))]
    for g, w, name in zip(got, want, ("inputG", "filterG", "biasG")):
        assert_bit_exact(g, w, name)


@pytest.mark.gpu
@pytest.mark.parametrize("width", ["128", "256", None])
@pytest.mark.parametrize("fdims", [(24, 3, 3, 32), (40, 1, 1, 128), (24, 1, 1, 256), (24, 3, 3, 128), (24, 1, 1, 1408)])
def test_conv2dGrad_narrow_layer_tile_widths(rt, oracle, switch_env, width, fdims):
    """up to 64 output channels: the filter gradient runs on 64 x 128 or 64 x 256 tiles (SWC_HIP_WGRAD_BN forces one;
    unset, the narrow tiles are taken where they cover the kh*kw*iC columns with over a tenth fewer: 288 and 128
    columns take them; 256 columns fill one wide tile exactly and keep it; 1152 columns (nine narrow tiles against
    1280 covered by five wide ones, a ratio of 0.9) sit just on the narrow side of the rule and 1408 (against 1536:
    0.917) just on the wide side).  Integer-valued operands: the gradients equal the oracle's bit for bit on either."""
    print("case conv2dGrad tile width", width, fdims, flush=True)
    if width is None:
        switch_env.delenv("SWC_HIP_WGRAD_BN", raising=False)
    else:
        switch_env.setenv("SWC_HIP_WGRAD_BN", width)
    rng = np.random.default_rng(fdims[0])
    k = fdims[1]
    pads = (k // 2,) * 4
    idims = (3, 21, 19, fdims[3])
    odims = idims[:3] + (fdims[0],)
    x = rng.integers(-2, 3, idims).astype(np.float32)
    f = rng.integers(-2, 3, fdims).astype(np.float32)
    og = rng.integers(-2, 3, odims).astype(np.float32)
    want = oracle.conv2dGrad(x, f, og, (k, k), (1, 1), pads)
    got = [t.numpy() for t in rt.conv2dGrad(*up(rt, x, f, og), (k, k), (1, 1), pads)]
    for g, w, name in zip(got, want, ("inputG", "filterG", "biasG")):
        assert_bit_exact(g, w, name)


@pytest.mark.parametrize("case", [
    # (idims, fdims, strides, pads, group)
    ((2, 9, 11, 8), (8, 3, 3, 8), (1, 1), (1, 1, 1, 1), 2),
    ((3, 12, 12, 16), (32, 3, 3, 16), (1, 1), (1, 1, 1, 1), 4),
    ((2, 13, 10, 6), (4, 3, 3, 6), (2, 2), (1, 1, 1, 1), 2),     # strided: the gather form of the input gradient
    ((2, 8, 8, 3), (6, 5, 5, 3), (1, 1), (2, 2, 2, 2), 3),      # three channels: the small-filter kernels
])
def test_conv2dGrad_groups(rt, oracle, case):
    """group > 1 as kernels.h:245-319 indexes it: computed as one group over a filter with the other groups'
    channels zeroed, the cross-group part of filterG zeroed afterwards.  Integer-valued operands: bit-exact."""
    idims, fdims, strides, pads, group = case
    print("case conv2dGrad groups", case, flush=True)
    rng = np.random.default_rng(group * 100 + fdims[0])
    k = fdims[1:3]
    odims = pool_out_dims(idims, k, strides, pads)[:3] + (fdims[0],)
    x = rng.integers(-2, 3, idims).astype(np.float32)
    f = rng.integers(-2, 3, fdims).astype(np.float32)
    og = rng.integers(-2, 3, odims).astype(np.float32)
    want = oracle.conv2dGrad(x, f, og, k, strides, pads, group)
    got = [t.numpy() for t in rt.conv2dGrad(*up(rt, x, f, og), k, strides, pads, group=group)]
    for g, w, name in zip(got, want, ("inputG", "filterG", "biasG")):
        assert_bit_exact(g, w, name)
    # the elements of filterG that pair an output channel with another group's input channel stay zero
    ocg, cg = fdims[0] // group, fdims[3] // group
    cross = (np.arange(fdims[0])[:, None] // ocg) != (np.arange(fdims[3])[None, :] // cg)
    assert not got[1].transpose(0, 3, 1, 2)[cross].any()
    assert rt.conv2dGrad_workspace_bytes(idims, fdims, strides, pads, group) > 0


@pytest.mark.gpu
def test_workspace_given_by_the_caller(rt, oracle):
    rng = np.random.default_rng(8)
    idims, fdims = (2, 12, 12, 8), (8, 3, 3, 8)
    x = rng.integers(-2, 3, idims).astype(np.float32)
    f = rng.integers(-2, 3, fdims).astype(np.float32)
    og = rng.integers(-2, 3, (2, 12, 12, 8)).astype(np.float32)
    want = oracle.conv2dGrad(x, f, og, (3, 3), (1, 1), (1, 1, 1, 1))
    from swcompiler_amd.hip import SwcHipError
    small = rt.empty((64,))
    rt.set_workspace(small)
    try:
        with pytest.raises(SwcHipError, match="workspace"):
            rt.conv2dGrad(*up(rt, x, f, og), (3, 3), (1, 1), (1, 1, 1, 1))
        big = rt.empty((1 << 22,))
        rt.set_workspace(big)
        got = [t.numpy() for t in rt.conv2dGrad(*up(rt, x, f, og), (3, 3), (1, 1), (1, 1, 1, 1))]
        for g, w in zip(got, want):
            assert_bit_exact(g, w, "with caller workspace")
    finally:
        rt.sync()
        rt.set_workspace(None)


def test_training_error_paths(rt):
    from swcompiler_amd.hip import SwcHipError
    x = rt.empty((1, 4, 4, 4))
    f = rt.empty((4, 3, 3, 4))
    og = rt.empty((1, 4, 4, 4))
    with pytest.raises(SwcHipError, match="group"):
        rt.conv2dGrad(x, f, og, (3, 3), (1, 1), (1, 1, 1, 1), group=3)   # divides neither channel count
    with pytest.raises(SwcHipError):
        rt.conv2dGrad(x, rt.empty((4, 3, 3, 8)), og, (3, 3), (1, 1), (1, 1, 1, 1))
    assert rt.lib.swc_hip_reluGrad_f(None, None, None, 4) != 0
    assert rt.lib.swc_hip_matrixTanhGrad_f(2, 4, x.ptr, 2, x.ptr, 4, x.ptr, 4) != 0     # lda < n


def test_conv2dGrad_full_size_properties(rt, oracle):
    """cfg4's first convolution at full size (32x56x56x64 -> 64): linearity in outputG (the gradients of
    g1 + g2 are the sums of the gradients, to rounding), a gradient that is zero except at one pixel checked
    against the oracle on that neighbourhood, and integer-valued operands against float64 einsum on a slab."""
    rng = np.random.default_rng(99)
    xs, fs = (32, 56, 56, 64), (64, 3, 3, 64)
    x = rng.integers(-2, 3, xs).astype(np.float32)
    f = rng.integers(-2, 3, fs).astype(np.float32)
    og = np.zeros(xs[:3] + (64,), np.float32)
    og[5, 10:13, 20:23, :] = rng.integers(-2, 3, (3, 3, 64))
    dx, df, dog = up(rt, x, f, og)
    ig, fg, bg = (t.numpy() for t in rt.conv2dGrad(dx, df, dog, (3, 3), (1, 1), (1, 1, 1, 1)))
    # only image 5, rows 9..13, columns 19..23 of the input can receive gradient; compare that crop with the oracle
    crop_x = x[5:6, 8:15, 18:25, :]
    crop_og = og[5:6, 9:14, 19:24, :]                     # valid convolution of the crop: 5x5 outputs
    want_ig, want_fg, want_bg = oracle.conv2dGrad(crop_x, f, crop_og, (3, 3), (1, 1), (0, 0, 0, 0))
    assert_bit_exact(ig[5:6, 8:15, 18:25, :], want_ig, "inputG crop")
    assert np.count_nonzero(ig) == np.count_nonzero(want_ig)
    assert_bit_exact(fg, want_fg, "filterG")
    assert_bit_exact(bg, want_bg, "biasG")
    # dense integer gradient: filterG against einsum in float64 for one tap, biasG exactly
    og2 = rng.integers(-1, 2, og.shape).astype(np.float32)
    ig2, fg2, bg2 = (t.numpy() for t in rt.conv2dGrad(dx, df, rt.upload(og2), (3, 3), (1, 1), (1, 1, 1, 1)))
    tap = np.einsum("nhwc,nhwo->oc", x.astype(np.float64), og2.astype(np.float64))     # centre tap (1,1)
    assert_bit_exact(fg2[:, 1, 1, :], tap.astype(np.float32), "filterG centre tap")
    keep = np.zeros((56, 56), bool)
    keep[1:, 1:] = True          # first tap (0,0) inside the image: oy >= 1 and ox >= 1 with pad 1
    assert_bit_exact(bg2, (og2 * keep[None, :, :, None]).sum(axis=(0, 1, 2), dtype=np.float64).astype(np.float32), "biasG")
    # linearity
    ig3, fg3, bg3 = (t.numpy() for t in rt.conv2dGrad(dx, df, rt.upload(og + og2), (3, 3), (1, 1), (1, 1, 1, 1)))
    assert_bit_exact(ig3, ig + ig2, "inputG linear")
    assert_bit_exact(fg3, fg + fg2, "filterG linear")


# ------------------------------------------------------------ the size queries hold for any operand alignment
def _shifted(rt, host, shift):
    """`host` on the device, `shift` floats past a 256-byte boundary (shift % 4 != 0: not on a 16-byte boundary)"""
    base = rt.empty((host.size + shift,))
    view = base.offset_view(shift, host.shape)
    rt.upload_into(view, host)
    return base, view


@pytest.mark.parametrize("case", range(8))
def test_conv2dGrad_query_covers_every_alignment(rt, oracle, case):
    """The query does not see the pointers; each of the call's three alignment tests (input, outputG, filterG) picks
    kernels with their own scratch needs.  With auto-workspace off and a buffer of exactly the queried size the call
    must run — and give the same gradients — for all eight combinations."""
    print("case conv2dGrad alignment", case, flush=True)
    idims, fdims, st, pd = (2, 14, 14, 8), (12, 3, 3, 8), (1, 1), (1, 1, 1, 1)
    rng = np.random.default_rng(77)
    n, oh, ow, _ = pool_out_dims(idims, fdims[1:3], st, pd)
    x = rng.integers(-3, 4, idims).astype(np.float32)
    f = rng.integers(-2, 3, fdims).astype(np.float32)
    og = rng.integers(-2, 3, (n, oh, ow, fdims[0])).astype(np.float32)
    want = oracle.conv2dGrad(x, f, og, fdims[1:3], st, pd)
    keep = []
    xb, dx = _shifted(rt, x, 1 if case & 1 else 0)
    ob, dog = _shifted(rt, og, 1 if case & 2 else 0)
    fgb = rt.empty((f.size + 1,))
    fg = fgb.offset_view(1 if case & 4 else 0, fdims)
    df, ig, bg = rt.upload(f), rt.empty(idims), rt.empty((fdims[0],))
    keep += [xb, ob, fgb]
    need = rt.conv2dGrad_workspace_bytes(idims, fdims, st, pd)
    ws = rt.empty((max(need, 4) // 4,))
    rt.sync()
    rt.set_workspace(ws)
    rt.enable_auto_workspace(False)
    try:
        rt.conv2dGrad(dx, df, dog, fdims[1:3], st, pd, out=(ig, fg, bg))
        got = [ig.numpy(), fg.numpy(), bg.numpy()]
    finally:
        rt.sync()
        rt.set_workspace(None)
        rt.enable_auto_workspace(True)
    for g, w, name in zip(got, want, ("inputG", "filterG", "biasG")):
        assert_bit_exact(g, w, f"{name}, alignment case {case}")   # integer-valued data: exact in any order
