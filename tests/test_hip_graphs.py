"""The five benchmark graphs end to end on the GPU against the oracle.

The unfused HIP sequence issues exactly the calls the reference's generator
emits; the fused one is what the HIP target emits.  Both must agree with the
oracle's unfused run on identical seeded inputs.  Batch sizes are reduced where
the single-threaded oracle would take minutes; full-size shapes are covered by
sampled-row checks in test_hip_parity.py and by the properties below.
"""
import numpy as np
import pytest

from swcompiler_amd import graphs
from tests.util import assert_bit_exact, rel_err, scaled_err, strict_rel_err

pytestmark = pytest.mark.gpu
TOL = 1e-4


@pytest.fixture(scope="module")
def rt():
    from swcompiler_amd.hip import runtime
    return runtime()


def to_dev(rt, t):
    return {k: rt.upload(v) for k, v in t.items()}


@pytest.mark.parametrize("cfg,batch", [(1, None), (2, 96), (3, 16)])
def test_graph_matches_oracle(rt, oracle, cfg, batch):
    print(f"case graph cfg{cfg} batch {batch}", flush=True)
    t = graphs.make_inputs(cfg, batch)
    want = graphs.run(cfg, oracle, t, fused=False)
    dt = to_dev(rt, t)
    for fused in (False, True):
        got = graphs.run(cfg, rt, dt, fused=fused).numpy()
        assert got.shape == want.shape
        assert rel_err(got, want) < TOL, f"cfg{cfg} fused={fused}"
        assert strict_rel_err(got, want) < TOL  # softmax outputs are strictly positive: the stated bar, literally


def _conv64(x, f, b, pad):
    """float64 direct convolution, NHWC / [oC,kh,kw,iC], stride 1."""
    n, h, w, c = x.shape
    co, kh, kw, _ = f.shape
    xp = np.zeros((n, h + 2 * pad, w + 2 * pad, c))
    xp[:, pad:pad + h, pad:pad + w] = x
    oh, ow = h + 2 * pad - kh + 1, w + 2 * pad - kw + 1
    y = np.zeros((n, oh, ow, co)) + b.astype(np.float64)
    for ky in range(kh):
        for kx in range(kw):
            y += xp[:, ky:ky + oh, kx:kx + ow] @ f[:, ky, kx].astype(np.float64).T
    return y


def test_cfg4_conv_block(rt, oracle):
    """Four chained 3x3 convs (K = 576..1152) + BN + ReLU.

    Per layer: the HIP kernels, fed the ORACLE's activations of the previous
    layer, match the oracle's next activations to 1e-4 of the accumulated
    magnitude (the per-op tolerance for contractions, tests/util.py scaled_err).
    Whole chain: rounding differences of an fp32 sum of ~1000 terms pass through
    three more contractions, so the end-to-end figure is held in the max norm
    and against a float64 evaluation of the same graph: the HIP output must be
    as close to the exact result as the reference's own fp32 arithmetic is."""
    t = graphs.make_inputs(4, 2)
    dt = to_dev(rt, t)
    h_or = t["x"]
    h64 = t["x"].astype(np.float64)
    for i in (1, 2, 3, 4):
        bn = [t[f"bn{i}_{k}"] for k in ("mean", "var", "scale", "bias")]
        dbn = [dt[f"bn{i}_{k}"] for k in ("mean", "var", "scale", "bias")]
        dh = rt.upload(h_or)
        conv = oracle.conv2d(h_or, t[f"f{i}"], t[f"cb{i}"], pads=(1, 1, 1, 1))
        act = oracle.relu(oracle.batchnormalization(conv, *bn, graphs.EPS))
        got_conv = rt.conv2d(dh, dt[f"f{i}"], dt[f"cb{i}"], pads=(1, 1, 1, 1))
        mag = oracle.conv2d(np.abs(h_or), np.abs(t[f"f{i}"]), t[f"cb{i}"], pads=(1, 1, 1, 1))
        assert scaled_err(got_conv.numpy(), conv, mag) < TOL, f"conv{i}"
        unfused = rt.relu(rt.batchnormalization(got_conv, *dbn, graphs.EPS)).numpy()
        fused = rt.conv2d(dh, dt[f"f{i}"], dt[f"cb{i}"], pads=(1, 1, 1, 1), bn=dbn, eps=graphs.EPS, relu=True).numpy()
        mag_bn = (mag + np.abs(bn[0])) * (bn[2] / np.sqrt(bn[1] + graphs.EPS)) + np.abs(bn[3])
        assert scaled_err(unfused, act, mag_bn) < TOL and scaled_err(fused, act, mag_bn) < TOL, f"conv{i}+bn+relu"
        y64 = _conv64(h64, t[f"f{i}"], t[f"cb{i}"], 1)
        mean, var, scale, bias = (v.astype(np.float64) for v in bn)
        h64 = np.maximum((y64 - mean) * (var + np.float32(graphs.EPS)) ** -0.5 * scale + bias, 0)
        h_or = act
        if i in (2, 4):
            h_or = oracle.maxpool(h_or, (2, 2), (2, 2))
            n, hh, ww, c = h64.shape
            h64 = h64.reshape(n, hh // 2, 2, ww // 2, 2, c).max(axis=(2, 4))
    oracle_err = np.max(np.abs(h_or - h64))
    for fused in (False, True):
        got = graphs.run(4, rt, dt, fused=fused).numpy()
        assert got.shape == h_or.shape
        assert np.max(np.abs(got - h_or)) / np.max(np.abs(h_or)) < TOL
        assert np.max(np.abs(got - h64)) <= 2 * oracle_err + 1e-7, (np.max(np.abs(got - h64)), oracle_err)


def test_cfg5_chain(rt, oracle):
    t = graphs.make_inputs(5, batch=4)   # 1024 softmax rows, [4,32,32,256] tensors
    want = graphs.run(5, oracle, t, fused=False)
    dt = to_dev(rt, t)
    for fused in (False, True):
        got = {k: v.numpy() for k, v in graphs.run(5, rt, dt, fused=fused).items()}
        nz = want["a"] > 1e-30
        assert strict_rel_err(got["a"][nz], want["a"][nz]) < TOL
        assert_bit_exact(got["b"], want["b"], "add+relu")
        assert rel_err(got["c"], want["c"]) < TOL


def test_full_size_properties(rt, oracle):
    """BASELINE sizes through size-independent properties."""
    t = graphs.make_inputs(5)
    dt = to_dev(rt, t)
    out = graphs.run(5, rt, dt, fused=True)
    a = out["a"].numpy()
    assert np.allclose(a.sum(1, dtype=np.float64), 1, atol=2e-5) and (a >= 0).all()
    assert np.array_equal(a.argmax(1), t["logits"].argmax(1))
    rows = np.array([0, 1, 4095, 32768, 65535])
    assert strict_rel_err(a[rows], oracle.matrixSoftmax(t["logits"][rows])) < TOL
    b = out["b"].numpy()
    assert_bit_exact(b, np.maximum(t["p"] + t["q"], np.float32(0)) + np.float32(0), "add+relu full size")
    c = out["c"].numpy()
    img = np.array([0, 255])
    bn = [t[f"bn_{k}"] for k in ("mean", "var", "scale", "bias")]
    want = oracle.maxpool(oracle.relu(oracle.batchnormalization(t["p"][img], *bn, graphs.EPS)), (2, 2), (2, 2))
    assert rel_err(c[img], want) < TOL
    # cfg4 full batch: first and last image against the oracle
    t4 = graphs.make_inputs(4)
    got = graphs.run(4, rt, to_dev(rt, t4), fused=True).numpy()
    sub = dict(t4)
    sub["x"] = t4["x"][[0, 31]]
    want = graphs.run(4, oracle, sub, fused=False)
    assert np.max(np.abs(got[[0, 31]] - want)) / np.max(np.abs(want)) < TOL  # chain: max norm, see test_cfg4_conv_block


@pytest.mark.parametrize("cfg,batch", [(1, None), (3, 16), (4, 2)])
def test_hip_graph_replay_equals_eager(rt, cfg, batch):
    """One step captured into a HIP graph; every replay — with eager work and
    synchronisations of the program's own in between — must reproduce the eager
    result bit for bit (same kernels, same launch parameters)."""
    t = graphs.make_inputs(cfg, batch)
    dt = to_dev(rt, t)
    ws = {}
    out = graphs.run(cfg, rt, dt, fused=True, ws=ws)   # eager pass: sets up kernels, allocates outputs
    eager = out.numpy().copy()
    handle = rt.capture(lambda: graphs.run(cfg, rt, dt, fused=True, ws=ws))
    scratch = rt.upload(np.ones(1000, np.float32))
    for i in range(4):
        rt.lib.swc_hip_fill_f(out.ptr, 0.0, out.size)          # wipe the output so a no-op replay would show
        rt.relu(scratch, out=scratch)                            # unrelated eager work between replays
        rt.sync()
        rt.graph_launch(handle)
        assert_bit_exact(out.numpy(), eager, f"replay {i}")
    # new input values through the same graph
    x2 = (t["x"] * np.float32(0.5)).astype(np.float32)
    rt._check(rt.lib.swc_hip_h2d(dt["x"].ptr, x2.ctypes.data, x2.nbytes), "h2d")
    rt.graph_launch(handle)
    replay2 = out.numpy().copy()
    t2 = dict(dt)
    eager2 = graphs.run(cfg, rt, t2, fused=True, ws=ws).numpy()
    assert_bit_exact(replay2, eager2, "replay on new input")
    assert not np.array_equal(replay2, eager)
    rt.graph_destroy(handle)


def test_library_workspace_is_not_replaced_under_a_recorded_graph(rt):
    """A graph recorded while the library's own scratch buffer (swc_hip_enable_auto_workspace) served a
    split-K product keeps that buffer's address in its kernel arguments: until the graph is destroyed an op that
    needs a larger buffer fails instead of freeing it, and so does swc_hip_set_workspace; the graph still replays."""
    from swcompiler_amd.hip import SwcHipError
    rng = np.random.default_rng(3)
    rt.sync()
    rt.set_workspace(None)                      # drop whatever earlier tests grew
    a = rt.upload(rng.standard_normal((160, 448)).astype(np.float32))
    w = rt.upload(rng.standard_normal((448, 200)).astype(np.float32))
    out = rt.empty((160, 200))
    small, big = rt.gemm_workspace_bytes(160, 200, 448), rt.gemm_workspace_bytes(256, 500, 1600)
    assert 0 < small < big - (1 << 20)          # (the library rounds its buffer up to 1 MiB)
    rt.fcbias(a, w, None, out=out)              # eager: the library allocates `small`
    eager = out.numpy().copy()
    handle = rt.capture(lambda: rt.fcbias(a, w, None, out=out))
    a2, w2 = rt.empty((256, 1600)), rt.empty((1600, 500))
    try:
        with pytest.raises(SwcHipError, match="recorded graph"):
            rt.fcbias(a2, w2, None)             # would need `big`
        ws = rt.empty((big // 4,))
        with pytest.raises(SwcHipError, match="recorded graph"):
            rt.set_workspace(ws)
        rt.lib.swc_hip_fill_f(out.ptr, 0.0, out.size)
        rt.graph_launch(handle)
        assert_bit_exact(out.numpy(), eager, "replay after the refused growth")
    finally:
        rt.graph_destroy(handle)
    rt.fcbias(a2, w2, None)                     # the graph is gone: the buffer may grow now
    rt.sync()


@pytest.mark.gpu
def test_shader_clock_watcher(rt):
    """The bench-only library's one-wavefront clock watcher (swc_hip_bench_clock_watch_*): it ends by itself, the
    work enqueued beside it runs undisturbed and correctly, and the clock it reads is a plausible shader clock —
    no higher under a long matrix product than on an idle chip."""
    idle = rt.shader_clock_ghz(lambda: None, 1.0, watch_ms=1.0)
    assert 0.5 < idle < 3.0, idle
    rng = np.random.default_rng(3)
    a, b = rng.standard_normal((1024, 1024)).astype(np.float32), rng.standard_normal((1024, 1024)).astype(np.float32)
    da, db, out = rt.upload(a), rt.upload(b), rt.empty((1024, 1024))
    busy = rt.shader_clock_ghz(lambda: rt.matrixMatrixMul(da, db, out=out), 0.03, watch_ms=1.0)
    assert 0.5 < busy <= idle + 0.05, (busy, idle)
    want = a.astype(np.float64) @ b.astype(np.float64)
    assert np.max(np.abs(out.numpy() - want)) < 1e-2
