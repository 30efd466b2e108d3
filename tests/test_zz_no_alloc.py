"""swc_hip_matrixMatrixFCBias_noalloc_f — the entry point that never allocates
(fixed scratch array inside the library's device code) — against
swc_hip_matrixMatrixFCBias_f on the same operands: the same kernels with the
same split of K, so the results must be bit-identical.  Two calls in a row, the
second smaller, share the one scratch array."""
import numpy as np
import pytest

from tests.util import assert_bit_exact

pytestmark = pytest.mark.gpu

NOALLOC_SCRATCH_BYTES = 16 << 20   # SWC_HIP_NOALLOC_SCRATCH_BYTES of include/swc_hip.h


@pytest.fixture(scope="module")
def rt():
    from swcompiler_amd.hip import runtime
    return runtime()


def _operands(rt, rng, m, n, k):
    a = rng.standard_normal((m, k), dtype=np.float32)
    w = (rng.standard_normal((k, n), dtype=np.float32) / np.sqrt(k)).astype(np.float32)
    b = rng.uniform(-0.01, 0.01, n).astype(np.float32)
    return a, w, b, rt.upload(a), rt.upload(w), rt.upload(b)


def test_noalloc_matches_workspace_entry_point_twice(rt, oracle):
    rng = np.random.default_rng(0x5C0DE)
    # a product of 33 ranges of K (12.7 MB of partial tiles), then a smaller one (16 ranges)
    for (m, n, k), relu in (((192, 500, 1056), True), ((160, 200, 448), False)):
        need = rt.gemm_workspace_bytes(m, n, k)
        assert 0 < need <= NOALLOC_SCRATCH_BYTES, (m, n, k, need)   # the shape does use the scratch array
        a, w, b, da, dw, db = _operands(rt, rng, m, n, k)
        print(f"noalloc case m={m} n={n} k={k} relu={relu} scratch={need}", flush=True)
        want = rt.fcbias(da, dw, db, relu=relu).numpy()
        got = rt.fcbias_noalloc(da, dw, db, relu=relu).numpy()
        assert_bit_exact(got, want, f"noalloc {m}x{n}x{k}")
        # and both against the CPU oracle (matrixMatrixMul_f + batchedadd_f [+ relu_f])
        ref = oracle.batchedadd(oracle.matrixMatrixMul(a, w), b)
        if relu:
            ref = oracle.relu(ref)
        scale = np.abs(a) @ np.abs(w) + np.abs(b)
        assert float(np.max(np.abs(got - ref) / scale)) < 1e-4


def test_noalloc_without_any_workspace(rt):
    """works where the ordinary entry point is refused: no workspace set, none allocated on demand"""
    from swcompiler_amd.hip import SwcHipError
    rng = np.random.default_rng(7)
    m, n, k = 192, 500, 1056
    a, w, b, da, dw, db = _operands(rt, rng, m, n, k)
    want = rt.fcbias(da, dw, db).numpy()
    rt.sync()
    rt.set_workspace(None)
    rt.enable_auto_workspace(False)
    try:
        with pytest.raises(SwcHipError, match="swc_hip_gemm_workspace_bytes"):
            rt.fcbias(da, dw, db)
        got = rt.fcbias_noalloc(da, dw, db).numpy()
    finally:
        rt.enable_auto_workspace(True)
    assert_bit_exact(got, want, "noalloc without workspace")


def test_noalloc_shapes_that_need_no_scratch(rt):
    rng = np.random.default_rng(11)
    for m, n, k in ((8, 512, 784), (300, 10, 96), (512, 512, 64)):
        assert rt.gemm_workspace_bytes(m, n, k) == 0
        a, w, b, da, dw, db = _operands(rt, rng, m, n, k)
        assert_bit_exact(rt.fcbias_noalloc(da, dw, db, relu=True).numpy(), rt.fcbias(da, dw, db, relu=True).numpy(),
                         f"noalloc {m}x{n}x{k}")


def test_noalloc_rejects_sizes_beyond_the_scratch(rt):
    from swcompiler_amd.hip import SwcHipError
    m, n, k = 64, 4096, 25088   # a thin product cut along K: its partial tiles exceed the fixed array
    assert rt.gemm_workspace_bytes(m, n, k) > NOALLOC_SCRATCH_BYTES
    da, dw, out = rt.empty((m, k)), rt.empty((k, n)), rt.empty((m, n))   # never read: the call is refused first
    with pytest.raises(SwcHipError, match="SWC_HIP_NOALLOC_SCRATCH_BYTES"):
        rt.fcbias_noalloc(da, dw, None, out=out)


def test_noalloc_recorded_in_a_graph(rt):
    """the use the header names: the call recorded into a HIP graph with no workspace anywhere, replayed several times
    with eager work and synchronisations in between; every replay gives the eager result"""
    rng = np.random.default_rng(21)
    m, n, k = 192, 500, 1056
    assert rt.gemm_workspace_bytes(m, n, k) > 0
    a, w, b, da, dw, db = _operands(rt, rng, m, n, k)
    want = rt.fcbias_noalloc(da, dw, db, relu=True).numpy()
    out, other = rt.empty((m, n)), rt.empty((m, n))
    rt.sync()
    rt.set_workspace(None)
    rt.enable_auto_workspace(False)
    try:
        graph = rt.capture(lambda: rt.fcbias_noalloc(da, dw, db, relu=True, out=out))
        for replay in range(4):
            rt.relu(other, out=out)                        # eager work between replays: overwrites the graph's output,
            rt.fcbias_noalloc(da, dw, db, out=other)       # and uses the same scratch array
            rt.sync()
            rt.graph_launch(graph)
            rt.sync()
            assert_bit_exact(out.numpy(), want, f"replay {replay}")
        rt.graph_destroy(graph)
    finally:
        rt.enable_auto_workspace(True)


def test_noalloc_leaves_free_device_memory_unchanged(rt):
    """hipMemGetInfo before and after a series of calls (after one warm-up call, which loads the kernels)"""
    import ctypes as C
    hip = C.CDLL("libamdhip64.so")
    rng = np.random.default_rng(22)
    a, w, b, da, dw, db = _operands(rt, rng, 192, 500, 1056)
    out = rt.empty((192, 500))
    rt.sync()
    rt.set_workspace(None)
    rt.enable_auto_workspace(False)

    def free_bytes():
        free, total = C.c_size_t(), C.c_size_t()
        assert hip.hipMemGetInfo(C.byref(free), C.byref(total)) == 0
        return free.value

    try:
        rt.fcbias_noalloc(da, dw, db, out=out)
        rt.sync()
        before = free_bytes()
        for _ in range(5):
            rt.fcbias_noalloc(da, dw, db, relu=True, out=out)
        rt.sync()
        assert free_bytes() == before
    finally:
        rt.enable_auto_workspace(True)


def test_noalloc_takes_operands_whose_kernel_needs_no_scratch(rt):
    """a shape whose split would overflow the array, on an A that is not on a 16-byte boundary: such operands run on
    the register-staged kernel, which is never split — the call is served, with the ordinary entry point's bits"""
    rng = np.random.default_rng(23)
    m, n, k = 64, 4096, 4096
    assert rt.gemm_workspace_bytes(m, n, k) > NOALLOC_SCRATCH_BYTES
    a = rng.standard_normal((m, k), dtype=np.float32)
    w = (rng.standard_normal((k, n), dtype=np.float32) / np.sqrt(k)).astype(np.float32)
    base = rt.empty((m * k + 4,))
    da = base.offset_view(1, (m, k))
    rt.upload_into(da, a)
    dw = rt.upload(w)
    want = rt.fcbias(da, dw, None).numpy()
    name = rt.last_kernel()
    assert "splitk" not in name, name
    got = rt.fcbias_noalloc(da, dw, None).numpy()
    assert_bit_exact(got, want, "noalloc on an unaligned A")
