"""The index arithmetic of the row-strip convolution kernel, checked on the CPU.

tests/host/strip_emu.cpp runs the kernel's data movement lane by lane — the same
header (swcompiler_amd/csrc/conv_strip_index.hpp) gives it the lane -> address
maps, swizzles, block assignment and the planner — and must reproduce the
oracle's conv2d_f bit for bit on integer-valued operands, for the planner's own
choice and for forced tile shapes.  No GPU."""
import ctypes as C
import os
import subprocess

import numpy as np
import pytest

from oracle.binding import pool_out_dims
from tests.util import assert_bit_exact

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


@pytest.fixture(scope="module")
def emu(tmp_path_factory):
    so = str(tmp_path_factory.mktemp("strip_emu") / "libstrip_emu.so")
    subprocess.check_call(["g++", "-std=c++17", "-O2", "-fPIC", "-shared", "-I",
                           os.path.join(ROOT, "swcompiler_amd", "csrc"), "-o", so,
                           os.path.join(ROOT, "tests", "host", "strip_emu.cpp")])
    lib = C.CDLL(so)
    ip, fp = C.POINTER(C.c_int), C.POINTER(C.c_float)
    lib.strip_emu_plan.argtypes, lib.strip_emu_plan.restype = [ip, C.c_int, ip], C.c_int
    lib.strip_emu_conv.argtypes, lib.strip_emu_conv.restype = [fp, fp, fp, fp, ip, C.c_int, ip], C.c_int
    return lib


def _geom(idims, fdims, strides, pads):
    odims = pool_out_dims(idims, fdims[1:3], strides, pads)[:3] + (fdims[0],)
    g = list(idims) + [odims[1], odims[2], odims[3], fdims[1], fdims[2], strides[0], strides[1], pads[0], pads[1]]
    return odims, (C.c_int * 13)(*g)


def _plan(emu, idims, fdims, strides, pads, cus):
    _, g = _geom(idims, fdims, strides, pads)
    out = (C.c_int * 11)()
    if not emu.strip_emu_plan(g, cus, out):
        return None
    return dict(zip(("R", "BN", "WM", "WN", "TMW", "TNW", "FW", "PW", "lds_bytes", "tiles", "eff_milli"), out))


def _run(emu, oracle, idims, fdims, strides, pads, cus, force=None, seed=0):
    rng = np.random.default_rng(seed)
    odims, g = _geom(idims, fdims, strides, pads)
    x = rng.integers(-3, 4, idims).astype(np.float32)
    f = rng.integers(-3, 4, fdims).astype(np.float32)
    b = rng.integers(-3, 4, fdims[0]).astype(np.float32)
    out = np.full(odims, np.nan, np.float32)
    fptr = lambda a: a.ctypes.data_as(C.POINTER(C.c_float))
    frc = (C.c_int * 3)(*force) if force else None
    ok = emu.strip_emu_conv(fptr(x), fptr(f), fptr(b), fptr(out), g, cus, frc)
    if not ok:
        return False
    assert_bit_exact(out, oracle.conv2d(x, f, b, fdims[1:3], strides, pads), f"strip emulation {idims} {fdims} {force}")
    return True


CASES = [
    # idims, fdims, strides, pads, cus
    ((2, 8, 8, 16), (16, 3, 3, 16), (1, 1), (1, 1, 1, 1), 4),
    ((3, 14, 14, 32), (32, 3, 3, 32), (1, 1), (1, 1, 1, 1), 8),      # 196 pixels per image: 12.25 blocks
    ((1, 12, 10, 16), (48, 3, 3, 16), (1, 1), (0, 0, 0, 0), 3),      # no padding, 48 channels
    ((2, 9, 9, 16), (32, 5, 5, 16), (1, 1), (2, 2, 2, 2), 2),        # 5 x 5 taps
    ((2, 13, 11, 16), (16, 3, 3, 16), (2, 2), (1, 1, 1, 1), 4),      # stride 2
    ((1, 7, 56, 16), (64, 3, 3, 16), (1, 1), (1, 1, 1, 1), 1),       # 392 pixels, as a 1/256 share of 56 x 56 x 32
]


@pytest.mark.parametrize("case", CASES)
def test_emulated_strip_kernel_matches_oracle(emu, oracle, case):
    idims, fdims, strides, pads, cus = case
    assert _run(emu, oracle, idims, fdims, strides, pads, cus, seed=sum(idims)), "the planner found no plan"


@pytest.mark.parametrize("force", [(1, 16, 8), (2, 16, 8), (7, 32, 4), (14, 32, 4), (14, 32, 8), (14, 16, 8), (7, 16, 8)])
def test_emulated_forced_plans(emu, oracle, force):
    """tile shapes the planner would not pick for this layer: ragged last blocks, wave rows without blocks"""
    assert _run(emu, oracle, (2, 14, 14, 32), (32, 3, 3, 32), (1, 1), (1, 1, 1, 1), 8, force=force, seed=force[0])


def test_planner_on_the_conv_block_configuration(emu):
    """the four layers of the ResNet-stage-like block on 256 compute units: one tile per compute unit each,
    a whole number of tiles per compute unit, at least 80 % of the matrix cores' time estimated useful"""
    layers = [((32, 56, 56, 64), (64, 3, 3, 64)), ((32, 56, 56, 64), (128, 3, 3, 64)),
              ((32, 28, 28, 128), (128, 3, 3, 128))]
    for idims, fdims in layers:
        p = _plan(emu, idims, fdims, (1, 1), (1, 1, 1, 1), 256)
        assert p is not None and p["tiles"] % 256 == 0 and p["eff_milli"] >= 800 and p["TNW"] >= 2, p
        assert p["lds_bytes"] <= 160 * 1024


def test_planner_refuses_what_the_kernel_cannot_take(emu):
    assert _plan(emu, (1, 8, 8, 3), (16, 3, 3, 3), (1, 1), (1, 1, 1, 1), 256) is None      # 3 channels
    assert _plan(emu, (1, 8, 8, 16), (20, 3, 3, 16), (1, 1), (1, 1, 1, 1), 256) is None    # 20 output channels
