"""The C-ABI library loads without a GPU and exports every symbol that
include/swc_hip.h declares; calls before init fail cleanly."""
import os
import re

import pytest

from swcompiler_amd import hip

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def declared_symbols():
    text = open(os.path.join(ROOT, "include", "swc_hip.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(swc_hip_\w+)\s*\(", text)))


def test_header_and_binding_agree():
    assert declared_symbols() == sorted(hip.EXPORTS)


def test_library_exports_every_declared_symbol():
    lib = hip.load_library()
    for name in declared_symbols():
        assert hasattr(lib, name), name


def test_bench_library_exports_its_header():
    """include/swc_hip_bench.h (measurement helpers, not part of the drop-in ABI) against libswc_hip_bench.so"""
    import ctypes
    text = open(os.path.join(ROOT, "include", "swc_hip_bench.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    names = sorted(set(re.findall(r"\b(swc_hip_bench_\w+)\s*\(", text)))
    assert names == ["swc_hip_bench_clock_watch_start", "swc_hip_bench_clock_watch_wait", "swc_hip_bench_probe_mfma_f32"]
    lib = ctypes.CDLL(os.path.join(ROOT, "swcompiler_amd", "libswc_hip_bench.so"))
    for name in names:
        assert hasattr(lib, name), name
    # nothing of it leaks into the product header
    assert "swc_hip_bench" not in open(os.path.join(ROOT, "include", "swc_hip.h")).read()


def test_calls_fail_cleanly_without_device_or_init():
    if os.path.exists("/dev/kfd"):
        pytest.skip("a GPU is present; the no-device path cannot be forced")
    lib = hip.load_library()
    assert lib.swc_hip_relu_f(None, None, 0) == 4          # SWC_HIP_ENOTINIT
    assert b"swc_hip_init" in lib.swc_hip_last_error()
    assert lib.swc_hip_malloc(16) is None
    assert lib.swc_hip_init(0) == 3                        # SWC_HIP_ERUNTIME: no device
    with pytest.raises(hip.SwcHipError):
        hip.SwcHip(0)
