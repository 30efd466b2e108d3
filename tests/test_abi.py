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
