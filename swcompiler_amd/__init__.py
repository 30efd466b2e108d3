"""swcompiler_amd — MI355X (gfx950) execution backend for SWCompiler graphs.

Contents:
  csrc/           hand-written HIP kernels and the C-ABI runtime (libswc_hip.so,
                  declared in include/swc_hip.h)
  hip.py          ctypes binding of that C ABI (used by tests and bench.py)
  graphs.py       the benchmark graphs as op sequences on device buffers
  swc/            the C++ compiler side: SWC graph API, passes, HipCodegen

There is no CPU fallback anywhere in this package: if libswc_hip.so is missing
or no gfx950 device is present, calls raise.
"""
from .hip import SwcHip, SwcHipError, DeviceArray, lib_path, load_library  # noqa: F401
