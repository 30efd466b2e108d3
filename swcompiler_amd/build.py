"""Compiles libswc_hip.so (every HIP source under csrc/) for gfx950, in-tree.

    python -m swcompiler_amd.build

hipcc cross-compiles without a GPU.  Packed-fp32 instruction selection is
switched off for all device code (-packed-fp32-ops): the compiler otherwise
forms v_pk_*_f32 from ordinary float code, and bit-exact parity with the CPU
kernels matters more here than the last percent of VALU rate.
"""
import glob
import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(HERE)
LIB = os.path.join(HERE, "libswc_hip.so")
BENCH_LIB = os.path.join(HERE, "libswc_hip_bench.so")
HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
FLAGS = ["--offload-arch=gfx950", "-O3", "-std=c++20", "-fPIC",
         "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
         "-Wno-unused-command-line-argument", "-Wno-unknown-attributes"] + os.environ.get("SWC_HIP_HIPCC_FLAGS", "").split()


def sources():
    return sorted(glob.glob(os.path.join(HERE, "csrc", "*.hip")))


def build_lib(verbose=True, jobs=8):
    """Compile each .hip to an object (in parallel), then link the shared library."""
    objdir = os.path.join(HERE, "csrc", "build")
    os.makedirs(objdir, exist_ok=True)
    inc = ["-I", os.path.join(ROOT, "include"), "-I", os.path.join(HERE, "csrc"),
           "-I", os.path.join(HERE, "swc", "src")]   # devices/HipDevice.h: the device description shared with the code generator
    procs, objs = [], []
    for src in sources():
        obj = os.path.join(objdir, os.path.basename(src)[:-4] + ".o")
        objs.append(obj)
        cmd = [HIPCC] + FLAGS + inc + ["-c", src, "-o", obj]
        if verbose:
            print(" ".join(cmd), flush=True)
        procs.append((src, subprocess.Popen(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)))
        while sum(p.poll() is None for _, p in procs) >= jobs:
            procs[0][1].wait()
    failed = False
    for src, p in procs:
        out, _ = p.communicate()
        out = "\n".join(l for l in out.splitlines() if "packed-fp32-ops" not in l and l.strip())
        if p.returncode != 0:
            failed = True
            print(f"FAILED {src}\n{out}", file=sys.stderr)
        elif out and verbose:
            print(out)
    if failed:
        raise RuntimeError("hipcc failed")
    cmd = [HIPCC, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", LIB] + objs
    if verbose:
        print(" ".join(cmd), flush=True)
    subprocess.check_call(cmd)
    # the bench-only helper library (include/swc_hip_bench.h): not part of the product ABI
    cmd = [HIPCC] + FLAGS + ["-I", os.path.join(ROOT, "include"), "-shared", "-o", BENCH_LIB] + \
        sorted(glob.glob(os.path.join(HERE, "csrc", "bench", "*.hip")))
    if verbose:
        print(" ".join(cmd), flush=True)
    out = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    if out.returncode != 0:
        print(out.stdout, file=sys.stderr)
        raise RuntimeError("hipcc failed (bench library)")
    return LIB


if __name__ == "__main__":
    build_lib()
    print("built", LIB)
