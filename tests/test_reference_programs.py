"""The reference's own example programs (test/*.cpp of the reference tree), compiled unchanged, from where they lie,
against this build's `SWC.h` and library: the drop-in claim for the upstream face of the boundary.  Runs only where
the reference tree is (never on the GPU box).

* every program that targets one device compiles (the multi-rank ones name ParallelCodegen / the parallel passes,
  which are not part of this build);
* the single-device ones run and generate a program; the generated program builds against the reference's own
  `utils/` kernels;
* test/engine/testEngineMLPInfer.cpp end to end: its generated batch loop over records made of the reference's
  eight MNIST digits classifies every one of them correctly (the labels of mnist_images_8.meta.txt).
"""
import glob
import os
import shutil
import subprocess

import numpy as np
import pytest

from tests.test_codegen import GEN, REF_UTILS, ROOT, SWC

REF_TESTS = "/root/reference/test"
pytestmark = pytest.mark.skipif(not os.path.isdir(REF_TESTS), reason="the reference tree is not here")

MULTI_RANK = {"benchmark/benchParallelLowering", "old/testParaMLPTraining", "parallel/testJointGraph",
              "parallel/testLenetDistTrain", "parallel/testMLPDistTrain", "parallel/testParallelInfer",
              "parallel/testParallelInferStrategyB", "parallel/testParallelInferStrategyC",
              "parallel/testParallelInferStrategyD", "testParallelPattern"}


@pytest.fixture(scope="module")
def lib():
    if not os.path.exists(GEN):
        subprocess.check_call(["make", "-C", SWC, "-j8"], stdout=subprocess.DEVNULL)
    return os.path.join(SWC, "libswc.a")


def programs():
    return sorted(os.path.relpath(p, REF_TESTS)[:-4] for p in glob.glob(REF_TESTS + "/**/*.cpp", recursive=True))


def compile_program(name, lib, out=None):
    cmd = ["g++", "-std=c++11", "-w", "-I", os.path.join(SWC, "include"), "-I", os.path.join(SWC, "src"),
           os.path.join(REF_TESTS, name + ".cpp")]
    cmd += ["-fsyntax-only"] if out is None else [lib, "-o", out]
    return subprocess.run(cmd, capture_output=True, text=True)


def test_every_single_device_program_compiles_and_links(lib, tmp_path):
    """compiled AND linked against libswc.a (a declaration without a definition would pass a syntax check)"""
    names = programs()
    assert len(names) >= 30 and MULTI_RANK <= set(names)
    single = [n for n in names if n not in MULTI_RANK]
    assert len(single) >= 22 and "cuda/testGPUInfer" in single and "old/testGraphPartition" in single
    from concurrent.futures import ThreadPoolExecutor
    def build(n):
        r = compile_program(n, lib, os.path.join(tmp_path, n.replace("/", "_") + ".bin"))
        return n, (r.stderr.splitlines()[:3] if r.returncode else None)
    with ThreadPoolExecutor(4) as pool:
        failed = {n: e for n, e in pool.map(build, single) if e}
    assert not failed, failed


def build_generated(tmp_path):
    subprocess.check_call(["g++", "-std=c++11", "-O2", "-w", "-I", REF_UTILS, "-I", os.path.join(ROOT, "include"), "Graph.cpp",
                           os.path.join(REF_UTILS, "utils", "DataLoader.cpp"), "-o", "generated.bin"], cwd=tmp_path)
    return os.path.join(tmp_path, "generated.bin")


@pytest.mark.parametrize("name,calls", [
    ("testMLP", ["matrixMatrixMul_f(", "matrixTanh_f("]),
    ("testConvnet", ["conv2dGrad_f(", "maxpoolGrad_f(", "sgd_f(", "matrixSoftmaxWithLossGrad_f(", "addOp(net, "]),   # TRAIN(...)
    ("testSnapshot", ["matrixSoftmaxGrad_f(", "sgd_f(", "addOp(net, ", "loadFromSnapShot("]),                       # getTrainNet
    ("old/testTraining", ["matrixTanhGrad_f(", "sgd_f("]),
])
def test_program_generates_code_that_builds(lib, tmp_path, name, calls):
    exe = os.path.join(tmp_path, "program.bin")
    r = compile_program(name, lib, exe)
    assert r.returncode == 0, r.stderr[-2000:]
    subprocess.run([exe], cwd=tmp_path, check=True, capture_output=True, timeout=120)
    code = open(os.path.join(tmp_path, "Graph.cpp")).read()
    for c in calls:
        assert c in code, c
    build_generated(tmp_path)


def test_gpu_example_retargeted_by_the_environment(lib, tmp_path):
    """test/cuda/testGPUInfer.cpp — the reference's only GPU example: two hand-built SubGraph nodes labelled for
    GPU 0 and GPU 1, a plain Codegen with Config::cuda — unchanged, with SWC_TARGET=hip: the generator writes the
    nested graphs' ops in place of their nodes, both on the one device, keeps the hand-placed Scatter/Gather nodes
    with their offsets, and places the rest of the graph on the device too.  Without the variable the CUDA target
    is refused with a message."""
    from tests.test_codegen import build_hip
    exe = os.path.join(tmp_path, "program.bin")
    assert compile_program("cuda/testGPUInfer", lib, exe).returncode == 0
    r = subprocess.run([exe], cwd=tmp_path, capture_output=True, text=True, timeout=120)
    assert r.returncode != 0 and "use Config::hip" in r.stderr
    subprocess.run([exe], cwd=tmp_path, check=True, capture_output=True, timeout=120, env=dict(os.environ, SWC_TARGET="hip"))
    code = open(os.path.join(tmp_path, "Graph.cpp")).read()
    head, body = code.split("// call op routine functions")
    for name in ("weight0_gpu0, weight0", "weight0_gpu1, weight0", "bias0_gpu0, bias0", "bias0_gpu1, bias0"):
        assert f"swc_hip_h2d({name}," in head            # parameters: uploaded once, to both copies
    assert "swc_hip_h2d(data0_gpu0, data0, 12544)" in body and "swc_hip_h2d(data0_gpu1, data0 + 3136, 12544)" in body
    assert "swc_hip_d2h(data2, data2_gpu0, 8192)" in body and "swc_hip_d2h(data2 + 2048, data2_gpu1, 8192)" in body
    assert body.count("swc_hip_matrixMatrixMul_f(4, 512, 784,") == 2 and body.count("swc_hip_matrixTanh_f(4, 512,") == 2
    assert "swc_hip_matrixSoftmax_f(8, 10," in body and "swc_hip_argMax_i(" in body
    assert "cuda" not in code and "gpu1_baseptr" not in code   # one device, one arena
    build_hip(tmp_path)


def test_graph_partition_example(lib, tmp_path):
    """test/old/testGraphPartition.cpp: IRGraph::buildSubGraphs cuts the first layer into two SubGraph nodes; the
    program runs, and with SWC_TARGET=hip its graph becomes a HIP program that builds"""
    from tests.test_codegen import build_hip
    exe = os.path.join(tmp_path, "program.bin")
    assert compile_program("old/testGraphPartition", lib, exe).returncode == 0
    out = subprocess.run([exe], cwd=tmp_path, check=True, capture_output=True, text=True, timeout=120,
                         env=dict(os.environ, SWC_TARGET="hip")).stdout
    assert "build SubGraph Ok" in out and out.count("subGraph Node") == 2
    code = open(os.path.join(tmp_path, "Graph.cpp")).read()
    assert code.count("swc_hip_matrixTanh_f(4, 512,") == 2
    # each slice reads and writes ITS rows (the reference's buildSubGraphs leaves both at the first slice's)
    assert "swc_hip_h2d(data0_sub, data0, 12544)" in code and "swc_hip_h2d(data0_sub1, data0 + 3136, 12544)" in code
    assert "swc_hip_d2h(data2, data2_sub, 8192)" in code and "swc_hip_d2h(data2 + 2048, data2_sub1, 8192)" in code
    build_hip(tmp_path)


def test_engine_mlp_infer_example_retargeted_by_the_environment(lib, tmp_path):
    """the same unchanged program with SWC_TARGET=hip: Engine::compile places the graph on the GPU and the HIP
    generator writes the program (built here against include/swc_hip.h; it runs where a GPU is)"""
    from tests.test_codegen import build_hip
    exe = os.path.join(tmp_path, "program.bin")
    assert compile_program("engine/testEngineMLPInfer", lib, exe).returncode == 0
    subprocess.run([exe], cwd=tmp_path, check=True, capture_output=True, timeout=120, env=dict(os.environ, SWC_TARGET="hip"))
    code = open(os.path.join(tmp_path, "Graph.cpp")).read()
    loop = code[code.index("while(loader.next("):code.index("} //while")]
    assert "swc_hip_matrixMatrixFCBiasSoftmax_f(" in loop and "swc_hip_argMax_i(" in loop and "swc_hip_accuracy_i(" in loop
    assert loop.count("swc_hip_h2d(") == 2 and "matrixMatrixMul_f(" not in code
    build_hip(tmp_path)


def test_engine_mlp_infer_example_end_to_end(lib, tmp_path):
    exe = os.path.join(tmp_path, "program.bin")
    assert compile_program("engine/testEngineMLPInfer", lib, exe).returncode == 0
    subprocess.run([exe], cwd=tmp_path, check=True, capture_output=True, timeout=120)
    assert os.path.exists(os.path.join(tmp_path, "mlp_def.dot"))
    # the files the generated program reads: the reference's weights, and 10000 records made of its eight digits
    gold = os.path.join(ROOT, "tests", "golden", "mnist8")
    for f in ("mlp_weight0.bin", "mlp_bias0.bin", "mlp_weight1.bin", "mlp_bias1.bin"):
        shutil.copy(os.path.join(gold, f), tmp_path)
    os.mkdir(os.path.join(tmp_path, "input"))
    shutil.copy(os.path.join(gold, "mnist_images_8.bin"), os.path.join(tmp_path, "input"))
    images = np.fromfile(os.path.join(gold, "mnist_images_8.bin"), np.float32).reshape(8, 784)
    labels = [5, 0, 4, 1, 9, 2, 1, 3]                      # mnist_images_8.meta.txt
    record = b"".join(bytes([l]) + img.tobytes() for l, img in zip(labels, images))
    with open(os.path.join(tmp_path, "mnist_labels_images_10k.bin"), "wb") as f:
        for _ in range(1250):
            f.write(record)
    out = subprocess.run([build_generated(tmp_path)], cwd=tmp_path, check=True, capture_output=True, text=True, timeout=300).stdout
    lines = out.strip().splitlines()
    assert lines[-2] == "iterations 1250" and lines[-1].split() == ["10000", "10000"], lines[-3:]
