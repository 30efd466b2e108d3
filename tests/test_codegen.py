"""The compiler side: SWC API -> passes -> CPU / HIP code generators.

CPU (no GPU needed): graphs built through the SWC API compile, the CPU program
calls the reference's kernels in the reference's order (checked by running it
against the reference's own utils/kernels.h where the reference tree exists,
else against the oracle through oracle/compat) and its outputs equal the
oracle's graph run bit for bit; the HIP program has the expected structure and
builds against include/swc_hip.h + libswc_hip.so.
GPU: the HIP program runs on the MI355X and matches the oracle.
"""
import os
import re
import shutil
import subprocess

import numpy as np
import pytest

from swcompiler_amd import graphs
from tests.util import assert_bit_exact, rel_err, strict_rel_err

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
SWC = os.path.join(ROOT, "swcompiler_amd", "swc")
GEN = os.path.join(SWC, "test", "bin", "genGraphs")
REF_UTILS = "/root/reference/src/codegen"
TOL = 1e-4


@pytest.fixture(scope="module")
def gen():
    if not os.path.exists(GEN):
        subprocess.check_call(["make", "-C", SWC, "-j8"], stdout=subprocess.DEVNULL)
    return GEN


def file_map(cfg, t):
    """graphs.make_inputs key -> file stem read by the programs genGraphs builds"""
    m = {}
    for k in t:
        if k in ("x", "logits", "p", "q"):
            m[k] = k
        elif re.fullmatch(r"w\d", k):
            m[k] = f"fc{k[1]}_w"
        elif re.fullmatch(r"b\d", k):
            m[k] = f"fc{k[1]}_b"
        elif re.fullmatch(r"f\d", k):
            m[k] = f"conv{k[1]}_f"
        elif re.fullmatch(r"cb\d", k):
            m[k] = f"conv{k[2]}_b"
        elif k.startswith("bn"):
            m[k] = k
    return m


def write_inputs(cfg, t, workdir):
    for k, stem in file_map(cfg, t).items():
        t[k].tofile(os.path.join(workdir, stem + ".bin"))


def generate(gen, model, target, workdir, batch=0, iters=0, nofuse=False, graph=False, prefetch=False, snapshot=0):
    args = [gen, model, target, str(batch), str(iters)] + (["nofuse"] if nofuse else []) + (["graph"] if graph else []) + \
           (["prefetch"] if prefetch else [])
    if snapshot:
        args += ["-"] * (6 - len(args)) + [str(snapshot)]
    code = subprocess.run(args, cwd=workdir, check=True, capture_output=True, text=True).stdout
    assert open(os.path.join(workdir, "Graph.cpp")).read() == code
    return code


def build_cpu(workdir, with_loader=False, force_compat=False):
    if os.path.isdir(REF_UTILS) and not force_compat:   # the reference's own image.h / kernels.h (/ DataLoader)
        cmd = ["g++", "-std=c++11", "-O2", "-w", "-I", REF_UTILS, "-I", os.path.join(ROOT, "include"), "Graph.cpp"]
        if with_loader:
            cmd.append(os.path.join(REF_UTILS, "utils", "DataLoader.cpp"))
        cmd += ["-o", "net_cpu.bin"]
    else:
        odir = os.path.join(ROOT, "oracle")
        cmd = ["g++", "-std=c++11", "-O2", "-I", os.path.join(odir, "compat"), "-I", os.path.join(ROOT, "include"),
               "Graph.cpp", "-L", odir, "-Wl,-rpath," + odir, "-loracle", "-o", "net_cpu.bin"]
    subprocess.check_call(cmd, cwd=workdir)
    return os.path.join(workdir, "net_cpu.bin")


def build_hip(workdir):
    libdir = os.path.join(ROOT, "swcompiler_amd")
    subprocess.check_call(["g++", "-std=c++11", "-O2", "-I", os.path.join(ROOT, "include"), "Graph.cpp", "-L", libdir,
                           "-Wl,-rpath," + libdir, "-lswc_hip", "-o", "net_hip.bin"], cwd=workdir)
    return os.path.join(workdir, "net_hip.bin")


MODELS = [("cfg1", 1, 8, "softmax_out"), ("cfg2", 2, 16, "softmax_out"), ("cfg3", 3, 4, "softmax_out"),
          ("cfg4", 4, 1, "pool4_out"), ("cfg5a", 5, 1, "softmax_out"), ("cfg5b", 5, 1, "relu_out"),
          ("cfg5c", 5, 1, "pool_out")]


def oracle_run(oracle, model, cfg, t):
    out = graphs.run(cfg, oracle, t, fused=False)
    return out[model[-1]] if cfg == 5 else out


def model_batch(model, batch):
    return batch * 256 if model == "cfg5a" else batch   # cfg5a counts softmax rows


@pytest.mark.parametrize("model,cfg,batch,outname", MODELS)
def test_cpu_program_equals_oracle_bit_for_bit(gen, oracle, tmp_path, model, cfg, batch, outname):
    t = graphs.make_inputs(cfg, batch)
    write_inputs(cfg, t, tmp_path)
    code = generate(gen, model, "cpu", tmp_path, model_batch(model, batch))
    assert "swc_hip" not in code and '#include "utils/kernels.h"' in code
    if model in ("cfg1", "cfg2", "cfg3"):   # FCBias is lowered exactly as the reference does it
        assert "matrixMatrixMul_f(" in code and "batchedadd_f(" in code and "_mm_out" in code
    exe = build_cpu(tmp_path)
    subprocess.check_call([exe], cwd=tmp_path, stdout=subprocess.DEVNULL)
    want = oracle_run(oracle, model, cfg, t)
    got = np.fromfile(os.path.join(tmp_path, outname + ".bin"), np.float32).reshape(want.shape)
    assert_bit_exact(got, want, model)


def test_mnist8_cpu_program_prints_the_reference_labels(gen, tmp_path, golden):
    for f in os.listdir(os.path.join(ROOT, "tests", "golden", "mnist8")):
        shutil.copy(os.path.join(ROOT, "tests", "golden", "mnist8", f), tmp_path)
    generate(gen, "mnist8", "cpu", tmp_path)
    exe = build_cpu(tmp_path)
    out = subprocess.run([exe], cwd=tmp_path, check=True, capture_output=True, text=True).stdout
    rows = [[int(v) for v in line.split()] for line in out.strip().splitlines()]
    assert [r[0] for r in rows] == [5, 0, 4, 1, 9, 2, 1, 3]
    assert_bit_exact(np.array(rows, np.int32), golden["mnist8_top3"], "printed top-3")


def test_hip_program_structure_and_build(gen, tmp_path):
    code = generate(gen, "cfg4", "hip", tmp_path, 2)
    # fused: four launches — conv+bn+relu twice, conv+bn+relu with the 2x2 pooling in its epilogue twice — and
    # nothing else on the device
    assert code.count("swc_hip_conv2dFused_f(") == 2 and code.count("swc_hip_conv2dFusedMaxpool_f(") == 2
    assert "swc_hip_batchnorm" not in code and "swc_hip_relu_f" not in code and "swc_hip_maxpool_f(" not in code
    assert "const size_t conv2_convDims[] = {2, 56, 56, 128};" in code and "const size_t conv2_outDims[] = {2, 28, 28, 128};" in code
    assert re.search(r"swc_hip_conv2dFusedMaxpool_f\(\w+, \w+, \w+, \w+, conv2_convDims, conv2_inDims, conv2_filterDims, "
                     r"conv2_biasDims, conv2_filterSizes, conv2_strides, conv2_pads, 1, \w+, \w+, \w+, \w+, [0-9.e-]+, 1, "
                     r"conv2_outDims, conv2_poolSizes, conv2_poolStrides, conv2_poolPads\)", code)
    # the convolution's own output is no tensor of the program any more
    assert code.count("swc_hip_conv2dFusedMaxpool_workspace_bytes(o, i, f, k, s, p, 1, po, pk, ps, pp)") == 2
    # every device tensor sits on a 256-byte boundary of the arena
    offs = [int(v) for v in re.findall(r"gpu0_baseptr \+ (\d+)\)", code)]
    assert offs and all(o % 256 == 0 for o in offs)
    # the host arena is page-locked memory of the library's, the device arena one allocation
    assert "cpu0_baseptr = (char*)swc_hip_host_malloc(" in code and "swc_hip_host_free(cpu0_baseptr)" in code
    assert code.count("swc_hip_malloc(") == 2   # workspace and arena
    # parameters are uploaded once, before the op calls; the result comes back once, after them
    body = code[code.index("// call op routine functions"):]
    assert "swc_hip_h2d" not in body and body.count("swc_hip_d2h(") == 1
    assert code.count("swc_hip_h2d(") == 1 + 4 * 6   # x + per layer filter, bias, 4 bn params
    build_hip(tmp_path)

    unfused = generate(gen, "cfg4", "hip", tmp_path, 2, nofuse=True)
    assert unfused.count("swc_hip_conv2d_f(") == 4 and unfused.count("swc_hip_batchnormalization_f(") == 4
    assert unfused.count("swc_hip_relu_f(") == 4

    mlp = generate(gen, "cfg2", "hip", tmp_path, 64)
    assert mlp.count("swc_hip_matrixMatrixFCBias_f(") == 2 and "swc_hip_batchedadd_f" not in mlp
    # the classifier head and its softmax are one call
    assert re.search(r"swc_hip_matrixMatrixFCBiasSoftmax_f\(64, 10, 4096, ", mlp) and "swc_hip_matrixSoftmax_f" not in mlp
    unfused_mlp = generate(gen, "cfg2", "hip", tmp_path, 64, nofuse=True)
    assert unfused_mlp.count("swc_hip_matrixMatrixFCBias_f(") == 3 and unfused_mlp.count("swc_hip_matrixSoftmax_f(") == 1
    assert re.search(r"swc_hip_matrixMatrixFCBias_f\(64, 4096, 784, .*, 1\)\);", mlp)
    # the program sizes and owns the scratch memory of its FC calls: one query per call, one buffer, given
    # to the library before the first op and taken back before it is freed
    assert mlp.count("swc_hip_gemm_workspace_bytes(") == 3 and "swc_hip_gemm_workspace_bytes(64, 4096, 784)" in mlp
    assert mlp.index("swc_hip_set_workspace(gpu0_ws, gpu0_ws_bytes)") < mlp.index("// call op routine functions")
    assert mlp.index("swc_hip_set_workspace(nullptr, 0)") < mlp.index("swc_hip_free(gpu0_ws)")
    # ... and of its convolutions: one query per conv, with the conv's own shape arrays
    assert code.count("swc_hip_conv2d_workspace_bytes(o, i, f, k, s, p, 1)") == 2
    assert "const size_t o[] = {2, 56, 56, 64};" in code and "const size_t f[] = {128, 3, 3, 64};" in code
    assert code.index("swc_hip_set_workspace(gpu0_ws, gpu0_ws_bytes)") < code.index("// call op routine functions")
    lenet = generate(gen, "cfg3", "hip", tmp_path, 4)
    # LeNet: both layers pool in their epilogue (the first in the direct kernel, the second in the tile kernel)
    assert lenet.count("swc_hip_conv2dFused_f(") == 0 and lenet.count("swc_hip_conv2dFusedMaxpool_f(") == 2
    assert lenet.count("swc_hip_maxpool_f(") == 0 and "swc_hip_matrixMatrixFCBias_f(4, 500, 800" in lenet
    bnpool = generate(gen, "cfg5c", "hip", tmp_path, 1)
    assert bnpool.count("swc_hip_batchnormReluMaxpool_f(") == 1 and "swc_hip_maxpool_f" not in bnpool
    assert "swc_hip_batchnormRelu_f" not in bnpool and "swc_hip_batchnormalization_f" not in bnpool
    bnpool = generate(gen, "cfg5c", "hip", tmp_path, 1, nofuse=True)
    assert bnpool.count("swc_hip_batchnormalization_f(") == 1 and bnpool.count("swc_hip_maxpool_f(") == 1
    timed = generate(gen, "cfg5b", "hip", tmp_path, 1, iters=10)
    assert "swc_hip_vecAddRelu_f(" in timed and "swc_time_ms_per_iter" in timed and "swc_iter < 10" in timed


@pytest.mark.gpu
@pytest.mark.parametrize("model,cfg,batch,outname", MODELS)
@pytest.mark.parametrize("nofuse", [False, True])
def test_hip_program_matches_oracle(gen, oracle, tmp_path, model, cfg, batch, outname, nofuse):
    print(f"case generated {model} batch {batch} nofuse={nofuse}", flush=True)
    t = graphs.make_inputs(cfg, batch)
    write_inputs(cfg, t, tmp_path)
    generate(gen, model, "hip", tmp_path, model_batch(model, batch), nofuse=nofuse)
    exe = build_hip(tmp_path)
    subprocess.run([exe], cwd=tmp_path, check=True, timeout=120, stdout=subprocess.DEVNULL)
    want = oracle_run(oracle, model, cfg, t)
    got = np.fromfile(os.path.join(tmp_path, outname + "_host.bin"), np.float32).reshape(want.shape)
    if model == "cfg5b":
        assert_bit_exact(got, want, model)
    elif model == "cfg4":
        assert np.max(np.abs(got - want)) / np.max(np.abs(want)) < TOL
    elif model == "cfg5c":
        assert rel_err(got, want) < TOL
    else:
        nz = want > 1e-30
        assert strict_rel_err(got[nz], want[nz]) < TOL


@pytest.mark.gpu
def test_mnist8_hip_program_prints_the_reference_labels(gen, tmp_path, golden):
    for f in os.listdir(os.path.join(ROOT, "tests", "golden", "mnist8")):
        shutil.copy(os.path.join(ROOT, "tests", "golden", "mnist8", f), tmp_path)
    generate(gen, "mnist8", "hip", tmp_path)
    exe = build_hip(tmp_path)
    out = subprocess.run([exe], cwd=tmp_path, check=True, capture_output=True, text=True, timeout=120).stdout
    rows = [[int(v) for v in line.split()] for line in out.strip().splitlines()]
    assert [r[0] for r in rows] == [5, 0, 4, 1, 9, 2, 1, 3]
    assert_bit_exact(np.array(rows, np.int32), golden["mnist8_top3"], "printed top-3")
    prob = np.fromfile(os.path.join(tmp_path, "data4_host.bin"), np.float32).reshape(8, 10)
    assert strict_rel_err(prob, golden["mnist8_prob"]) < TOL
    top3 = np.fromfile(os.path.join(tmp_path, "top3_host.bin"), np.int32).reshape(8, 3)
    assert_bit_exact(top3, golden["mnist8_top3"], "dumped top-3")


def test_subgraph_program_structure(gen, tmp_path):
    """IRGraph::buildSubGraphs + SubGraph nodes labelled for two GPUs + a plain Codegen (the reference's route to a
    GPU): on this target both nested graphs are emitted in place, on the one device"""
    for f in os.listdir(os.path.join(ROOT, "tests", "golden", "mnist8")):
        shutil.copy(os.path.join(ROOT, "tests", "golden", "mnist8", f), tmp_path)
    code = generate(gen, "mnist8_subgraphs", "hip", tmp_path)
    head, body = code.split("// call op routine functions")
    assert head.count("swc_hip_h2d(weight0_sub") == 2 and head.count("swc_hip_h2d(bias0_sub") == 2
    assert "swc_hip_h2d(data0_sub, data0, 12544)" in body and "swc_hip_h2d(data0_sub1, data0 + 3136, 12544)" in body
    assert "swc_hip_d2h(data2, data2_sub, 8192)" in body and "swc_hip_d2h(data2 + 2048, data2_sub1, 8192)" in body
    assert "SubGraph" not in body and "gpu1_baseptr" not in code
    build_hip(tmp_path)


@pytest.mark.gpu
def test_subgraph_program_prints_the_reference_labels(gen, tmp_path, golden):
    """the same program run: the reference's MNIST labels, and the probabilities of the un-partitioned program"""
    for f in os.listdir(os.path.join(ROOT, "tests", "golden", "mnist8")):
        shutil.copy(os.path.join(ROOT, "tests", "golden", "mnist8", f), tmp_path)
    generate(gen, "mnist8_subgraphs", "hip", tmp_path)
    exe = build_hip(tmp_path)
    out = subprocess.run([exe], cwd=tmp_path, check=True, capture_output=True, text=True, timeout=120).stdout
    rows = [[int(v) for v in line.split()] for line in out.strip().splitlines()]
    assert [r[0] for r in rows] == [5, 0, 4, 1, 9, 2, 1, 3]
    assert_bit_exact(np.array(rows, np.int32), golden["mnist8_top3"], "printed top-3")
    prob = np.fromfile(os.path.join(tmp_path, "data4_host.bin"), np.float32).reshape(8, 10)
    assert strict_rel_err(prob, golden["mnist8_prob"]) < TOL


# ------------------------------------------------------ batch loop (dataloader)
def write_record_file(tmp_path, samples, seed=5):
    """`samples` records of <1-byte label><784 fp32>; half of the images are the reference's eight
    MNIST digits (so some predictions are right), the rest noise."""
    d = os.path.join(ROOT, "tests", "golden", "mnist8")
    for f in os.listdir(d):
        shutil.copy(os.path.join(d, f), tmp_path)
    img8 = np.fromfile(os.path.join(d, "mnist_images_8.bin"), np.float32).reshape(8, 784)
    lab8 = [5, 0, 4, 1, 9, 2, 1, 3]
    rng = np.random.default_rng(seed)
    images, labels = [], []
    for i in range(samples):
        if i % 2 == 0:
            j = int(rng.integers(0, 8))
            images.append(img8[j])
            labels.append(lab8[j])
        else:
            images.append(rng.uniform(0, 1, 784).astype(np.float32))
            labels.append(int(rng.integers(0, 10)))
    with open(os.path.join(tmp_path, "mnist_labels_images.bin"), "wb") as f:
        for lab, img in zip(labels, images):
            f.write(bytes([lab]))
            f.write(np.asarray(img, np.float32).tobytes())
    return np.stack(images), np.array(labels)


def expected_counters(oracle, images, labels):
    d = os.path.join(ROOT, "tests", "golden", "mnist8")
    ld = lambda n, shape: np.fromfile(os.path.join(d, n), np.float32).reshape(shape)
    w0, b0, w1, b1 = ld("mlp_weight0.bin", (784, 512)), ld("mlp_bias0.bin", (512,)), ld("mlp_weight1.bin", (512, 10)), ld("mlp_bias1.bin", (10,))
    n = (len(images) // 8) * 8
    prob = oracle.matrixSoftmax(oracle.fcbias(oracle.matrixTanh(oracle.fcbias(images[:n], w0, b0)), w1, b1))
    right = int((oracle.argMax(prob, 1).ravel() == labels[:n]).sum())
    return right, n


def parse_counters(stdout):
    lines = stdout.strip().splitlines()
    assert lines[-2].startswith("iterations"), stdout
    return tuple(int(v) for v in lines[-1].split())


@pytest.mark.parametrize("compat", [False, True])
def test_batch_loop_cpu_program(gen, oracle, tmp_path, compat):
    """compat=False: the reference's DataLoader.cpp and kernels (where the reference tree exists);
    compat=True: this repository's DataLoader (include/swc_host_utils.h) and the oracle."""
    images, labels = write_record_file(tmp_path, 44)   # 5 mini-batches of 8, 4 records left over
    code = generate(gen, "mnist_loader", "cpu", tmp_path, 44)
    assert "while(loader.next(selected, data0))" in code and "DataLoader loader(" in code
    exe = build_cpu(tmp_path, with_loader=True, force_compat=compat)
    out = subprocess.run([exe], cwd=tmp_path, check=True, capture_output=True, text=True).stdout
    assert parse_counters(out) == expected_counters(oracle, images, labels)
    assert parse_counters(out)[1] == 40 and parse_counters(out)[0] >= 15


def test_batch_loop_hip_program_structure(gen, tmp_path):
    code = generate(gen, "mnist_loader", "hip", tmp_path, 44)
    body = code[code.index("while(loader.next(selected, data0))"):]
    loop, tail = body[:body.index("} //while")], body[body.index("} //while"):]
    # inside the loop: the data batch and its labels go up, ArgMax and Accuracy run on the device, and the
    # counters come back only where they are displayed
    assert loop.count("swc_hip_h2d(") == 2 and "swc_hip_h2d(data0_dev, data0" in loop
    assert "swc_hip_h2d(selected_dev, selected, 32)" in loop
    assert "swc_hip_accuracy_i(top1, selected_dev, accur, 8, 1)" in loop and "accuracy_i(top1_host" not in code
    shown = loop[loop.index("if (iter % "):]
    assert loop.count("swc_hip_d2h(") == 1 and shown.index("swc_hip_d2h(accur_host, accur, 8)") < shown.index("printMatrix(accur_host, 1, 2)")
    # after the loop: the counters of the last batch reach the host once more (for the output dump)
    assert tail.count("swc_hip_d2h(accur_host, accur, 8)") == 1
    # the counters start at zero on the device
    assert "swc_hip_fill_i(accur, 0, 2)" in code[:code.index("while(loader")]
    # before the loop: the four parameter uploads
    assert code[:code.index("while(loader")].count("swc_hip_h2d(") == 4
    build_hip(tmp_path)
    # with hip_graph: the device ops of an iteration are recorded once before the loop (after an eager pass) and
    # each batch is upload, one graph launch, download, host ops
    code = generate(gen, "mnist_loader", "hip", tmp_path, 44, graph=True)
    head, body = code.split("while(loader.next(selected, data0))")
    assert head.count("swc_hip_graph_begin()") == 1 and head.count("swc_hip_matrixMatrixFCBiasSoftmax_f(") == 2
    assert head.index("swc_hip_sync()", head.index("warm-up pass")) < head.index("swc_hip_graph_begin()")
    loop = body[:body.index("} //while")]
    assert loop.count("swc_hip_graph_launch(swc_graph)") == 1 and "swc_hip_matrixMatrixFCBias" not in loop
    assert loop.index("swc_hip_h2d(data0_dev") < loop.index("swc_hip_h2d(selected_dev") < loop.index("swc_hip_graph_launch")
    assert loop.index("swc_hip_graph_launch") < loop.index("swc_hip_d2h(accur_host") and "swc_hip_accuracy_i" not in loop
    # the warm-up pass has counted a batch of whatever the arena held: the counters are cleared again before recording
    warm = head[head.index("warm-up pass"):head.index("swc_hip_graph_begin()")]
    assert warm.index("swc_hip_accuracy_i(") < warm.index("swc_hip_fill_i(accur, 0, 2)")
    assert "swc_hip_graph_destroy(swc_graph)" in body
    build_hip(tmp_path)


def test_prefetching_batch_loop_structure(gen, tmp_path):
    """Config::hip_prefetch: the loader reads and the copy stream uploads batch i+1 while the graph of batch i runs."""
    code = generate(gen, "mnist_loader", "hip", tmp_path, 44, prefetch=True)
    head, body = code.split("while (swc_more) {")
    assert "while(loader.next(" not in code
    assert head.count("loader.next(selected, data0)") == 1 and head.count("swc_hip_copy_h2d_async(") == 2
    assert "void *data0_dev_stage = swc_hip_malloc(25088);" in head and "void *selected_dev_stage = swc_hip_malloc(32);" in head
    loop = body[:body.index("} //while")]
    order = ["swc_hip_copy_sync()", "swc_hip_ops_wait_copies()", "swc_hip_d2d(data0_dev, data0_dev_stage, 25088)",
             "swc_hip_d2d(selected_dev, selected_dev_stage, 32)", "swc_hip_copy_wait_ops()", "swc_hip_graph_launch(swc_graph)",
             "swc_more = loader.next(selected, data0)", "swc_hip_copy_h2d_async(data0_dev_stage, data0, 25088)",
             "swc_hip_copy_h2d_async(selected_dev_stage, selected, 32)", "iter++"]
    positions = [loop.index(s) for s in order]
    assert positions == sorted(positions)
    assert "swc_hip_h2d(" not in loop      # no synchronous upload is left in the loop
    assert body.count("swc_hip_free(data0_dev_stage)") == 1
    build_hip(tmp_path)


def test_prefetching_is_dropped_when_the_host_reads_the_loaders_buffers(gen, tmp_path):
    """With prefetching the loader refills its host buffers right after the graph launch; a displayed tensor (or a host
    op) that reads one of them would show the next batch, so such a program keeps the plain loop."""
    code = generate(gen, "mnist_loader+labels", "hip", tmp_path, 44, prefetch=True)
    assert "no prefetching" in code and "swc_hip_copy_h2d_async" not in code and "_stage" not in code
    assert "while(loader.next(" in code and "swc_hip_graph_launch(swc_graph)" in code
    body = code[code.index("while(loader.next("):]
    assert "printMatrix(selected" in body.replace("cpu0_", "") or "printMatrix(" in body
    build_hip(tmp_path)
    # the same model without the label on display prefetches
    assert "swc_hip_copy_h2d_async" in generate(gen, "mnist_loader", "hip", tmp_path, 44, prefetch=True)


@pytest.mark.gpu
@pytest.mark.parametrize("graph,prefetch", [(False, False), (True, False), (True, True)])
def test_batch_loop_hip_program(gen, oracle, tmp_path, graph, prefetch):
    print("case batch loop, graph =", graph, "prefetch =", prefetch, flush=True)
    images, labels = write_record_file(tmp_path, 44)
    generate(gen, "mnist_loader", "hip", tmp_path, 44, graph=graph and not prefetch, prefetch=prefetch)
    exe = build_hip(tmp_path)
    out = subprocess.run([exe], cwd=tmp_path, check=True, capture_output=True, text=True, timeout=120).stdout
    assert parse_counters(out) == expected_counters(oracle, images, labels)


# ------------------------------------------- layout ops at an NCHW import boundary
def nchw_block_expected(oracle, x, w, cb):
    xh, wh = oracle.transpose(x, (0, 2, 3, 1)), oracle.transpose(w, (0, 2, 3, 1))
    y = oracle.relu(oracle.conv2d(xh, wh, cb, (3, 3), (1, 1), (1, 1, 1, 1)))
    return oracle.transpose(oracle.avgpool(y, (2, 2), (2, 2)), (0, 3, 1, 2))


def nchw_inputs(tmp_path):
    rng = np.random.default_rng(8)
    x = rng.standard_normal((2, 8, 12, 12)).astype(np.float32)
    w = (rng.standard_normal((16, 8, 3, 3)) / 8).astype(np.float32)
    cb = (rng.standard_normal(16) * 0.1).astype(np.float32)
    for name, a in (("x", x), ("w", w), ("cb", cb)):
        a.tofile(os.path.join(tmp_path, name + ".bin"))
    return x, w, cb


def test_nchw_block_cpu_program(gen, oracle, tmp_path):
    x, w, cb = nchw_inputs(tmp_path)
    code = generate(gen, "nchw", "cpu", tmp_path, 2)
    assert code.count("transpose4d_f(") == 3 and "avgpool_f(" in code
    subprocess.check_call([build_cpu(tmp_path)], cwd=tmp_path, stdout=subprocess.DEVNULL)
    want = nchw_block_expected(oracle, x, w, cb)
    got = np.fromfile(os.path.join(tmp_path, "y_nchw.bin"), np.float32).reshape(want.shape)
    assert want.shape == (2, 16, 6, 6)
    assert_bit_exact(got, want, "nchw block")


@pytest.mark.gpu
def test_nchw_block_hip_program(gen, oracle, tmp_path):
    x, w, cb = nchw_inputs(tmp_path)
    code = generate(gen, "nchw", "hip", tmp_path, 2)
    assert code.count("swc_hip_transpose4d_f(") == 3 and "swc_hip_avgpool_f(" in code and "swc_hip_conv2dFused_f(" in code
    subprocess.run([build_hip(tmp_path)], cwd=tmp_path, check=True, timeout=120, stdout=subprocess.DEVNULL)
    want = nchw_block_expected(oracle, x, w, cb)
    got = np.fromfile(os.path.join(tmp_path, "y_nchw_host.bin"), np.float32).reshape(want.shape)
    assert rel_err(got, want) < TOL


@pytest.mark.gpu
@pytest.mark.parametrize("graph", [False, True])
def test_timed_hip_program(gen, oracle, tmp_path, graph):
    """Config::time_iters (and Config::hip_graph): the program still produces the right output and
    prints a per-iteration time."""
    t = graphs.make_inputs(3, 8)
    write_inputs(3, t, tmp_path)
    code = generate(gen, "cfg3", "hip", tmp_path, 8, iters=20, graph=graph)
    assert ("swc_hip_graph_launch(swc_graph)" in code) == graph
    exe = build_hip(tmp_path)
    out = subprocess.run([exe], cwd=tmp_path, check=True, capture_output=True, text=True, timeout=120).stdout
    ms = float(re.search(r"swc_time_ms_per_iter ([0-9.eE+-]+)", out).group(1))
    assert 0 < ms < 50
    want = oracle_run(oracle, "cfg3", 3, t)
    got = np.fromfile(os.path.join(tmp_path, "softmax_out_host.bin"), np.float32).reshape(want.shape)
    assert strict_rel_err(got, want) < TOL


def test_graph_ir_and_passes_cpp_unit_tests(gen):
    """swcompiler_amd/swc/test/testPasses.cpp: topology, shape inference, clone, FC lowering, renaming,
    fusion, device placement, transpose cancelling and dead-node elimination, checked in C++."""
    exe = os.path.join(SWC, "test", "bin", "testPasses")
    out = subprocess.run([exe], capture_output=True, text=True)
    assert out.returncode == 0, out.stderr
    assert "all pass checks ok" in out.stdout


# ------------------------------------------------ placement written by hand
def manual_inputs(tmp_path):
    rng = np.random.default_rng(21)
    x = rng.standard_normal((16, 64)).astype(np.float32)
    w = (rng.standard_normal((64, 24)) / 8).astype(np.float32)
    b = (rng.standard_normal(24) * 0.1).astype(np.float32)
    for name, a in (("x", x), ("w", w), ("bias", b)):
        a.tofile(os.path.join(tmp_path, name + ".bin"))
    return x, w, b


def test_manual_placement_structure(gen, tmp_path):
    manual_inputs(tmp_path)
    code = generate(gen, "manual", "hip", tmp_path, 16)
    # the hand-placed graph went through the CPU-target passes: FCBias lowered, on the device
    assert "swc_hip_matrixMatrixMul_f(16, 24, 64, x_d, 64, w_d, 24, fc_mm_out, 24)" in code
    assert "swc_hip_batchedadd_f(y_d, fc_mm_out, bias_d, 16, 24)" in code and "swc_hip_matrixTanh_f(" in code
    head, body = code.split("// call op routine functions")
    assert head.count("swc_hip_h2d(") == 2 and body.count("swc_hip_h2d(x_d, x,") == 1 and body.count("swc_hip_d2h(z, z_d,") == 1
    build_hip(tmp_path)


@pytest.mark.gpu
def test_manual_placement_runs(gen, oracle, tmp_path):
    x, w, b = manual_inputs(tmp_path)
    generate(gen, "manual", "hip", tmp_path, 16)
    subprocess.run([build_hip(tmp_path)], cwd=tmp_path, check=True, timeout=120, stdout=subprocess.DEVNULL)
    want = oracle.matrixTanh(oracle.fcbias(x, w, b))
    got = np.fromfile(os.path.join(tmp_path, "z.bin"), np.float32).reshape(want.shape)
    assert rel_err(got, want) < TOL
