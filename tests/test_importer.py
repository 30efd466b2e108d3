"""Caffe2 import (reference: src/importer/Caffe2Importer.cpp, test/importer/testResnetImport.cpp).

The reference's own tests import ResNet50 / VGG19 / LeNet files that it downloads; none is in the reference
tree.  Here a small residual network is written in the Caffe2 file format by the encoder below (binary wire
format as protobuf serialises proto2 messages, and the text format), imported through the SWC API, compiled
for the CPU and the HIP target, and checked against the same network computed with the oracle's kernels.
"""
import os
import struct
import subprocess

import numpy as np
import pytest

from tests.test_codegen import GEN, SWC, TOL, build_cpu, build_hip, generate
from swcompiler_amd.caffe2_files import enc_net, make_resnet50, text_net
from tests.util import assert_bit_exact, rel_err


@pytest.fixture(scope="module")
def gen():
    if not os.path.exists(GEN):
        subprocess.check_call(["make", "-C", SWC, "-j8"], stdout=subprocess.DEVNULL)
    return GEN


# ------------------------------------------------ the network
def make_weights():
    rng = np.random.default_rng(2019)
    f32 = lambda a: np.asarray(a, np.float32)
    w = {
        "gpu_0/conv1_w": f32(rng.standard_normal((8, 3, 3, 3)) / 5),      # OIHW, as Caffe2 stores them
        "gpu_0/conv1_b": f32(rng.standard_normal(8) / 10),
        "gpu_0/res_w": f32(rng.standard_normal((8, 8, 3, 3)) / 8),
        "gpu_0/pred_w": f32(rng.standard_normal((10, 72)) / 8),            # [out, in], in = (c, h, w) flattened
        "gpu_0/pred_b": f32(rng.standard_normal(10) / 10),
    }
    for bn in ("gpu_0/conv1_bn", "gpu_0/res_bn"):
        w[bn + "_s"] = f32(rng.uniform(0.5, 1.5, 8))
        w[bn + "_b"] = f32(rng.standard_normal(8) / 10)
        w[bn + "_rm"] = f32(rng.standard_normal(8) / 10)
        w[bn + "_riv"] = f32(rng.uniform(0.5, 2.0, 8))
    return w


def make_nets(weights):
    init = [dict(type="GivenTensorFill", input=[], output=[k], arg=dict(shape=list(v.shape), values=v))
            for k, v in weights.items()]
    init.append(dict(type="ConstantFill", input=[], output=["gpu_0/data"], arg=dict(shape=[1], value=0.0)))   # the caller's wins
    g = "gpu_0/"
    bn = lambda x: [g + x + s for s in ("_s", "_b", "_rm", "_riv")]
    predict = [
        dict(type="Conv", input=[g + "data", g + "conv1_w", g + "conv1_b"], output=[g + "conv1"],
             arg=dict(kernel=3, pad=1, stride=1, order="NCHW", exhaustive_search=0)),
        dict(type="SpatialBN", input=[g + "conv1"] + bn("conv1_bn"), output=[g + "conv1_bn"],
             arg=dict(epsilon=float(np.float32(1e-5)), is_test=1, order="NCHW")),
        dict(type="Relu", input=[g + "conv1_bn"], output=[g + "conv1_bn"]),                      # in place
        dict(type="MaxPool", input=[g + "conv1_bn"], output=[g + "pool1"], arg=dict(kernel=2, stride=2, order="NCHW")),
        dict(type="Conv", input=[g + "pool1", g + "res_w"], output=[g + "res"],                    # no bias blob
             arg=dict(kernels=[3, 3], pads=[1, 1, 1, 1], strides=[1, 1])),
        dict(type="SpatialBN", input=[g + "res"] + bn("res_bn"), output=[g + "res_bn"], arg=dict(is_test=1)),
        dict(type="Sum", input=[g + "res_bn", g + "pool1"], output=[g + "res_bn"]),                # in place
        dict(type="Relu", input=[g + "res_bn"], output=[g + "res_bn"]),
        dict(type="AveragePool", input=[g + "res_bn"], output=[g + "pool2"], arg=dict(kernel_h=2, kernel_w=2, stride_h=2, stride_w=2)),
        dict(type="Dropout", input=[g + "pool2"], output=[g + "drop"], arg=dict(ratio=0.5, is_test=1)),
        dict(type="FC", input=[g + "drop", g + "pred_w", g + "pred_b"], output=[g + "pred"]),
        dict(type="Softmax", input=[g + "pred"], output=[g + "softmax"]),
    ]
    return predict, init


def expected(oracle, data, w):
    g = "gpu_0/"
    ohwi = lambda f: oracle.transpose(f, (0, 2, 3, 1))
    bn = lambda x, p: oracle.batchnormalization(x, w[g + p + "_rm"], w[g + p + "_riv"], w[g + p + "_s"], w[g + p + "_b"],
                                                float(np.float32(1e-5)))
    y = oracle.conv2d(data, ohwi(w[g + "conv1_w"]), w[g + "conv1_b"], (3, 3), (1, 1), (1, 1, 1, 1))
    pool1 = oracle.maxpool(oracle.relu(bn(y, "conv1_bn")), (2, 2), (2, 2))
    r = oracle.conv2d(pool1, ohwi(w[g + "res_w"]), np.zeros(8, np.float32), (3, 3), (1, 1), (1, 1, 1, 1))
    r = oracle.relu(oracle.vecAdd(bn(r, "res_bn").ravel(), pool1.ravel()).reshape(pool1.shape))
    pool2 = oracle.avgpool(r, (2, 2), (2, 2))
    flat = oracle.transpose(pool2, (0, 3, 1, 2)).reshape(data.shape[0], -1)      # (c, h, w) order, as trained
    pred = oracle.fcbias(flat, oracle.transpose(w[g + "pred_w"], (1, 0)), w[g + "pred_b"])
    prob = oracle.matrixSoftmax(pred)
    return prob, oracle.argMax(prob, 3)


def run_net(oracle, predict, w, data):
    """The operators of a predict_net executed with the oracle's kernels: activations NHWC, weights as stored
    (Conv OIHW, FC [out, in] over an NCHW-flattened input) — what the imported graph must compute."""
    blobs = dict(w)
    blobs["gpu_0/data"] = data
    pair = lambda a, one, h, wd, lst, default: ((a[one],) * 2 if one in a else (a[h], a[wd]) if h in a else
                                                tuple(a[lst]) if lst in a else default)
    for op in predict:
        a, x = op.get("arg", {}), [blobs[n] for n in op["input"]]
        pads = (a["pad"],) * 4 if "pad" in a else tuple(a.get("pads", (0, 0, 0, 0)))
        if op["type"] == "Conv":
            f = oracle.transpose(x[1], (0, 2, 3, 1))
            bias = x[2] if len(x) > 2 else np.zeros(f.shape[0], np.float32)
            y = oracle.conv2d(x[0], f, bias, pair(a, "kernel", "kernel_h", "kernel_w", "kernels", f.shape[1:3]),
                              pair(a, "stride", "stride_h", "stride_w", "strides", (1, 1)), pads)
        elif op["type"] == "SpatialBN":
            y = oracle.batchnormalization(x[0], x[3], x[4], x[1], x[2], a.get("epsilon", float(np.float32(1e-5))))
        elif op["type"] == "Relu":
            y = oracle.relu(x[0].ravel()).reshape(x[0].shape)
        elif op["type"] == "Sum":
            y = oracle.vecAdd(x[0].ravel(), x[1].ravel()).reshape(x[0].shape)
        elif op["type"] in ("MaxPool", "AveragePool"):
            k = pair(a, "kernel", "kernel_h", "kernel_w", "kernels", None)
            if a.get("global_pooling"):
                k = x[0].shape[1:3]
            fn = oracle.maxpool if op["type"] == "MaxPool" else oracle.avgpool
            y = fn(x[0], k, pair(a, "stride", "stride_h", "stride_w", "strides", (1, 1)), pads)
        elif op["type"] == "Dropout":
            y = x[0]
        elif op["type"] == "FC":
            flat = oracle.transpose(x[0], (0, 3, 1, 2)) if x[0].ndim == 4 else x[0]
            y = oracle.fcbias(flat.reshape(flat.shape[0], -1), oracle.transpose(x[1], (1, 0)), x[2])
        elif op["type"] == "Softmax":
            y = oracle.matrixSoftmax(x[0])
        else:
            raise ValueError(op["type"])
        blobs[op["output"][0]] = y
    return blobs


def write_resnet50(tmp_path, batch, **kw):
    predict, init, w = make_resnet50(**kw)
    open(os.path.join(tmp_path, "predict_net.pb"), "wb").write(enc_net("resnet50", predict, packed=True))
    open(os.path.join(tmp_path, "init_net.pb"), "wb").write(enc_net("resnet50_init", init, packed=True))
    image = kw.get("image", 224)
    data = np.random.default_rng(11).standard_normal((batch, image, image, 3)).astype(np.float32)
    data.tofile(os.path.join(tmp_path, "data.bin"))
    return predict, w, data


def write_model(tmp_path, binary, packed=False):
    w = make_weights()
    predict, init = make_nets(w)
    if binary:
        open(os.path.join(tmp_path, "predict_net.pb"), "wb").write(enc_net("mini_resnet", predict, packed))
        open(os.path.join(tmp_path, "init_net.pb"), "wb").write(enc_net("mini_resnet_init", init, packed))
    else:
        open(os.path.join(tmp_path, "predict_net.pbtxt"), "w").write(text_net("mini_resnet", predict))
        open(os.path.join(tmp_path, "init_net.pbtxt"), "w").write(text_net("mini_resnet_init", init))
    data = np.random.default_rng(7).standard_normal((2, 12, 12, 3)).astype(np.float32)
    data.tofile(os.path.join(tmp_path, "data.bin"))
    return w, data


def read_outputs(tmp_path, suffix, batch=2, classes=10):
    prob = np.fromfile(os.path.join(tmp_path, f"gpu_0_softmax{suffix}.bin"), np.float32).reshape(batch, classes)
    top3 = np.fromfile(os.path.join(tmp_path, f"top3{suffix}.bin"), np.int32).reshape(batch, 3)
    return prob, top3


# ------------------------------------------------ tests
@pytest.mark.parametrize("binary,packed", [(True, False), (True, True), (False, False)])
def test_import_cpu_program(gen, oracle, tmp_path, binary, packed):
    w, data = write_model(tmp_path, binary, packed)
    code = generate(gen, "caffe2" if binary else "caffe2txt", "cpu", tmp_path, 2)
    # the graph the reference's importer builds: a transpose per Conv / FC weight and one in front of the FC
    assert code.count("transpose4d_f(") == 3 and code.count("transpose2d_f(") == 1
    assert code.count("conv2d_f(") == 2 and code.count("batchnormalization_f(") == 2 and code.count("relu_f(") == 2
    assert "vecAdd_f(" in code and "maxpool_f(" in code and "avgpool_f(" in code and "matrixSoftmax_f(" in code
    # every weight blob became a raw fp32 file the program loads
    for name, v in w.items():
        path = os.path.join(tmp_path, "weights", name.replace("/", "_") + ".bin")
        assert_bit_exact(np.fromfile(path, np.float32).reshape(v.shape), v, name)
        assert f'"weights/{name.replace("/", "_")}.bin"' in code
    out = subprocess.run([build_cpu(tmp_path)], cwd=tmp_path, check=True, capture_output=True, text=True).stdout
    prob, top3 = read_outputs(tmp_path, "")
    want_prob, want_top3 = expected(oracle, data, w)
    assert_bit_exact(run_net(oracle, make_nets(w)[0], w, data)["gpu_0/softmax"], want_prob, "the two statements of the network")
    assert_bit_exact(prob, want_prob, "probabilities")
    assert_bit_exact(top3, want_top3, "top-3")
    assert [int(v) for v in out.split()[-6:]] == want_top3.ravel().tolist()      # the Debug print


def test_text_and_binary_files_give_the_same_program(gen, tmp_path):
    a, b = os.path.join(tmp_path, "a"), os.path.join(tmp_path, "b")
    os.mkdir(a), os.mkdir(b)
    write_model(a, True)
    write_model(b, False)
    assert generate(gen, "caffe2", "cpu", a, 2) == generate(gen, "caffe2txt", "cpu", b, 2)
    assert generate(gen, "caffe2", "hip", a, 2) == generate(gen, "caffe2txt", "hip", b, 2)


def test_import_hip_program_structure(gen, tmp_path):
    write_model(tmp_path, True)
    code = generate(gen, "caffe2", "hip", tmp_path, 2)
    # conv+BN+ReLU with the pooling behind it is one call (a first layer: the direct kernel pools in its epilogue), and
    # so is conv+BN+Sum+ReLU (the other summand, pool1, is the call's `residual`); the weight transposes run once,
    # before the op sequence
    assert code.count("swc_hip_conv2dFusedMaxpool_f(") == 1 and code.count("swc_hip_conv2dFused_f(") == 0
    assert "swc_hip_vecAdd" not in code and "swc_hip_maxpool_f(" not in code
    assert code.count("swc_hip_conv2dFusedAdd_f(") == 1 and "1e-05, gpu_0_pool1, 1));" in code
    head, body = code.split("// call op routine functions")
    assert head.count("swc_hip_transpose4d_f(") == 2 and head.count("swc_hip_transpose2d_f(") == 1
    assert body.count("swc_hip_transpose4d_f(") == 1 and "swc_hip_transpose2d_f(" not in body
    assert "swc_hip_matrixMatrixFCBiasSoftmax_f(2, 10, 72" in body
    build_hip(tmp_path)


@pytest.mark.parametrize("damage", ["unsupported op", "truncated", "missing blob", "value count"])
def test_import_errors(gen, tmp_path, damage):
    w = make_weights()
    predict, init = make_nets(w)
    if damage == "unsupported op":
        predict.insert(3, dict(type="LRN", input=["gpu_0/conv1_bn"], output=["gpu_0/conv1_bn"]))
        message = "unsupported Caffe2 operator LRN"
    elif damage == "missing blob":
        init = [o for o in init if o["output"] != ["gpu_0/res_w"]]
        message = "blob gpu_0/res_w"
    elif damage == "value count":
        init[0]["arg"]["shape"] = [8, 3, 3, 4]
        message = "216 values for a shape of 288 elements"
    else:
        message = "not a serialized NetDef"
    pred_bytes = enc_net("mini", predict)
    if damage == "truncated":
        pred_bytes = pred_bytes[:len(pred_bytes) // 2 + 1]
    open(os.path.join(tmp_path, "predict_net.pb"), "wb").write(pred_bytes)
    open(os.path.join(tmp_path, "init_net.pb"), "wb").write(enc_net("mini_init", init))
    r = subprocess.run([gen, "caffe2", "cpu", "2"], cwd=tmp_path, capture_output=True, text=True)
    assert r.returncode != 0 and message in r.stderr + r.stdout


@pytest.mark.gpu
@pytest.mark.parametrize("graph", [False, True])
def test_import_hip_program(gen, oracle, tmp_path, graph):
    print("case caffe2 import, graph =", graph, flush=True)
    w, data = write_model(tmp_path, True)
    generate(gen, "caffe2", "hip", tmp_path, 2, iters=3 if graph else 0, graph=graph)
    subprocess.run([build_hip(tmp_path)], cwd=tmp_path, check=True, timeout=120, stdout=subprocess.DEVNULL)
    prob, top3 = read_outputs(tmp_path, "_host")
    want_prob, want_top3 = expected(oracle, data, w)
    assert rel_err(prob, want_prob) < TOL
    assert_bit_exact(top3, want_top3, "top-3")


# A ResNet-50 of reduced width and resolution (all 16 bottleneck blocks, every layer type and stride of the real
# one): 1/4 of the channels, 64 x 64 images.
SMALL_RESNET = dict(width=16, classes=100, image=64)


def test_resnet50_import_cpu_program(gen, oracle, tmp_path):
    predict, w, data = write_resnet50(tmp_path, 1, **SMALL_RESNET)
    code = generate(gen, "caffe2@64", "cpu", tmp_path, 1)
    assert code.count("conv2d_f(") == 53 and code.count("batchnormalization_f(") == 53 and code.count("vecAdd_f(") == 16
    subprocess.run([build_cpu(tmp_path)], cwd=tmp_path, check=True, stdout=subprocess.DEVNULL)
    prob, top3 = read_outputs(tmp_path, "", 1, 100)
    want = run_net(oracle, predict, w, data)["gpu_0/softmax"]
    assert_bit_exact(prob, want, "probabilities")
    assert_bit_exact(top3, oracle.argMax(want, 3), "top-3")


@pytest.mark.gpu
def test_resnet50_import_hip_program(gen, oracle, tmp_path):
    print("case resnet50 import", flush=True)
    predict, w, data = write_resnet50(tmp_path, 4, **SMALL_RESNET)
    code = generate(gen, "caffe2@64", "hip", tmp_path, 4)
    head, body = code.split("// call op routine functions")
    # the 53 filter transposes and the FC weight's run once; in the op sequence only pool5 is reordered for the FC
    assert head.count("swc_hip_transpose4d_f(") == 53 and head.count("swc_hip_transpose2d_f(") == 1
    assert body.count("swc_hip_transpose4d_f(") == 1 and "swc_hip_conv2dFused_f(" not in head
    # the last convolution of each of the 16 blocks takes the block's sum and ReLU along
    assert body.count("swc_hip_conv2dFused_f(") == 37 and body.count("swc_hip_conv2dFusedAdd_f(") == 16
    assert "swc_hip_vecAdd" not in body
    subprocess.run([build_hip(tmp_path)], cwd=tmp_path, check=True, timeout=120, stdout=subprocess.DEVNULL)
    prob, top3 = read_outputs(tmp_path, "_host", 4, 100)
    want = run_net(oracle, predict, w, data)["gpu_0/softmax"]
    assert rel_err(prob, want) < TOL
    assert (top3[:, 0] == oracle.argMax(want, 1)[:, 0]).all()


@pytest.mark.gpu
def test_resnet50_full_size_hip_program(gen, oracle, tmp_path):
    """All of ResNet-50 at its real size (25.6 M parameters, 224 x 224 images, 1000 classes), one image: the 7x7/2
    first layer on padded channels, 1x1 and strided 1x1 convolutions, 3x3/2 pooling with padding, 7x7 average
    pooling and a 2048 -> 1000 FC, against the oracle's run of the same network."""
    print("case resnet50 full size", flush=True)
    predict, w, data = write_resnet50(tmp_path, 1)
    generate(gen, "caffe2@224", "hip", tmp_path, 1)
    subprocess.run([build_hip(tmp_path)], cwd=tmp_path, check=True, timeout=120, stdout=subprocess.DEVNULL)
    prob, top3 = read_outputs(tmp_path, "_host", 1, 1000)
    want = run_net(oracle, predict, w, data)["gpu_0/softmax"]
    assert rel_err(prob, want) < TOL
    assert top3[0, 0] == int(np.argmax(want))


# ------------------------------------------------ the other two networks the reference's tests import
def conv_relu(ops, w, rng, name, src, cin, cout, k, pad, relu=True):
    g = "gpu_0/"
    w[g + name + "_w"] = (rng.standard_normal((cout, cin, k, k)) / np.sqrt(cin * k * k)).astype(np.float32)
    w[g + name + "_b"] = (rng.standard_normal(cout) * 0.1).astype(np.float32)
    ops.append(dict(type="Conv", input=[g + src, g + name + "_w", g + name + "_b"], output=[g + name],
                    arg=dict(kernel=k, pad=pad, stride=1)))
    if relu:
        ops.append(dict(type="Relu", input=[g + name], output=[g + name]))
    return name


def fc(ops, w, rng, name, src, cin, cout, relu=False, dropout=False):
    g = "gpu_0/"
    w[g + name + "_w"] = (rng.standard_normal((cout, cin)) / np.sqrt(cin)).astype(np.float32)
    w[g + name + "_b"] = (rng.standard_normal(cout) * 0.1).astype(np.float32)
    ops.append(dict(type="FC", input=[g + src, g + name + "_w", g + name + "_b"], output=[g + name]))
    if relu:
        ops.append(dict(type="Relu", input=[g + name], output=[g + name]))
    if dropout:
        ops.append(dict(type="Dropout", input=[g + name], output=[g + name + "_drop"], arg=dict(ratio=0.5, is_test=1)))
        return name + "_drop"
    return name


def make_lenet():
    """Caffe2's lenet_mnist (test/importer/testLeNetImport.cpp): conv 5x5 -> pool -> conv 5x5 -> pool -> FC 500 ->
    ReLU -> FC 10 -> softmax on 28 x 28 x 1 images."""
    rng, w, ops, g = np.random.default_rng(1998), {}, [], "gpu_0/"
    x = conv_relu(ops, w, rng, "conv1", "data", 1, 20, 5, 0, relu=False)
    ops.append(dict(type="MaxPool", input=[g + x], output=[g + "pool1"], arg=dict(kernel=2, stride=2)))
    x = conv_relu(ops, w, rng, "conv2", "pool1", 20, 50, 5, 0, relu=False)
    ops.append(dict(type="MaxPool", input=[g + x], output=[g + "pool2"], arg=dict(kernel=2, stride=2)))
    x = fc(ops, w, rng, "fc3", "pool2", 800, 500, relu=True)
    x = fc(ops, w, rng, "pred", x, 500, 10)
    ops.append(dict(type="Softmax", input=[g + x], output=[g + "softmax"]))
    return ops, w, (28, 1, 10)


def make_vgg(width=8, image=32, classes=20):
    """VGG-19's layer sequence (test/importer/testVGG19Import.cpp) at 1/8 of its width on 32 x 32 images: 2-2-4-4-4
    convolutions 3x3 + ReLU with 2x2 pooling between the groups, FC + ReLU + Dropout twice, FC, softmax."""
    rng, w, ops, g = np.random.default_rng(2014), {}, [], "gpu_0/"
    x, cin, hw = "data", 3, image
    for group, (n, mult) in enumerate(((2, 1), (2, 2), (4, 4), (4, 8), (4, 8))):
        for i in range(n):
            x = conv_relu(ops, w, rng, f"conv{group + 1}_{i + 1}", x, cin, width * mult, 3, 1)
            cin = width * mult
        ops.append(dict(type="MaxPool", input=[g + x], output=[g + f"pool{group + 1}"], arg=dict(kernel=2, stride=2)))
        x, hw = f"pool{group + 1}", hw // 2
    x = fc(ops, w, rng, "fc6", x, cin * hw * hw, 64 * width, relu=True, dropout=True)
    x = fc(ops, w, rng, "fc7", x, 64 * width, 64 * width, relu=True, dropout=True)
    x = fc(ops, w, rng, "fc8", x, 64 * width, classes)
    ops.append(dict(type="Softmax", input=[g + x], output=[g + "softmax"]))
    return ops, w, (image, 3, classes)


def write_net(tmp_path, batch, predict, w, image, channels):
    init = [dict(type="GivenTensorFill", input=[], output=[k], arg=dict(shape=list(v.shape), values=v)) for k, v in w.items()]
    open(os.path.join(tmp_path, "predict_net.pb"), "wb").write(enc_net("net", predict, packed=True))
    open(os.path.join(tmp_path, "init_net.pb"), "wb").write(enc_net("net_init", init, packed=True))
    data = np.random.default_rng(13).uniform(0, 1, (batch, image, image, channels)).astype(np.float32)
    data.tofile(os.path.join(tmp_path, "data.bin"))
    return data


@pytest.mark.parametrize("make", [make_lenet, make_vgg])
def test_lenet_and_vgg_import_cpu_program(gen, oracle, tmp_path, make):
    predict, w, (image, channels, classes) = make()
    data = write_net(tmp_path, 2, predict, w, image, channels)
    generate(gen, f"caffe2@{image}x{channels}", "cpu", tmp_path, 2)
    subprocess.run([build_cpu(tmp_path)], cwd=tmp_path, check=True, stdout=subprocess.DEVNULL)
    prob, top3 = read_outputs(tmp_path, "", 2, classes)
    want = run_net(oracle, predict, w, data)["gpu_0/softmax"]
    assert_bit_exact(prob, want, "probabilities")
    assert_bit_exact(top3, oracle.argMax(want, 3), "top-3")


@pytest.mark.gpu
@pytest.mark.parametrize("make", [make_lenet, make_vgg])
def test_lenet_and_vgg_import_hip_program(gen, oracle, tmp_path, make):
    print("case import", make.__name__, flush=True)
    predict, w, (image, channels, classes) = make()
    data = write_net(tmp_path, 8, predict, w, image, channels)
    code = generate(gen, f"caffe2@{image}x{channels}", "hip", tmp_path, 8)
    assert "swc_hip_relu_f(" not in code.split("// call op routine functions")[1] or make is make_lenet   # VGG: every ReLU fused
    subprocess.run([build_hip(tmp_path)], cwd=tmp_path, check=True, timeout=120, stdout=subprocess.DEVNULL)
    prob, top3 = read_outputs(tmp_path, "_host", 8, classes)
    want = run_net(oracle, predict, w, data)["gpu_0/softmax"]
    assert rel_err(prob, want) < TOL
    assert (top3[:, 0] == oracle.argMax(want, 1)[:, 0]).all()


# ------------------------------------------------ the same files through the protobuf library
# The fixtures above are written by this file's own encoder and read by the importer's own decoder: a shared
# misreading of the reference's src/importer/caffe2.proto would pass.  Here the messages are built with the
# protobuf library of the Python environment from descriptors that carry the field numbers and types of that
# file (Argument: caffe2.proto:152-166, DeviceOption: 192-207, OperatorDef: 210-268, NetDef: 270-309), serialised
# by the library — unpacked as proto2 declares the repeated scalars, and packed as newer writers emit them — and
# printed by its text format; the importer must read them exactly as it reads the hand-written files.
_CLASSES = {}


def caffe2_classes(packed):
    if packed not in _CLASSES:
        _CLASSES[packed] = _caffe2_classes(packed)
    return _CLASSES[packed]


def _caffe2_classes(packed):
    from google.protobuf import descriptor_pb2, descriptor_pool, message_factory
    F = descriptor_pb2.FieldDescriptorProto
    pkg = "c2p" if packed else "c2u"
    fd = descriptor_pb2.FileDescriptorProto(name=pkg + ".proto", package=pkg, syntax="proto2")

    def msg(name, fields):
        m = fd.message_type.add(name=name)
        for fname, number, ftype, label, type_name in fields:
            f = m.field.add(name=fname, number=number, type=ftype, label=label)
            if type_name:
                f.type_name = "." + pkg + "." + type_name
            if packed and label == F.LABEL_REPEATED and ftype in (F.TYPE_FLOAT, F.TYPE_INT64):
                f.options.packed = True
    O, R = F.LABEL_OPTIONAL, F.LABEL_REPEATED
    msg("Argument", [("name", 1, F.TYPE_STRING, O, None), ("f", 2, F.TYPE_FLOAT, O, None), ("i", 3, F.TYPE_INT64, O, None),
                     ("s", 4, F.TYPE_BYTES, O, None), ("floats", 5, F.TYPE_FLOAT, R, None), ("ints", 6, F.TYPE_INT64, R, None),
                     ("strings", 7, F.TYPE_BYTES, R, None)])
    msg("DeviceOption", [("device_type", 1, F.TYPE_INT32, O, None), ("device_id", 2, F.TYPE_INT32, O, None)])
    msg("OperatorDef", [("input", 1, F.TYPE_STRING, R, None), ("output", 2, F.TYPE_STRING, R, None),
                        ("name", 3, F.TYPE_STRING, O, None), ("type", 4, F.TYPE_STRING, O, None),
                        ("arg", 5, F.TYPE_MESSAGE, R, "Argument"), ("device_option", 6, F.TYPE_MESSAGE, O, "DeviceOption"),
                        ("engine", 7, F.TYPE_STRING, O, None), ("is_gradient_op", 9, F.TYPE_BOOL, O, None)])
    msg("NetDef", [("name", 1, F.TYPE_STRING, O, None), ("op", 2, F.TYPE_MESSAGE, R, "OperatorDef"),
                   ("type", 3, F.TYPE_STRING, O, None), ("device_option", 5, F.TYPE_MESSAGE, O, "DeviceOption"),
                   ("arg", 6, F.TYPE_MESSAGE, R, "Argument"), ("external_input", 7, F.TYPE_STRING, R, None),
                   ("external_output", 8, F.TYPE_STRING, R, None)])
    pool = descriptor_pool.DescriptorPool()
    pool.Add(fd)
    return message_factory.GetMessageClass(pool.FindMessageTypeByName(pkg + ".NetDef"))


def library_net(name, ops, packed):
    net = caffe2_classes(packed)(name=name)
    for o in ops:
        op = net.op.add(name="", type=o["type"], engine="CUDNN", is_gradient_op=False)
        op.input.extend(o["input"])
        op.output.extend(o["output"])
        op.device_option.device_type = 1
        op.device_option.device_id = 0
        for k, v in o.get("arg", {}).items():
            a = op.arg.add(name=k)
            if isinstance(v, float):
                a.f = v
            elif isinstance(v, int):
                a.i = v
            elif isinstance(v, str):
                a.s = v.encode()
            elif isinstance(v, np.ndarray):
                a.floats.extend(float(x) for x in v.ravel())
            else:
                a.ints.extend(int(x) for x in v)
    net.external_input.append("gpu_0/data")
    return net


def program_and_weights(gen, model, workdir):
    code = generate(gen, model, "cpu", workdir, 2)
    wdir = os.path.join(workdir, "weights")
    return code, {f: open(os.path.join(wdir, f), "rb").read() for f in sorted(os.listdir(wdir))}


def test_files_written_by_the_protobuf_library_import_identically(gen, tmp_path):
    pytest.importorskip("google.protobuf")
    from google.protobuf import text_format
    w = make_weights()
    predict, init = make_nets(w)
    dirs = {}
    for tag_ in ("hand", "lib_unpacked", "lib_packed", "lib_text"):
        dirs[tag_] = os.path.join(tmp_path, tag_)
        os.mkdir(dirs[tag_])
        write_model(dirs[tag_], True)                       # (data.bin; its model files are replaced below)
        if tag_ != "hand":
            for f in ("predict_net.pb", "init_net.pb"):
                os.remove(os.path.join(dirs[tag_], f))
    for packed in (False, True):
        d = dirs["lib_packed" if packed else "lib_unpacked"]
        for fname, nm, ops in (("predict_net.pb", "mini_resnet", predict), ("init_net.pb", "mini_resnet_init", init)):
            msg = library_net(nm, ops, packed)
            open(os.path.join(d, fname), "wb").write(msg.SerializeToString())
            # and the other way round: the library reads this file's own encoder's bytes as the same message
            back = caffe2_classes(packed)()
            back.ParseFromString(enc_net(nm, ops, packed))
            plain = caffe2_classes(packed)()
            plain.CopyFrom(msg)
            for op in plain.op:
                op.ClearField("device_option")          # (the hand encoder's binary files carry none)
            assert back == plain, fname
    for fname, nm, ops in (("predict_net.pbtxt", "mini_resnet", predict), ("init_net.pbtxt", "mini_resnet_init", init)):
        open(os.path.join(dirs["lib_text"], fname), "w").write(text_format.MessageToString(library_net(nm, ops, False)))
    want = program_and_weights(gen, "caffe2", dirs["hand"])
    assert len(want[1]) == len(w)
    assert program_and_weights(gen, "caffe2", dirs["lib_unpacked"]) == want
    assert program_and_weights(gen, "caffe2", dirs["lib_packed"]) == want
    assert program_and_weights(gen, "caffe2txt", dirs["lib_text"]) == want
