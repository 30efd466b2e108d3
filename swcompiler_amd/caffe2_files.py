"""Writer of Caffe2 model files (predict_net / init_net), binary and text, without protobuf.

The importer (reference: src/importer/Caffe2Importer.cpp) reads what the Caffe2 model zoo ships; none of those files is
in the reference, so its tests and the benchmark of the import path write their own in the same format: the wire format
as protobuf serialises the proto2 messages of caffe2.proto, and the text format.  A network is a list of operators,
each a dict(type=, input=[...], output=[...], arg={name: float | int | str | float32 array | list of ints}).
"""
import struct

import numpy as np


def varint(n):
    n &= (1 << 64) - 1          # negative int64 values take ten bytes
    out = bytearray()
    while True:
        out.append((n & 0x7f) | (0x80 if n > 0x7f else 0))
        n >>= 7
        if not n:
            return bytes(out)


def tag(field, wire_type):
    return varint(field << 3 | wire_type)


def delimited(field, payload):
    return tag(field, 2) + varint(len(payload)) + payload


def enc_arg(name, value, packed=False):
    """Argument (caffe2.proto:152-166): name=1, f=2, i=3, s=4, floats=5, ints=6"""
    out = delimited(1, name.encode())
    if isinstance(value, float):
        out += tag(2, 5) + struct.pack("<f", value)
    elif isinstance(value, int):
        out += tag(3, 0) + varint(value)
    elif isinstance(value, str):
        out += delimited(4, value.encode())
    elif isinstance(value, np.ndarray) and value.dtype == np.float32:
        if packed:
            out += delimited(5, value.astype("<f4").tobytes())
        else:
            out += b"".join(tag(5, 5) + struct.pack("<f", v) for v in value.ravel())
    else:                                                  # list of ints
        if packed:
            out += delimited(6, b"".join(varint(int(v)) for v in value))
        else:
            out += b"".join(tag(6, 0) + varint(int(v)) for v in value)
    return out


def enc_op(op, packed=False):
    """OperatorDef (caffe2.proto:208-268): input=1, output=2, name=3, type=4, arg=5 (+ engine=7, skipped by the importer)"""
    out = b"".join(delimited(1, s.encode()) for s in op["input"])
    out += b"".join(delimited(2, s.encode()) for s in op["output"])
    out += delimited(3, b"") + delimited(4, op["type"].encode())
    out += b"".join(delimited(5, enc_arg(k, v, packed)) for k, v in op.get("arg", {}).items())
    return out + delimited(7, b"CUDNN") + tag(9, 0) + varint(0)


def enc_net(name, ops, packed=False):
    """NetDef (caffe2.proto:270-309): name=1, op=2, external_input=7"""
    return delimited(1, name.encode()) + b"".join(delimited(2, enc_op(o, packed)) for o in ops) + delimited(7, b"gpu_0/data")


def text_net(name, ops):
    def q(s):
        return '"' + s.replace("\\", "\\\\").replace('"', '\\"') + '"'
    lines = [f"name: {q(name)}  # written by swcompiler_amd.caffe2_files"]
    for o in ops:
        lines.append("op {")
        lines += [f"  input: {q(s)}" for s in o["input"]] + [f"  output: {q(s)}" for s in o["output"]]
        lines += ['  name: ""', f"  type: {q(o['type'])}"]
        for k, v in o.get("arg", {}).items():
            lines.append("  arg {")
            lines.append(f"    name: {q(k)}")
            if isinstance(v, float):
                lines.append(f"    f: {v!r}")
            elif isinstance(v, int):
                lines.append(f"    i: {v}")
            elif isinstance(v, str):
                lines.append(f"    s: {q(v)}")
            elif isinstance(v, np.ndarray):
                lines += [f"    floats: {float(x)!r}" for x in v.ravel()]   # repr of the float32 value as a double: exact
            else:
                lines += [f"    ints: {int(x)}" for x in v]
            lines.append("  }")
        lines += ['  engine: "CUDNN"', "  device_option { device_type: 1 cuda_gpu_id: 0 }", "}"]
    lines.append('external_input: "gpu_0/data"')
    return "\n".join(lines) + "\n"


def make_resnet50(width=64, blocks=(3, 4, 6, 3), classes=1000, image=224, seed=50):
    """ResNet-50 as the Caffe2 model zoo stores it (bias-free convolutions each followed by SpatialBN, in-place
    Relu and Sum, stride on the first 1x1 of a stage, 3x3/2 max pooling with pad 1, average pooling over the last
    map, FC, Softmax) with random weights; `width` = channels of the first stage's 3x3 (64 in the real model)."""
    rng = np.random.default_rng(seed)
    w, ops, g = {}, [], "gpu_0/"

    def conv_bn(name, src, cin, cout, k, stride, relu):
        w[g + name + "_w"] = (rng.standard_normal((cout, cin, k, k)) * np.sqrt(2.0 / (cin * k * k))).astype(np.float32)
        ops.append(dict(type="Conv", input=[g + src, g + name + "_w"], output=[g + name],
                        arg=dict(kernel=k, stride=stride, pad=k // 2, order="NCHW")))
        bn = name + "_bn"
        w[g + bn + "_s"] = rng.uniform(0.5, 1.0, cout).astype(np.float32)
        w[g + bn + "_b"] = (rng.standard_normal(cout) * 0.1).astype(np.float32)
        w[g + bn + "_rm"] = (rng.standard_normal(cout) * 0.1).astype(np.float32)
        w[g + bn + "_riv"] = rng.uniform(0.5, 2.0, cout).astype(np.float32)
        ops.append(dict(type="SpatialBN", input=[g + name] + [g + bn + s for s in ("_s", "_b", "_rm", "_riv")],
                        output=[g + bn], arg=dict(epsilon=float(np.float32(1e-5)), is_test=1, order="NCHW")))
        if relu:
            ops.append(dict(type="Relu", input=[g + bn], output=[g + bn]))
        return bn

    x = conv_bn("conv1", "data", 3, width, 7, 2, True)
    ops.append(dict(type="MaxPool", input=[g + x], output=[g + "pool1"], arg=dict(kernel=3, stride=2, pad=1)))
    x, cin, hw = "pool1", width, (image + 6 - 7) // 2 + 1
    hw = (hw + 2 - 3) // 2 + 1
    for stage, n in enumerate(blocks):
        mid, cout = width << stage, (width << stage) * 4
        for b in range(n):
            name = f"res{stage + 2}_{b}"
            stride = 2 if stage > 0 and b == 0 else 1
            short = x if (cin == cout and stride == 1) else conv_bn(name + "_branch1", x, cin, cout, 1, stride, False)
            y = conv_bn(name + "_branch2a", x, cin, mid, 1, stride, True)
            y = conv_bn(name + "_branch2b", y, mid, mid, 3, 1, True)
            y = conv_bn(name + "_branch2c", y, mid, cout, 1, 1, False)
            ops.append(dict(type="Sum", input=[g + y, g + short], output=[g + y]))
            ops.append(dict(type="Relu", input=[g + y], output=[g + y]))
            x, cin = y, cout
            hw = (hw - 1) // stride + 1
    ops.append(dict(type="AveragePool", input=[g + x], output=[g + "pool5"], arg=dict(kernel=hw, stride=1)))
    w[g + "pred_w"] = (rng.standard_normal((classes, cin)) / np.sqrt(cin)).astype(np.float32)
    w[g + "pred_b"] = (rng.standard_normal(classes) * 0.1).astype(np.float32)
    ops.append(dict(type="FC", input=[g + "pool5", g + "pred_w", g + "pred_b"], output=[g + "pred"]))
    ops.append(dict(type="Softmax", input=[g + "pred"], output=[g + "softmax"]))
    init = [dict(type="GivenTensorFill", input=[], output=[k], arg=dict(shape=list(v.shape), values=v)) for k, v in w.items()]
    return ops, init, w
