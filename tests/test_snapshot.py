"""Snapshots of training programs (reference: TrainingConfig::snapshot, src/codegen/Codegen.cpp:659-812,
src/codegen/utils/utils.h:23-68; the loader's restart position, src/codegen/utils/DataLoader.cpp:161-168).

The file format is pinned with the protobuf library (the Python package, which the generated programs do not
use): a message type with the field numbers of the reference's caffe2.proto parses what the programs write,
serializes it back to the same bytes, and what it writes — unpacked or packed — restores a program.  A run that
is restored from the snapshot of iteration 8 ends with the parameters of the uninterrupted run, bit for bit on the
CPU; a snapshot of the CPU program restores the HIP program and the other way round.
"""
import os
import subprocess

import numpy as np
import pytest

from tests.test_codegen import GEN, REF_UTILS, ROOT, SWC, build_cpu, build_hip, generate, write_record_file

SAMPLES, EVERY = 64, 4          # 2 epochs of 8 mini-batches: iterations 1..16, snapshots at 4, 8, 12, 16
MLP = dict(fc0_w=(784, 64), fc0_b=(64,), fc1_w=(64, 10), fc1_b=(10,))
LENET = dict(conv0_w=(16, 5, 5, 1), conv0_b=(16,), conv1_w=(16, 5, 5, 16), conv1_b=(16,), fc0_w=(144, 10), fc0_b=(10,))


@pytest.fixture(scope="module")
def gen():
    if not os.path.exists(GEN):
        subprocess.check_call(["make", "-C", SWC, "-j8"], stdout=subprocess.DEVNULL)
    return GEN


def netdef_class(packed=False):
    """NetDef / OperatorDef / Argument with the fields a snapshot uses, numbered as in caffe2.proto:152-166,
    210-218, 270-294"""
    from google.protobuf import descriptor_pb2, descriptor_pool, message_factory
    F = descriptor_pb2.FieldDescriptorProto
    pkg = "snap_packed" if packed else "snap"
    fd = descriptor_pb2.FileDescriptorProto(name=pkg + ".proto", package=pkg, syntax="proto2")
    arg = fd.message_type.add(name="Argument")
    arg.field.add(name="name", number=1, type=F.TYPE_STRING, label=F.LABEL_OPTIONAL)
    arg.field.add(name="i", number=3, type=F.TYPE_INT64, label=F.LABEL_OPTIONAL)
    floats = arg.field.add(name="floats", number=5, type=F.TYPE_FLOAT, label=F.LABEL_REPEATED)
    if packed:
        floats.options.packed = True
    op = fd.message_type.add(name="OperatorDef")
    op.field.add(name="name", number=3, type=F.TYPE_STRING, label=F.LABEL_OPTIONAL)
    op.field.add(name="arg", number=5, type=F.TYPE_MESSAGE, label=F.LABEL_REPEATED, type_name="." + pkg + ".Argument")
    net = fd.message_type.add(name="NetDef")
    net.field.add(name="op", number=2, type=F.TYPE_MESSAGE, label=F.LABEL_REPEATED, type_name="." + pkg + ".OperatorDef")
    net.field.add(name="arg", number=6, type=F.TYPE_MESSAGE, label=F.LABEL_REPEATED, type_name="." + pkg + ".Argument")
    pool = descriptor_pool.DescriptorPool()
    pool.Add(fd)
    return message_factory.GetMessageClass(pool.FindMessageTypeByName(pkg + ".NetDef"))


def run(exe, cwd, *flags):
    return subprocess.run([exe, *flags], cwd=cwd, check=True, capture_output=True, text=True, timeout=120).stdout


def final_params(tmp_path, shapes, suffix=""):
    out = {}
    for name, shape in shapes.items():
        files = [f for f in os.listdir(tmp_path) if f.startswith(name) and f.endswith(suffix + ".bin") and "momentum" not in f]
        assert len(files) == 1, (name, files)
        out[name] = np.fromfile(os.path.join(tmp_path, files[0]), np.float32).reshape(shape)
    return out


@pytest.mark.parametrize("compat", [False, True])
def test_snapshot_file_and_restored_cpu_run(gen, tmp_path, compat):
    write_record_file(tmp_path, SAMPLES)
    code = generate(gen, "mlp_train", "cpu", tmp_path, SAMPLES, snapshot=EVERY)
    assert code.count("addOp(net, ") == 2 * len(MLP) and "initTensorXavier(fc0_w, 50176, 784)" in code
    assert code.index("iter++") < code.index('std::cout << "iter = "') < code.index("iterations ")
    exe = build_cpu(tmp_path, with_loader=True, force_compat=compat)
    out = run(exe, tmp_path)
    assert [l for l in out.splitlines() if l.startswith("save snapshot")] == \
        ["save snapshot to snapshot_iter%d.model" % i for i in (4, 8, 12, 16)]
    full = final_params(tmp_path, MLP)

    # the file of the last iteration, read by the protobuf library: the final parameters, their momenta, the count
    NetDef = netdef_class()
    raw = open(os.path.join(tmp_path, "snapshot_iter16.model"), "rb").read()
    net = NetDef.FromString(raw)
    assert [o.name for o in net.op] == list(MLP) + [n + "_momentum" for n in reversed(list(MLP))]
    assert all(len(o.arg) == 1 and o.arg[0].name == "values" for o in net.op)
    for o in net.op[:len(MLP)]:
        assert np.array_equal(np.array(o.arg[0].floats, np.float32).view(np.uint32), full[o.name].ravel().view(np.uint32)), o.name
    assert any(np.any(np.array(o.arg[0].floats)) for o in net.op[len(MLP):])
    assert len(net.arg) == 1 and net.arg[0].name == "iter" and net.arg[0].i == 16
    assert net.SerializeToString(deterministic=True) == raw          # byte for byte what protobuf itself writes

    # restored at iteration 8, the run ends where the uninterrupted one ended
    for spelling in (["--snapshot=snapshot_iter8.model"], ["-snapshot", "snapshot_iter8.model"]):
        os.remove(os.path.join(tmp_path, "fc0_w.bin"))
        out = run(exe, tmp_path, *spelling)
        assert "restoring from snapshot snapshot_iter8.model" in out and "snapshot iter= 8" in out
        assert [l for l in out.splitlines() if l.startswith("iterations ")] == ["iterations 12", "iterations 16"]
        again = final_params(tmp_path, MLP)
        for name in MLP:
            assert np.array_equal(again[name].view(np.uint32), full[name].view(np.uint32)), name

    # files written by the protobuf library restore the program too: as the reference writes them, and packed
    half = NetDef.FromString(open(os.path.join(tmp_path, "snapshot_iter8.model"), "rb").read())
    Packed = netdef_class(packed=True)
    for fname, blob in (("by_protobuf.model", half.SerializeToString()),
                        ("packed.model", Packed.FromString(half.SerializeToString()).SerializeToString())):
        with open(os.path.join(tmp_path, fname), "wb") as f:
            f.write(blob)
        run(exe, tmp_path, "--snapshot=" + fname)
        again = final_params(tmp_path, MLP)
        for name in MLP:
            assert np.array_equal(again[name].view(np.uint32), full[name].view(np.uint32)), (fname, name)
    assert len(Packed.FromString(half.SerializeToString()).SerializeToString()) < len(half.SerializeToString())

    # a snapshot of another model is refused; a file that is not there, too
    bad = NetDef()
    o = bad.op.add(name="fc0_w")
    o.arg.add(name="values").floats.extend([1.0, 2.0])
    with open(os.path.join(tmp_path, "bad.model"), "wb") as f:
        f.write(bad.SerializeToString())
    r = subprocess.run([exe, "--snapshot=bad.model"], cwd=tmp_path, capture_output=True, text=True)
    assert r.returncode != 0 and "fc0_w does not have 50176 elements" in r.stdout
    r = subprocess.run([exe, "--snapshot=none.model"], cwd=tmp_path, capture_output=True, text=True)
    assert r.returncode != 0 and "Error loading none.model" in r.stdout


def test_loader_continues_where_the_snapshot_was_taken(tmp_path):
    """DataLoader::shift(n) of include/swc_host_utils.h: the loader goes on as after n mini-batches, also when a
    mini-batch runs over the end of the file into the next epoch (reference: DataLoader.cpp:125-168)"""
    images, labels = write_record_file(tmp_path, 20)
    src = r'''
#include "swc_host_utils.h"
int main(int argc, char **argv) {
    DataLoader loader("mnist_labels_images.bin", ONE_BYTE_AS_INT, FOUR_BYTES_AS_FLOAT, 3, 20, {8}, {8, 784});
    loader.shift(std::atoi(argv[1]));
    int label[8]; static float data[8 * 784];
    while (loader.next(label, data)) { for (int i = 0; i < 8; ++i) std::cout << label[i] << ":" << data[i * 784 + 300] << " "; std::cout << "\n"; }
    return argc ? 0 : 1;
}'''
    with open(os.path.join(tmp_path, "loader.cpp"), "w") as f:
        f.write(src)
    subprocess.check_call(["g++", "-std=c++11", "-O1", "-I", os.path.join(ROOT, "include"), "loader.cpp",
                           "-o", "loader.bin"], cwd=tmp_path)
    whole = run(os.path.join(tmp_path, "loader.bin"), tmp_path, "0").splitlines()
    assert len(whole) == 7                       # 3 x 20 records, 8 per mini-batch; the last 4 records are dropped
    want = [int(labels[(b * 8 + i) % 20]) for b in range(7) for i in range(8)]
    assert [int(tok.split(":")[0]) for line in whole for tok in line.split()] == want
    for n in (1, 2, 3, 5, 6):                    # 3 and 5: the next mini-batch starts in the middle of an epoch's tail
        assert run(os.path.join(tmp_path, "loader.bin"), tmp_path, str(n)).splitlines() == whole[n:], n


@pytest.mark.skipif(not os.path.isdir(REF_UTILS), reason="the reference tree is not here")
@pytest.mark.parametrize("samples,epochs,batch", [(20, 3, 8), (24, 2, 8), (5, 4, 3)])
def test_loader_reads_what_the_reference_loader_reads(tmp_path, samples, epochs, batch):
    """records of <1-byte label><12 data bytes>, bytes above 127 among them, through this repository's DataLoader
    and through the reference's (compiled from where it lies): the same mini-batches, from the start and after shift"""
    rng = np.random.default_rng(samples)
    rng.integers(0, 256, (samples, 13), dtype=np.uint8).tofile(os.path.join(tmp_path, "records.bin"))
    src = r'''
#include <cstdlib>
#include <iostream>
#include HEADER
int main(int argc, char **argv) {
    std::string file = "records.bin";
    DataLoader loader(file, ONE_BYTE_AS_INT, ONE_BYTE_AS_INT, EPOCHS, SAMPLES, {BATCH}, {BATCH, 3, 4});
    int label[BATCH]; float data[BATCH * 12];
    // (the reference opens its file in the first next(): a shift before that moves its counters but not its file
    // position, which a shift is meant to move too — the comparison is made where both have a file to seek in)
    if (std::atoi(argv[1])) { loader.next(label, data); loader.shift(std::atoi(argv[1])); }
    while (loader.next(label, data)) {
        std::cout << "batch";
        for (int i = 0; i < BATCH; ++i) { std::cout << " " << label[i]; for (int j = 0; j < 12; ++j) std::cout << "," << data[i * 12 + j]; }
        std::cout << "\n";
    }
    return argc ? 0 : 1;
}'''
    with open(os.path.join(tmp_path, "loader.cpp"), "w") as f:
        f.write(src)
    defs = ["-DEPOCHS=%d" % epochs, "-DSAMPLES=%d" % samples, "-DBATCH=%d" % batch]
    subprocess.check_call(["g++", "-std=c++11", "-O1", "-w", "-I", os.path.join(ROOT, "include"), '-DHEADER="swc_host_utils.h"',
                           *defs, "loader.cpp", "-o", "mine.bin"], cwd=tmp_path)
    subprocess.check_call(["g++", "-std=c++11", "-O1", "-w", "-I", REF_UTILS, '-DHEADER="utils/DataLoader.h"', *defs, "loader.cpp",
                           os.path.join(REF_UTILS, "utils", "DataLoader.cpp"), "-o", "theirs.bin"], cwd=tmp_path)
    total = samples * epochs // batch
    for n in (0, 1, 2, total // 2, total - 1):
        mine = [l for l in run(os.path.join(tmp_path, "mine.bin"), tmp_path, str(n)).splitlines() if l.startswith("batch")]
        theirs = [l for l in run(os.path.join(tmp_path, "theirs.bin"), tmp_path, str(n)).splitlines() if l.startswith("batch")]
        assert mine == theirs and len(mine) == total - n, n
    assert "-" in "".join(mine)          # bytes above 127 are read as negative numbers by both


def test_snapshot_hip_program_structure(gen, tmp_path):
    write_record_file(tmp_path, SAMPLES)
    code = generate(gen, "lenet_train", "hip", tmp_path, SAMPLES, graph=True, snapshot=EVERY)
    loop = code[code.index("while(loader.next("):code.index("} //while")]
    snap = loop[loop.index('std::cout << "iter = "'):loop.index("save snapshot to")]
    # every parameter and every momentum comes down from the device into the host tensor the snapshot names
    assert snap.count("swc_hip_d2h(") == 2 * len(LENET) == snap.count("addOp(net, ")
    for name in LENET:
        for t in (name, name + "_momentum"):
            assert snap.index("swc_hip_d2h(%s, %s_dev, " % (t, t)) < snap.index('addOp(net, "%s", %s, ' % (t, t))
    # restored values are in the host tensors before the uploads
    assert code.index('loadFromSnapShot(swc_snapshot, "conv0_w", conv0_w, 400)') < code.index("swc_hip_h2d(conv0_w_dev, conv0_w, ")
    assert code.index("loader.shift(snap_iter)") < code.index("one-time parameter upload")
    build_hip(tmp_path)


@pytest.mark.gpu
@pytest.mark.parametrize("model,shapes", [("mlp_train", MLP), ("lenet_train", LENET)])
@pytest.mark.parametrize("mode", ["eager", "graph"])
def test_snapshot_hip_program(gen, tmp_path, model, shapes, mode):
    print("case snapshot", model, mode, flush=True)
    write_record_file(tmp_path, SAMPLES)
    generate(gen, model, "hip", tmp_path, SAMPLES, graph=mode == "graph", snapshot=EVERY)
    exe = build_hip(tmp_path)
    out = run(exe, tmp_path)
    assert out.count("save snapshot to") == 4
    full = final_params(tmp_path, shapes, "_host")
    NetDef = netdef_class()
    last = NetDef.FromString(open(os.path.join(tmp_path, "snapshot_iter16.model"), "rb").read())
    for o in last.op:
        if o.name in shapes:     # what the last snapshot holds is what the program leaves at its end
            assert np.array_equal(np.array(o.arg[0].floats, np.float32), full[o.name].ravel()), o.name
    first = NetDef.FromString(open(os.path.join(tmp_path, "snapshot_iter8.model"), "rb").read())
    start = {o.name: np.array(o.arg[0].floats, np.float32) for o in first.op}
    assert all(np.any(start[n + "_momentum"]) for n in shapes)
    # the same kernels in the same order on the same values: the restored run repeats iterations 9..16 exactly
    out = run(exe, tmp_path, "--snapshot=snapshot_iter8.model")
    assert "snapshot iter= 8" in out and out.count("save snapshot to") == 2
    again = final_params(tmp_path, shapes, "_host")
    for name in shapes:
        assert np.array_equal(again[name], full[name]), name
        assert not np.array_equal(full[name].ravel(), start[name]), name

    # the CPU program goes on from the HIP program's snapshot, and the other way round
    cpu_dir = os.path.join(tmp_path, "cpu")
    os.mkdir(cpu_dir)
    write_record_file(cpu_dir, SAMPLES)
    generate(gen, model, "cpu", cpu_dir, SAMPLES, snapshot=EVERY)
    cpu = build_cpu(cpu_dir, with_loader=True, force_compat=True)
    run(cpu, cpu_dir, "--snapshot=" + os.path.join(tmp_path, "snapshot_iter8.model"))
    on_cpu = final_params(cpu_dir, shapes)
    run(exe, tmp_path, "--snapshot=" + os.path.join(cpu_dir, "snapshot_iter12.model"))
    back = final_params(tmp_path, shapes, "_host")
    for name in shapes:
        change = np.abs(full[name].ravel() - start[name]).max()
        assert np.abs(on_cpu[name] - full[name]).max() < 1e-3 * change + 1e-6, name
        assert np.abs(back[name] - full[name]).max() < 1e-3 * change + 1e-6, name
