"""Training programs: Config::train_mode -> autodiff pass -> CPU / HIP code generators (reference:
src/pass/AutodiffPass.cpp, src/op/dlOp/dlOpAD.cpp, the training branch of src/codegen/Codegen.cpp and
test/engine/testEngineLenetDistTrain.cpp without MPI).

CPU: the generated program calls the reference's training kernels in the reference's order; its final parameters
equal, bit for bit, the same loop written out in Python over the oracle's kernels.  GPU: the HIP program's final
parameters and its losses follow the CPU program's within the tolerance of the forward path.
"""
import os
import subprocess

import numpy as np
import pytest

from tests.test_codegen import GEN, SWC, TOL, build_cpu, build_hip, generate, write_record_file
from tests.util import assert_bit_exact

LR, DECAY, MOMENTUM, BATCH, SAMPLES, EPOCHS = 0.01, 0.001, 0.9, 8, 64, 2


@pytest.fixture(scope="module")
def gen():
    if not os.path.exists(GEN):
        subprocess.check_call(["make", "-C", SWC, "-j8"], stdout=subprocess.DEVNULL)
    return GEN


def make_params(model, tmp_path):
    rng = np.random.default_rng(11)
    shapes = (dict(fc0_w=(784, 64), fc0_b=(64,), fc1_w=(64, 10), fc1_b=(10,)) if model == "mlp_train" else
              dict(conv0_w=(16, 5, 5, 1), conv0_b=(16,), conv1_w=(16, 5, 5, 16), conv1_b=(16,), fc0_w=(144, 10), fc0_b=(10,)))
    params = {}
    for name, shape in shapes.items():
        fan_in = int(np.prod(shape[1:])) if name.startswith("conv") else shape[0]
        p = (rng.standard_normal(shape) / np.sqrt(fan_in)).astype(np.float32) if name.endswith("_w") else \
            (rng.standard_normal(shape) * 0.1).astype(np.float32)
        p.tofile(os.path.join(tmp_path, name + ".bin"))
        params[name] = p
    return params


def fc_backward(oracle, x2d, w, dy):
    """what MatrixMatrixFCBiasGrad is lowered to; the bias gradient as batchedreduceadd_f leaves it: the sums of
    dy's ROWS in the first `rows` entries of a zero-initialised vector (kernels.h:554-563 at the call of
    Codegen.cpp:1517-1531)"""
    dx = oracle.matrixMatrixMul(dy, oracle.transpose(w, (1, 0)))
    dw = oracle.matrixMatrixMul(oracle.transpose(x2d, (1, 0)), dy)
    db = np.zeros(w.shape[1], np.float32)
    db[:dy.shape[0]] = oracle.batchedreduceadd(dy)
    return dx, dw, db


def train_reference(oracle, model, params, images, labels):
    """the generated training program, written out over the oracle's kernels"""
    p = {k: v.copy() for k, v in params.items()}
    mom = {k: np.zeros_like(v) for k, v in params.items()}
    losses = []
    conv = dict(kernels=(5, 5), strides=(1, 1), pads=(2, 2, 2, 2))

    def step(k, g):
        p[k], mom[k] = oracle.sgd(p[k], g, mom[k], LR, DECAY, MOMENTUM, BATCH)
    n_iter = SAMPLES * EPOCHS // BATCH
    for it in range(n_iter):
        idx = [(it * BATCH + j) % SAMPLES for j in range(BATCH)]
        sel = labels[idx].astype(np.int32)
        if model == "mlp_train":
            x = images[idx]
            y0 = oracle.fcbias(x, p["fc0_w"], p["fc0_b"])
            h = oracle.matrixTanh(y0)
            logits = oracle.fcbias(h, p["fc1_w"], p["fc1_b"])
            prob, loss = oracle.matrixSoftmaxWithLoss(logits, sel)
            dlogits = oracle.matrixSoftmaxGrad(prob, sel, with_loss=True)
            dh, dw1, db1 = fc_backward(oracle, h, p["fc1_w"], dlogits)
            dy0 = oracle.matrixTanhGrad(h, dh)
            _, dw0, db0 = fc_backward(oracle, x, p["fc0_w"], dy0)
            grads = dict(fc1_w=dw1, fc1_b=db1, fc0_w=dw0, fc0_b=db0)
        else:
            x = images[idx].reshape(BATCH, 28, 28, 1)
            c0 = oracle.conv2d(x, p["conv0_w"], p["conv0_b"], **conv)
            m0 = oracle.maxpool(c0, (3, 3), (3, 3))
            r0 = oracle.relu(m0.ravel()).reshape(m0.shape)
            c1 = oracle.conv2d(r0, p["conv1_w"], p["conv1_b"], **conv)
            m1 = oracle.maxpool(c1, (3, 3), (3, 3))
            r1 = oracle.relu(m1.ravel()).reshape(m1.shape)
            flat = r1.reshape(BATCH, -1)
            logits = oracle.fcbias(flat, p["fc0_w"], p["fc0_b"])
            prob, loss = oracle.matrixSoftmaxWithLoss(logits, sel)
            dlogits = oracle.matrixSoftmaxGrad(prob, sel, with_loss=True)
            dflat, dwf, dbf = fc_backward(oracle, flat, p["fc0_w"], dlogits)
            dm1 = oracle.reluGrad(m1.ravel(), dflat.ravel()).reshape(m1.shape)
            dc1 = oracle.maxpoolGrad(c1, dm1, (3, 3), (3, 3))
            dr0, dw1, db1 = oracle.conv2dGrad(r0, p["conv1_w"], dc1, **conv)
            dm0 = oracle.reluGrad(m0.ravel(), dr0.ravel()).reshape(m0.shape)
            dc0 = oracle.maxpoolGrad(c0, dm0, (3, 3), (3, 3))
            _, dw0, db0 = oracle.conv2dGrad(x, p["conv0_w"], dc0, **conv)
            grads = dict(fc0_w=dwf, fc0_b=dbf, conv1_w=dw1, conv1_b=db1, conv0_w=dw0, conv0_b=db0)
        for k, g in grads.items():
            step(k, g)
        losses.append(float(loss))
    return p, losses


def printed_losses(out):
    lines = out.split("\n")
    return [float(lines[i + 1].split()[0]) for i, l in enumerate(lines) if l.startswith("iterations ")]


@pytest.mark.parametrize("model", ["mlp_train", "lenet_train"])
@pytest.mark.parametrize("compat", [False, True])
def test_training_cpu_program(gen, oracle, tmp_path, model, compat):
    images, labels = write_record_file(tmp_path, SAMPLES)
    params = make_params(model, tmp_path)
    code = generate(gen, model, "cpu", tmp_path, SAMPLES)
    assert code.count("sgd_f(") == len(params) and "matrixSoftmaxWithLoss_f(" in code and "matrixSoftmaxWithLossGrad_f(" in code
    assert code.count("batchedreduceadd_f(") == (2 if model == "mlp_train" else 1)
    if model == "lenet_train":
        assert code.count("conv2dGrad_f(") == 2 and code.count("maxpoolGrad_f(") == 2 and code.count("reluGrad_f(") == 2
    exe = build_cpu(tmp_path, with_loader=True, force_compat=compat)
    out = subprocess.run([exe], cwd=tmp_path, check=True, capture_output=True, text=True).stdout
    want, losses = train_reference(oracle, model, params, images, labels)
    for name in params:
        got = np.fromfile(os.path.join(tmp_path, name + ".bin"), np.float32).reshape(params[name].shape)
        assert not np.array_equal(got, params[name]), name + " was not trained"
        assert_bit_exact(got, want[name], name)
    shown = printed_losses(out)
    assert len(shown) == 4 and np.allclose(shown, losses[3::4], atol=2e-3)     # printed with three decimals
    assert losses[-1] < losses[0]


@pytest.mark.parametrize("model", ["mlp_train", "lenet_train"])
def test_training_hip_program_structure(gen, tmp_path, model):
    write_record_file(tmp_path, SAMPLES)
    n_params = len(make_params(model, tmp_path))
    code = generate(gen, model, "hip", tmp_path, SAMPLES, graph=True)
    head, body = code.split("while(loader.next(selected, data0))")
    loop = body[:body.index("} //while")]
    # the whole step — forward, gradients, optimizer — is one recorded graph; per batch: two uploads and its launch
    assert head.count("swc_hip_graph_begin()") == 1 and head.count("swc_hip_sgd_f(") == 2 * n_params
    assert loop.count("swc_hip_h2d(") == 2 and loop.count("swc_hip_graph_launch(swc_graph)") == 1 and "swc_hip_sgd_f" not in loop
    # parameters and momenta go up before the warm-up pass and again after it (it takes an optimizer step of its
    # own); the updated parameters come back once, after the loop; the loss where it is shown
    assert head.count("swc_hip_h2d(") == 4 * n_params
    warm = head[head.index("warm-up pass"):head.index("swc_hip_graph_begin()")]
    assert warm.index("swc_hip_sgd_f(") < warm.index("before the warm-up pass") and warm.count("swc_hip_h2d(") == 2 * n_params
    tail = body[body.index("} //while"):]
    assert tail.count("swc_hip_d2h(") == n_params + 1 and loop.count("swc_hip_d2h(") == 1
    assert "swc_hip_d2h(loss_host, loss, 4)" in loop[loop.index("if (iter % 4 == 0)"):]
    build_hip(tmp_path)


@pytest.mark.gpu
@pytest.mark.parametrize("model", ["mlp_train", "lenet_train"])
@pytest.mark.parametrize("mode", ["eager", "graph", "prefetch"])
def test_training_hip_program(gen, oracle, tmp_path, model, mode):
    print("case training", model, mode, flush=True)
    images, labels = write_record_file(tmp_path, SAMPLES)
    params = make_params(model, tmp_path)
    generate(gen, model, "hip", tmp_path, SAMPLES, graph=mode == "graph", prefetch=mode == "prefetch")
    out = subprocess.run([build_hip(tmp_path)], cwd=tmp_path, check=True, capture_output=True, text=True, timeout=120).stdout
    want, losses = train_reference(oracle, model, params, images, labels)
    for name in params:
        files = [f for f in os.listdir(tmp_path) if f.startswith(name) and f.endswith("_host.bin")]
        assert len(files) == 1, (name, files)
        got = np.fromfile(os.path.join(tmp_path, files[0]), np.float32).reshape(params[name].shape)
        change = np.abs(want[name] - params[name]).max()
        assert change > 0 and np.abs(got - want[name]).max() < 1e-3 * change + 1e-6, name
    assert np.allclose(printed_losses(out), losses[3::4], atol=2e-3)


@pytest.mark.parametrize("model", ["mlp_train_label", "mlp_train_getnet"])
def test_training_through_a_labelled_softmax_cpu(gen, oracle, tmp_path, model):
    """The older way to end a training graph: the label is the second operand of MatrixSoftmax, whose gradient op
    is MatrixSoftmaxGrad (reference: src/op/dlOp/dlOpAD.cpp:213-247, Codegen.cpp:2429-2444); once through
    Engine::compile, once through getTrainNet and hand-run passes as the reference's test/testSnapshot.cpp does.
    matrixSoftmaxGrad_f is the arithmetic of matrixSoftmaxWithLossGrad_f, so the parameters end where the
    MatrixSoftmaxWithLoss network's end."""
    images, labels = write_record_file(tmp_path, SAMPLES)
    params = make_params("mlp_train", tmp_path)
    code = generate(gen, model, "cpu", tmp_path, SAMPLES)
    assert "matrixSoftmaxGrad_f(8, 10, fc1_out_grad, 10, prob, 10, selected);" in code and "WithLoss" not in code
    assert code.count("sgd_f(") == len(params)
    exe = build_cpu(tmp_path, with_loader=True)
    subprocess.run([exe], cwd=tmp_path, check=True, capture_output=True, text=True)
    want, _ = train_reference(oracle, "mlp_train", params, images, labels)
    for name in params:
        got = np.fromfile(os.path.join(tmp_path, name + ".bin"), np.float32).reshape(params[name].shape)
        assert_bit_exact(got, want[name], name)


@pytest.mark.gpu
def test_training_through_a_labelled_softmax_hip(gen, oracle, tmp_path):
    print("case training mlp_train_label graph", flush=True)
    images, labels = write_record_file(tmp_path, SAMPLES)
    params = make_params("mlp_train", tmp_path)
    code = generate(gen, "mlp_train_label", "hip", tmp_path, SAMPLES, graph=True)
    assert "swc_hip_matrixSoftmaxGrad_f(8, 10, fc1_out_grad, 10, prob, 10, selected_dev)" in code
    subprocess.run([build_hip(tmp_path)], cwd=tmp_path, check=True, capture_output=True, text=True, timeout=120)
    want, _ = train_reference(oracle, "mlp_train", params, images, labels)
    for name in params:
        files = [f for f in os.listdir(tmp_path) if f.startswith(name) and f.endswith("_host.bin")]
        assert len(files) == 1, (name, files)
        got = np.fromfile(os.path.join(tmp_path, files[0]), np.float32).reshape(params[name].shape)
        change = np.abs(want[name] - params[name]).max()
        assert change > 0 and np.abs(got - want[name]).max() < 1e-3 * change + 1e-6, name
