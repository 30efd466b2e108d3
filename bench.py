#!/usr/bin/env python3
"""Benchmark of the SWCompiler inference path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--headline-only] [--no-cpu]
    python bench.py --clocks        (the shader clock under single kernels, a line of its own)

Headline workload (the configuration the metric is quoted on): the wide MLP,
batch 4096 x 784 -> FC 4096 + ReLU -> FC 4096 + ReLU -> FC 10 + softmax (one call), fp32,
as the HIP target emits it (bias and ReLU in the GEMM epilogue).  One step = one
pass of that graph over one batch already resident in HBM.  Prints ONE JSON
line; `value` is samples/s over exactly K timed steps.

Also in the line:
  roofline      the dominant kernel (the tiled fp32-MFMA GEMM gemm_dma2<2,4,4,2,false,8>: both of its
                launches per step, 4096x784x4096 and 4096x4096x4096), timed
                with HIP events on the library's stream inside the timed region
  kernels       per-launch times of the headline graph.  Every kernel row carries two durations: `ms`, between
                events around the single launch inside the eager step (which adds the 2-5 us a pair of events
                costs), and `ms_loop`, the average over 20 back-to-back launches of that op between ONE pair of
                events; `frac`, `tflops`, `gbs` come from `ms_loop`, `frac_in_step` from `ms`
  parity        measured distance between what the timed graph computed on the GPU and what the reference's own
                CPU kernels computed from the same buffers in the cpu_baseline leg (strict on significant outputs,
                floored, max norm, bit-exact), with its bar; configs.cfgN.parity for the other configurations; the
                run exits non-zero after printing if a bar is broken
  graph_replay  the same K steps replayed as one HIP graph per step (no per-kernel
                events in the loop): what a launch-bound small graph gains; `shader_clock_ghz`: the clock the
                chip ran at meanwhile (one-wavefront watcher of the bench-only library on a stream of its own;
                the datasheet peaks assume 2.4 GHz)
  incl_transfers  the step with the input batch uploaded and the result downloaded
                each time (never the headline value); `overlapped_uploads`: the same with
                the next batch's upload on a second stream while this batch is computed
  peaks_measured  fp32 MFMA rate of a register-only loop and a streaming copy on this
                device, beside the datasheet peaks the fractions are computed from; and what a pair of
                events reads with nothing / a 1 KB kernel between them (the floor under every per-op figure)
  configs       the other synthetic configurations (samples/s and, per kernel,
                TFLOP/s or GB/s with the fraction of the MI355X peak)
                plus `training_kernels`: conv2dGrad, reluGrad, sgd, maxpoolGrad at those sizes, and `resnet50_b32`:
                ResNet-50 (synthetic weights) imported from Caffe2 model files, fused and run as a HIP graph by the
                generated program, with a table of its layers by class
  cpu_baseline  the reference's own CPU kernels (oracle/_ref, g++ -std=c++11 -O2,
                one thread) on the first rows of the same batch; every other configuration
                carries its own under configs.cfgN.cpu_baseline (whole batch, same buffers)

Ops never allocate: the harness sizes one scratch buffer with the library's
swc_hip_*_workspace_bytes queries over every shape it runs and hands it over
with swc_hip_set_workspace, as a generated program does.

The CPU checker is used only for the cpu_baseline leg.
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

import numpy as np  # noqa: E402

PEAK_TFLOPS_FP32_MFMA = 157.3
PEAK_HBM_GBS = 8000.0
ROOFLINE_KERNEL = "gemm_dma2<2,4,4,2,false,8>"   # 256x256 tiles, eight wavefronts: what both large FCs dispatch to
# the sources of that kernel: profiles/traffic.json records their hash when its counters are read, and a figure
# measured on other sources is not reported
ROOFLINE_SOURCES = ["swcompiler_amd/csrc/gemm.hip", "swcompiler_amd/csrc/mfma_dma2.hpp", "swcompiler_amd/csrc/mfma_dma.hpp",
                    "swcompiler_amd/csrc/mfma_tile.hpp"]


def sources_sha256():
    import hashlib
    h = hashlib.sha256()
    for rel in ROOFLINE_SOURCES:
        with open(os.path.join(ROOT, rel), "rb") as f:
            h.update(f.read())
    return h.hexdigest()


def traffic_from_counters(fetch_csv, write_csv):
    """--traffic-from: reads the two rocprofv3 --pmc runs of `bench.py --headline-only --no-cpu --calibrate` (FETCH_SIZE,
    then WRITE_SIZE; KiB per dispatch), scales each by what the same counter reads for the calibration pass (relu_f
    over 2^26 floats: 256 MiB read, 256 MiB written) and writes profiles/traffic.json with the hash of the kernel's
    sources."""
    import csv
    import datetime
    import re

    def short(name):   # "void (anonymous namespace)::gemm_dma2<2, 4, 4, 2, false, 8>(float const*, ...)" -> "gemm_dma2<2,4,4,2,false,8>"
        name = re.sub(r"\(anonymous namespace\)::", "", name.replace("void ", ""))
        depth, out = 0, ""
        for ch in name:
            if ch == "(" and depth == 0:
                break
            depth += ch == "<"
            depth -= ch == ">"
            out += ch
        return out.replace(" ", "")

    def per_kernel(path, counter):
        vals = {}
        for row in csv.DictReader(open(path)):
            if row["Counter_Name"] == counter:
                vals.setdefault((short(row["Kernel_Name"]), int(row["Grid_Size"])), []).append(float(row["Counter_Value"]))
        return vals

    fetch, write = per_kernel(fetch_csv, "FETCH_SIZE"), per_kernel(write_csv, "WRITE_SIZE")
    cal = ("flat_vec4<OpRelu,true>", 1 << 24)   # 2^26 floats, four per thread
    true_kib = float(1 << 18)
    f_scale = true_kib / (sum(fetch[cal]) / len(fetch[cal]))
    w_scale = true_kib / (sum(write[cal]) / len(write[cal]))
    out = {"_comment": "HBM bytes per launch from rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE (written by bench.py --traffic-from; "
                       "the commands are in profiles/wide_mlp_gemm.txt); bench.py copies the figure of the dominant kernel "
                       "into roofline.traffic while the kernel's sources still hash to sources_sha256"}
    for kernel in (ROOFLINE_KERNEL, "gemm_skinny_stream<3,true>"):
        f = [v for (k, _), vs in fetch.items() if k == kernel for v in vs]
        w = [v for (k, _), vs in write.items() if k == kernel for v in vs]
        if not f or not w:
            continue
        fk, wk = sum(f) / len(f), sum(w) / len(w)
        out[kernel] = dict(fetch_kib_counter=fk, fetch_scale=f_scale, write_kib_counter=wk, write_scale=w_scale,
                           bytes_per_launch=int((fk * f_scale + wk * w_scale) * 1024), dispatches=len(f),
                           measured=dict(date=datetime.date.today().isoformat(), sources_sha256=sources_sha256(),
                                         sources=ROOFLINE_SOURCES, command="see profiles/wide_mlp_gemm.txt"))
    with open(os.path.join(ROOT, "profiles", "traffic.json"), "w") as fh:
        json.dump(out, fh, indent=1)
    print(json.dumps(out, indent=1))


class Timed:
    """Proxy of the runtime that records a HIP event before and after every op."""

    def __init__(self, rt):
        self.rt = rt
        self.log = []   # (op name, slot0, slot1, work dict)
        self.slot = 0

    def reset(self):
        self.log, self.slot = [], 0

    def _wrap(self, name, work_fn):
        fn = getattr(self.rt, name)

        def call(*a, **kw):
            s0 = self.slot
            self.slot += 2
            self.rt.event_record(s0)
            out = fn(*a, **kw)
            self.rt.event_record(s0 + 1)
            self.log.append((name, s0, s0 + 1, work_fn(out, *a, **kw), lambda: fn(*a, **kw)))
            return out
        return call

    def __getattr__(self, name):
        return self._wrap(name, WORK[name])

    def results(self):
        rows = []
        for name, s0, s1, work, _ in self.log:
            ms = self.rt.event_elapsed_ms(s0, s1)
            rows.append(dict(op=name, ms=ms, **work))
        return rows

    def loop_times(self, iters=20, warm=3):
        """Average duration of one launch of every op of the last logged step, over `iters` back-to-back launches
        of that op between ONE pair of events: the op's kernels and the gaps between its launches, without the
        2-5 us that a pair of events around a single launch adds."""
        out = []
        for _, _, _, _, again in self.log:
            for _ in range(warm):
                again()
            self.rt.event_record(0)
            for _ in range(iters):
                again()
            self.rt.event_record(1)
            out.append(self.rt.event_elapsed_ms(0, 1) / iters)
        return out


def _gemm_work(res, a, b, *r, **kw):
    m, k = a.shape
    n = b.shape[1]
    work = dict(shape=f"{m}x{k}x{n}", flop=2.0 * m * n * k)
    if n <= 16:   # a classifier head: one pass over A is what bounds it, not the arithmetic
        work["bytes"] = 4.0 * (m * k + k * n + m * n)
    return work


def _conv_work(res, x, f, *r, **kw):
    m = res.size // res.shape[3]
    k = f.shape[1] * f.shape[2] * f.shape[3]
    if kw.get("pool"):   # the result is the pooled tensor: four convolution pixels per element
        m *= 4
        return dict(shape=f"{list(x.shape)}*{list(f.shape)} + maxpool 2x2", flop=2.0 * m * f.shape[0] * k)
    return dict(shape=f"{list(x.shape)}*{list(f.shape)}", flop=2.0 * m * f.shape[0] * k)


def _bytes(per_in=0, per_out=0, n_in=1):
    def fn(res, x, *r, **kw):
        return dict(shape=str(list(x.shape)), bytes=float(x.size * per_in * n_in + res.size * per_out))
    return fn


# algorithmic work per op: GEMM 2mnk, conv 2*M*oC*K; bandwidth ops count every
# input element read once and every output element written once (4 B each).
WORK = {
    "matrixMatrixMul": _gemm_work, "fcbias": _gemm_work, "conv2d": _conv_work,
    "relu": _bytes(4, 4), "batchedadd": _bytes(4, 4), "vecAdd": _bytes(4, 4, n_in=2),
    "batchnormalization": _bytes(4, 4), "maxpool": _bytes(4, 4), "matrixSoftmax": _bytes(4, 4),
    "batchnormReluMaxpool": _bytes(4, 4),
}


def rate(row):
    """adds achieved rate and roofline fraction to a kernel row: from `ms_loop` (average launch duration over
    back-to-back launches) where the row has one, else from `ms`; rows with both also get `frac_in_step`, the same
    fraction from the events around the single launch inside the eager step"""
    if "ms_loop" in row:
        in_step = rate(dict((k, v) for k, v in row.items() if k != "ms_loop"))
        row["frac_in_step"] = in_step["frac"]
    s = row.get("ms_loop", row["ms"]) * 1e-3
    if "flop" in row and "bytes" in row:   # GEMM with N <= 16: both figures, judged against the HBM roofline
        row["tflops"] = row["flop"] / s / 1e12
        row["gbs"] = row["bytes"] / s / 1e9
        row["frac"] = row["gbs"] / PEAK_HBM_GBS
        row["bound"] = "hbm"
    elif "flop" in row:
        row["tflops"] = row["flop"] / s / 1e12
        row["frac"] = row["tflops"] / PEAK_TFLOPS_FP32_MFMA
        row["bound"] = "mfma"
    else:
        row["gbs"] = row["bytes"] / s / 1e9
        row["frac"] = row["gbs"] / PEAK_HBM_GBS
        row["bound"] = "hbm"
    return row


def merge_rows(all_rows, loop_ms=None):
    """average per-launch rows of repeated steps (same op order every step); loop_ms: per op, the average launch
    duration over back-to-back launches (Timed.loop_times)"""
    n = len(all_rows)
    out = []
    for i, row in enumerate(all_rows[0]):
        r = dict(row)
        times = sorted(step[i]["ms"] for step in all_rows)
        r["ms"] = sum(times) / n          # events around the single launch inside the step, averaged over the steps
        r["ms_median"] = times[n // 2]
        r["ms_min"] = times[0]
        if loop_ms is not None:
            r["ms_loop"] = loop_ms[i]
        out.append(rate(r))
    return out


def with_transfers(rt, graphs, cfg, steps):
    """The same step with the input batch uploaded and the result downloaded every step
    (page-locked host memory, synchronous copies: what a generated program's batch loop does)."""
    t = graphs.make_inputs(cfg)
    dt = {k: rt.upload(v) for k, v in t.items()}
    batch = graphs.batch_of(cfg, t)
    ws = {}
    out = graphs.run(cfg, rt, dt, fused=True, ws=ws)
    # page-locked host buffers, as the host arena of a generated program is
    host_x, host_out = rt.pinned_empty(t["x"].shape), rt.pinned_empty(out.shape)
    host_x[...] = t["x"]
    rt.sync()
    t0 = time.perf_counter()
    for _ in range(steps):
        rt.upload_into(dt["x"], host_x)
        out = graphs.run(cfg, rt, dt, fused=True, ws=ws)
        rt.download_into(host_out, out)
    wall = time.perf_counter() - t0
    res = dict(samples_per_s=batch * steps / wall, ms_per_step=wall * 1e3 / steps,
               h2d_bytes=int(host_x.nbytes), d2h_bytes=int(host_out.nbytes), host_memory="page-locked")
    # the same with the upload of the next batch on the library's copy stream while this one is computed:
    # the batch lands in a staging buffer, a device-to-device copy hands it to the graph's input
    stage = rt.empty(t["x"].shape)
    rt.copy_h2d_async(stage, host_x)
    t0 = time.perf_counter()
    for _ in range(steps):
        rt.copy_sync()            # the batch has arrived (and host_x may be refilled)
        rt.ops_wait_copies()
        rt.d2d(dt["x"], stage)
        rt.copy_wait_ops()        # the next upload starts when the staging buffer has been read
        out = graphs.run(cfg, rt, dt, fused=True, ws=ws)
        rt.copy_h2d_async(stage, host_x)
        rt.download_into(host_out, out)
    rt.copy_sync()
    wall = time.perf_counter() - t0
    res["overlapped_uploads"] = dict(samples_per_s=batch * steps / wall, ms_per_step=wall * 1e3 / steps)
    stage.free()
    rt.free_pinned(host_x)
    rt.free_pinned(host_out)
    return res


def measured_peaks(rt):
    """What this device sustains on the two rooflines: a register-only fp32 MFMA loop
    (short and ~10 ms long: the clock settles lower under sustained matrix load) and a
    256 MiB-in / 256 MiB-out streaming pass (relu_f)."""
    short = rt.probe_mfma_tflops(200)
    long_ = rt.probe_mfma_tflops(20000)
    x = rt.upload(np.ones(1 << 26, np.float32))
    y = rt.empty(x.shape)
    rt.relu(x, out=y)
    times = []
    for i in range(10):
        rt.event_record(0)
        rt.relu(x, out=y)
        rt.event_record(1)
        times.append(rt.event_elapsed_ms(0, 1))
    x.free()
    y.free()
    # what a pair of events costs by itself: every per-op figure below carries it (it matters for kernels of a few us)
    gaps = []
    for i in range(20):
        rt.event_record(0)
        rt.event_record(1)
        rt.sync()
        gaps.append(rt.event_elapsed_ms(0, 1) * 1e3)
    tiny = rt.upload(np.ones(256, np.float32))
    tiny_out = rt.empty((256,))
    around_tiny = []
    for i in range(20):
        rt.event_record(0)
        rt.relu(tiny, out=tiny_out)
        rt.event_record(1)
        rt.sync()
        around_tiny.append(rt.event_elapsed_ms(0, 1) * 1e3)
    return dict(event_pair_empty_us=float(np.median(gaps)), event_pair_around_a_1kb_kernel_us=float(np.median(around_tiny)),
                mfma_f32_tflops_short=short[0], mfma_f32_short_ms=short[1], mfma_f32_tflops_sustained=long_[0],
                mfma_f32_sustained_ms=long_[1], stream_copy_gbs=2 * (1 << 28) / (min(times) * 1e-3) / 1e9,
                datasheet=dict(mfma_f32_tflops=PEAK_TFLOPS_FP32_MFMA, hbm_gbs=PEAK_HBM_GBS))


def run_config(rt, graphs, cfg, steps, warmup):
    t = graphs.make_inputs(cfg)
    dt = {k: rt.upload(v) for k, v in t.items()}
    batch = graphs.batch_of(cfg, t)
    ws = {}
    for _ in range(max(warmup, 1)):
        graphs.run(cfg, rt, dt, fused=True, ws=ws)
    rt.sync()
    timed = Timed(rt)
    per_step = []
    t0 = time.perf_counter()
    rt.timer_begin()
    for _ in range(steps):
        timed.log = []
        graphs.run(cfg, timed, dt, fused=True, ws=ws)
        per_step.append(timed.log)
    gpu_ms = rt.timer_end_ms()
    rt.sync()
    wall = time.perf_counter() - t0
    # events were recorded into distinct slots per step; read them now
    all_rows = []
    for log in per_step:
        timed.log = log
        all_rows.append(timed.results())
    timed.log = per_step[-1]
    rows = merge_rows(all_rows, timed.loop_times())
    result = graphs.run(cfg, rt, dt, fused=True, ws=ws)   # what the timed steps computed, for the parity figures
    result = {k: v.numpy() for k, v in result.items()} if isinstance(result, dict) else result.numpy()
    # the same step as one HIP graph: K replays, nothing else in the loop
    handle = rt.capture(lambda: graphs.run(cfg, rt, dt, fused=True, ws=ws))
    for _ in range(3):
        rt.graph_launch(handle)
    rt.sync()
    t0 = time.perf_counter()
    for _ in range(steps):
        rt.graph_launch(handle)
    rt.sync()
    graph_wall = time.perf_counter() - t0
    # the shader clock while that graph replays back to back (the datasheet peaks assume 2.4 GHz; under sustained
    # matrix work the chip settles lower, by an amount that depends on the kernel and on the data)
    clock = rt.shader_clock_ghz(lambda: rt.graph_launch(handle), graph_wall * 1e3 / steps)
    rt.graph_destroy(handle)
    return dict(batch=batch, wall_s=wall, gpu_ms=gpu_ms, ms_per_step=wall * 1e3 / steps,
                samples_per_s=batch * steps / wall, kernels=rows, result=result,
                graph_replay=dict(ms_per_step=graph_wall * 1e3 / steps, samples_per_s=batch * steps / graph_wall,
                                  shader_clock_ghz=clock))


def run_training(rt, iters=20):
    """The training kernels at the sizes of the conv block and of the bandwidth configuration: gradients of the
    four convolutions (2 x the forward flop: input and filter gradient; the bias gradient's adds are not
    counted), ReLU gradient (12 B/elt), SGD step (20 B/elt) and 2x2 pooling gradient (9 B per input elt)."""
    rng = np.random.default_rng(0x7EA1)
    rows = []

    def timed(fn):
        for _ in range(3):
            fn()
        rt.event_record(0)
        for _ in range(iters):
            fn()
        rt.event_record(1)
        return rt.event_elapsed_ms(0, 1) / iters

    for xs, oc in [((32, 56, 56, 64), 64), ((32, 56, 56, 64), 128), ((32, 28, 28, 128), 128)]:
        x = rt.upload(rng.standard_normal(xs).astype(np.float32))
        f = rt.upload((rng.standard_normal((oc, 3, 3, xs[3])) / np.sqrt(9 * xs[3])).astype(np.float32))
        og = rt.upload(rng.standard_normal(xs[:3] + (oc,)).astype(np.float32))
        ig, fg, bg = rt.empty(xs), rt.empty(f.shape), rt.empty((oc,))
        ms = timed(lambda: rt.conv2dGrad(x, f, og, (3, 3), (1, 1), (1, 1, 1, 1), out=(ig, fg, bg)))
        flop = 2.0 * 2.0 * xs[0] * xs[1] * xs[2] * oc * 9 * xs[3]
        rows.append(rate(dict(op="conv2dGrad", shape=f"{list(xs)}*{list(f.shape)}", ms=ms, flop=flop)))
        for t in (x, f, og, ig, fg, bg):
            t.free()
    n = 256 * 32 * 32 * 256
    a, b = rt.upload(rng.standard_normal(n).astype(np.float32)), rt.upload(rng.standard_normal(n).astype(np.float32))
    c = rt.empty((n,))
    rows.append(rate(dict(op="reluGrad", shape=f"[{n}]", ms=timed(lambda: rt.reluGrad(a, b, out=c)), bytes=12.0 * n)))
    mom = rt.upload(np.zeros(n, np.float32))
    rows.append(rate(dict(op="sgd", shape=f"[{n}]", ms=timed(lambda: rt.sgd(a, b, mom, 0.01, 0.001, 0.9, 32)), bytes=20.0 * n)))
    x4 = a.reshape(256, 32, 32, 256)
    og = rt.upload(rng.standard_normal((256, 16, 16, 256)).astype(np.float32))
    rows.append(rate(dict(op="maxpoolGrad", shape="[256, 32, 32, 256] 2x2/2",
                          ms=timed(lambda: rt.maxpoolGrad(x4, og, (2, 2), (2, 2), out=c)), bytes=9.0 * n)))
    return rows


def run_resnet50(rt, workspace, batch=32, iters=20):
    """The import path at a real workload (reference: test/importer/testResnetImport.cpp:19-51): ResNet-50 as the Caffe2
    model zoo stores it, with synthetic weights (25.6 M parameters), written as a pair of .pb files, imported by
    Caffe2Importer, fused, emitted by the HIP generator, built and run as one HIP graph per batch: `ms_per_batch` is
    the program's own timer over `iters` replays.  Beside it, per class of layer, the layers of that class timed
    through the C ABI as the program calls them (fused epilogues; average over back-to-back launches): what share
    of the matrix or HBM peak each class reaches."""
    import shutil
    import subprocess
    import tempfile
    from swcompiler_amd.caffe2_files import enc_net, make_resnet50
    swc = os.path.join(ROOT, "swcompiler_amd", "swc")
    gen = os.path.join(swc, "test", "bin", "genGraphs")
    if not os.path.exists(gen) or shutil.which("g++") is None:
        return dict(error="genGraphs is not built or there is no g++ here")
    predict, init, w = make_resnet50()
    out = dict(model="ResNet-50, Caffe2 model-zoo structure, synthetic weights, 224 x 224 x 3, fp32", batch=batch,
               parameters=int(sum(v.size for v in w.values())))
    work = tempfile.mkdtemp(prefix="swc_resnet50_")
    try:
        open(os.path.join(work, "predict_net.pb"), "wb").write(enc_net("resnet50", predict, packed=True))
        open(os.path.join(work, "init_net.pb"), "wb").write(enc_net("resnet50_init", init, packed=True))
        np.random.default_rng(11).standard_normal((batch, 224, 224, 3)).astype(np.float32).tofile(os.path.join(work, "data.bin"))
        libdir = os.path.join(ROOT, "swcompiler_amd")
        subprocess.run([gen, "caffe2@224", "hip", str(batch), str(iters), "graph"], cwd=work, check=True, capture_output=True, timeout=120)
        subprocess.run(["g++", "-std=c++11", "-O2", "-I", os.path.join(ROOT, "include"), "Graph.cpp", "-L", libdir,
                        "-Wl,-rpath," + libdir, "-lswc_hip", "-o", "net_hip.bin"], cwd=work, check=True, capture_output=True, timeout=120)
        rt.sync()
        res = subprocess.run([os.path.join(work, "net_hip.bin")], cwd=work, check=True, capture_output=True, text=True, timeout=300).stdout
        ms = float(res.split("swc_time_ms_per_iter")[1].split()[0])
        out.update(ms_per_batch=ms, samples_per_s=batch / ms * 1e3)
    except Exception as e:
        out["error"] = f"{type(e).__name__}: {str(e)[:300]}"
    finally:
        shutil.rmtree(work, ignore_errors=True)

    # ---- the layers by class, as the generated program calls them
    def timed(fn, n=10):
        for _ in range(2):
            fn()
        rt.event_record(0)
        for _ in range(n):
            fn()
        rt.event_record(1)
        return rt.event_elapsed_ms(0, 1) / n

    rng = np.random.default_rng(5)
    shape = {"gpu_0/data": (224, 224, 3)}
    need = rt.gemm_workspace_bytes(batch, 1000, 2048)
    for op in predict:   # one scratch buffer for the layers of this leg, as the generated program sets one
        if op["type"] == "Conv":
            src, (oc, ic, k) = shape[op["input"][0]], w[op["input"][1]].shape[:3]
            s, pad = op["arg"]["stride"], op["arg"]["pad"]
            need = max(need, rt.conv2d_workspace_bytes((batch,) + src, (oc, k, k, ic), (s, s), (pad,) * 4))
            shape[op["output"][0]] = ((src[0] + 2 * pad - k) // s + 1,) * 2 + (oc,)
        elif op["type"] in ("MaxPool", "AveragePool"):
            src, a = shape[op["input"][0]], op["arg"]
            shape[op["output"][0]] = ((src[0] + 2 * a.get("pad", 0) - a["kernel"]) // a["stride"] + 1,) * 2 + (src[2],)
        else:
            shape[op["output"][0]] = shape[op["input"][0]]
    scratch = rt.empty((need // 4 + 64,))
    rt.set_workspace(scratch)
    shape = {"gpu_0/data": (224, 224, 3)}
    relu_after, summed = set(), set()
    for op in predict:
        if op["type"] == "Relu":
            relu_after.add(op["input"][0])
        if op["type"] == "Sum":
            summed.add(op["input"][0])
    classes, seen, total_flop = {}, {}, 0.0

    def add(cls, ms, flop=0.0, nbytes=0.0):
        c = classes.setdefault(cls, dict(layers=0, ms=0.0, flop=0.0, bytes=0.0))
        c["layers"] += 1
        c["ms"] += ms
        c["flop"] += flop
        c["bytes"] += nbytes

    for op in predict:
        a, src = op.get("arg", {}), shape[op["input"][0]]
        if op["type"] == "Conv":
            oc, ic, k = w[op["input"][1]].shape[:3]
            s, pad = a["stride"], a["pad"]
            oh = (src[0] + 2 * pad - k) // s + 1
            name = op["output"][0]
            shape[name] = (oh, oh, oc)
            bn = name + "_bn"
            key = (src, oc, k, s, bn in relu_after, bn in summed)
            flop = 2.0 * batch * oh * oh * oc * ic * k * k
            total_flop += flop
            if key not in seen:
                x = rt.upload(rng.standard_normal((batch,) + src).astype(np.float32))
                f = rt.upload((rng.standard_normal((oc, k, k, ic)) * np.sqrt(2.0 / (ic * k * k))).astype(np.float32))
                b = rt.upload(np.zeros(oc, np.float32))
                par = [rt.upload(rng.uniform(0.5, 1.5, oc).astype(np.float32)) for _ in range(4)]
                y = rt.empty((batch, oh, oh, oc))
                res = rt.upload(rng.standard_normal((batch, oh, oh, oc)).astype(np.float32)) if key[5] else None
                fn = lambda: rt.conv2d(x, f, b, (k, k), (s, s), (pad,) * 4, bn=par, eps=1e-5, relu=key[4] or key[5],   # noqa: E731
                                       residual=res, out=y)
                seen[key] = (timed(fn), rt.last_kernel())
                for t in [x, f, b, y] + par + ([res] if res is not None else []):
                    t.free()
            cls = "conv 7x7 stride 2 (first layer)" if k == 7 else f"conv {k}x{k}" + (f" stride {s}" if s > 1 else "")
            add(cls, seen[key][0], flop=flop)
        elif op["type"] in ("MaxPool", "AveragePool"):
            k, s, pad = a["kernel"], a["stride"], a.get("pad", 0)
            oh = (src[0] + 2 * pad - k) // s + 1
            shape[op["output"][0]] = (oh, oh, src[2])
            x = rt.upload(rng.standard_normal((batch,) + src).astype(np.float32))
            y = rt.empty((batch, oh, oh, src[2]))
            pool = rt.maxpool if op["type"] == "MaxPool" else rt.avgpool
            ms = timed(lambda: pool(x, (k, k), (s, s), (pad,) * 4, out=y))
            add(f"{'max' if op['type'] == 'MaxPool' else 'average'} pooling {k}x{k} stride {s}", ms, nbytes=4.0 * (x.size + y.size))
            x.free(), y.free()
        elif op["type"] == "FC":
            n, kdim = w[op["input"][1]].shape
            x, wt, b = rt.upload(rng.standard_normal((batch, kdim)).astype(np.float32)), rt.upload(rng.standard_normal((kdim, n)).astype(np.float32)), rt.upload(np.zeros(n, np.float32))
            y = rt.empty((batch, n))
            ms = timed(lambda: rt.fcbias(x, wt, b, softmax=True, out=y))
            add("FC 2048 -> 1000 + softmax", ms, flop=2.0 * batch * n * kdim, nbytes=4.0 * (kdim * n + n + batch * (kdim + n)))
            total_flop += 2.0 * batch * n * kdim
            shape[op["output"][0]] = src
            for t in (x, wt, b, y):
                t.free()
        else:
            shape[op["output"][0]] = src
    rt.set_workspace(workspace)
    scratch.free()
    table = []
    for cls, c in classes.items():
        row = dict(layer_class=cls, layers=c["layers"], ms=c["ms"])
        if c["flop"] and not cls.startswith("FC"):
            row.update(flop=c["flop"], tflops=c["flop"] / c["ms"] / 1e9, frac=c["flop"] / c["ms"] / 1e9 / PEAK_TFLOPS_FP32_MFMA, bound="mfma")
        else:   # pools, and the FC of 32 rows (one pass over its 8 MB of weights)
            row.update(bytes=c["bytes"], gbs=c["bytes"] / c["ms"] / 1e6, frac=c["bytes"] / c["ms"] / 1e6 / PEAK_HBM_GBS, bound="hbm")
        table.append(row)
    out["layer_classes"] = table
    out["flop_per_batch"] = total_flop
    out["layers_ms_sum"] = sum(c["ms"] for c in classes.values())
    out["conv_shapes"] = [dict(input=list(k[0]), oc=k[1], k=k[2], stride=k[3], relu=k[4], residual=k[5], ms=ms, kernel=name,
                               frac=2.0 * batch * ((k[0][0] - 1) // k[3] + 1) ** 2 * k[1] * k[0][2] * k[2] ** 2 / ms / 1e9 / PEAK_TFLOPS_FP32_MFMA)
                          for k, (ms, name) in seen.items()]
    if "ms_per_batch" in out:
        out["tflops"] = total_flop / out["ms_per_batch"] / 1e9
        out["frac_of_mfma_peak"] = out["tflops"] / PEAK_TFLOPS_FP32_MFMA
    return out


def run_bn_pool_separately(rt, graphs, iters=20):
    """BN+ReLU and max-pool of the bandwidth configuration as two launches (the target emits one fused call,
    which is what that configuration's step times): the two kernels' own rates against the HBM roofline."""
    t = graphs.make_inputs(5)
    x = rt.upload(t["p"])
    bn = [rt.upload(t[f"bn_{k}"]) for k in ("mean", "var", "scale", "bias")]
    h, y = rt.empty(x.shape), rt.empty((x.shape[0], x.shape[1] // 2, x.shape[2] // 2, x.shape[3]))
    rows = []
    for op, fn, nbytes in (("batchnormalization", lambda: rt.batchnormalization(x, *bn, graphs.EPS, relu=True, out=h),
                            8.0 * x.size),
                           ("maxpool", lambda: rt.maxpool(h, (2, 2), (2, 2), out=y), 4.0 * x.size + 4.0 * y.size)):
        for _ in range(3):
            fn()
        rt.event_record(0)
        for _ in range(iters):
            fn()
        rt.event_record(1)
        rows.append(rate(dict(op=op, shape=str(list(x.shape)), ms=rt.event_elapsed_ms(0, 1) / iters, bytes=nbytes)))
    for a in [x, h, y] + bn:
        a.free()
    return rows


def clock_report(rt):
    """--clocks: the shader clock (GHz) the chip holds under single kernels in a loop, by operand distribution: the
    4096^3 product and the three cfg4 convolution shapes.  One JSON line; not part of the benchmark line."""
    rng = np.random.default_rng(0)

    def timed(fn, n):
        for _ in range(3):
            fn()
        rt.sync()
        rt.event_record(0)
        for _ in range(n):
            fn()
        rt.event_record(1)
        rt.sync()
        return rt.event_elapsed_ms(0, 1) / n

    kinds = [("normal", lambda s: rng.standard_normal(s)), ("relu(normal)", lambda s: np.maximum(rng.standard_normal(s), 0)),
             ("ones", lambda s: np.ones(s))]
    rows = [dict(work="idle", clock_ghz=rt.shader_clock_ghz(lambda: None, 1.0))]
    b = rt.upload((rng.standard_normal((4096, 4096)) / 64).astype(np.float32))
    c = rt.empty((4096, 4096))
    for name, make in kinds:
        a = rt.upload(make((4096, 4096)).astype(np.float32))
        fn = lambda: rt.matrixMatrixMul(a, b, out=c)   # noqa: E731
        ms = timed(fn, 10)
        rows.append(dict(work="gemm 4096^3", a=name, us=ms * 1e3, tflops=2 * 4096 ** 3 / ms / 1e9,
                         clock_ghz=rt.shader_clock_ghz(fn, ms), kernel=rt.last_kernel()))
        a.free()
    for idims, oc in (((32, 56, 56, 64), 64), ((32, 56, 56, 64), 128), ((32, 28, 28, 128), 128)):
        f = rt.upload((rng.standard_normal((oc, 3, 3, idims[3])) / np.sqrt(9 * idims[3])).astype(np.float32))
        bias = rt.upload(np.zeros(oc, np.float32))
        out = rt.empty(idims[:3] + (oc,))
        for name, make in kinds[:2]:
            x = rt.upload(make(idims).astype(np.float32))
            fn = lambda: rt.conv2d(x, f, bias, out=out, pads=(1, 1, 1, 1), relu=True)   # noqa: E731
            ms = timed(fn, 20)
            rows.append(dict(work=f"conv {list(idims)} -> {oc}, 3x3", input=name, us=ms * 1e3,
                             tflops=2.0 * np.prod(idims[:3]) * oc * 9 * idims[3] / ms / 1e9,
                             clock_ghz=rt.shader_clock_ghz(fn, ms), kernel=rt.last_kernel()))
            x.free()
    return dict(shader_clock=rows, datasheet_clock_ghz=2.4)


def cpu_baselines(graphs, rows=64):
    """The reference's CPU kernels (the unfused call sequence its generator emits, one thread, g++ -std=c++11 -O2,
    src/codegen/MakefileBuilder.h:34) on the buffers of every configuration: the whole batch, three timed
    iterations, for the MLP, LeNet and the bandwidth chain; one iteration for the conv block (about 10 s); the
    first `rows` rows of the wide MLP's batch, whose whole batch would take about 11 minutes."""
    from oracle import binding
    if binding.ref_available():
        be, kind = binding.load_ref(), "reference"
    else:
        be, kind = binding.load_oracle(), "port"
    out, results = {}, {}
    for cfg, iters in ((1, 3), (2, 1), (3, 3), (4, 1), (5, 3)):
        t = graphs.make_inputs(cfg)
        batch = graphs.batch_of(cfg, t)
        sample = f"the whole batch of {batch}, {iters} timed iteration{'s' if iters > 1 else ''}"
        if cfg == 2:
            t["x"] = np.ascontiguousarray(t["x"][:rows])
            sample = f"first {rows} of the {batch} rows of the same batch, one iteration"
            batch = rows
        times = []
        for _ in range(iters):
            t0 = time.perf_counter()
            results[f"cfg{cfg}"] = graphs.run(cfg, be, t, fused=False)
            times.append(time.perf_counter() - t0)
        dt = min(times)
        out[f"cfg{cfg}"] = dict(value=batch / dt, unit="samples/s", cores=1, kind=kind, seconds=dt,
                                seconds_all=times,
                                sample=sample + "; the whole graph as the reference emits it (one kernels.h call per "
                                       f"op node), one thread, g++ -std=c++11 -O2; {os.cpu_count()} host cpus visible")
    return out, results


def distance(got, want):
    """Measured distance between the device's and the reference's result of one graph output (the definitions of
    tests/util.py and tests/test_parity_report.py): strict_on_significant = max |g-r|/|r| over the outputs with
    |r| >= 1e-3 max|r|; floored = max |g-r| / max(|r|, 1e-3 max|r|) over all outputs; max_norm = max|g-r| / max|r|."""
    g, r = np.asarray(got, np.float64).ravel(), np.asarray(want, np.float64).ravel()
    top = float(np.max(np.abs(r)))
    big = np.abs(r) >= 1e-3 * top
    diff = np.abs(g - r)
    same = bool(np.array_equal(np.ascontiguousarray(got, np.float32).view(np.uint32), np.ascontiguousarray(want, np.float32).view(np.uint32)))
    return dict(strict_on_significant=float(np.max(diff[big] / np.abs(r[big]))),
                floored=float(np.max(diff / np.maximum(np.abs(r), 1e-3 * top))),
                max_norm=float(np.max(diff)) / top, bit_exact=same, outputs=int(r.size))


def parity_report(device, reference, cpu_rows):
    """Per configuration: the distances between what the timed (fused) graphs computed on the GPU and what the
    reference's own kernels computed from the same buffers in the cpu_baseline leg, with the bar each is held to.
    Softmax outputs (cfg1-3, cfg5a) and BN+ReLU+max-pool (cfg5c): 1e-4 strict on the significant outputs and floored;
    add+ReLU (cfg5b): bit-exact; the conv block (cfg4: four chained contractions of K = 576-1152 on N(0,1) data, each
    followed by BN and ReLU): 1e-4 in the max norm — the per-layer bars are held by the tests."""
    report, failed = {}, []
    for name in sorted(reference):
        got, want = device[name], reference[name]
        if name == "cfg2":
            got = got[:cpu_rows]
        if isinstance(want, dict):
            rows = {k: distance(got[k], want[k]) for k in sorted(want)}
            rows["a"]["bar"], rows["b"]["bar"], rows["c"]["bar"] = "strict, floored < 1e-4", "bit-exact", "strict, floored < 1e-4"
            ok = (rows["a"]["strict_on_significant"] < 1e-4 and rows["a"]["floored"] < 1e-4 and rows["b"]["bit_exact"] and
                  rows["c"]["strict_on_significant"] < 1e-4 and rows["c"]["floored"] < 1e-4)
            entry = dict(outputs=rows, ok=ok)
        elif name == "cfg4":
            entry = distance(got, want)
            entry["bar"] = "max_norm < 1e-4"
            entry["ok"] = entry["max_norm"] < 1e-4
        else:
            entry = distance(got, want)
            entry["bar"] = "strict_on_significant, floored < 1e-4"
            entry["ok"] = entry["strict_on_significant"] < 1e-4 and entry["floored"] < 1e-4
        if name == "cfg2":
            entry["rows"] = f"the first {cpu_rows} of the batch's 4096 rows"
        if not entry["ok"]:
            failed.append(name)
        report[name] = entry
    return report, failed


def bench_workspace(rt, graphs):
    """One scratch buffer for every op this harness runs: the maximum of the library's size queries over the FC
    and convolution shapes of the five configurations and the training-kernel leg."""
    need = 0
    for m, n, k in ((8, 512, 784), (8, 10, 512), (4096, 4096, 784), (4096, 4096, 4096), (4096, 10, 4096),
                    (256, 500, 800), (256, 10, 500)):
        need = max(need, rt.gemm_workspace_bytes(m, n, k))
    p1 = (1, 1, 1, 1)
    convs = [((256, 28, 28, 1), (20, 5, 5, 1), (0,) * 4), ((256, 12, 12, 20), (50, 5, 5, 20), (0,) * 4),
             ((32, 56, 56, 64), (64, 3, 3, 64), p1), ((32, 56, 56, 64), (128, 3, 3, 64), p1),
             ((32, 28, 28, 128), (128, 3, 3, 128), p1)]
    for xs, fs, pads in convs:
        need = max(need, rt.conv2d_workspace_bytes(xs, fs, (1, 1), pads))
    for xs, fs, pads in convs[:2] + convs[3:]:   # the layers that pool in their epilogue
        need = max(need, rt.conv2d_maxpool_workspace_bytes(xs, fs, (1, 1), pads, ((2, 2), (2, 2))))
    for xs, fs, pads in convs[2:]:
        need = max(need, rt.conv2dGrad_workspace_bytes(xs, fs, (1, 1), pads))
    if not need:
        return None
    ws = rt.empty((need // 4 + 64,))
    rt.set_workspace(ws)
    return ws


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=10)
    ap.add_argument("--headline-only", action="store_true", help="skip the other configurations")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--cpu-rows", type=int, default=64)
    ap.add_argument("--calibrate", action="store_true",
                    help="also launch relu_f on 2^26 floats three times: a plain 256 MiB-in/256 MiB-out pass whose "
                         "FETCH_SIZE/WRITE_SIZE readings calibrate the counters for the traffic figures")
    ap.add_argument("--traffic-from", nargs=2, metavar=("FETCH_CSV", "WRITE_CSV"),
                    help="instead of the benchmark: write profiles/traffic.json from two rocprofv3 --pmc counter files")
    ap.add_argument("--no-resnet", action="store_true", help="skip the `resnet50_b32` leg (the only one that starts other programs)")
    ap.add_argument("--resnet50", action="store_true",
                    help="instead of the benchmark: only the `resnet50_b32` leg (the import path), printed as its own JSON line")
    ap.add_argument("--clocks", action="store_true",
                    help="instead of the benchmark: print the shader clock held under single kernels, by operand distribution")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py: this build runs on one GPU only (nothing is sharded); use --gpus 1")
    if args.traffic_from:
        traffic_from_counters(*args.traffic_from)
        return

    from swcompiler_amd import graphs
    from swcompiler_amd.hip import SwcHip
    rt = SwcHip(0, auto_workspace=False)   # ops fail rather than allocate: the buffer below must cover them all
    workspace = bench_workspace(rt, graphs)
    if args.clocks:
        print(json.dumps(clock_report(rt)))
        rt.sync()
        rt.set_workspace(None)
        return

    if args.resnet50:
        print(json.dumps(run_resnet50(rt, workspace)))
        rt.sync()
        rt.set_workspace(None)
        return

    if args.calibrate:
        x = rt.upload(np.ones(1 << 26, np.float32))
        y = rt.empty(x.shape)
        for _ in range(3):
            rt.relu(x, out=y)
        rt.sync()
        x.free()
        y.free()

    head = run_config(rt, graphs, 2, args.steps, args.warmup)
    device_results = {"cfg2": head.pop("result")}
    gemm = [r for r in head["kernels"] if r["op"] == "fcbias" and not r["shape"].endswith("x10")]
    flop = sum(r["flop"] for r in gemm)
    secs = sum(r["ms"] for r in gemm) * 1e-3
    achieved = flop / secs / 1e12
    # the kernel the roofline object names must be the one both large FC calls dispatched to in THIS run
    ran = []
    for x, w in ((rt.empty((4096, 784)), rt.empty((784, 4096))), (rt.empty((4096, 4096)), rt.empty((4096, 4096)))):
        rt.fcbias(x, w, None, relu=True)
        ran.append(rt.last_kernel())
    rt.sync()
    if any(name != ROOFLINE_KERNEL for name in ran):
        sys.exit(f"bench.py: the large FC layers ran on {ran}, not on ROOFLINE_KERNEL = {ROOFLINE_KERNEL}: "
                 f"update ROOFLINE_KERNEL and re-measure profiles/traffic.json before reporting a roofline")
    traffic, traffic_source = None, None
    tpath = os.path.join(ROOT, "profiles", "traffic.json")
    if os.path.exists(tpath):   # measured separately under rocprofv3 --pmc (a counter run cannot share the timed run)
        entry = json.load(open(tpath)).get(ROOFLINE_KERNEL, {})
        traffic_source = dict(file="profiles/traffic.json", **entry.get("measured", {}))
        if traffic_source.get("sources_sha256") == sources_sha256():
            traffic = entry.get("bytes_per_launch")
        else:   # the kernel's sources changed since its counters were read: no figure rather than a stale one
            traffic_source["stale"] = "the kernel's sources no longer hash to sources_sha256: re-measure (bench.py --traffic-from)"
    out = {
        "metric": "samples/s per graph; TFLOP/s (FC/conv) & GB/s (eltwise) vs MI355X roofline",
        "value": head["samples_per_s"], "unit": "samples/s", "n_gpus": 1, "steps": args.steps,
        "warmup": args.warmup, "ms_per_step": head["ms_per_step"], "higher_is_better": True,
        "scaling": "weak", "vs_baseline": None, "dtype": "f32", "data": "synthetic",
        "config": {"workload": "wide MLP: batch 4096x784 -> FC4096+ReLU -> FC4096+ReLU -> FC10 -> softmax, fp32 "
                               "(BASELINE.json configs[1]), fused epilogues",
                   "global_batch": head["batch"], "device": rt.device_name()},
        "roofline": {"bound": "mfma", "achieved": achieved, "peak": PEAK_TFLOPS_FP32_MFMA, "unit": "TFLOP/s",
                     "frac": achieved / PEAK_TFLOPS_FP32_MFMA, "traffic": traffic, "traffic_source": traffic_source,
                     "kernel": ROOFLINE_KERNEL + " (both launches per step: 4096x784x4096 and 4096x4096x4096)",
                     "flop_per_launch": flop / len(gemm), "avg_launch_ms": secs * 1e3 / len(gemm),
                     # for information, not part of frac: the clock the step ran at and the MFMA peak at that clock
                     "shader_clock_ghz": head["graph_replay"]["shader_clock_ghz"],
                     "peak_at_that_clock": PEAK_TFLOPS_FP32_MFMA * head["graph_replay"]["shader_clock_ghz"] / 2.4},
        "gpu_ms_per_step": head["gpu_ms"] / args.steps,
        "graph_replay": head["graph_replay"],
        "incl_transfers": with_transfers(rt, graphs, 2, max(5, min(args.steps, 20))),
        "kernels": head["kernels"],
    }
    if not args.headline_only:
        out["peaks_measured"] = measured_peaks(rt)
    if not args.headline_only:
        others = {}
        for cfg in (1, 3, 4, 5):
            steps = max(5, min(args.steps, 20))
            r = run_config(rt, graphs, cfg, steps, max(2, min(args.warmup, 5)))
            device_results[f"cfg{cfg}"] = r.pop("result")
            others[f"cfg{cfg}"] = dict(batch=r["batch"], samples_per_s=r["samples_per_s"], ms_per_step=r["ms_per_step"],
                                       gpu_ms_per_step=r["gpu_ms"] / steps, graph_replay=r["graph_replay"],
                                       kernels=r["kernels"])
        others["cfg5"]["kernels_unfused"] = run_bn_pool_separately(rt, graphs)
        others["training_kernels"] = dict(kernels=run_training(rt))
        if not args.no_resnet:
            others["resnet50_b32"] = run_resnet50(rt, workspace)
        out["configs"] = others
    failed = []
    if not args.no_cpu:
        cpu, reference = cpu_baselines(graphs, args.cpu_rows)
        if args.headline_only:
            reference = {"cfg2": reference["cfg2"]}
        report, failed = parity_report(device_results, reference, args.cpu_rows)
        out["parity"] = report["cfg2"]
        for name, entry in report.items():
            if name != "cfg2" and "configs" in out:
                out["configs"][name]["parity"] = entry
        out["cpu_baseline"] = cpu["cfg2"]
        for name, entry in cpu.items():
            if name != "cfg2" and "configs" in out:
                out["configs"][name]["cpu_baseline"] = entry
        out.setdefault("configs", {})["cfg2"] = dict(cpu_baseline=cpu["cfg2"], parity=report["cfg2"],
                                                     note="the headline workload: see the top level")
    rt.sync()
    rt.set_workspace(None)
    print(json.dumps(out))
    if failed:
        sys.exit(f"bench.py: the device results of {failed} are outside their parity bar (see `parity` in the line above)")


if __name__ == "__main__":
    main()
