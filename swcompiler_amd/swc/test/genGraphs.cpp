// Builds one of the benchmark graphs through the SWC API, compiles it for the
// CPU or the HIP target and writes Graph.cpp + G_Makefile into the current
// directory.  User-level code: only `SWC.h` and the DSL macros, in the style of
// the reference's test/engine/testEngineMLPInfer.cpp.
//
//   genGraphs <model> <cpu|hip> [batch] [time_iters] [nofuse|graph|prefetch|-] [snapshot]
//   model: mnist8 | mnist_loader | mlp_train | lenet_train | nchw | manual | caffe2[txt][@size[xchannels]] | cfg1 | cfg2 | cfg3 | cfg4 | cfg5a | cfg5b | cfg5c
//   mnist_loader: [batch] is the number of records in mnist_labels_images.bin
//   [snapshot] (training models): TrainingConfig::snapshot; the parameters then start from Xavier / zero
//   initialisers instead of files
//
// Every parameter/input tensor is initialised from "<name>.bin" in the
// directory the generated program runs in; outputs are dumped to "<name>.bin".
#include <cstdlib>
#include <iostream>
#include <string>

#include "SWC.h"

using namespace swc;
using namespace swc::op;
using namespace std;

static void fromFile(Tensor *t, const string &name) { t->setTensorInit(TensorInitType::FILE, name + ".bin"); }

// x -> FCBias(w,b) [-> Relu] -> returns the output tensor node
static TensorNode *fc(IRGraph *g, const string &name, TensorNode *x, size_t k, size_t n, bool relu) {
    auto *w = new TensorNode(name + "_w", new Tensor({k, n}));
    auto *b = new TensorNode(name + "_b", new Tensor({n}));
    fromFile(w->getTensor(), name + "_w");
    fromFile(b->getTensor(), name + "_b");
    auto *op = new OpNode(name, new MatrixMatrixFCBiasOp());
    op->exlinkUpperNode(x, w, b);
    auto *y = new TensorNode(name + "_out", new Tensor({x->getDims()[0], n}), op);
    g->pushTensorNode(w, b, y);
    g->pushOpNode(op);
    if (!relu) return y;
    auto *r = new OpNode(name + "_relu", new ReluOp());
    r->exlinkUpperNode(y);
    auto *z = new TensorNode(name + "_act", new Tensor({x->getDims()[0], n}), r);
    g->pushTensorNode(z);
    g->pushOpNode(r);
    return z;
}

static TensorNode *unary(IRGraph *g, const string &name, Op *op, TensorNode *x) {
    auto *o = new OpNode(name, op);
    o->exlinkUpperNode(x);
    auto *y = new TensorNode(name + "_out", new Tensor(new TensorShape(x->getDims())), o);
    g->pushOpNode(o);
    g->pushTensorNode(y);
    return y;
}

static TensorNode *conv(IRGraph *g, const string &name, TensorNode *x, size_t oc, size_t k, size_t pad) {
    const size_t ic = x->getDims()[3];
    auto *f = new TensorNode(name + "_f", new Tensor({oc, k, k, ic}));
    auto *b = new TensorNode(name + "_b", new Tensor({oc}));
    fromFile(f->getTensor(), name + "_f");
    fromFile(b->getTensor(), name + "_b");
    vector<size_t> kernels{k, k}, strides{1, 1}, pads{pad, pad, pad, pad};
    DYOP(c, Conv2dOp, kernels, strides, pads);
    c->setName(name);
    LINKUPPER(c, x, f, b);
    auto *y = new TensorNode(name + "_out", new Tensor({0}), c);   // shape filled in by initTensorNodes()
    g->pushTensorNode(f, b, y);
    g->pushOpNode(c);
    return y;
}

static TensorNode *bn(IRGraph *g, const string &name, TensorNode *x) {
    const size_t c = x->getDims().size() == 4 && x->getDims()[3] ? x->getDims()[3] : 0;
    TensorNode *p[4];
    const char *suffix[4] = {"_scale", "_bias", "_mean", "_var"};
    for (int i = 0; i < 4; ++i) {
        p[i] = new TensorNode(name + suffix[i], new Tensor({c}));
        fromFile(p[i]->getTensor(), name + suffix[i]);
        g->pushTensorNode(p[i]);
    }
    auto *o = new OpNode(name, new BatchNormalizationOp(1e-5f));
    o->exlinkUpperNode(x, p[0], p[1], p[2], p[3]);
    auto *y = new TensorNode(name + "_out", new Tensor({0}), o);
    g->pushOpNode(o);
    g->pushTensorNode(y);
    return y;
}

static TensorNode *pool(IRGraph *g, const string &name, TensorNode *x) {
    vector<size_t> kernels{2, 2}, strides{2, 2}, pads{0, 0, 0, 0};
    auto *o = new OpNode(name, new MaxPoolOp(kernels, strides, pads));
    o->exlinkUpperNode(x);
    auto *y = new TensorNode(name + "_out", new Tensor({0}), o);
    g->pushOpNode(o);
    g->pushTensorNode(y);
    return y;
}

static TensorNode *lazyUnary(IRGraph *g, const string &name, Op *op, TensorNode *x) {
    auto *o = new OpNode(name, op);
    o->exlinkUpperNode(x);
    auto *y = new TensorNode(name + "_out", new Tensor({0}), o);
    g->pushOpNode(o);
    g->pushTensorNode(y);
    return y;
}

int main(int argc, char **argv) {
    if (argc < 3) {
        cerr << "usage: genGraphs <model> <cpu|hip> [batch] [time_iters] [nofuse|graph|prefetch]\n";
        return 2;
    }
    string model = argv[1];
    // "mnist_loader+labels": the data-loader model with the label batch among the displayed tensors
    const bool show_labels = model == "mnist_loader+labels";
    if (show_labels) model = "mnist_loader";
    const string target = argv[2];
    const size_t batch = argc > 3 ? strtoul(argv[3], nullptr, 10) : 0;
    const size_t iters = argc > 4 ? strtoul(argv[4], nullptr, 10) : 0;
    const bool nofuse = argc > 5 && string(argv[5]) == "nofuse";
    const bool prefetch = argc > 5 && string(argv[5]) == "prefetch";   // (implies graph)
    const bool useGraph = prefetch || (argc > 5 && string(argv[5]) == "graph");
    const size_t snapshot = argc > 6 ? strtoul(argv[6], nullptr, 10) : 0;   // training models: TrainingConfig::snapshot

    // mlp_train_label: the MLP with the label linked to a MatrixSoftmax node (the older way to end a training graph);
    // mlp_train_getnet: the same graph taken through getTrainNet and hand-run passes to codegen::Codegen, in the
    // style of the reference's test/testSnapshot.cpp (no Engine)
    const bool labelled = model == "mlp_train_label" || model == "mlp_train_getnet";
    const bool training = model == "mlp_train" || model == "lenet_train" || labelled;

    G(graph);
    TensorNode *out = nullptr;

    if (model == "mnist8") {
        // the reference's MNIST example: FCBias -> Tanh -> FCBias -> Softmax -> ArgMax(3) -> print
        TENSOR(data0, 8, 784);
        TENSOR(weight0, 784, 512);
        TENSOR(bias0, 512);
        INIT(data0, TensorInitType::FILE, "mnist_images_8.bin");
        INIT(weight0, TensorInitType::FILE, "mlp_weight0.bin");
        INIT(bias0, TensorInitType::FILE, "mlp_bias0.bin");
        OP(fc0, MatrixMatrixFCBiasOp);
        LINKUPPER(fc0, data0, weight0, bias0);
        TENSOR(data1, 8, 512);
        LINKUPPER(data1, fc0);
        OP(tanh0, MatrixTanhOp);
        LINKUPPER(tanh0, data1);
        TENSOR(data2, 8, 512);
        LINKUPPER(data2, tanh0);
        TENSOR(weight1, 512, 10);
        TENSOR(bias1, 10);
        INIT(weight1, TensorInitType::FILE, "mlp_weight1.bin");
        INIT(bias1, TensorInitType::FILE, "mlp_bias1.bin");
        OP(fc1, MatrixMatrixFCBiasOp);
        LINKUPPER(fc1, data2, weight1, bias1);
        TENSOR(data3, 8, 10);
        LINKUPPER(data3, fc1);
        OP(softmax, MatrixSoftmaxOp);
        LINKUPPER(softmax, data3);
        TENSOR(data4, 8, 10);
        LINKUPPER(data4, softmax);
        auto *argmax_o = new OpNode("argmax", new ArgMaxOp(3));
        argmax_o->exlinkUpperNode(data4);
        auto *top3_t = new TensorNode("top3", new Tensor({8, 3}, DataType::Int32_t), argmax_o);
        auto *print_o = new OpNode("print", new DebugOp());
        print_o->exlinkUpperNode(top3_t);
        GpT(graph, data0, weight0, bias0, data1, data2, weight1, bias1, data3, data4, top3_t);
        GpO(graph, fc0, tanh0, fc1, softmax, argmax_o, print_o);
        graph->addLogicalOutNodes(data4, top3_t);   // dump the probabilities and the top-3 table
    } else if (model == "mnist8_subgraphs") {
        // The reference's route to a GPU (test/cuda/testGPUInfer.cpp, test/old/testGraphPartition.cpp): the first
        // layer of the MNIST example is cut out into two nested graphs, one per half of the batch, each labelled
        // for a GPU of its own, and a plain Codegen is asked for the CUDA target.  On this one-device target
        // (Config::hip, or SWC_TARGET=hip in the environment) both halves run on the one GPU.
        TENSOR(data0, 8, 784);
        TENSOR(weight0, 784, 512);
        TENSOR(bias0, 512);
        INIT(data0, TensorInitType::FILE, "mnist_images_8.bin");
        INIT(weight0, TensorInitType::FILE, "mlp_weight0.bin");
        INIT(bias0, TensorInitType::FILE, "mlp_bias0.bin");
        OP(fc0, MatrixMatrixFCBiasOp);
        LINKUPPER(fc0, data0, weight0, bias0);
        TENSOR(data1, 8, 512);
        LINKUPPER(data1, fc0);
        OP(tanh0, MatrixTanhOp);
        LINKUPPER(tanh0, data1);
        TENSOR(data2, 8, 512);
        LINKUPPER(data2, tanh0);
        TENSOR(weight1, 512, 10);
        TENSOR(bias1, 10);
        INIT(weight1, TensorInitType::FILE, "mlp_weight1.bin");
        INIT(bias1, TensorInitType::FILE, "mlp_bias1.bin");
        OP(fc1, MatrixMatrixFCBiasOp);
        LINKUPPER(fc1, data2, weight1, bias1);
        TENSOR(data3, 8, 10);
        LINKUPPER(data3, fc1);
        OP(softmax, MatrixSoftmaxOp);
        LINKUPPER(softmax, data3);
        TENSOR(data4, 8, 10);
        LINKUPPER(data4, softmax);
        auto *argmax_o = new OpNode("argmax", new ArgMaxOp(3));
        argmax_o->exlinkUpperNode(data4);
        auto *top3_t = new TensorNode("top3", new Tensor({8, 3}, DataType::Int32_t), argmax_o);
        auto *print_o = new OpNode("print", new DebugOp());
        print_o->exlinkUpperNode(top3_t);
        GpT(graph, data0, weight0, bias0, data1, data2, weight1, bias1, data3, data4, top3_t);
        GpO(graph, fc0, tanh0, fc1, softmax, argmax_o, print_o);
        graph->addLogicalOutNodes(data4, top3_t);

        if (!graph->buildSubGraphs(data0, data2, ParallelStrategy::SLICE, 0, 2)) {
            cerr << "buildSubGraphs failed" << endl;
            return 1;
        }
        graph->findInOut();
        graph->updateTopology();
        pass::Optimizer opt(graph);
        opt.runOptimizer();
        int dev = 0;
        for (int i = 0; i < graph->opNodeNum(); ++i) {
            auto *sub = dynamic_cast<SubGraphOp *>(graph->getOpNode(i)->getOp());
            if (!sub) continue;
            IRGraph *inner = sub->getGraph();
            // (buildSubGraphs has given the second slice's Scatter and Gather the element offsets of its rows: what the
            // reference's two-GPU example sets by hand, test/cuda/testGPUInfer.cpp:177-178, 205-206)
            inner->setDeviceLabel(Device(0, DeviceType::GPU, dev++));
            inner->findInOut();
            inner->updateTopology();
            opt.setGraph(inner);
            opt.runOptimizer();
        }
        Config config;
        config.cuda = true;
        config.cuda_stream = true;
        config.cublas = true;
        config.hip = target == "hip";   // (or SWC_TARGET=hip)
        config.dump_outputs = true;
        codegen::Codegen generator(graph, config);
        cout << generator.generate();
        return dev == 2 ? 0 : 1;
    } else if (model == "mnist_loader") {
        // the reference's test/engine/testEngineMLPInfer.cpp: batch loop over a record file,
        // FCBias -> Tanh -> FCBias -> Softmax -> ArgMax(1) -> Accuracy, counters printed at the end
        TENSOR(data0, 8, 784);
        TENSOR(weight0, 784, 512);
        TENSOR(bias0, 512);
        INIT(weight0, TensorInitType::FILE, "mlp_weight0.bin");
        INIT(bias0, TensorInitType::FILE, "mlp_bias0.bin");
        OP(fc0, MatrixMatrixFCBiasOp);
        LINKUPPER(fc0, data0, weight0, bias0);
        TENSOR(data1, 8, 512);
        LINKUPPER(data1, fc0);
        OP(tanh0, MatrixTanhOp);
        LINKUPPER(tanh0, data1);
        TENSOR(data2, 8, 512);
        LINKUPPER(data2, tanh0);
        TENSOR(weight1, 512, 10);
        TENSOR(bias1, 10);
        INIT(weight1, TensorInitType::FILE, "mlp_weight1.bin");
        INIT(bias1, TensorInitType::FILE, "mlp_bias1.bin");
        OP(fc1, MatrixMatrixFCBiasOp);
        LINKUPPER(fc1, data2, weight1, bias1);
        TENSOR(data3, 8, 10);
        LINKUPPER(data3, fc1);
        Tensor *labelt = new Tensor({8}, DataType::Int32_t);
        TensorNode *label = new TensorNode("selected", labelt);
        OP(softmax, MatrixSoftmaxOp);
        LINKUPPER(softmax, data3);
        TENSOR(data4, 8, 10);
        LINKUPPER(data4, softmax);
        auto *argmax_o = new OpNode("argmax", new ArgMaxOp(1));
        argmax_o->exlinkUpperNode(data4);
        auto *top1_t = new TensorNode("top1", new Tensor({8, 1}, DataType::Int32_t), argmax_o);
        OP(accuracy_o, AccuracyOp);
        LINKUPPER(accuracy_o, top1_t, label);
        auto *accuracy_t = new TensorNode("accur", new Tensor({1, 2}, DataType::Int32_t), accuracy_o);
        accuracy_t->getTensor()->setTensorInit(TensorInitType::CONSTANT, 0);
        GpT(graph, data0, weight0, bias0, data1, data2, weight1, bias1, data3, data4, label, top1_t, accuracy_t);
        GpO(graph, fc0, tanh0, fc1, softmax, argmax_o, accuracy_o);
        graph->setInferDataNodes(label, data0);
        graph->addDisplayTensorNodes(accuracy_t);
        if (show_labels) graph->addDisplayTensorNodes(label);   // the display block then reads the loader's host buffer
    } else if (training) {
        // Training programs in the style of the reference's test/engine/testEngineLenetDistTrain.cpp (one process,
        // no MPI): the inference graph ends in MatrixSoftmaxWithLoss, the parameters are marked for training, and
        // Config::train_mode lets Engine::compile add the gradient ops and the SGD updates.  [batch] = records in
        // mnist_labels_images.bin; mini-batches of 8; every parameter starts from "<name>.bin".
        const size_t mb = 8;
        auto param = [&](const string &name, Tensor *t) {
            auto *n = new TensorNode(name, t);
            // (only tensors that start from an initialiser are part of a snapshot, as in the reference)
            if (!snapshot) fromFile(t, name);
            else if (t->getNDim() == 1) t->setTensorInit(TensorInitType::ZERO);
            else t->setTensorInit(TensorInitType::XAVIER, (float)(t->size() / t->getDim(t->getNDim() == 2 ? 1 : 0)));
            n->setTraining(1);
            graph->pushTensorNode(n);
            return n;
        };
        auto apply = [&](const string &name, Op *o, std::initializer_list<TensorNode *> ins) {
            auto *opn = new OpNode(name, o);
            for (TensorNode *i : ins) opn->exlinkUpperNode(i);
            auto *y = new TensorNode(name + "_out", new Tensor({0}), opn);
            graph->pushOpNode(opn);
            graph->pushTensorNode(y);
            return y;
        };
        TensorNode *data, *h;
        if (model == "mlp_train" || labelled) {
            data = new TensorNode("data0", new Tensor({mb, 784}));
            graph->pushTensorNode(data);
            h = apply("fc0", new MatrixMatrixFCBiasOp(), {data, param("fc0_w", new Tensor({784, 64})), param("fc0_b", new Tensor({64}))});
            h = apply("tanh0", new MatrixTanhOp(), {h});
            h = apply("fc1", new MatrixMatrixFCBiasOp(), {h, param("fc1_w", new Tensor({64, 10})), param("fc1_b", new Tensor({10}))});
        } else {
            data = new TensorNode("data0", new Tensor({mb, 28, 28, 1}));
            graph->pushTensorNode(data);
            vector<size_t> ck{5, 5}, cs{1, 1}, cp{2, 2, 2, 2}, pk{3, 3}, ps{3, 3}, pp{0, 0, 0, 0};
            h = apply("conv0", new Conv2dOp(ck, cs, cp), {data, param("conv0_w", new Tensor({16, 5, 5, 1})), param("conv0_b", new Tensor({16}))});
            h = apply("pool0", new MaxPoolOp(pk, ps, pp), {h});
            h = apply("relu0", new ReluOp(), {h});
            h = apply("conv1", new Conv2dOp(ck, cs, cp), {h, param("conv1_w", new Tensor({16, 5, 5, 16})), param("conv1_b", new Tensor({16}))});
            h = apply("pool1", new MaxPoolOp(pk, ps, pp), {h});
            h = apply("relu1", new ReluOp(), {h});
            h = apply("fc0", new MatrixMatrixFCBiasOp(), {h, param("fc0_w", new Tensor({144, 10})), param("fc0_b", new Tensor({10}))});
        }
        auto *label = new TensorNode("selected", new Tensor({mb}, DataType::Int32_t));
        auto *loss_op = new OpNode("softmax", labelled ? static_cast<Op *>(new MatrixSoftmaxOp()) : new MatrixSoftmaxWithLossOp());
        loss_op->exlinkUpperNode(h, label);
        auto *prob = new TensorNode("prob", new Tensor({0}), loss_op);
        graph->pushOpNode(loss_op);
        graph->pushTensorNode(label, prob);
        if (labelled) {
            graph->initTensorNodes();
            graph->setTrainDataNodes(label, data);
            graph->addDisplayTensorNodes(prob);
        } else {
            auto *loss = new TensorNode("loss", new Tensor({1}), loss_op);
            graph->pushTensorNode(loss);
            graph->initTensorNodes();
            graph->setTrainDataNodes(label, data);
            graph->addDisplayTensorNodes(loss);
        }
    } else if (model == "manual") {
        // placement written out by hand, the way the reference's test/cuda/testGPUInfer.cpp does it:
        // device twins, ScatterOp / GatherOp nodes, Label::setDeviceLabel, run-once parameter uploads,
        // and the code generator injected with Engine::setCodegenerator — no Config::hip, no placement pass
        const size_t b = batch ? batch : 16;
        const Device gpu0(0, DeviceType::GPU, 0);
        TENSOR(x, b, 64);
        TENSOR(w, 64, 24);
        TENSOR(bias, 24);
        INIT(x, TensorInitType::FILE, "x.bin");
        INIT(w, TensorInitType::FILE, "w.bin");
        INIT(bias, TensorInitType::FILE, "bias.bin");
        TENSOR(x_d, b, 64);
        TENSOR(w_d, 64, 24);
        TENSOR(bias_d, 24);
        OP(up_x, ScatterOp);
        OP(up_w, ScatterOp);
        OP(up_b, ScatterOp);
        up_w->setRunOnce();
        up_b->setRunOnce();
        LINKUPPER(up_x, x);
        LINKUPPER(x_d, up_x);
        LINKUPPER(up_w, w);
        LINKUPPER(w_d, up_w);
        LINKUPPER(up_b, bias);
        LINKUPPER(bias_d, up_b);
        OP(fc, MatrixMatrixFCBiasOp);
        LINKUPPER(fc, x_d, w_d, bias_d);
        TENSOR(y_d, b, 24);
        LINKUPPER(y_d, fc);
        OP(act, MatrixTanhOp);
        LINKUPPER(act, y_d);
        TENSOR(z_d, b, 24);
        LINKUPPER(z_d, act);
        OP(down, GatherOp);
        LINKUPPER(down, z_d);
        TENSOR(z, b, 24);
        LINKUPPER(z, down);
        for (IRNode *n : {(IRNode *)x_d, (IRNode *)w_d, (IRNode *)bias_d, (IRNode *)y_d, (IRNode *)z_d, (IRNode *)up_x,
                          (IRNode *)up_w, (IRNode *)up_b, (IRNode *)fc, (IRNode *)act, (IRNode *)down})
            n->getLabel()->setDeviceLabel(gpu0);
        GpT(graph, x, w, bias, x_d, w_d, bias_d, y_d, z_d, z);
        GpO(graph, up_x, up_w, up_b, fc, act, down);
        graph->findInOut();
        graph->updateTopology();
        Config config;
        config.dump_outputs = true;
        graph->setConfig(config);
        Engine engine(graph);
        engine.compile();   // CPU-target passes: FCBias is lowered to MatrixMatrixMul + MatrixVectorAdd, on the GPU label
        engine.setCodegenerator(new codegen::HipCodegen(graph, config));
        cout << engine.genCode();
        return 0;
    } else if (model == "nchw") {
        // an NCHW-trained block at the import boundary: data NCHW -> NHWC, filter OIHW -> OHWI
        // (the reference's importer inserts TransposeOp(NCHW2NHWC) the same way,
        // src/importer/Caffe2Importer.cpp:220-229), conv + relu + average pool, result back to NCHW
        const size_t b = batch ? batch : 2;
        auto *x = new TensorNode("x", new Tensor({b, 8, 12, 12}, DataType::Float_t, layout_nchw));
        auto *w = new TensorNode("w", new Tensor({16, 8, 3, 3}, DataType::Float_t, layout_nchw));
        auto *cb = new TensorNode("cb", new Tensor({16}));
        fromFile(x->getTensor(), "x");
        fromFile(w->getTensor(), "w");
        fromFile(cb->getTensor(), "cb");
        auto *tx = new OpNode("x_to_nhwc", new TransposeOp(NCHW2NHWC));
        tx->exlinkUpperNode(x);
        auto *xh = new TensorNode("x_nhwc", new Tensor({0}), tx);
        auto *tw = new OpNode("w_to_ohwi", new TransposeOp(NCHW2NHWC));
        tw->exlinkUpperNode(w);
        auto *wh = new TensorNode("w_ohwi", new Tensor({0}), tw);
        vector<size_t> kernels{3, 3}, strides{1, 1}, pads{1, 1, 1, 1};
        DYOP(conv0, Conv2dOp, kernels, strides, pads);
        LINKUPPER(conv0, xh, wh, cb);
        auto *y = new TensorNode("conv0_out", new Tensor({0}), conv0);
        graph->pushTensorNode(x, w, cb, xh, wh, y);
        graph->pushOpNode(tx, tw, conv0);
        graph->initTensorNodes();
        TensorNode *h = lazyUnary(graph, "relu0", new ReluOp(), y);
        vector<size_t> pk{2, 2}, ps{2, 2}, pp{0, 0, 0, 0};
        auto *ap = new OpNode("avgpool0", new AvgPoolOp(pk, ps, pp));
        ap->exlinkUpperNode(h);
        auto *pooled = new TensorNode("avgpool0_out", new Tensor({0}), ap);
        auto *back = new OpNode("to_nchw", new TransposeOp(NHWC2NCHW));
        back->exlinkUpperNode(pooled);
        out = new TensorNode("y_nchw", new Tensor({0}), back);
        graph->pushTensorNode(pooled, out);
        graph->pushOpNode(ap, back);
    } else if (model == "cfg1" || model == "cfg2") {
        const bool wide = model == "cfg2";
        const size_t b = batch ? batch : (wide ? 4096 : 8), hidden = wide ? 4096 : 512;
        auto *x = new TensorNode("x", new Tensor({b, 784}));
        fromFile(x->getTensor(), "x");
        graph->pushTensorNode(x);
        TensorNode *h = fc(graph, "fc1", x, 784, hidden, true);
        if (wide) h = fc(graph, "fc2", h, hidden, hidden, true);
        h = fc(graph, wide ? "fc3" : "fc2", h, hidden, 10, false);
        out = unary(graph, "softmax", new MatrixSoftmaxOp(), h);
    } else if (model == "cfg3") {
        const size_t b = batch ? batch : 256;
        auto *x = new TensorNode("x", new Tensor({b, 28, 28, 1}));
        fromFile(x->getTensor(), "x");
        graph->pushTensorNode(x);
        TensorNode *h = conv(graph, "conv1", x, 20, 5, 0);
        graph->initTensorNodes();
        h = pool(graph, "pool1", lazyUnary(graph, "relu1", new ReluOp(), h));
        graph->initTensorNodes();
        h = conv(graph, "conv2", h, 50, 5, 0);
        h = pool(graph, "pool2", lazyUnary(graph, "relu2", new ReluOp(), h));
        graph->initTensorNodes();
        h = fc(graph, "fc1", h, 800, 500, true);   // 4-D input: read as [b, 4*4*50]
        h = fc(graph, "fc2", h, 500, 10, false);
        out = unary(graph, "softmax", new MatrixSoftmaxOp(), h);
    } else if (model == "cfg4") {
        const size_t b = batch ? batch : 32;
        auto *x = new TensorNode("x", new Tensor({b, 56, 56, 64}));
        fromFile(x->getTensor(), "x");
        graph->pushTensorNode(x);
        const size_t oc[4] = {64, 128, 128, 128};
        TensorNode *h = x;
        for (int i = 0; i < 4; ++i) {
            const string n = to_string(i + 1);
            h = conv(graph, "conv" + n, h, oc[i], 3, 1);
            graph->initTensorNodes();
            h = lazyUnary(graph, "relu" + n, new ReluOp(), bn(graph, "bn" + n, h));
            if (i == 1 || i == 3) h = pool(graph, "pool" + n, h);
            graph->initTensorNodes();
        }
        out = h;
    } else if (model == "cfg5a") {
        const size_t rows = batch ? batch : 65536;
        auto *x = new TensorNode("logits", new Tensor({rows, 1000}));
        fromFile(x->getTensor(), "logits");
        graph->pushTensorNode(x);
        out = unary(graph, "softmax", new MatrixSoftmaxOp(), x);
    } else if (model == "cfg5b" || model == "cfg5c") {
        const size_t b = batch ? batch : 256;
        auto *p = new TensorNode("p", new Tensor({b, 32, 32, 256}));
        fromFile(p->getTensor(), "p");
        graph->pushTensorNode(p);
        if (model == "cfg5b") {
            auto *q = new TensorNode("q", new Tensor({b, 32, 32, 256}));
            fromFile(q->getTensor(), "q");
            OP(add, ElementAddOp);
            LINKUPPER(add, p, q);
            auto *s = new TensorNode("sum", new Tensor({b, 32, 32, 256}), add);
            graph->pushTensorNode(q, s);
            graph->pushOpNode(add);
            out = unary(graph, "relu", new ReluOp(), s);
        } else {
            TensorNode *h = bn(graph, "bn", p);
            graph->initTensorNodes();
            h = lazyUnary(graph, "relu", new ReluOp(), h);
            out = pool(graph, "pool", h);
            graph->initTensorNodes();
        }
    } else if (model.rfind("caffe2", 0) == 0) {
        // the reference's test/importer/testResnetImport.cpp: the caller defines the data tensor in NHWC, the
        // network and its weights come from a Caffe2 predict_net / init_net pair in the current directory
        // (binary .pb, or .pbtxt for "caffe2txt"), ArgMax(3) + a Debug print follow the softmax.
        // "caffe2@64": images of 64 x 64 (default 12 x 12) with 3 channels; "caffe2@28x1": 28 x 28 with one.
        const size_t b = batch ? batch : 2;
        size_t hw = 12, channels = 3;
        if (model.find('@') != string::npos) {
            const string size = model.substr(model.find('@') + 1);
            hw = stoul(size);
            if (size.find('x') != string::npos) channels = stoul(size.substr(size.find('x') + 1));
            model = model.substr(0, model.find('@'));
        }
        if (model != "caffe2" && model != "caffe2txt") {
            cerr << "unknown model " << model << "\n";
            return 2;
        }
        vector<TensorNode *> udef;
        auto *data = new TensorNode("gpu_0/data", new Tensor({b, hw, hw, channels}));
        data->getTensor()->setTensorInit(TensorInitType::FILE, "data.bin");
        udef.push_back(data);
        const string ext = model == "caffe2" ? ".pb" : ".pbtxt";
        Caffe2Importer importer(graph, "predict_net" + ext, "init_net" + ext, udef, "weights");
        auto *softmax_t = static_cast<TensorNode *>(graph->getNodeByName("gpu_0/softmax"));
        if (!softmax_t) {
            cerr << "gpu_0/softmax not found\n";
            return 2;
        }
        auto *argmax_o = new OpNode("argmax", new ArgMaxOp(3));
        argmax_o->exlinkUpperNode(softmax_t);
        auto *top3_t = new TensorNode("top3", new Tensor({b, 3}, DataType::Int32_t), argmax_o);
        auto *print_o = new OpNode("print", new DebugOp());
        print_o->exlinkUpperNode(top3_t);
        graph->pushOpNode(argmax_o, print_o);
        graph->pushTensorNode(top3_t);
        graph->addLogicalOutNodes(softmax_t, top3_t);
    } else {
        cerr << "unknown model " << model << "\n";
        return 2;
    }
    (void)out;

    graph->initTensorNodes();
    graph->findInOut();
    graph->updateTopology();

    Config config;
    config.hip = target == "hip";
    config.hip_fusion = !nofuse;
    config.time_iters = iters;
    config.hip_graph = useGraph;
    config.hip_prefetch = prefetch;
    config.dump_outputs = true;
    if (training) {
        config.train_mode = true;
        config.train_config.optimizer = "sgd";
        config.train_config.lr = 0.01f;
        config.train_config.decay = 0.001f;
        config.train_config.momentum = 0.9f;
        config.train_config.batch = 8;
        config.train_config.train_data_file = "mnist_labels_images.bin";
        config.train_config.label_bytes = BytesProto::ONE_BYTE_AS_INT;
        config.train_config.data_bytes = BytesProto::FOUR_BYTES_AS_FLOAT;
        config.train_config.train_data_samples = batch;
        config.train_config.max_epoch = 2;
        config.train_config.display = 4;
        config.train_config.snapshot = snapshot;
    }
    if (model == "mnist_loader") {
        config.use_dataloader = true;
        config.dataloader_src = "mnist_labels_images.bin";
        config.label_bytes = BytesProto::ONE_BYTE_AS_INT;
        config.data_bytes = BytesProto::FOUR_BYTES_AS_FLOAT;
        config.dataloader_samples = batch;
        config.display = batch / 8;   // print once, after the last mini-batch
    }
    graph->setConfig(config);

    if (model == "mlp_train_getnet") {
        IRGraph *net = getTrainNet(graph, config.train_config);
        net->setTrainDataNodes(static_cast<TensorNode *>(net->getNodeByName("selected")),
                               static_cast<TensorNode *>(net->getNodeByName("data0")));
        net->addDisplayTensorNodes(static_cast<TensorNode *>(net->getNodeByName("prob")));
        net->updateTopology();
        pass::RenamingNodePass renaming(net);
        pass::LabelingPass labeling(net);
        pass::LoweringPass lowering(net);
        pass::PassManager manager;
        manager.add(&renaming);
        manager.add(&labeling);
        manager.add(&lowering);
        manager.add(&labeling);
        manager.run();
        for (int i = 0; i < net->tensorNodeNum(); ++i)   // what the program leaves behind: the trained parameters
            if (net->getTensorNode(i)->getTraining()) net->getTensorNode(i)->getLabel()->setIsOut(1);
        codegen::Codegen generator(net, config);
        cout << generator.generate();
        return 0;
    }

    Engine engine(graph);
    engine.compile();
    string code = engine.genCode();
    cout << code;
    return 0;
}
