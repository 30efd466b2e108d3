// Self-checking unit tests of the graph IR and the passes (no code is generated).
// Exit status 0 = all checks passed; prints the failing check otherwise.
#include <cstdlib>
#include <iostream>

#include "SWC.h"

using namespace swc;
using namespace swc::op;
using namespace swc::pass;
using namespace std;

static int failures = 0;
#define CHECK(cond)                                                                  \
    do {                                                                             \
        if (!(cond)) {                                                               \
            cerr << __FILE__ << ":" << __LINE__ << ": CHECK failed: " #cond << endl; \
            ++failures;                                                              \
        }                                                                            \
    } while (0)

static int countOps(IRGraph *g, const string &type) {
    int n = 0;
    for (int i = 0; i < g->opNodeNum(); ++i) n += g->getOpNode(i)->getOp()->getOpName() == type;
    return n;
}

static void testTopologyAndShapes() {
    TENSOR(x, 4, 10, 10, 3);
    TENSOR(f, 8, 3, 3, 3);
    TENSOR(b, 8);
    vector<size_t> k{3, 3}, s{2, 2}, p{1, 1, 1, 1};
    DYOP(conv, Conv2dOp, k, s, p);
    LINKUPPER(conv, x, f, b);
    auto *y = new TensorNode("y", new Tensor({0}), conv);
    vector<size_t> pk{2, 2}, ps{2, 2}, pp{0, 0, 0, 0};
    DYOP(pool, MaxPoolOp, pk, ps, pp);
    LINKUPPER(pool, y);
    auto *z = new TensorNode("z", new Tensor({0}), pool);
    G(g);
    GpT(g, x, f, b, y, z);
    GpO(g, conv, pool);
    g->initTensorNodes();
    g->findInOut();
    g->updateTopology();
    // (10 + 1 + 1 - 3) / 2 + 1 = 5 ; pooled (5 - 2) / 2 + 1 = 2
    CHECK((y->getDims() == vector<size_t>{4, 5, 5, 8}));
    CHECK((z->getDims() == vector<size_t>{4, 2, 2, 8}));
    CHECK(y->getTensor()->getMemLayoutTag() == "nhwc");
    CHECK(g->inNodeNum() == 3 && g->outNodeNum() == 1 && g->getOutNode(0) == z);
    CHECK(g->topologyNum() == 5 && conv->topologyId() == 1 && z->topologyId() == 4);
    CHECK(g->getNodeByName("pool") == pool && g->getNodeByName("nope") == nullptr);
    IRGraph *c = g->clone();
    CHECK(c->tensorNodeNum() == 5 && c->opNodeNum() == 2 && c->topologyNum() == 5);
    CHECK(c->getTensorNode(0) != x && c->getTensorNode(0)->getTensor() != x->getTensor());
    auto *cconv = static_cast<OpNode *>(c->getNodeByName("conv"));
    CHECK(cconv->parentNum() == 3 && cconv->getParentNode(1)->name() == "f");
}

static void testLoweringAndRenaming() {
    TENSOR(x, 8, 4, 4, 2);   // rank 4: FC views it as [8, 32]
    TENSOR(w, 32, 16);
    TENSOR(b, 16);
    OP(fc, MatrixMatrixFCBiasOp);
    LINKUPPER(fc, x, w, b);
    TENSOR(y, 8, 16);
    LINKUPPER(y, fc);
    G(g);
    GpT(g, x, w, b, y);
    GpO(g, fc);
    g->findInOut();
    g->updateTopology();
    Config cpu;
    g->setConfig(cpu);
    Engine e(g);
    e.compile();
    CHECK(countOps(g, "MatrixMatrixFCBias") == 0 && countOps(g, "MatrixMatrixMul") == 1);
    CHECK(countOps(g, "MatrixVectorAdd") == 1 && countOps(g, "Reshape") == 1);
    auto *mm = static_cast<OpNode *>(g->getNodeByName("fc_mm"));
    CHECK(mm && mm->getParentNode(0)->name() == "x_reshape" && mm->getParentNode(1) == w);
    CHECK(static_cast<TensorNode *>(mm->getParentNode(0))->getDims() == (vector<size_t>{8, 32}));
    CHECK(g->getNodeByName("fc_mm_out") != nullptr && y->getParentNode(0)->name() == "fc_add");
    CHECK(y->getLabel()->getIsOut() == 1);

    UniqueName un;
    CHECK(un("a/b.c-d") == "a_b_c_d" && un("a_b_c_d") == "a_b_c_d1" && un("a_b_c_d") == "a_b_c_d2");
}

static void testFusionAndPlacement() {
    TENSOR(x, 2, 8, 8, 4);
    TENSOR(f, 8, 3, 3, 4);
    TENSOR(cb, 8);
    x_Tensor->setTensorInit(TensorInitType::FILE, "x.bin");
    f_Tensor->setTensorInit(TensorInitType::FILE, "f.bin");
    cb_Tensor->setTensorInit(TensorInitType::ZERO);
    vector<size_t> k{3, 3}, s{1, 1}, p{1, 1, 1, 1};
    DYOP(conv, Conv2dOp, k, s, p);
    LINKUPPER(conv, x, f, cb);
    TENSOR(c, 2, 8, 8, 8);
    LINKUPPER(c, conv);
    TensorNode *bnp[4];
    const char *names[4] = {"scale", "bias", "mean", "var"};
    for (int i = 0; i < 4; ++i) {
        bnp[i] = new TensorNode(names[i], new Tensor({8}));
        bnp[i]->getTensor()->setTensorInit(TensorInitType::CONSTANT, 1);
    }
    DYOP(bn, BatchNormalizationOp, 1e-5f);
    LINKUPPER(bn, c, bnp[0], bnp[1], bnp[2], bnp[3]);
    TENSOR(n, 2, 8, 8, 8);
    LINKUPPER(n, bn);
    OP(relu, ReluOp);
    LINKUPPER(relu, n);
    TENSOR(r, 2, 8, 8, 8);
    LINKUPPER(r, relu);
    auto *print = new OpNode("print", new DebugOp());
    print->exlinkUpperNode(r);
    G(g);
    GpT(g, x, f, cb, c, bnp[0], bnp[1], bnp[2], bnp[3], n, r);
    GpO(g, conv, bn, relu, print);
    g->findInOut();
    g->updateTopology();
    Config hip;
    hip.hip = true;
    g->setConfig(hip);
    Engine e(g);
    e.compile();
    CHECK(countOps(g, "Conv2dBatchNorm") == 1 && countOps(g, "Conv2d") == 0);
    CHECK(countOps(g, "BatchNormalization") == 0 && countOps(g, "Relu") == 0);
    auto *fused = static_cast<OpNode *>(g->getNodeByName("conv"));
    CHECK(fused && fused->parentNum() == 7 && static_cast<Conv2dBatchNormOp *>(fused->getOp())->hasRelu());
    CHECK(fused->getParentNode(0)->name() == "x_dev" && fused->getParentNode(3)->name() == "scale_dev");
    CHECK(fused->getLabel()->getDeviceLabel().type == DeviceType::GPU);
    CHECK(countOps(g, "Scatter") == 7 && countOps(g, "Gather") == 1);
    for (int i = 0; i < g->opNodeNum(); ++i)
        if (g->getOpNode(i)->getOp()->getOpName() == "Scatter") CHECK(g->getOpNode(i)->isRunOnce());
    // the host op reads the gathered twin, the device tensor keeps its GPU label
    CHECK(print->getParentNode(0)->name() == "r_host" && r->getLabel()->getDeviceLabel().type == DeviceType::GPU);
    CHECK(print->getLabel()->getDeviceLabel().type == DeviceType::CPU);
}

static void testSubGraphs() {
    // x -> fc -> y -> tanh -> z -> relu -> r ; the part from x to z becomes nested graphs
    TENSOR(x, 8, 32);
    TENSOR(w, 32, 16);
    TENSOR(b, 16);
    OP(fc, MatrixMatrixFCBiasOp);
    LINKUPPER(fc, x, w, b);
    TENSOR(y, 8, 16);
    LINKUPPER(y, fc);
    OP(act, MatrixTanhOp);
    LINKUPPER(act, y);
    TENSOR(z, 8, 16);
    LINKUPPER(z, act);
    OP(relu, ReluOp);
    LINKUPPER(relu, z);
    TENSOR(r, 8, 16);
    LINKUPPER(r, relu);
    G(g);
    GpT(g, x, w, b, y, z, r);
    GpO(g, fc, act, relu);
    CHECK(g->extractSubGraph(r, x) == nullptr);   // x does not depend on r
    CHECK(g->buildSubGraphs(x, z, ParallelStrategy::SLICE, 0, 2));
    CHECK(countOps(g, "SubGraph") == 2 && countOps(g, "MatrixMatrixFCBias") == 0 && countOps(g, "Relu") == 1);
    CHECK(g->tensorNodeNum() == 5);               // x, w, b, z, r: y moved inside
    int seen = 0;
    for (int i = 0; i < g->opNodeNum(); ++i) {
        auto *sub = dynamic_cast<SubGraphOp *>(g->getOpNode(i)->getOp());
        if (!sub) continue;
        OpNode *node = g->getOpNode(i);
        CHECK(node->parentNum() == 3 && node->getParentNode(0) == x && node->childNum() == 1 && node->getChildNode(0) == z);
        IRGraph *in = sub->getGraph();
        CHECK(countOps(in, "Scatter") == 3 && countOps(in, "Gather") == 1 && countOps(in, "MatrixMatrixFCBias") == 1);
        auto *xs = static_cast<TensorNode *>(in->getNodeByName("x_sub"));
        auto *zs = static_cast<TensorNode *>(in->getNodeByName("z_sub"));
        CHECK(xs && zs && xs->getDims() == (vector<size_t>{4, 32}) && zs->getDims() == (vector<size_t>{4, 16}));
        auto *mirror = static_cast<TensorNode *>(in->getNodeByName("x"));
        CHECK(mirror && mirror->isExternal() && mirror->getTensor() == x->getTensor());
        in->setDeviceLabel(Device(0, DeviceType::GPU, seen));
        CHECK(mirror->getLabel()->getDeviceLabel().type == DeviceType::CPU);   // mirrors keep the outer device
        CHECK(xs->getLabel()->getDeviceLabel().id == seen);
        ++seen;
    }
    CHECK(seen == 2);
    CHECK(g->inlineSubGraphs(0) == 2);
    CHECK(countOps(g, "SubGraph") == 0 && countOps(g, "MatrixMatrixFCBias") == 2 && countOps(g, "Scatter") == 6);
    CHECK(z->parentNum() == 2 && z->getParentNode(0)->name() == "gather" && z->getParentNode(1)->name() == "gather");
    CHECK(x->childNum() == 2 && w->childNum() == 2);
    for (int i = 0; i < g->tensorNodeNum(); ++i) {
        const Device d = g->getTensorNode(i)->getLabel()->getDeviceLabel();
        CHECK(d.type == DeviceType::CPU || d.id == 0);   // every GPU label is the one device now
        CHECK(!g->getTensorNode(i)->isExternal());
    }
    CHECK(g->topologyNum() == 11);   // x, scatter, x_sub, fc, y, tanh, z_sub, gather, z, relu, r: one level each
}

static void testElimination() {
    TENSOR(x, 2, 3, 4, 5);
    auto *t1 = new OpNode("t1", new TransposeOp(NCHW2NHWC));
    t1->exlinkUpperNode(x);
    auto *m = new TensorNode("m", new Tensor({0}), t1);
    auto *t2 = new OpNode("t2", new TransposeOp(NHWC2NCHW));
    t2->exlinkUpperNode(m);
    auto *back = new TensorNode("back", new Tensor({0}), t2);
    OP(relu, ReluOp);
    LINKUPPER(relu, back);
    auto *y = new TensorNode("y", new Tensor({0}), relu);
    // a dead branch
    OP(dead, ReluOp);
    LINKUPPER(dead, x);
    auto *dz = new TensorNode("dz", new Tensor({0}), dead);
    G(g);
    GpT(g, x, m, back, y, dz);
    GpO(g, t1, t2, relu, dead);
    g->initTensorNodes();
    CHECK((m->getDims() == vector<size_t>{2, 4, 5, 3}) && (back->getDims() == vector<size_t>{2, 3, 4, 5}));
    g->findInOut();
    g->updateTopology();
    SETOUT(g, y);
    dz->getLabel()->setIsOut(0);
    ElimTransposePass et(g);
    et.run();
    CHECK(et.cancelledCount() == 1 && relu->getParentNode(0) == x);
    EliminationPass dce(g);
    dce.run();
    CHECK(g->opNodeNum() == 1 && g->getOpNode(0) == relu);
    CHECK(g->tensorNodeNum() == 2 && g->getNodeByName("m") == nullptr && g->getNodeByName("dz") == nullptr);
    // a non-inverse pair stays
    TENSOR(a, 2, 3, 4, 5);
    auto *u1 = new OpNode("u1", new TransposeOp(NCHW2NHWC));
    u1->exlinkUpperNode(a);
    auto *am = new TensorNode("am", new Tensor({0}), u1);
    auto *u2 = new OpNode("u2", new TransposeOp(NCHW2NHWC));
    u2->exlinkUpperNode(am);
    auto *ab = new TensorNode("ab", new Tensor({0}), u2);
    OP(r2, ReluOp);
    LINKUPPER(r2, ab);
    auto *ay = new TensorNode("ay", new Tensor({0}), r2);
    G(h);
    GpT(h, a, am, ab, ay);
    GpO(h, u1, u2, r2);
    h->initTensorNodes();
    ElimTransposePass et2(h);
    et2.run();
    CHECK(et2.cancelledCount() == 0 && r2->getParentNode(0) == ab);
}

// A residual block as an importer builds it: weights stored [oC,iC,kh,kw] behind a Transpose, conv -> BN ->
// Sum with the block's input -> Relu; then ArgMax and Accuracy.
static void testResidualBlockAndCounters() {
    TENSOR(x, 2, 6, 6, 8);
    auto *w = new TensorNode("w", new Tensor({8, 8, 3, 3}, DataType::Float_t, layout_nchw));
    w->getTensor()->setTensorInit(TensorInitType::FILE, "w.bin");
    auto *tw = new OpNode("w_T_op", new TransposeOp(NCHW2NHWC));
    tw->exlinkUpperNode(w);
    auto *wT = new TensorNode("w_T", new Tensor({8, 3, 3, 8}), tw);
    TENSOR(cb, 8);
    TENSOR(scale, 8);
    TENSOR(beta, 8);
    TENSOR(mean, 8);
    TENSOR(var, 8);
    vector<size_t> k{3, 3}, st{1, 1}, p{1, 1, 1, 1};
    DYOP(conv, Conv2dOp, k, st, p);
    LINKUPPER(conv, x, wT, cb);
    TENSOR(y, 2, 6, 6, 8);
    LINKUPPER(y, conv);
    auto *bn = new OpNode("bn", new BatchNormalizationOp(1e-5f));
    bn->exlinkUpperNode(y, scale, beta, mean, var);
    TENSOR(z, 2, 6, 6, 8);
    LINKUPPER(z, bn);
    OP(sum, ElementAddOp);
    LINKUPPER(sum, x, z);   // the convolution's result is the SECOND summand here
    auto *s1 = new TensorNode("z", z->getTensor(), sum);   // written in place, as Caffe2's Sum does
    OP(relu, ReluOp);
    LINKUPPER(relu, s1);
    auto *r = new TensorNode("z", z->getTensor(), relu);
    TENSOR(fw, 288, 10);
    TENSOR(fb, 10);
    OP(fc, MatrixMatrixFCBiasOp);
    LINKUPPER(fc, r, fw, fb);
    TENSOR(logits, 2, 10);
    LINKUPPER(logits, fc);
    auto *am = new OpNode("argmax", new ArgMaxOp(1));
    am->exlinkUpperNode(logits);
    auto *top1 = new TensorNode("top1", new Tensor({2, 1}, DataType::Int32_t), am);
    auto *label = new TensorNode("label", new Tensor({2}, DataType::Int32_t));
    OP(acc, AccuracyOp);
    LINKUPPER(acc, top1, label);
    auto *counters = new TensorNode("counters", new Tensor({1, 2}, DataType::Int32_t), acc);
    counters->getTensor()->setTensorInit(TensorInitType::CONSTANT, 0);
    G(g);
    GpT(g, x, w, wT, cb, scale, beta, mean, var, y, z, s1, r, fw, fb, logits, top1, label, counters);
    GpO(g, tw, conv, bn, sum, relu, fc, am, acc);
    g->findInOut();
    g->updateTopology();
    Config hip;
    hip.hip = true;
    g->setConfig(hip);
    Engine e(g);
    e.compile();
    CHECK(countOps(g, "Conv2dAdd") == 1 && countOps(g, "ElementAdd") + countOps(g, "ElementAddRelu") + countOps(g, "Relu") == 0);
    OpNode *fused = nullptr, *trans = nullptr, *accuracy = nullptr;
    for (int i = 0; i < g->opNodeNum(); ++i) {
        const string t = g->getOpNode(i)->getOp()->getOpName();
        if (t == "Conv2dAdd") fused = g->getOpNode(i);
        if (t == "Transpose") trans = g->getOpNode(i);
        if (t == "Accuracy") accuracy = g->getOpNode(i);
    }
    CHECK(fused && fused->parentNum() == 8 && fused->getParentNode(7)->name() == "x_dev");
    auto *fop = static_cast<Conv2dAddOp *>(fused->getOp());
    CHECK(fop->hasBatchNorm() && fop->hasRelu() && fused->getChildNode(0) == r);
    // the weight's layout change runs once, after its upload; the data tensor's consumers stay per-iteration
    CHECK(trans && trans->isRunOnce() && wT->getTensor()->getTensorInitType() == TensorInitType::PARENTOP);
    CHECK(!fused->isRunOnce());
    // Accuracy runs on the device: labels get a device twin, the counters live there and have a host twin
    CHECK(accuracy && accuracy->getLabel()->getDeviceLabel().type == DeviceType::GPU);
    CHECK(accuracy->getParentNode(1)->name() == "label_dev" && counters->getLabel()->getDeviceLabel().type == DeviceType::GPU);
    CHECK(g->getNodeByName("counters_host") != nullptr && g->getNodeByName("top1_host") == nullptr);
}

// Config::train_mode: FCBias -> Tanh -> FCBias -> SoftmaxWithLoss grows gradient ops, SGD nodes that rewrite
// their parameter in place, and (after lowering and elimination) no gradient for the data.
static void testAutodiff() {
    TENSOR(x, 8, 20);
    TENSOR(w0, 20, 16);
    TENSOR(b0, 16);
    TENSOR(w1, 16, 10);
    TENSOR(b1, 10);
    for (TensorNode *p : {w0, b0, w1, b1}) p->setTraining(1);
    OP(fc0, MatrixMatrixFCBiasOp);
    LINKUPPER(fc0, x, w0, b0);
    TENSOR(h0, 8, 16);
    LINKUPPER(h0, fc0);
    OP(act, MatrixTanhOp);
    LINKUPPER(act, h0);
    TENSOR(h1, 8, 16);
    LINKUPPER(h1, act);
    OP(fc1, MatrixMatrixFCBiasOp);
    LINKUPPER(fc1, h1, w1, b1);
    TENSOR(logits, 8, 10);
    LINKUPPER(logits, fc1);
    auto *label = new TensorNode("label", new Tensor({8}, DataType::Int32_t));
    OP(lossop, MatrixSoftmaxWithLossOp);
    LINKUPPER(lossop, logits, label);
    TENSOR(prob, 8, 10);
    LINKUPPER(prob, lossop);
    TENSOR(loss, 1);
    LINKUPPER(loss, lossop);
    G(g);
    GpT(g, x, w0, b0, w1, b1, h0, h1, logits, label, prob, loss);
    GpO(g, fc0, act, fc1, lossop);
    g->findInOut();
    g->updateTopology();
    g->setTrainDataNodes(label, x);
    g->addDisplayTensorNodes(loss);
    Config cfg;
    cfg.train_mode = true;
    cfg.train_config.optimizer = "sgd";
    cfg.train_config.batch = 8;
    g->setConfig(cfg);
    Engine e(g);
    e.compile();
    CHECK(countOps(g, "SGD") == 4 && countOps(g, "MatrixSoftmaxWithLossGrad") == 1 && countOps(g, "MatrixTanhGrad") == 1);
    CHECK(countOps(g, "MatrixMatrixFCBiasGrad") == 0 && countOps(g, "BatchedReduceAdd") == 2);
    // forward: 2 products (FCBias is lowered on the CPU target); backward: dW twice, dX once (the data needs none)
    CHECK(countOps(g, "MatrixMatrixMul") == 5 && countOps(g, "Transpose") == 3);
    CHECK(g->getNodeByName("x_grad") == nullptr && g->getNodeByName("w0_grad") != nullptr);
    auto *sgd = static_cast<OpNode *>(g->getNodeByName("w0_sgd"));
    CHECK(sgd && sgd->parentNum() == 3 && sgd->getParentNode(0) == w0 && sgd->getParentNode(1)->name() == "w0_grad");
    auto *updated = static_cast<TensorNode *>(sgd->getChildNode(0));
    CHECK(updated != w0 && updated->getTensor() == w0->getTensor() && updated->getLabel()->getIsOut());
    auto *step = static_cast<SGDOp *>(sgd->getOp());
    CHECK(step->getLR() == 0.001f && step->getDecay() == 0.001f && step->getMomentum() == 0.9f && step->getBatch() == 8);
    // every SGD node comes after every reader of its parameter
    CHECK(sgd->topologyId() > static_cast<OpNode *>(g->getNodeByName("fc0_mm"))->topologyId());
}

int main() {
    testTopologyAndShapes();
    testLoweringAndRenaming();
    testFusionAndPlacement();
    testSubGraphs();
    testElimination();
    testResidualBlockAndCounters();
    testAutodiff();
    if (failures) {
        cerr << failures << " check(s) failed" << endl;
        return 1;
    }
    cout << "all pass checks ok" << endl;
    return 0;
}
