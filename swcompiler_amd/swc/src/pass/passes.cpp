#include "passes.h"

#include <cassert>
#include <cctype>
#include <cstdlib>
#include <set>
#include <unordered_map>
#include <unordered_set>

#include "../graphIR/OpNode.h"
#include "../graphIR/TensorNode.h"
#include "../op/ops.h"

namespace swc {
namespace pass {

using namespace swc::op;

void Optimizer::runOptimizer() {
    PassManager pm;
    LabelingPass labeling(_graph);
    LoweringPass lowering(_graph);
    pm.add(&labeling);
    pm.add(&lowering);
    pm.add(&labeling);
    pm.run();
}

// ------------------------------------------------------------------ labeling
void LabelingPass::run() {
    const Config cfg = _graph->getConfig();
    for (int i = 0; i < _graph->tensorNodeNum(); ++i) {
        TensorNode *t = _graph->getTensorNode(i);
        Label *l = t->getLabel();
        l->setNodeNameLabel(t->name());
        l->setTypeNameLabel("Tensor");
        if (t->getTensor()) {
            l->setTraining(t->getTraining());
            l->setTensorInitTypeLabel(t->getTensor()->getTensorInitType());
        }
    }
    for (int i = 0; i < _graph->opNodeNum(); ++i) {
        OpNode *o = _graph->getOpNode(i);
        Label *l = o->getLabel();
        l->setNodeNameLabel(o->name());
        const std::string type = o->getOp()->getOpName();
        l->setTypeNameLabel(type);
        if (!cfg.enable_lowering) continue;
        // FC without bias always becomes a plain GEMM.  FC with bias is split
        // into GEMM + bias-add only for targets without a fused kernel: the CPU
        // generator; MKL-DNN and the HIP target keep it whole.
        if (type == "MatrixMatrixFC" || type == "MatrixMatrixFCBiasGrad") l->setLowerMark();   // (no target has a kernel for the latter)
        else if (type == "MatrixMatrixFCBias" && !cfg.mkldnn && !cfg.hip) l->setLowerMark();
    }
}

// ------------------------------------------------------------------ lowering
void LoweringPass::run() {
    // lowering edits the op list, so collect first
    std::vector<OpNode *> marked;
    for (int i = 0; i < _graph->opNodeNum(); ++i)
        if (_graph->getOpNode(i)->getLabel()->getLowerMark()) marked.push_back(_graph->getOpNode(i));
    for (OpNode *o : marked) {
        o->getLabel()->clearLowerMark();
        o->getOp()->lowering(_graph, o);
    }
}

// ------------------------------------------------------------------ renaming
std::string UniqueName::operator()(const std::string &in) {
    assert(!in.empty());
    std::string base = in;
    for (char &c : base)
        if (c == '/' || c == '.' || c == '-') c = '_';
    std::string name = base;
    auto it = seen_.find(base);
    if (it != seen_.end())
        do name = base + std::to_string(++it->second);
        while (seen_.count(name));
    seen_[name] = 0;
    return name;
}

void RenamingNodePass::run() {
    for (int i = 0; i < _graph->tensorNodeNum(); ++i) {
        TensorNode *t = _graph->getTensorNode(i);
        t->setName(unique_(t->name()));
    }
    for (int i = 0; i < _graph->opNodeNum(); ++i) {
        OpNode *o = _graph->getOpNode(i);
        o->setName(unique_(o->name()));
    }
}

// --------------------------------------------------------------- elimination
void EliminationPass::run() {
    // live = everything from which an output-marked node is reachable
    std::unordered_set<IRNode *> live;
    std::vector<IRNode *> work;
    auto seed = [&](IRNode *n) {
        if (n->getLabel()->getIsOut() && live.insert(n).second) work.push_back(n);
    };
    for (int i = 0; i < _graph->tensorNodeNum(); ++i) seed(_graph->getTensorNode(i));
    for (int i = 0; i < _graph->opNodeNum(); ++i) seed(_graph->getOpNode(i));
    while (!work.empty()) {
        IRNode *n = work.back();
        work.pop_back();
        for (IRNode *p : n->getParentNodes())
            if (live.insert(p).second) work.push_back(p);
    }
    // every result of a live op stays, read or not: the op's emitter addresses its results by position
    for (int i = 0; i < _graph->opNodeNum(); ++i)
        if (live.count(_graph->getOpNode(i)))
            for (IRNode *c : _graph->getOpNode(i)->getChildNodes()) live.insert(c);
    std::vector<TensorNode *> deadT;
    std::vector<OpNode *> deadO;
    for (int i = 0; i < _graph->tensorNodeNum(); ++i)
        if (!live.count(_graph->getTensorNode(i))) deadT.push_back(_graph->getTensorNode(i));
    for (int i = 0; i < _graph->opNodeNum(); ++i)
        if (!live.count(_graph->getOpNode(i))) deadO.push_back(_graph->getOpNode(i));
    auto detach = [](IRNode *n) {
        while (n->parentNum()) n->destroyUpperNode(n->getParentNode(0));
        while (n->childNum()) n->getChildNode(0)->destroyUpperNode(n);
    };
    for (auto *t : deadT) {
        detach(t);
        _graph->delTensorNode(t);
    }
    for (auto *o : deadO) {
        detach(o);
        _graph->delOpNode(o);
    }
    _graph->findInOut();
    _graph->updateTopology();
}

// ------------------------------------------------------------------ autodiff
void AutodiffPass::getMethods(const std::string &method, float lr, float decay, float momentum, size_t batch) {
    std::string m = method;
    for (char &c : m) c = (char)std::tolower((unsigned char)c);
    if (m != "sgd") {
        SWLOG_ERROR << "AutodiffPass: optimizer \"" << method << "\" is not implemented (sgd)" << std::endl;
        std::abort();
    }
    lr_ = lr, decay_ = decay, momentum_ = momentum, batch_ = batch;
}

void AutodiffPass::show() const {
    SWLOG_INFO << "AutodiffPass: sgd, lr " << lr_ << ", decay " << decay_ << ", momentum " << momentum_ << ", batch "
               << batch_ << std::endl;
}

void AutodiffPass::run(IRGraph *graph_train) {
    if (graph_train) {
        _graph->copyTo(graph_train);
        _graph = graph_train;
    }
    run();
}

void AutodiffPass::run() {
    std::vector<IRNode *> order;
    for (int i = 0; i < _graph->topologyNum(); ++i)
        for (int j = 0; j < _graph->getNumInTopoLevel(i); ++j) order.push_back(_graph->getNodeInTopo(i, j));
    std::unordered_map<IRNode *, TensorNode *> gradOf;

    // gradient op with the given operands; one gradient tensor per operand of the forward op, in operand order
    auto addGrad = [&](OpNode *fwd, Op *gradOp, const std::vector<IRNode *> &operands) {
        auto *g = new OpNode(fwd->name() + "_grad", gradOp);
        for (IRNode *p : operands) g->exlinkUpperNode(p);
        _graph->pushOpNode(g);
        for (int i = 0; i < fwd->parentNum(); ++i) {
            auto *t = static_cast<TensorNode *>(fwd->getParentNode(i));
            auto *gt = new TensorNode(t->name() + "_grad", new Tensor(new TensorShape(t->getDims())), g);
            gradOf[t] = gt;
            _graph->pushTensorNode(gt);
        }
        ++gradOps_;
    };

    for (auto it = order.rbegin(); it != order.rend(); ++it) {
        IRNode *node = *it;
        if (node->nodeType() == TENSOR_NODE) {
            auto *t = static_cast<TensorNode *>(node);
            if (gradOf.count(t)) {
                if (!t->getTraining()) continue;
                auto *momT = new Tensor(new TensorShape(t->getDims()));
                momT->setTensorInit(TensorInitType::CONSTANT, 0.f);
                auto *mom = new TensorNode(t->name() + "_momentum", momT);
                auto *sgd = new OpNode(t->name() + "_sgd", new SGDOp(lr_, decay_, momentum_, batch_));
                sgd->exlinkUpperNode(t, gradOf[t], mom);
                auto *updated = new TensorNode(t->name(), t->getTensor(), sgd);   // the same Tensor: in place
                updated->setTraining(t->getTraining());
                _graph->pushOpNode(sgd);
                _graph->pushTensorNode(mom, updated);
                _graph->addLogicalOutNodes(updated);
                ++sgdOps_;
            } else if (t->childNum() == 0) {
                // an end point (loss, probabilities): its gradient exists by name only, no op computes or reads it
                gradOf[t] = new TensorNode(t->name() + "_grad", new Tensor(new TensorShape(t->getDims())));
            }
            continue;
        }
        auto *op = static_cast<OpNode *>(node);
        const std::string type = op->getOp()->getOpName();
        auto in = [&](int i) { return op->getParentNode(i); };
        auto outGrad = [&]() -> IRNode * {
            auto *out = static_cast<TensorNode *>(op->getChildNode(0));
            if (!gradOf.count(out)) {
                SWLOG_ERROR << "AutodiffPass: no gradient reaches the output of " << op->name() << std::endl;
                std::abort();
            }
            return gradOf[out];
        };
        if (type == "MatrixMatrixFCBias") {
            addGrad(op, new MatrixMatrixFCBiasGradOp(), {in(0), in(1), in(2), outGrad()});
        } else if (type == "MatrixTanh") {
            addGrad(op, new MatrixTanhGradOp(), {in(0), op->getChildNode(0), outGrad()});
        } else if (type == "Relu") {
            addGrad(op, new ReluGradOp(), {in(0), outGrad()});
        } else if (type == "MaxPool") {
            auto *mp = static_cast<MaxPoolOp *>(op->getOp());
            addGrad(op, new MaxPoolGradOp(mp->getKernels(), mp->getStrides(), mp->getPads()),
                    {in(0), op->getChildNode(0), outGrad()});
        } else if (type == "Conv2d") {
            auto *cv = static_cast<Conv2dOp *>(op->getOp());
            addGrad(op, new Conv2dGradOp(cv->getKernels(), cv->getStrides(), cv->getPads(), (int)cv->getGroup()),
                    {in(0), in(1), outGrad()});
        } else if (type == "TensorDescend") {   // tensorOps.cpp:25-85: the gradient is unfolded the way the input was folded
            auto *d = static_cast<TensorDescendOp *>(op->getOp());
            addGrad(op, new TensorAscendOp(d->getNDim(), d->getStart(), d->getEnd()), {outGrad()});
        } else if (type == "TensorAscend") {
            auto *a = static_cast<TensorAscendOp *>(op->getOp());
            addGrad(op, new TensorDescendOp(a->getNDim(), a->getStart(), a->getEnd()), {outGrad()});
        } else if (type == "MatrixSoftmaxWithLoss") {
            addGrad(op, new MatrixSoftmaxWithLossGradOp(), {in(1), op->getChildNode(0)});   // label, prob
        } else if (type == "MatrixSoftmax" && op->parentNum() == 2) {   // a label as second operand: the network's end
            addGrad(op, new MatrixSoftmaxGradOp(), {in(0), in(1), op->getChildNode(0), outGrad()});
        } else {
            SWLOG_ERROR << "AutodiffPass: no gradient for op type " << type << " (node " << op->name() << ")" << std::endl;
            std::abort();
        }
    }
    _graph->findInOut();
    _graph->updateTopology();
}

} // namespace pass

IRGraph *getTrainNet(IRGraph *graph, TrainingConfig &profile) {
    IRGraph *net = graph->clone();
    net->findInOut();
    net->updateTopology();
    pass::AutodiffPass autodiff(net);
    autodiff.getMethods("sgd", profile.lr, profile.decay, profile.momentum, profile.batch);
    autodiff.run();
    return net;
}

namespace pass {

// -------------------------------------------------------- transpose cancelling
void ElimTransposePass::run() {
    for (int i = 0; i < _graph->opNodeNum(); ++i) {
        OpNode *first = _graph->getOpNode(i);
        auto *t1 = dynamic_cast<TransposeOp *>(first->getOp());
        if (!t1 || first->parentNum() != 1 || first->childNum() != 1) continue;
        IRNode *source = first->getParentNode(0);
        IRNode *mid = first->getChildNode(0);
        const std::vector<size_t> a = t1->getShuffle();
        std::vector<IRNode *> readers(mid->getChildNodes());
        for (IRNode *r : readers) {
            if (r->nodeType() != OP_NODE) continue;
            auto *second = static_cast<OpNode *>(r);
            auto *t2 = dynamic_cast<TransposeOp *>(second->getOp());
            if (!t2 || second->childNum() != 1) continue;
            const std::vector<size_t> b = t2->getShuffle();
            bool inverse = a.size() == b.size();
            for (size_t k = 0; inverse && k < b.size(); ++k) inverse = b[k] < a.size() && a[b[k]] == k;
            if (!inverse) continue;
            IRNode *result = second->getChildNode(0);
            std::vector<IRNode *> users(result->getChildNodes());
            for (IRNode *u : users) result->replaceUseKeepOrder(u, source);
            ++cancelled_;
        }
    }
    _graph->findInOut();
    _graph->updateTopology();
}

// -------------------------------------------------------------------- fusion
namespace {

bool isType(IRNode *n, const char *type) {
    return n->nodeType() == OP_NODE && static_cast<OpNode *>(n)->getOp()->getOpName() == type;
}

// the op consuming `producer`'s only output, if that output has exactly one
// consumer, is not a graph output and the consumer has the wanted type
OpNode *soleConsumer(OpNode *producer, const char *type, IRGraph *g) {
    if (producer->childNum() != 1) return nullptr;
    IRNode *t = producer->getChildNode(0);
    if (t->childNum() != 1 || t->getLabel()->getIsOut()) return nullptr;
    for (IRNode *lo : g->getLogicalOutNodes())
        if (lo == t) return nullptr;
    IRNode *c = t->getChildNode(0);
    if (!isType(c, type) || c->getParentNode(0) != t) return nullptr;
    return static_cast<OpNode *>(c);
}

// Replaces producer -> mid -> consumer -> out by fusedNode -> out, where
// fusedNode takes producer's operands followed by consumer's operands 1.. .
void splice(IRGraph *g, OpNode *producer, OpNode *consumer, Op *fusedOp) {
    auto *mid = static_cast<TensorNode *>(producer->getChildNode(0));
    auto *out = static_cast<TensorNode *>(consumer->getChildNode(0));
    auto *fused = new OpNode(producer->name(), fusedOp);
    *fused->getLabel() = *producer->getLabel();
    fused->getLabel()->setTypeNameLabel(fusedOp->getOpName());
    std::vector<IRNode *> operands(producer->getParentNodes());
    for (int i = 1; i < consumer->parentNum(); ++i) operands.push_back(consumer->getParentNode(i));
    while (producer->parentNum()) producer->destroyUpperNode(producer->getParentNode(0));
    mid->destroyUpperNode(producer);
    while (consumer->parentNum()) consumer->destroyUpperNode(consumer->getParentNode(0));
    out->destroyUpperNode(consumer);
    for (IRNode *p : operands) fused->exlinkUpperNode(p);
    out->exlinkUpperNode(fused);
    g->delOpNode(producer);
    g->delOpNode(consumer);
    g->delTensorNode(mid);
    g->pushOpNode(fused);
}

// The ElementAdd / ElementAddRelu node that is the only reader of `producer`'s result (which is no graph output)
// and whose other operand is a different tensor; null if there is none, or while a Relu behind a plain
// ElementAdd is still to be merged into it.
OpNode *soleAddConsumer(OpNode *producer, IRGraph *g, IRNode *&other) {
    if (producer->childNum() != 1) return nullptr;
    IRNode *t = producer->getChildNode(0);
    if (t->childNum() != 1 || t->getLabel()->getIsOut()) return nullptr;
    for (IRNode *lo : g->getLogicalOutNodes())
        if (lo == t) return nullptr;
    IRNode *c = t->getChildNode(0);
    if (!(isType(c, "ElementAdd") || isType(c, "ElementAddRelu")) || c->parentNum() != 2) return nullptr;
    auto *add = static_cast<OpNode *>(c);
    other = add->getParentNode(0) == t ? add->getParentNode(1) : add->getParentNode(0);
    if (other == t) return nullptr;
    if (isType(c, "ElementAdd") && soleConsumer(add, "Relu", g)) return nullptr;
    return add;
}

// producer -> mid -> add(mid, other) -> out  becomes  fused(producer's operands..., other) -> out
void spliceAdd(IRGraph *g, OpNode *producer, OpNode *add, IRNode *other, Op *fusedOp) {
    auto *mid = static_cast<TensorNode *>(producer->getChildNode(0));
    auto *out = static_cast<TensorNode *>(add->getChildNode(0));
    auto *fused = new OpNode(producer->name(), fusedOp);
    *fused->getLabel() = *producer->getLabel();
    fused->getLabel()->setTypeNameLabel(fusedOp->getOpName());
    std::vector<IRNode *> operands(producer->getParentNodes());
    operands.push_back(other);
    while (producer->parentNum()) producer->destroyUpperNode(producer->getParentNode(0));
    mid->destroyUpperNode(producer);
    while (add->parentNum()) add->destroyUpperNode(add->getParentNode(0));
    out->destroyUpperNode(add);
    for (IRNode *p : operands) fused->exlinkUpperNode(p);
    out->exlinkUpperNode(fused);
    g->delOpNode(producer);
    g->delOpNode(add);
    g->delTensorNode(mid);
    g->pushOpNode(fused);
}

} // namespace

// The MaxPool that may move into the epilogue of the convolution `conv` feeding it: 2 x 2 windows, stride 2, no
// padding, over a convolution output with even height and width, and an input-channel count the MFMA tile kernels
// take as it is (a multiple of 4) — what swc_hip_conv2dFusedMaxpool_f does in one launch.
static OpNode *poolBehind(OpNode *conv, IRGraph *g) {
    OpNode *pool = soleConsumer(conv, "MaxPool", g);
    if (!pool) return nullptr;
    auto *mp = static_cast<MaxPoolOp *>(pool->getOp());
    const auto k = mp->getKernels(), s = mp->getStrides(), p = mp->getPads();
    if (k != std::vector<size_t>{2, 2} || s != std::vector<size_t>{2, 2}) return nullptr;
    for (size_t v : p)
        if (v) return nullptr;
    Tensor *y = static_cast<TensorNode *>(conv->getChildNode(0))->getTensor();
    Tensor *x = static_cast<TensorNode *>(conv->getParentNode(0))->getTensor();
    if (y->getNDim() != 4 || y->getDim(1) % 2 || y->getDim(2) % 2) return nullptr;
    // channel counts the tile kernels take as they are, or a first layer for the direct kernel (a short filter and up
    // to 20 output channels: a thread then holds a window's four pixels); any other layer would pool in a second
    // kernel anyway
    Tensor *f = static_cast<TensorNode *>(conv->getParentNode(1))->getTensor();
    const size_t taps = f->getNDim() == 4 ? f->getDim(1) * f->getDim(2) * f->getDim(3) : 0;
    const bool direct = taps && taps <= 128 && y->getDim(3) <= 20;
    if (x->getDim(3) % 4 && !direct) return nullptr;
    return pool;
}
static Op *pooledConv(Conv2dOp *conv, bool bn, float eps, bool relu, OpNode *pool) {
    auto *mp = static_cast<MaxPoolOp *>(pool->getOp());
    auto k = conv->getKernels(), s = conv->getStrides(), p = conv->getPads();
    return new Conv2dMaxPoolOp(k, s, p, bn, eps, relu, mp->getKernels(), mp->getStrides(), mp->getPads());
}

void HipFusionPass::run() {
    bool changed = true;
    while (changed) {
        changed = false;
        for (int i = 0; i < _graph->opNodeNum() && !changed; ++i) {
            OpNode *o = _graph->getOpNode(i);
            const std::string type = o->getOp()->getOpName();
            if (type == "MatrixMatrixFCBias") {
                if (OpNode *r = soleConsumer(o, "Relu", _graph)) {
                    splice(_graph, o, r, new MatrixMatrixFCBiasReluOp());
                    changed = true;
                } else if (OpNode *sm = soleConsumer(o, "MatrixSoftmax", _graph)) {
                    splice(_graph, o, sm, new MatrixMatrixFCBiasSoftmaxOp());
                    changed = true;
                }
            } else if (type == "Conv2d") {
                auto *conv = static_cast<Conv2dOp *>(o->getOp());
                auto k = conv->getKernels(), s = conv->getStrides(), p = conv->getPads();
                if (conv->getGroup() != 1) continue;
                if (OpNode *bn = soleConsumer(o, "BatchNormalization", _graph)) {
                    const float eps = static_cast<BatchNormalizationOp *>(bn->getOp())->getEpsilon();
                    splice(_graph, o, bn, new Conv2dBatchNormOp(k, s, p, eps, false));
                    changed = true;
                } else if (OpNode *r = soleConsumer(o, "Relu", _graph)) {
                    splice(_graph, o, r, new Conv2dWithActivationOp(k, s, p, SWC_ACTIVATION_RELU));
                    changed = true;
                } else if (IRNode *other = nullptr; OpNode *add = soleAddConsumer(o, _graph, other)) {
                    spliceAdd(_graph, o, add, other, new Conv2dAddOp(k, s, p, false, 0.f, isType(add, "ElementAddRelu")));
                    changed = true;
                } else if (OpNode *pool = poolBehind(o, _graph)) {
                    splice(_graph, o, pool, pooledConv(conv, false, 0.f, false, pool));
                    changed = true;
                }
            } else if (type == "Conv2dWithActivation") {
                auto *ca = static_cast<Conv2dWithActivationOp *>(o->getOp());
                if (ca->getGroup() != 1 || ca->getActivationType() != SWC_ACTIVATION_RELU) continue;
                if (OpNode *pool = poolBehind(o, _graph)) {
                    splice(_graph, o, pool, pooledConv(ca, false, 0.f, true, pool));
                    changed = true;
                }
            } else if (type == "Conv2dBatchNorm") {
                auto *cb = static_cast<Conv2dBatchNormOp *>(o->getOp());
                if (cb->hasRelu()) {
                    if (OpNode *pool = poolBehind(o, _graph)) {
                        splice(_graph, o, pool, pooledConv(cb, true, cb->getEpsilon(), true, pool));
                        changed = true;
                        ++fused_;
                    }
                    continue;
                }
                auto k = cb->getKernels(), s = cb->getStrides(), p = cb->getPads();
                if (OpNode *r = soleConsumer(o, "Relu", _graph)) {
                    splice(_graph, o, r, new Conv2dBatchNormOp(k, s, p, cb->getEpsilon(), true));
                    changed = true;
                } else if (IRNode *other = nullptr; OpNode *add = soleAddConsumer(o, _graph, other)) {
                    spliceAdd(_graph, o, add, other,
                              new Conv2dAddOp(k, s, p, true, cb->getEpsilon(), isType(add, "ElementAddRelu")));
                    changed = true;
                } else if (OpNode *pool = poolBehind(o, _graph)) {
                    splice(_graph, o, pool, pooledConv(cb, true, cb->getEpsilon(), false, pool));
                    changed = true;
                }
            } else if (type == "BatchNormalization") {
                if (OpNode *r = soleConsumer(o, "Relu", _graph)) {
                    const float eps = static_cast<BatchNormalizationOp *>(o->getOp())->getEpsilon();
                    splice(_graph, o, r, new BatchNormalizationReluOp(eps));
                    changed = true;
                }
            } else if (type == "BatchNormalizationRelu") {
                if (OpNode *pool = soleConsumer(o, "MaxPool", _graph)) {
                    auto *mp = static_cast<MaxPoolOp *>(pool->getOp());
                    const float eps = static_cast<BatchNormalizationReluOp *>(o->getOp())->getEpsilon();
                    splice(_graph, o, pool, new BatchNormReluMaxPoolOp(eps, mp->getKernels(), mp->getStrides(), mp->getPads()));
                    changed = true;
                }
            } else if (type == "ElementAdd") {
                if (OpNode *r = soleConsumer(o, "Relu", _graph)) {
                    splice(_graph, o, r, new ElementAddReluOp());
                    changed = true;
                }
            }
            if (changed) ++fused_;
        }
    }
    _graph->findInOut();
    _graph->updateTopology();
}

// ---------------------------------------------------------- device placement
bool DeviceMemoryLoweringPass::runsOnGpu(const std::string &t) {
    static const std::set<std::string> gpu = {
        "MatrixMatrixMul", "MatrixVectorAdd", "BatchedAdd", "MatrixMatrixFCBias", "MatrixMatrixFCBiasRelu",
        "MatrixMatrixFCBiasSoftmax", "Reshape", "TensorDescend", "TensorAscend", "MatrixTanh", "MatrixSoftmax", "ElementAdd", "ElementAddRelu", "Relu", "Dropout",
        "Conv2d", "Conv2dWithActivation", "Conv2dBatchNorm", "Conv2dAdd", "Conv2dMaxPool", "MaxPool", "AveragePool", "Transpose",
        "BatchNormalization",
        "BatchNormalizationRelu", "BatchNormReluMaxPool", "ArgMax", "Accuracy",
        "MatrixSoftmaxWithLoss", "MatrixSoftmaxWithLossGrad", "MatrixSoftmaxGrad", "BatchedReduceAdd", "MatrixTanhGrad", "ReluGrad",
        "MaxPoolGrad", "Conv2dGrad", "SGD"};
    return gpu.count(t) != 0;
}

void DeviceMemoryLoweringPass::run() {
    const Device gpu(0, DeviceType::GPU, device_);
    const Config cfg = _graph->getConfig();

    std::vector<OpNode *> ops;
    for (int i = 0; i < _graph->opNodeNum(); ++i) ops.push_back(_graph->getOpNode(i));

    // 1. label compute ops and what they produce
    for (OpNode *o : ops) {
        if (!runsOnGpu(o->getOp()->getOpName())) continue;
        o->getLabel()->setDeviceLabel(gpu);
        for (IRNode *c : o->getChildNodes()) c->getLabel()->setDeviceLabel(gpu);
    }
    auto onGpu = [&](IRNode *n) { return n->getLabel()->getDeviceLabel() == gpu; };

    std::vector<TensorNode *> tensors;
    for (int i = 0; i < _graph->tensorNodeNum(); ++i) tensors.push_back(_graph->getTensorNode(i));

    for (TensorNode *t : tensors) {
        if (!onGpu(t)) {
            // 2. host tensor read by GPU ops: device twin + Scatter
            std::vector<IRNode *> gpuReaders;
            for (IRNode *c : t->getChildNodes()) {
                // the mask operand of a Dropout node is not read at inference: it needs no device copy
                if (c->nodeType() == OP_NODE && static_cast<OpNode *>(c)->getOp()->getOpName() == "Dropout" &&
                    c->parentNum() > 1 && c->getParentNode(1) == t && c->getParentNode(0) != t)
                    continue;
                // (a Scatter node placed by hand IS the upload of this host tensor: its operand stays on the host)
                if (c->nodeType() == OP_NODE && static_cast<OpNode *>(c)->getOp()->getOpName() == "Scatter") continue;
                if (onGpu(c) && std::find(gpuReaders.begin(), gpuReaders.end(), c) == gpuReaders.end())
                    gpuReaders.push_back(c);
            }
            if (gpuReaders.empty()) continue;
            auto *twin = new TensorNode(t->name() + "_dev", t->getTensor()->clone());
            twin->getTensor()->setTensorInit(TensorInitType::NONE);
            twin->getLabel()->setDeviceLabel(gpu);
            auto *scatter = new OpNode(t->name() + "_h2d", new ScatterOp());
            scatter->getLabel()->setDeviceLabel(gpu);
            scatter->getLabel()->setTypeNameLabel("Scatter");
            const bool perIteration =
                cfg.train_mode ? (t == _graph->getTrainDataNode() || t == _graph->getTrainLabelNode())
                               : cfg.use_dataloader && (t == _graph->getInferDataNode() || t == _graph->getInferLabelNode());
            const bool parameter = t->parentNum() == 0 && !perIteration;
            if (parameter) {
                scatter->setRunOnce();
                twin->getTensor()->setTensorInit(TensorInitType::PARENTOP);
            }
            for (IRNode *reader : gpuReaders) t->replaceUseKeepOrder(reader, twin);
            // a device node that names the same Tensor (the parameter as an SGD node rewrites it in place) means
            // the device copy from now on
            for (TensorNode *other : tensors)
                if (other != t && other->getTensor() == t->getTensor() && onGpu(other)) other->setTensor(twin->getTensor());
            scatter->exlinkUpperNode(t);
            twin->exlinkUpperNode(scatter);
            _graph->pushOpNode(scatter);
            _graph->pushTensorNode(twin);
            ++scatters_;
        } else {
            // 3. GPU tensor that leaves the device: host twin + Gather
            std::vector<IRNode *> hostReaders;
            for (IRNode *c : t->getChildNodes()) {
                // (a Gather node placed by hand IS the download of this device tensor)
                if (c->nodeType() == OP_NODE && static_cast<OpNode *>(c)->getOp()->getOpName() == "Gather") continue;
                if (!onGpu(c) && std::find(hostReaders.begin(), hostReaders.end(), c) == hostReaders.end())
                    hostReaders.push_back(c);
            }
            bool gathered = false;   // already downloaded by a hand-placed Gather: no second copy as an output
            for (IRNode *c : t->getChildNodes())
                gathered |= c->nodeType() == OP_NODE && static_cast<OpNode *>(c)->getOp()->getOpName() == "Gather";
            // (a training graph marks its outputs — the updated parameters, the displayed loss; a gradient nobody
            // reads, such as the one a conv2dGrad computes for the data, is not one)
            bool isOutput = t->getLabel()->getIsOut() != 0 || (!cfg.train_mode && t->childNum() == 0);
            for (IRNode *lo : _graph->getLogicalOutNodes())
                if (lo == t) isOutput = true;
            if (hostReaders.empty() && (!isOutput || gathered)) continue;
            auto *twin = new TensorNode(t->name() + "_host", t->getTensor()->clone());
            twin->getTensor()->setTensorInit(TensorInitType::NONE);
            twin->getLabel()->setDeviceLabel(Device());
            auto *gather = new OpNode(t->name() + "_d2h", new GatherOp());
            gather->getLabel()->setDeviceLabel(gpu);
            gather->getLabel()->setTypeNameLabel("Gather");
            for (IRNode *reader : hostReaders) t->replaceUseKeepOrder(reader, twin);
            gather->exlinkUpperNode(t);
            twin->exlinkUpperNode(gather);
            if (isOutput) {
                twin->getLabel()->setIsOut(1);
                t->getLabel()->setIsOut(0);
            }
            _graph->pushOpNode(gather);
            _graph->pushTensorNode(twin);
            ++gathers_;
        }
    }
    _graph->findInOut();
    _graph->updateTopology();

    // 4. the layout change of a weight (the Transpose an importer puts behind a Conv or FC weight stored in
    //    another order) has the same result in every iteration: it runs once, after the uploads, like them.
    //    A weight is recognised by its use: an uploaded parameter whose transposed copy is read only as a
    //    second or later operand (operand 0 carries the data).
    for (int i = 0; i < _graph->topologyNum(); ++i)
        for (int j = 0; j < _graph->getNumInTopoLevel(i); ++j) {
            IRNode *node = _graph->getNodeInTopo(i, j);
            if (node->nodeType() != OP_NODE || !onGpu(node)) continue;
            auto *op = static_cast<OpNode *>(node);
            if (op->isRunOnce() || op->getOp()->getOpName() != "Transpose" || op->parentNum() != 1 || op->childNum() != 1)
                continue;
            auto *src = static_cast<TensorNode *>(op->getParentNode(0));
            auto *dst = static_cast<TensorNode *>(op->getChildNode(0));
            bool uploaded = src->parentNum() == 1 && static_cast<OpNode *>(src->getParentNode(0))->isRunOnce() &&
                            src->getTensor()->getTensorInitType() == TensorInitType::PARENTOP && !cfg.train_mode;
            for (TensorNode *other : tensors)   // a parameter that an op rewrites in place is no constant
                if (other != src && other->getTensor() == src->getTensor()) uploaded = false;
            if (!uploaded || dst->getLabel()->getIsOut() || dst->childNum() == 0 ||
                dst->getTensor()->getTensorInitType() != TensorInitType::NONE)
                continue;
            bool weightOnly = true;
            for (IRNode *reader : dst->getChildNodes())
                weightOnly = weightOnly && reader->nodeType() == OP_NODE && onGpu(reader) && reader->parentNum() > 1 &&
                             reader->getParentNode(0) != dst;
            if (!weightOnly) continue;
            op->setRunOnce();
            dst->getTensor()->setTensorInit(TensorInitType::PARENTOP);
            ++hoisted_;
        }
}

} // namespace pass
} // namespace swc
