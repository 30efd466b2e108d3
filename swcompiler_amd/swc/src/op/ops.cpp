#include "ops.h"

#include <cassert>
#include <cstdlib>
#include <sstream>

#include "../graphIR/IRGraph.h"
#include "../graphIR/OpNode.h"
#include "../graphIR/TensorNode.h"

namespace swc {
namespace op {

namespace {
std::vector<size_t> dimsOfParent(OpNode *node, int i) {
    return static_cast<TensorNode *>(node->getParentNode(i))->getDims();
}
std::string join(const std::vector<size_t> &v) {
    std::ostringstream os;
    for (size_t i = 0; i < v.size(); ++i) os << (i ? "," : "") << v[i];
    return os.str();
}
// (in + pad_begin + pad_end - k) / s + 1 on H and W (reference: dlOp.cpp:195-196)
std::vector<size_t> windowedShape(const std::vector<size_t> &idims, const std::vector<size_t> &k,
                                  const std::vector<size_t> &s, const std::vector<size_t> &p, size_t channels) {
    assert(idims.size() == 4 && k.size() == 2 && s.size() == 2 && p.size() == 4);
    return {idims[0], (idims[1] + p[0] + p[2] - k[0]) / s[0] + 1, (idims[2] + p[1] + p[3] - k[1]) / s[1] + 1,
            channels};
}
} // namespace

void Op::checkValid(OpNode *node) {
    if (_nInput > 0 && node->parentNum() != _nInput) {
        SWLOG_ERROR << node->name() << " (" << _opClassName << ") expects " << _nInput << " inputs, has "
                    << node->parentNum() << std::endl;
        std::abort();
    }
    if (_nOutput > 0 && node->childNum() != _nOutput) {
        SWLOG_ERROR << node->name() << " (" << _opClassName << ") expects " << _nOutput << " outputs, has "
                    << node->childNum() << std::endl;
        std::abort();
    }
}

void Op::outTensorShapeGen(OpNode *node, size_t, TensorShape *shape) { shape->setShape(dimsOfParent(node, 0)); }

void MatrixSoftmaxOp::checkValid(OpNode *node) {
    if (node->parentNum() < 1 || node->parentNum() > 2 || node->childNum() != 1) {
        SWLOG_ERROR << node->name() << " (MatrixSoftmax) expects 1 input (+ optional label) and 1 output" << std::endl;
        std::abort();
    }
}

static void fcShape(OpNode *node, TensorShape *shape) {
    shape->setShape({dimsOfParent(node, 0)[0], dimsOfParent(node, 1)[1]});
}
void MatrixMatrixMulOp::outTensorShapeGen(OpNode *node, size_t, TensorShape *shape) { fcShape(node, shape); }
void MatrixMatrixFCOp::outTensorShapeGen(OpNode *node, size_t, TensorShape *shape) { fcShape(node, shape); }
void MatrixMatrixFCBiasOp::outTensorShapeGen(OpNode *node, size_t, TensorShape *shape) { fcShape(node, shape); }
void MatrixMatrixFCBiasReluOp::outTensorShapeGen(OpNode *node, size_t, TensorShape *shape) { fcShape(node, shape); }
void MatrixMatrixFCBiasSoftmaxOp::outTensorShapeGen(OpNode *node, size_t, TensorShape *shape) { fcShape(node, shape); }

void ReshapeOp::outTensorShapeGen(OpNode *node, size_t, TensorShape *shape) {
    if (!oshape_.empty()) shape->setShape(oshape_);
    else shape->setShape(dimsOfParent(node, 0));
}

void Conv2dOp::outTensorShapeGen(OpNode *node, size_t, TensorShape *shape) {
    shape->setShape(windowedShape(dimsOfParent(node, 0), kernels_, strides_, pads_, dimsOfParent(node, 1)[0]));
}
void MaxPoolOp::outTensorShapeGen(OpNode *node, size_t, TensorShape *shape) {
    const auto idims = dimsOfParent(node, 0);
    shape->setShape(windowedShape(idims, kernels_, strides_, pads_, idims[3]));
}
void BatchNormReluMaxPoolOp::outTensorShapeGen(OpNode *node, size_t, TensorShape *shape) {
    const auto idims = dimsOfParent(node, 0);
    shape->setShape(windowedShape(idims, kernels_, strides_, pads_, idims[3]));
}
std::vector<size_t> Conv2dMaxPoolOp::convOutDims(const std::vector<size_t> &idims, size_t oc) const {
    return windowedShape(idims, kernels_, strides_, pads_, oc);
}
void Conv2dMaxPoolOp::outTensorShapeGen(OpNode *node, size_t, TensorShape *shape) {
    const auto cdims = convOutDims(dimsOfParent(node, 0), dimsOfParent(node, 1)[0]);
    shape->setShape(windowedShape(cdims, pool_kernels_, pool_strides_, pool_pads_, cdims[3]));
}
void AvgPoolOp::outTensorShapeGen(OpNode *node, size_t, TensorShape *shape) {
    const auto idims = dimsOfParent(node, 0);
    shape->setShape(windowedShape(idims, kernels_, strides_, pads_, idims[3]));
}
void TransposeOp::outTensorShapeGen(OpNode *node, size_t, TensorShape *shape) {
    const auto idims = dimsOfParent(node, 0);
    std::vector<size_t> odims;
    for (size_t s : shuffle_) odims.push_back(idims.at(s));
    shape->setShape(odims);
}
std::string Conv2dOp::getOpInfo() {
    return Op::getOpInfo() + "kernels: " + join(kernels_) + "\\nstrides: " + join(strides_) + "\\npads: " +
           join(pads_) + "\\n";
}
std::string MaxPoolOp::getOpInfo() {
    return Op::getOpInfo() + "kernels: " + join(kernels_) + "\\nstrides: " + join(strides_) + "\\npads: " +
           join(pads_) + "\\n";
}

void ArgMaxOp::outTensorShapeGen(OpNode *node, size_t, TensorShape *shape) {
    shape->setShape({dimsOfParent(node, 0)[0], (size_t)topK_});
}

// FC lowering.  Rewrites
//     in, w[, b] -> FC[Bias] -> out
// into
//     in [-> Reshape -> in_reshape] , w -> MatrixMatrixMul -> <fc>_mm_out [, b -> MatrixVectorAdd] -> out
// which is the shape the reference's CPU generator needs (it has no emitter for
// FCBias; src/op/dlOp/dlOpEinsum.cpp:37-80,154-237).  New nodes inherit the FC
// node's device label.
static void lowerFC(IRGraph *graph, IRNode *node, bool withBias) {
    assert(node->parentNum() == (withBias ? 3 : 2) && node->childNum() == 1);
    const Device dev = node->getLabel()->getDeviceLabel();
    auto *input = static_cast<TensorNode *>(node->getParentNode(0));
    auto *weight = static_cast<TensorNode *>(node->getParentNode(1));
    auto *bias = withBias ? static_cast<TensorNode *>(node->getParentNode(2)) : nullptr;
    auto *out = static_cast<TensorNode *>(node->getChildNode(0));
    const size_t rows = input->getDims()[0], cols = weight->getDims()[1];

    TensorNode *x = input;
    if (input->getNDim() > 2) {
        auto rc = input->getTensor()->viewAs2D(1);
        std::vector<size_t> flat = {rc.first, rc.second};
        auto *reshape = new OpNode(input->name() + "_reshape_op", new ReshapeOp(flat));
        x = new TensorNode(input->name() + "_reshape", new Tensor({rc.first, rc.second}));
        reshape->exlinkUpperNode(input);
        x->exlinkUpperNode(reshape);
        reshape->getLabel()->setDeviceLabel(dev);
        x->getLabel()->setDeviceLabel(dev);
        graph->pushOpNode(reshape);
        graph->pushTensorNode(x);
    }

    auto *mm = new OpNode(node->name() + "_mm", new MatrixMatrixMulOp());
    mm->getLabel()->setDeviceLabel(dev);
    mm->exlinkUpperNode(x, weight);
    graph->pushOpNode(mm);

    // detach the FC node
    if (withBias) node->destroyUpperNode(input, weight, bias);
    else node->destroyUpperNode(input, weight);
    out->destroyUpperNode(node);

    if (withBias) {
        auto *mmOut = new TensorNode(mm->name() + "_out", {rows, cols}, mm);
        mmOut->getLabel()->setDeviceLabel(dev);
        auto *add = new OpNode(node->name() + "_add", new MatrixVectorAddOp());
        add->getLabel()->setDeviceLabel(dev);
        add->exlinkUpperNode(mmOut, bias);
        out->exlinkUpperNode(add);
        graph->pushTensorNode(mmOut);
        graph->pushOpNode(add);
    } else {
        out->exlinkUpperNode(mm);
    }
    graph->delOpNode(static_cast<OpNode *>(node));
    graph->updateTopology();
}

// prob has the logits' shape, loss is one number
void MatrixSoftmaxWithLossOp::outTensorShapeGen(OpNode *node, size_t index, TensorShape *shape) {
    if (index == 0) shape->setShape(static_cast<TensorNode *>(node->getParentNode(0))->getDims());
    else shape->setShape({1});
}

// Y = X W + b (reference: src/op/dlOp/dlOpEinsum.cpp:239-318):
//   dX = dY * W^T      dW = X^T * dY      db = column sums of dY
// X of rank > 2 is read as [dim0, rest] through a Reshape alias; dX keeps X's shape (same storage size).
void MatrixMatrixFCBiasGradOp::lowering(IRGraph *graph, IRNode *node) {
    auto *input = static_cast<TensorNode *>(node->getParentNode(0));
    auto *weight = static_cast<TensorNode *>(node->getParentNode(1));
    auto *bias = static_cast<TensorNode *>(node->getParentNode(2));
    auto *outputG = static_cast<TensorNode *>(node->getParentNode(3));
    auto *inputG = static_cast<TensorNode *>(node->getChildNode(0));
    auto *weightG = static_cast<TensorNode *>(node->getChildNode(1));
    auto *biasG = static_cast<TensorNode *>(node->getChildNode(2));

    auto *wT_op = new OpNode("op_" + weight->name() + "_T", new TransposeOp({1, 0}));
    wT_op->exlinkUpperNode(weight);
    auto *wT = new TensorNode(weight->name() + "_T", new Tensor(weight->getTensor()->getShuffledTensorShape({1, 0})), wT_op);
    auto *dx = new OpNode(node->name() + "_dx_mm", new MatrixMatrixMulOp());
    dx->exlinkUpperNode(outputG, wT);

    TensorNode *x2d = input;
    if (input->getTensor()->getNDim() > 2) {
        const auto rc = input->getTensor()->viewAs2D(1);
        std::vector<size_t> flat{rc.first, rc.second};
        auto *reshape = new OpNode(input->name() + "_reshape_op", new ReshapeOp(flat));
        reshape->exlinkUpperNode(input);
        x2d = new TensorNode(input->name() + "_reshape", new Tensor({rc.first, rc.second}), reshape);
        graph->pushOpNode(reshape);
        graph->pushTensorNode(x2d);
    }
    auto *xT_op = new OpNode("op_" + x2d->name() + "_T", new TransposeOp({1, 0}));
    xT_op->exlinkUpperNode(x2d);
    auto *xT = new TensorNode(x2d->name() + "_T", new Tensor(x2d->getTensor()->getShuffledTensorShape({1, 0})), xT_op);
    auto *dw = new OpNode(node->name() + "_dw_mm", new MatrixMatrixMulOp());
    dw->exlinkUpperNode(xT, outputG);
    auto *db = new OpNode(node->name() + "_db_bra", new BatchedReduceAddOp());
    db->exlinkUpperNode(outputG);

    node->destroyUpperNode(input);
    node->destroyUpperNode(weight);
    node->destroyUpperNode(bias);
    node->destroyUpperNode(outputG);
    inputG->destroyUpperNode(node);
    weightG->destroyUpperNode(node);
    biasG->destroyUpperNode(node);
    inputG->exlinkUpperNode(dx);
    weightG->exlinkUpperNode(dw);
    biasG->exlinkUpperNode(db);
    graph->delOpNode(static_cast<OpNode *>(node));
    graph->pushOpNode(wT_op, xT_op, dx, dw, db);
    graph->pushTensorNode(wT, xT);
    graph->updateTopology();
}

void MatrixMatrixFCOp::lowering(IRGraph *graph, IRNode *node) { lowerFC(graph, node, false); }
void MatrixMatrixFCBiasOp::lowering(IRGraph *graph, IRNode *node) { lowerFC(graph, node, true); }

} // namespace op
} // namespace swc
