#include "IRGraph.h"

#include <cassert>
#include <deque>
#include <unordered_map>

#include <queue>
#include <unordered_set>

#include "../op/ops.h"
#include "OpNode.h"
#include "TensorNode.h"

namespace swc {

IRNode *IRGraph::getNodeByName(std::string name) const {
    for (auto *t : tensors_)
        if (t->name() == name) return t;
    for (auto *o : ops_)
        if (o->name() == name) return o;
    return nullptr;
}

void IRGraph::findInOut() {
    inNodes_.clear();
    outNodes_.clear();
    auto visit = [&](IRNode *n) {
        if (n->parentNum() == 0) inNodes_.push_back(n);
        if (n->childNum() == 0) outNodes_.push_back(n);
    };
    for (auto *t : tensors_) visit(t);
    for (auto *o : ops_) visit(o);
}

void IRGraph::updateTopology() {
    // longest-path levels by Kahn's algorithm over the nodes this graph owns
    std::unordered_map<IRNode *, int> pending, level;
    std::vector<IRNode *> all;
    for (auto *t : tensors_) all.push_back(t);
    for (auto *o : ops_) all.push_back(o);
    std::deque<IRNode *> ready;
    for (IRNode *n : all) {
        int inside = 0;
        for (IRNode *p : n->getParentNodes())
            if (std::find(all.begin(), all.end(), p) != all.end()) ++inside;
        pending[n] = inside;
        level[n] = 0;
        if (inside == 0) ready.push_back(n);
    }
    levels_.clear();
    size_t done = 0;
    while (!ready.empty()) {
        IRNode *n = ready.front();
        ready.pop_front();
        ++done;
        const int lv = level[n];
        n->setTopologyId(lv);
        if ((int)levels_.size() <= lv) levels_.resize(lv + 1);
        levels_[lv].push_back(n);
        for (IRNode *c : n->getChildNodes()) {
            auto it = pending.find(c);
            if (it == pending.end()) continue;
            level[c] = std::max(level[c], lv + 1);
            if (--it->second == 0) ready.push_back(c);
        }
    }
    assert(done == all.size() && "IRGraph::updateTopology: graph has a cycle");
    (void)done;
}

void IRGraph::initTensorNodes() {
    updateTopology();
    for (auto &lvl : levels_)
        for (IRNode *n : lvl) {
            if (n->nodeType() != TENSOR_NODE || n->parentNum() == 0) continue;
            auto *tn = static_cast<TensorNode *>(n);
            auto *producer = static_cast<OpNode *>(n->getParentNode(0));
            size_t index = 0;
            for (int i = 0; i < producer->childNum(); ++i)
                if (producer->getChildNode(i) == n) index = (size_t)i;
            Tensor *t = tn->getTensor();
            const bool unset = !t || t->getNDim() == 0 || t->size() == 0;
            if (!unset) continue;
            auto *shape = new TensorShape(std::vector<size_t>{});
            producer->outTensorShapeGen(index, shape);
            if (!t) tn->setTensor(new Tensor(shape));
            else t->reset(shape, t->getDataType());
        }
}

void IRGraph::setOutMark() {
    for (IRNode *n : outNodes_) n->getLabel()->setIsOut();
    setLogicalOutMark();
}
void IRGraph::setLogicalOutMark() {
    for (IRNode *n : logicalOutNodes_) n->getLabel()->setIsOut();
}
void IRGraph::clearOutMark() {
    for (IRNode *n : outNodes_) n->getLabel()->setIsOut(0);
}

// (external nodes are mirrors of nodes of an outer graph and keep that graph's device, as in the reference,
// src/graphIR/IRGraph.cpp:585-601)
void IRGraph::setDeviceLabel(Device dev) {
    dev_ = dev;
    for (auto *t : tensors_)
        if (!t->isExternal()) t->getLabel()->setDeviceLabel(dev);
    for (auto *o : ops_)
        if (!o->isExternal()) o->getLabel()->setDeviceLabel(dev);
}

IRGraph *IRGraph::clone() const {
    auto *g = new IRGraph();
    copyTo(g);
    return g;
}

void IRGraph::copyTo(IRGraph *g) const {
    std::unordered_map<const IRNode *, IRNode *> twin;
    for (auto *t : tensors_) {
        // (a mirror of an outer graph's node goes on naming that node's Tensor)
        auto *c = t->isExternal() ? static_cast<TensorNode *>(t->clone()) : static_cast<TensorNode *>(t->deepClone());
        twin[t] = c;
        g->tensors_.push_back(c);
    }
    for (auto *o : ops_) {
        auto *c = o->clone();
        twin[o] = c;
        g->ops_.push_back(c);
    }
    // operand order and result order are both preserved
    auto relink = [&](const IRNode *orig) {
        for (IRNode *p : orig->getParentNodes()) {
            auto it = twin.find(p);
            if (it != twin.end()) twin[orig]->pushParentNode(it->second);
        }
        for (IRNode *c : orig->getChildNodes()) {
            auto it = twin.find(c);
            if (it != twin.end()) twin[orig]->pushChildNode(it->second);
        }
    };
    for (auto *t : tensors_) relink(t);
    for (auto *o : ops_) relink(o);
    g->config_ = config_;
    g->dev_ = dev_;
    auto map = [&](TensorNode *n) { return n ? static_cast<TensorNode *>(twin[n]) : nullptr; };
    g->inferData_ = map(inferData_);
    g->inferLabel_ = map(inferLabel_);
    g->trainData_ = map(trainData_);
    g->trainLabel_ = map(trainLabel_);
    for (auto *d : displayNodes_) g->displayNodes_.push_back(map(d));
    for (auto *l : logicalOutNodes_) g->logicalOutNodes_.push_back(twin[l]);
    g->findInOut();
    g->updateTopology();
}

// ---------------------------------------------------------------- nested graphs
OpNode *IRGraph::extractSubGraph(TensorNode *in, TensorNode *out) {
    // everything `out` depends on, walking up and stopping at `in`
    std::unordered_set<IRNode *> part{out};
    std::queue<IRNode *> todo;
    todo.push(out);
    while (!todo.empty()) {
        IRNode *cur = todo.front();
        todo.pop();
        if (cur == in) continue;
        for (IRNode *p : cur->getParentNodes())
            if (part.insert(p).second) todo.push(p);
    }
    if (!part.count(in)) return nullptr;

    auto *inner = new IRGraph();
    auto *sub_op = new op::SubGraphOp();
    sub_op->setGraph(inner);
    auto *sub_node = new OpNode("subG", sub_op);

    // an outer tensor the part reads: mirror -> Scatter -> working copy, which takes the outer node's place
    // as operand of the part's ops
    auto bring_in = [&](TensorNode *outer, bool once) {
        TensorNode *mirror = static_cast<TensorNode *>(outer->clone());
        mirror->setExternal(true);
        auto *scatter = new OpNode("scatter", new op::ScatterOp());
        if (once) scatter->setRunOnce();
        scatter->exlinkUpperNode(mirror);
        auto *work = new TensorNode(outer->name() + "_sub", new Tensor(outer->getTensor()->getTensorShape()), scatter);
        for (IRNode *reader : std::vector<IRNode *>(outer->getChildNodes()))
            if (part.count(reader)) outer->replaceUseKeepOrder(reader, work);
        inner->pushTensorNode(mirror, work);
        inner->pushOpNode(scatter);
    };

    // (in a fixed order: the nodes as the graph lists them, not the hash set's)
    std::vector<IRNode *> ordered;
    for (auto *t : tensors_)
        if (part.count(t)) ordered.push_back(t);
    for (auto *o : ops_)
        if (part.count(o)) ordered.push_back(o);
    for (IRNode *n : ordered) {
        if (n->nodeType() == OP_NODE) {
            inner->pushOpNode(static_cast<OpNode *>(n));
            delOpNode(static_cast<OpNode *>(n));
            continue;
        }
        auto *t = static_cast<TensorNode *>(n);
        if (t == in) {
            bring_in(t, false);
        } else if (t == out) {
            assert(t->parentNum() == 1 && "the output of the part has one producer");
            IRNode *producer = t->getParentNode(0);
            auto *work = new TensorNode(t->name() + "_sub", new Tensor(t->getTensor()->getTensorShape()));
            t->destroyUpperNode(producer);
            work->exlinkUpperNode(producer);
            TensorNode *mirror = static_cast<TensorNode *>(t->clone());
            mirror->setExternal(true);
            auto *gather = new OpNode("gather", new op::GatherOp());
            gather->exlinkUpperNode(work);
            mirror->exlinkUpperNode(gather);
            inner->pushTensorNode(work, mirror);
            inner->pushOpNode(gather);
        } else if (t->parentNum() == 0) {   // a parameter of one of the part's ops: stays outside, uploaded once
            bring_in(t, true);
            sub_node->exlinkUpperNode(t);
        } else {
            inner->pushTensorNode(t);
            delTensorNode(t);
        }
    }
    // outside: in (and the parameters) -> subG -> out
    std::vector<IRNode *> params(sub_node->getParentNodes());
    for (IRNode *p : params) sub_node->destroyUpperNode(p);
    sub_node->exlinkUpperNode(in);
    for (IRNode *p : params) sub_node->exlinkUpperNode(p);
    out->exlinkUpperNode(sub_node);
    pushOpNode(sub_node);
    inner->findInOut();
    inner->updateTopology();
    return sub_node;
}

bool IRGraph::buildSubGraphs(TensorNode *in, TensorNode *out, ParallelStrategy strategy, int axis, int num) {
    assert(strategy == ParallelStrategy::SLICE && axis == 0 && "slices along axis 0 only");
    (void)strategy;
    const std::vector<size_t> whole = in->getDims();
    if (num < 1 || whole.empty() || whole[0] % (size_t)num) return false;
    OpNode *first = extractSubGraph(in, out);
    if (!first) return false;
    std::vector<size_t> part_dims = whole;
    part_dims[axis] = whole[0] / (size_t)num;

    // the working copy of `in` shrinks to one slice, and every tensor computed from it follows
    auto reshape_inner = [&](IRGraph *g) {
        auto *work = static_cast<TensorNode *>(g->getNodeByName(in->name() + "_sub"));
        if (!work) return false;
        work->setTensor(new Tensor(new TensorShape(new std::vector<size_t>(part_dims))));
        g->updateTopology();
        for (int i = 0; i < g->topologyNum(); ++i)
            for (IRNode *n : g->getNodeInTopoLevel(i)) {
                if (n->nodeType() != TENSOR_NODE || n->parentNum() == 0 || n == work || n->isExternal()) continue;
                auto *producer = static_cast<OpNode *>(n->getParentNode(0));
                const std::string type = producer->getOp()->getOpName();
                if (type == "Scatter" || type == "Gather") continue;   // copies keep the shape they were made with
                size_t index = 0;
                for (int c = 0; c < producer->childNum(); ++c)
                    if (producer->getChildNode(c) == n) index = (size_t)c;
                auto *shape = new TensorShape(std::vector<size_t>{});
                producer->outTensorShapeGen(index, shape);
                auto *tn = static_cast<TensorNode *>(n);
                tn->setTensor(new Tensor(shape, tn->getTensor() ? tn->getTensor()->getDataType() : DataType::Float_t));
            }
        return true;
    };
    // Slice i reads rows [i, i + 1) * whole[0] / num of `in` and writes the same rows of `out`: its Scatter and Gather
    // nodes get ops of their own (a clone shares its ops with the original) with the slice's element offset, as the
    // reference's two-GPU example sets them by hand (test/cuda/testGPUInfer.cpp:177-178, 205-206).  The reference's
    // buildSubGraphs leaves every offset at zero (src/graphIR/IRGraph.cpp:47-96): all its slices read and write the
    // first one's rows.
    size_t in_slice = 1, out_slice = 1;
    for (size_t d : part_dims) in_slice *= d;
    const std::vector<size_t> out_dims = out->getDims();
    if (out_dims.empty() || out_dims[0] % (size_t)num) return false;
    for (size_t d : out_dims) out_slice *= d;
    out_slice /= (size_t)num;
    auto place_slice = [&](IRGraph *g, int i) {
        IRNode *work_in = g->getNodeByName(in->name() + "_sub"), *work_out = g->getNodeByName(out->name() + "_sub");
        if (!work_in || !work_out || work_in->parentNum() != 1 || work_out->childNum() < 1) return false;
        auto *scatter = static_cast<OpNode *>(work_in->getParentNode(0));
        OpNode *gather = nullptr;
        for (int c = 0; c < work_out->childNum(); ++c) {
            auto *reader = static_cast<OpNode *>(work_out->getChildNode(c));
            if (reader->nodeType() == OP_NODE && reader->getOp()->getOpName() == "Gather") gather = reader;
        }
        if (scatter->getOp()->getOpName() != "Scatter" || !gather) return false;
        scatter->setOp(new op::ScatterOp((size_t)i * in_slice));
        gather->setOp(new op::GatherOp((size_t)i * out_slice));
        return true;
    };
    IRGraph *inner = static_cast<op::SubGraphOp *>(first->getOp())->getGraph();
    if (!reshape_inner(inner) || !place_slice(inner, 0)) return false;
    for (int i = 1; i < num; ++i) {
        IRGraph *copy = inner->clone();
        if (!reshape_inner(copy) || !place_slice(copy, i)) return false;
        auto *sub_op = new op::SubGraphOp();
        sub_op->setGraph(copy);
        auto *node = new OpNode("subG", sub_op);
        for (IRNode *p : first->getParentNodes()) node->exlinkUpperNode(p);
        for (IRNode *c : std::vector<IRNode *>(first->getChildNodes())) c->exlinkUpperNode(node);
        pushOpNode(node);
    }
    return true;
}

int IRGraph::inlineSubGraphs(int device) {
    int replaced = 0;
    for (bool again = true; again;) {
        again = false;
        for (OpNode *node : std::vector<OpNode *>(ops_)) {
            auto *sub = dynamic_cast<op::SubGraphOp *>(node->getOp());
            if (!sub) continue;
            IRGraph *inner = sub->getGraph();
            // the SubGraph node's own links go: its nested graph's Scatter and Gather nodes carry the dependences
            for (IRNode *p : std::vector<IRNode *>(node->getParentNodes())) node->destroyUpperNode(p);
            for (IRNode *c : std::vector<IRNode *>(node->getChildNodes())) c->destroyUpperNode(node);
            delOpNode(node);
            ++replaced;
            if (!inner) continue;
            again = true;   // (its nodes may include SubGraph nodes of their own)
            for (int i = 0; i < inner->tensorNodeNum(); ++i) {
                TensorNode *t = inner->getTensorNode(i);
                TensorNode *outer = nullptr;
                if (t->isExternal())
                    for (auto *mine : tensors_)
                        if (mine->getTensor() == t->getTensor()) {
                            outer = mine;
                            break;
                        }
                if (!outer) {   // an ordinary inner node (or a mirror of nothing here): it moves out as it is
                    t->setExternal(false);
                    pushTensorNode(t);
                    continue;
                }
                // a mirror: the outer node takes its place as operand (of a Scatter) and as result (of a Gather)
                for (IRNode *reader : std::vector<IRNode *>(t->getChildNodes())) t->replaceUseKeepOrder(reader, outer);
                for (IRNode *producer : std::vector<IRNode *>(t->getParentNodes())) {
                    t->destroyUpperNode(producer);
                    outer->exlinkUpperNode(producer);
                }
            }
            for (int i = 0; i < inner->opNodeNum(); ++i) pushOpNode(inner->getOpNode(i));
        }
    }
    if (replaced) {
        auto collapse = [&](IRNode *n) {
            Device d = n->getLabel()->getDeviceLabel();
            if (d.type == DeviceType::GPU && d.id != device) n->getLabel()->setDeviceLabel(Device(d.rank, DeviceType::GPU, device));
        };
        for (auto *t : tensors_) collapse(t);
        for (auto *o : ops_) collapse(o);
        findInOut();
        updateTopology();
    }
    return replaced;
}

} // namespace swc
