#include "IRGraph.h"

#include <cassert>
#include <deque>
#include <unordered_map>

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

void IRGraph::setDeviceLabel(Device dev) {
    dev_ = dev;
    for (auto *t : tensors_) t->getLabel()->setDeviceLabel(dev);
    for (auto *o : ops_) o->getLabel()->setDeviceLabel(dev);
}

IRGraph *IRGraph::clone() const {
    auto *g = new IRGraph();
    copyTo(g);
    return g;
}

void IRGraph::copyTo(IRGraph *g) const {
    std::unordered_map<const IRNode *, IRNode *> twin;
    for (auto *t : tensors_) {
        auto *c = t->deepClone();
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

} // namespace swc
