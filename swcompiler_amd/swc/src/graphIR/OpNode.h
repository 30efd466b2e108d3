// Graph node that carries an Op (reference surface: src/graphIR/OpNode.h:23-86).
#ifndef SWC_OPNODE_H_
#define SWC_OPNODE_H_
#include <sstream>

#include "../op/Op.h"
#include "IRNode.h"

namespace swc {
class OpNode : public IRNode {
    op::Op *op_{nullptr};
    bool run_{true}, runOnce_{false};

  public:
    explicit OpNode(std::string name) : IRNode(OP_NODE, std::move(name)) {}
    OpNode(std::string name, op::Op *op) : IRNode(OP_NODE, std::move(name)), op_(op) {}
    void destroy() override {}
    void setOp(op::Op *op) { op_ = op; }
    op::Op *getOp() const { return op_; }
    const std::string getOpName() const { return op_->getOpName(); }
    // shares the Op object; links are not copied
    OpNode *clone() const override {
        auto *n = new OpNode(name(), op_);
        *n->getLabel() = *getLabel();
        n->runOnce_ = runOnce_;
        return n;
    }
    OpNode *deepClone() const override { return clone(); }
    std::string toString() const { return "OpNode " + name() + " : " + (op_ ? op_->getOpName() : "?"); }

    // A run-once node (a parameter upload) is emitted before the execute loop
    // and reports itself runnable a single time.
    void setRunOnce() { runOnce_ = true; }
    bool isRunOnce() const { return runOnce_; }
    bool runable() {
        const bool r = run_;
        if (runOnce_) run_ = false;
        return r;
    }
    void checkValid() override { op_->checkValid(this); }
    void outTensorShapeGen(size_t index, TensorShape *shape) { op_->outTensorShapeGen(this, index, shape); }
};
} // namespace swc
// The reference's header of the same name has this directive at file scope (src/graphIR/OpNode.h:16), and its
// user programs — the importer examples, for one — name ops without `swc::op::` because of it.
using namespace swc::op;

#endif
