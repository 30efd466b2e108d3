// Graph node that carries a Tensor (reference surface: src/graphIR/TensorNode.h:24-78).
#ifndef SWC_TENSORNODE_H_
#define SWC_TENSORNODE_H_
#include <sstream>

#include "../tensor/tensor.h"
#include "IRNode.h"

namespace swc {
class TensorNode : public IRNode {
    Tensor *tensor_{nullptr};

  public:
    explicit TensorNode(std::string name, IRNode *parent = nullptr) : IRNode(TENSOR_NODE, std::move(name), parent) {}
    TensorNode(std::string name, Tensor *tensor, IRNode *parent = nullptr)
        : IRNode(TENSOR_NODE, std::move(name), parent), tensor_(tensor) {}
    TensorNode(std::string name, const std::initializer_list<size_t> &shape, IRNode *parent = nullptr,
               DataType dtype = DataType::Float_t, mem_layout_t layout = layout_default)
        : IRNode(TENSOR_NODE, std::move(name), parent), tensor_(new Tensor(shape, dtype, layout)) {}

    void destroy() override {}
    void setTensor(Tensor *t) { tensor_ = t; }
    Tensor *getTensor() const { return tensor_; }
    void setTraining(int t) { tensor_->setTraining(t); }
    int getTraining() const { return tensor_->getTraining(); }
    DataType getDataType() const { return tensor_->getDataType(); }
    std::vector<size_t> getDims() const { return tensor_->getDims(); }
    size_t getNDim() const { return (size_t)tensor_->getNDim(); }
    void setMemLayout(mem_layout_t l) { tensor_->setMemLayout(l); }
    mem_layout_t getMemLayout() const { return tensor_->getMemLayout(); }

    // same Tensor object (an alias of the buffer), fresh label, no links
    TensorNode *clone() const override {
        auto *n = new TensorNode(name(), tensor_);
        n->setExternal(isExternal());
        *n->getLabel() = *getLabel();
        return n;
    }
    // own copy of the Tensor metadata (a distinct buffer)
    TensorNode *deepClone() const override {
        auto *n = new TensorNode(name(), tensor_ ? tensor_->clone() : nullptr);
        n->setExternal(isExternal());
        *n->getLabel() = *getLabel();
        return n;
    }
    std::string toString() const {
        std::ostringstream os;
        os << "TensorNode " << name() << " [";
        if (tensor_)
            for (int i = 0; i < tensor_->getNDim(); ++i) os << (i ? "," : "") << tensor_->getDim(i);
        os << "]";
        return os.str();
    }
};
} // namespace swc
#endif
