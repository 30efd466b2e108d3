// Base of every operator (reference surface: src/op/Op.h:35-153).  An Op knows
// its arity, can infer its output shape from the parents of its OpNode, and may
// rewrite itself into simpler ops (lowering).
#ifndef SWC_OP_H_
#define SWC_OP_H_
#include <string>
#include <vector>

#include "../SWLOG.h"
#include "../common.h"

namespace swc {
class Tensor;
class TensorShape;
class IRGraph;
class IRNode;
class OpNode;

namespace op {

enum activation_type { SWC_ACTIVATION_RELU, SWC_ACTIVATION_TANH, SWC_ACTIVATION_SIGMOID };

class Op {
  protected:
    const OpType _opType;
    const int _nInput, _nOutput;
    std::vector<int> _inputNDims, _outputNDims;
    const std::string _opClassName;

  public:
    Op(OpType opType = BASIC_OP, int nInput = 0, int nOutput = 0, std::string opClassName = "")
        : _opType(opType), _nInput(nInput), _nOutput(nOutput), _opClassName(std::move(opClassName)) {}
    virtual ~Op() {}
    virtual void destroy() {}
    OpType getOpType() const { return _opType; }
    const std::string getOpName() const { return _opClassName; }
    int getnInput() const { return _nInput; }
    int getnOutput() const { return _nOutput; }
    int getInputDims(int n) const { return _inputNDims.at(n); }
    int getOutputDims(int n) const { return _outputNDims.at(n); }
    virtual std::string getOpInfo() { return " " + _opClassName + "\\n"; }
    virtual void lowering(IRGraph *, IRNode *) {}
    virtual void einsumLowering(IRGraph *graph, IRNode *node) { lowering(graph, node); }
    // arity check against the node's links; aborts with a message on mismatch
    virtual void checkValid(OpNode *node);
    // default: output has the shape of operand 0
    virtual void outTensorShapeGen(OpNode *node, size_t index, TensorShape *tShape);
};

} // namespace op
} // namespace swc
#endif
