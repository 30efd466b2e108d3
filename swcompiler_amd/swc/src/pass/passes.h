// The graph passes of the inference pipeline.
//
//   LabelingPass             type-name labels + lowering marks       (reference: src/pass/LabelingPass.h:34-125)
//   LoweringPass             Op::lowering on marked nodes            (src/pass/LoweringPass.h:34-59)
//   RenamingNodePass         C-identifier-safe unique node names     (src/pass/RenamingNodePass.h:23-83)
//   EliminationPass          dead-node removal from the output marks (src/pass/EliminationPass.cpp:34-154)
//   ElimTransposePass        cancels inverse transpose pairs         (src/pass/ElimTransposePass.h:23-88)
//   HipFusionPass            NEW: chains -> one fused libswc_hip call
//   DeviceMemoryLoweringPass NEW: places compute on GPU 0, inserts host<->device transfer nodes
#ifndef SWC_PASSES_H_
#define SWC_PASSES_H_
#include <string>
#include <unordered_map>

#include "../diff/AutoDiff.h"
#include "OptimizePass.h"

namespace swc {
class OpNode;
class TensorNode;
namespace pass {

class LabelingPass : public OptimizePass {
  public:
    explicit LabelingPass(IRGraph *graph) : OptimizePass(graph) {}
    void run() override;
};

class LoweringPass : public OptimizePass {
  public:
    explicit LoweringPass(IRGraph *graph) : OptimizePass(graph) {}
    void run() override;
};

// '/', '.', '-' become '_'; a repeated name gets the smallest unused numeric suffix.
class UniqueName {
    std::unordered_map<std::string, int> seen_;

  public:
    std::string operator()(const std::string &name);
    void clear() { seen_.clear(); }
};

class RenamingNodePass : public OptimizePass {
    UniqueName unique_;

  public:
    explicit RenamingNodePass(IRGraph *graph) : OptimizePass(graph) {}
    void setGraph(IRGraph *graph) {
        _graph = graph;
        unique_.clear();
    }
    void run() override;
};

class EliminationPass : public OptimizePass {
  public:
    explicit EliminationPass(IRGraph *graph) : OptimizePass(graph) {}
    void run() override;
};

// Turns an inference graph that ends in a loss into a training graph (reference:
// src/pass/AutodiffPass.cpp:69-117, src/op/dlOp/dlOpAD.cpp, src/graphIR/TensorNode.cpp:66-134).  Nodes are
// visited in reverse topological order: a tensor without readers seeds a gradient; an op gets its gradient op
// (operands as the reference links them) and a gradient tensor per operand; a tensor marked for training gets
// an SGD node reading (parameter, gradient, momentum) whose result is a second node of the SAME Tensor — the
// parameter is updated in place — registered as a logical graph output.  As in the reference a tensor read by
// several ops keeps the gradient of the reader visited last (no summation), and only "sgd" is implemented.
class AutodiffPass : public OptimizePass {
    float lr_{0.001f}, decay_{0.001f}, momentum_{0.9f};
    size_t batch_{1};
    int gradOps_{0}, sgdOps_{0};

  public:
    explicit AutodiffPass(IRGraph *graph) : OptimizePass(graph) {}
    void getMethods(const std::string &method, float lr, float decay, float momentum, size_t batch);
    void getMethods() {}   // the settings this object already has
    void show() const;     // logs the optimizer and its settings
    void run() override;
    // copies the graph into `graph_train` (a graph the caller has made, empty) and differentiates the copy; with
    // nullptr the pass's own graph is differentiated (reference: src/pass/AutodiffPass.h:100-105; the TRAIN macro)
    void run(IRGraph *graph_train);
    int gradOpCount() const { return gradOps_; }
    int sgdCount() const { return sgdOps_; }
};


// Transpose(a) followed by Transpose(b) with a[b[i]] == i is the identity: the
// readers of the second result are rewired to the first operand (the pair itself
// is left for EliminationPass).  Reference: src/pass/ElimTransposePass.h:23-88.
class ElimTransposePass : public OptimizePass {
    int cancelled_{0};

  public:
    explicit ElimTransposePass(IRGraph *graph) : OptimizePass(graph) {}
    void run() override;
    int cancelledCount() const { return cancelled_; }
};

// Rewrites, wherever the intermediate tensor has a single consumer and is not a
// graph output:
//   MatrixMatrixFCBias -> Relu                    => MatrixMatrixFCBiasRelu
//   MatrixMatrixFCBias -> MatrixSoftmax           => MatrixMatrixFCBiasSoftmax
//   Conv2d -> BatchNormalization [-> Relu]        => Conv2dBatchNorm(relu)
//   Conv2d -> Relu                                => Conv2dWithActivation(RELU)
//   BatchNormalization -> Relu                    => BatchNormalizationRelu
//   BatchNormalizationRelu -> MaxPool             => BatchNormReluMaxPool
//   ElementAdd -> Relu                            => ElementAddRelu
//   Conv2d | Conv2dBatchNorm -> ElementAdd[Relu]  => Conv2dAdd (the other summand becomes its last operand)
//   Conv2d | Conv2dWithActivation | Conv2dBatchNorm -> MaxPool 2x2/2, no padding, over an even-sized output of a
//       convolution with iC % 4 == 0                 => Conv2dMaxPool (the pooling in the convolution's epilogue)
// Each right-hand side is one kernel launch of libswc_hip whose result equals
// the left-hand sequence of reference kernels.
class HipFusionPass : public OptimizePass {
    int fused_{0};

  public:
    explicit HipFusionPass(IRGraph *graph) : OptimizePass(graph) {}
    void run() override;
    int fusedCount() const { return fused_; }
};

// Device placement for the single-GPU HIP target.  Every op libswc_hip
// implements is labelled Device{0, GPU, id} together with its outputs; every
// host tensor read by a GPU op gets a device twin fed by a ScatterOp (run-once
// when the tensor is a parameter, i.e. has an initialiser and is not the
// per-iteration data/label input); every GPU tensor that is a graph output or
// is read by a host op (Debug, Accuracy) gets a host twin fed by a GatherOp.
// The Transpose an importer puts behind a weight (an uploaded parameter whose
// transposed copy is read only as a second or later operand) becomes run-once itself.
// After the pass the graph itself says where each buffer lives and where each
// transfer happens; the code generator only walks it.
class DeviceMemoryLoweringPass : public OptimizePass {
    int device_;
    int scatters_{0}, gathers_{0}, hoisted_{0};

  public:
    DeviceMemoryLoweringPass(IRGraph *graph, int device = 0) : OptimizePass(graph), device_(device) {}
    void run() override;
    static bool runsOnGpu(const std::string &typeName);
    int scatterCount() const { return scatters_; }
    int gatherCount() const { return gathers_; }
    int hoistedCount() const { return hoisted_; }   // weight transposes made run-once
};

} // namespace pass
} // namespace swc
#endif
