// Operator classes of the inference path (reference surface:
// src/op/basicOp/basicOps.h:26-95 and src/op/dlOp/dlOp.h).  Class names,
// constructor arguments and type-name strings are the reference's because user
// programs and the code generators key on them.  Classes below the "HIP target"
// banner have no counterpart there: they are what the fusion pass rewrites
// chains into and what HipCodegen emits one fused kernel call for.
#ifndef SWC_OPS_H_
#define SWC_OPS_H_
#include <initializer_list>
#include <string>
#include <vector>

#include "Op.h"

namespace swc {
namespace op {

// ---- GEMM family -----------------------------------------------------------
class MatrixMatrixMulOp : public Op {   // out[m,n] = in[m,k] * w[k,n]
  public:
    MatrixMatrixMulOp() : Op(BASIC_OP, 2, 1, "MatrixMatrixMul") {}
    void outTensorShapeGen(OpNode *node, size_t index, TensorShape *shape) override;
};
class MatrixVectorAddOp : public Op {   // out[r,j] = in[r,j] + bias[j]
  public:
    MatrixVectorAddOp() : Op(BASIC_OP, 2, 1, "MatrixVectorAdd") {}
};
class BatchedAddOp : public Op {
  public:
    BatchedAddOp() : Op(DL_OP, 2, 1, "BatchedAdd") {}
};
// Fully connected layer without / with bias.  Inputs of rank > 2 are viewed as
// [dim0, rest].  On the CPU target both are lowered to MatrixMatrixMul
// (+ MatrixVectorAdd) with an intermediate tensor; the HIP target keeps FCBias
// whole and runs it as one GEMM with the bias in the epilogue.
class MatrixMatrixFCOp : public Op {
  public:
    MatrixMatrixFCOp() : Op(DL_OP, 2, 1, "MatrixMatrixFC") {}
    void outTensorShapeGen(OpNode *node, size_t index, TensorShape *shape) override;
    void lowering(IRGraph *graph, IRNode *node) override;
};
class MatrixMatrixFCBiasOp : public Op {
  public:
    MatrixMatrixFCBiasOp() : Op(DL_OP, 3, 1, "MatrixMatrixFCBias") {}
    void outTensorShapeGen(OpNode *node, size_t index, TensorShape *shape) override;
    void lowering(IRGraph *graph, IRNode *node) override;
};
class ReshapeOp : public Op {           // alias of the input buffer with a new shape
    std::vector<size_t> oshape_;

  public:
    ReshapeOp() : Op(DL_OP, 1, 1, "Reshape") {}
    explicit ReshapeOp(std::vector<size_t> &shape) : Op(DL_OP, 1, 1, "Reshape"), oshape_(shape) {}
    std::vector<size_t> getOutShape() const { return oshape_; }
    void outTensorShapeGen(OpNode *node, size_t index, TensorShape *shape) override;
};

// Dimensions start..end of an nDim tensor folded into one (TensorDescend) and unfolded again (TensorAscend): a view
// of the same buffer, like Reshape (reference: src/op/tensorOp/tensorOps.h:18-70; emitted as a pointer alias,
// src/codegen/Codegen.cpp:1487-1499).  Each is the other's gradient op.
class TensorDescendOp : public Op {
    int nDim_, start_, end_;

  public:
    TensorDescendOp(int nDim, int start, int end) : Op(TENSOR_OP, 1, 1, "TensorDescend"), nDim_(nDim), start_(start), end_(end) {}
    int getNDim() const { return nDim_; }
    int getStart() const { return start_; }
    int getEnd() const { return end_; }
};
class TensorAscendOp : public Op {
    int nDim_, start_, end_;

  public:
    TensorAscendOp(int nDim, int start, int end) : Op(TENSOR_OP, 1, 1, "TensorAscend"), nDim_(nDim), start_(start), end_(end) {}
    int getNDim() const { return nDim_; }
    int getStart() const { return start_; }
    int getEnd() const { return end_; }
};
// Local response normalisation: declared so that programs naming it compile (reference: src/op/dlOp/dlOp.h:765-784);
// like the reference's generators, this build's emit no code for it.
class LRNOp : public Op {
  public:
    LRNOp() : Op(DL_OP, 1, 1, "LRN") {}
};

// ---- element-wise / row-wise ----------------------------------------------
class MatrixTanhOp : public Op {
  public:
    MatrixTanhOp() : Op(DL_OP, 1, 1, "MatrixTanh") {}
};
class MatrixSoftmaxOp : public Op {
  public:
    MatrixSoftmaxOp() : Op(DL_OP, 1, 1, "MatrixSoftmax") {}
    void checkValid(OpNode *node) override;   // the reference's tests also link a label tensor; tolerated
};
class ElementAddOp : public Op {
  public:
    ElementAddOp() : Op(DL_OP, 2, 1, "ElementAdd") {}
};
class ReluOp : public Op {
  public:
    ReluOp() : Op(DL_OP, 1, 1, "Relu") {}
};
class DropoutOp : public Op {           // inference: identity on operand 0 (operand 1 is the mask)
    float ratio_;

  public:
    explicit DropoutOp(float ratio) : Op(DL_OP, 2, 1, "Dropout"), ratio_(ratio) {}
    float getRatio() const { return ratio_; }
};

// ---- NHWC spatial ops -------------------------------------------------------
// kernels {kh,kw}, strides {sh,sw}, pads {top,left,bottom,right};
// out = (in + pad_begin + pad_end - k) / s + 1   (reference: dlOp.cpp:195-196)
class Conv2dOp : public Op {            // parents: input NHWC, filter [oC,kh,kw,iC], bias [oC]
  protected:
    std::vector<size_t> kernels_, strides_, pads_;
    int group_{1};
    Conv2dOp(const char *type, int nIn, std::vector<size_t> &k, std::vector<size_t> &s, std::vector<size_t> &p)
        : Op(DL_OP, nIn, 1, type), kernels_(k), strides_(s), pads_(p) {}

  public:
    Conv2dOp() : Op(DL_OP, 3, 1, "Conv2d") {}
    Conv2dOp(std::vector<size_t> &kernels, std::vector<size_t> &strides, std::vector<size_t> &pads)
        : Op(DL_OP, 3, 1, "Conv2d"), kernels_(kernels), strides_(strides), pads_(pads) {}
    std::vector<size_t> getPads() const { return pads_; }
    std::vector<size_t> getKernels() const { return kernels_; }
    std::vector<size_t> getStrides() const { return strides_; }
    size_t getGroup() const { return (size_t)group_; }
    std::string getOpInfo() override;
    void outTensorShapeGen(OpNode *node, size_t index, TensorShape *shape) override;
};
class MaxPoolOp : public Op {
    std::vector<size_t> kernels_, strides_, pads_;

  public:
    MaxPoolOp() : Op(DL_OP, 1, 1, "MaxPool") {}
    MaxPoolOp(std::vector<size_t> &kernels, std::vector<size_t> &strides, std::vector<size_t> &pads)
        : Op(DL_OP, 1, 1, "MaxPool"), kernels_(kernels), strides_(strides), pads_(pads) {}
    std::vector<size_t> getPads() const { return pads_; }
    std::vector<size_t> getKernels() const { return kernels_; }
    std::vector<size_t> getStrides() const { return strides_; }
    std::string getOpInfo() override;
    void outTensorShapeGen(OpNode *node, size_t index, TensorShape *shape) override;
};
class AvgPoolOp : public Op {           // sum of in-bounds taps / (kh*kw)
    std::vector<size_t> kernels_, strides_, pads_;

  public:
    AvgPoolOp() : Op(DL_OP, 1, 1, "AveragePool") {}
    AvgPoolOp(std::vector<size_t> &kernels, std::vector<size_t> &strides, std::vector<size_t> &pads)
        : Op(DL_OP, 1, 1, "AveragePool"), kernels_(kernels), strides_(strides), pads_(pads) {}
    std::vector<size_t> getPads() const { return pads_; }
    std::vector<size_t> getKernels() const { return kernels_; }
    std::vector<size_t> getStrides() const { return strides_; }
    void outTensorShapeGen(OpNode *node, size_t index, TensorShape *shape) override;
};
// Axis permutation: output axis a is input axis shuffle[a] (NCHW2NHWC, NHWC2NCHW, {1,0}).
class TransposeOp : public Op {
    std::vector<size_t> shuffle_;

  public:
    TransposeOp(const std::initializer_list<size_t> &shuffle) : Op(DL_OP, 1, 1, "Transpose"), shuffle_(shuffle) {}
    std::vector<size_t> getShuffle() const { return shuffle_; }
    void outTensorShapeGen(OpNode *node, size_t index, TensorShape *shape) override;
};
class BatchNormalizationOp : public Op {   // parents: input, scale, bias, mean, var
    float epsilon_;

  public:
    explicit BatchNormalizationOp(float eps) : Op(DL_OP, 5, 1, "BatchNormalization"), epsilon_(eps) {}
    float getEpsilon() const { return epsilon_; }
};

// ---- classification tail (int32 tensors) ------------------------------------
class ArgMaxOp : public Op {            // out[m, topK] int32
    int topK_;

  public:
    explicit ArgMaxOp(int topK) : Op(DL_OP, 1, 1, "ArgMax"), topK_(topK) {}
    int getTopK() const { return topK_; }
    void outTensorShapeGen(OpNode *node, size_t index, TensorShape *shape) override;
};
class AccuracyOp : public Op {          // parents: pred[m,k] int32, label[m] int32 -> {right, total} counters
  public:
    AccuracyOp() : Op(DL_OP, 2, 1, "Accuracy") {}
};
class DebugOp : public Op {             // prints its operand; output aliases it
  public:
    DebugOp() : Op(DL_OP, 1, 1, "Debug") {}
};

// ---- placement ops ----------------------------------------------------------
// Scatter copies its single parent tensor (host) into its single child tensor
// (device); Gather the other way.  `offset` is in elements of the host side.
class ScatterOp : public Op {
    size_t offset_{0};
    int axis_{-1}, degree_{1};

  public:
    ScatterOp() : Op(DL_OP, 0, 0, "Scatter") {}
    explicit ScatterOp(size_t offset) : Op(DL_OP, 0, 0, "Scatter"), offset_(offset) {}
    ScatterOp(int axis, int degree) : Op(DL_OP, 0, 0, "Scatter"), axis_(axis), degree_(degree) {}
    void setOffset(size_t o) { offset_ = o; }
    size_t getOffset() const { return offset_; }
    int getAxis() const { return axis_; }
    int getDegree() const { return degree_; }
};
class GatherOp : public Op {
    size_t offset_{0};
    int axis_{-1}, degree_{1};

  public:
    GatherOp() : Op(DL_OP, 0, 0, "Gather") {}
    explicit GatherOp(size_t offset) : Op(DL_OP, 0, 0, "Gather"), offset_(offset) {}
    GatherOp(int axis, int degree) : Op(DL_OP, 0, 0, "Gather"), axis_(axis), degree_(degree) {}
    void setOffset(size_t o) { offset_ = o; }
    size_t getOffset() const { return offset_; }
    int getAxis() const { return axis_; }
    int getDegree() const { return degree_; }
};
class SubGraphOp : public Op {
    IRGraph *graph_{nullptr};

  public:
    SubGraphOp() : Op(DL_OP, 0, 0, "SubGraph") {}
    void setGraph(IRGraph *g) { graph_ = g; }
    IRGraph *getGraph() const { return graph_; }
};

// =============================== HIP target =================================
// One node per fused kernel call of libswc_hip.

// MatrixMatrixFCBias followed by Relu: swc_hip_matrixMatrixFCBias_f(..., relu=1)
class MatrixMatrixFCBiasReluOp : public Op {
  public:
    MatrixMatrixFCBiasReluOp() : Op(DL_OP, 3, 1, "MatrixMatrixFCBiasRelu") {}
    void outTensorShapeGen(OpNode *node, size_t index, TensorShape *shape) override;
};
// MatrixMatrixFCBias followed by MatrixSoftmax: swc_hip_matrixMatrixFCBiasSoftmax_f
class MatrixMatrixFCBiasSoftmaxOp : public Op {
  public:
    MatrixMatrixFCBiasSoftmaxOp() : Op(DL_OP, 3, 1, "MatrixMatrixFCBiasSoftmax") {}
    void outTensorShapeGen(OpNode *node, size_t index, TensorShape *shape) override;
};
// ElementAdd followed by Relu: swc_hip_vecAddRelu_f
class ElementAddReluOp : public Op {
  public:
    ElementAddReluOp() : Op(DL_OP, 2, 1, "ElementAddRelu") {}
};
// BatchNormalization followed by Relu: swc_hip_batchnormRelu_f
class BatchNormalizationReluOp : public Op {
    float epsilon_;

  public:
    explicit BatchNormalizationReluOp(float eps) : Op(DL_OP, 5, 1, "BatchNormalizationRelu"), epsilon_(eps) {}
    float getEpsilon() const { return epsilon_; }
};
// BatchNormalization, Relu, then MaxPool over the result: swc_hip_batchnormReluMaxpool_f
class BatchNormReluMaxPoolOp : public Op {
    float epsilon_;
    std::vector<size_t> kernels_, strides_, pads_;

  public:
    BatchNormReluMaxPoolOp(float eps, std::vector<size_t> kernels, std::vector<size_t> strides, std::vector<size_t> pads)
        : Op(DL_OP, 5, 1, "BatchNormReluMaxPool"), epsilon_(eps), kernels_(std::move(kernels)),
          strides_(std::move(strides)), pads_(std::move(pads)) {}
    float getEpsilon() const { return epsilon_; }
    std::vector<size_t> getPads() const { return pads_; }
    std::vector<size_t> getKernels() const { return kernels_; }
    std::vector<size_t> getStrides() const { return strides_; }
    void outTensorShapeGen(OpNode *node, size_t index, TensorShape *shape) override;
};
// Conv2d followed by an activation: the class the reference declares
// (src/op/dlOp/dlOp.h:655-700) but never emits code for.  Only ReLU here.
class Conv2dWithActivationOp : public Conv2dOp {
    activation_type activation_;

  public:
    Conv2dWithActivationOp(std::vector<size_t> &kernels, std::vector<size_t> &strides, std::vector<size_t> &pads,
                           activation_type act)
        : Conv2dOp("Conv2dWithActivation", 3, kernels, strides, pads), activation_(act) {}
    activation_type getActivationType() const { return activation_; }
};
// Conv2d + BatchNormalization (+ Relu): parents input, filter, bias, then the
// batchnorm's scale, bias, mean, var.  swc_hip_conv2dFused_f
class Conv2dBatchNormOp : public Conv2dOp {
    float epsilon_;
    bool relu_;

  public:
    Conv2dBatchNormOp(std::vector<size_t> &kernels, std::vector<size_t> &strides, std::vector<size_t> &pads,
                      float eps, bool relu)
        : Conv2dOp("Conv2dBatchNorm", 7, kernels, strides, pads), epsilon_(eps), relu_(relu) {}
    float getEpsilon() const { return epsilon_; }
    bool hasRelu() const { return relu_; }
};
// ---- training: the loss, the gradient ops the autodiff pass creates, the optimizer step ----
// (reference: src/op/dlOp/dlOp.h:61-75, 121-141, 182-193, 213-222, 243-256, 290-336, 600-640, 715-770)
// parents: logits [m,n], label [m] int32 -> prob [m,n], loss [1]
class MatrixSoftmaxWithLossOp : public Op {
  public:
    MatrixSoftmaxWithLossOp() : Op(DL_OP, 2, 2, "MatrixSoftmaxWithLoss") {}
    void outTensorShapeGen(OpNode *node, size_t index, TensorShape *shape) override;
};
// parents: label, prob -> gradient of the logits
// the older way to train: a label linked to MatrixSoftmax as its second operand (reference:
// src/op/dlOp/dlOpAD.cpp:213-247); parents input, label, output, outputGrad -> inputGrad (, labelGrad: by name only)
class MatrixSoftmaxGradOp : public Op {
  public:
    MatrixSoftmaxGradOp() : Op(DL_OP, 4, 1, "MatrixSoftmaxGrad") {}
};
class MatrixSoftmaxWithLossGradOp : public Op {
  public:
    MatrixSoftmaxWithLossGradOp() : Op(DL_OP, 2, 1, "MatrixSoftmaxWithLossGrad") {}
};
// parents: input, weight, bias, outputGrad -> inputGrad, weightGrad, biasGrad; always lowered to
// Transpose + MatrixMatrixMul (twice) + BatchedReduceAdd
class MatrixMatrixFCBiasGradOp : public Op {
  public:
    MatrixMatrixFCBiasGradOp() : Op(DL_OP, 4, 3, "MatrixMatrixFCBiasGrad") {}
    void lowering(IRGraph *graph, IRNode *node) override;
};
class BatchedReduceAddOp : public Op {    // out[j] = sum over rows of in[r, j]
  public:
    BatchedReduceAddOp() : Op(DL_OP, 1, 1, "BatchedReduceAdd") {}
};
class MatrixTanhGradOp : public Op {      // parents: input, output, outputGrad
  public:
    MatrixTanhGradOp() : Op(DL_OP, 3, 1, "MatrixTanhGrad") {}
};
class ReluGradOp : public Op {            // parents: input, outputGrad
  public:
    ReluGradOp() : Op(DL_OP, 2, 1, "ReluGrad") {}
};
class MaxPoolGradOp : public Op {         // parents: input, output, outputGrad
    std::vector<size_t> kernels_, strides_, pads_;

  public:
    MaxPoolGradOp(const std::vector<size_t> &kernels, const std::vector<size_t> &strides, const std::vector<size_t> &pads)
        : Op(DL_OP, 3, 1, "MaxPoolGrad"), kernels_(kernels), strides_(strides), pads_(pads) {}
    std::vector<size_t> getPads() const { return pads_; }
    std::vector<size_t> getKernels() const { return kernels_; }
    std::vector<size_t> getStrides() const { return strides_; }
};
class Conv2dGradOp : public Op {          // parents: input, filter, outputGrad -> inputGrad, filterGrad, biasGrad
    std::vector<size_t> kernels_, strides_, pads_;
    int group_;

  public:
    Conv2dGradOp(const std::vector<size_t> &kernels, const std::vector<size_t> &strides, const std::vector<size_t> &pads,
                 int group)
        : Op(DL_OP, 3, 3, "Conv2dGrad"), kernels_(kernels), strides_(strides), pads_(pads), group_(group) {}
    std::vector<size_t> getPads() const { return pads_; }
    std::vector<size_t> getKernels() const { return kernels_; }
    std::vector<size_t> getStrides() const { return strides_; }
    size_t getGroup() const { return (size_t)group_; }
};
// parents: parameter, its gradient, its momentum -> the parameter again (same Tensor: updated in place)
class SGDOp : public Op {
    float lr_, decay_, momentum_;
    size_t batch_;

  public:
    SGDOp(float lr, float decay, float momentum, size_t batch)
        : Op(DL_OP, 3, 1, "SGD"), lr_(lr), decay_(decay), momentum_(momentum), batch_(batch) {}
    float getLR() const { return lr_; }
    float getDecay() const { return decay_; }
    float getMomentum() const { return momentum_; }
    size_t getBatch() const { return batch_; }
};

// Conv2d (+ BatchNormalization) + ElementAdd (+ Relu): the last convolution of a residual block with the sum
// and the activation that follow it.  Parents: input, filter, bias, [bn scale, bias, mean, var,] the other
// summand.  swc_hip_conv2dFusedAdd_f
class Conv2dAddOp : public Conv2dOp {
    float epsilon_;
    bool bn_, relu_;

  public:
    Conv2dAddOp(std::vector<size_t> &kernels, std::vector<size_t> &strides, std::vector<size_t> &pads, bool bn, float eps,
                bool relu)
        : Conv2dOp("Conv2dAdd", bn ? 8 : 4, kernels, strides, pads), epsilon_(eps), bn_(bn), relu_(relu) {}
    float getEpsilon() const { return epsilon_; }
    bool hasBatchNorm() const { return bn_; }
    bool hasRelu() const { return relu_; }
};
// Conv2d (+ BatchNormalization) (+ Relu) followed by MaxPool: parents as Conv2d (3) or Conv2dBatchNorm (7); the
// output is the pooled tensor, the convolution's own output never exists.  swc_hip_conv2dFusedMaxpool_f
class Conv2dMaxPoolOp : public Conv2dOp {
    float epsilon_;
    bool bn_, relu_;
    std::vector<size_t> pool_kernels_, pool_strides_, pool_pads_;

  public:
    Conv2dMaxPoolOp(std::vector<size_t> &kernels, std::vector<size_t> &strides, std::vector<size_t> &pads, bool bn, float eps,
                    bool relu, std::vector<size_t> pk, std::vector<size_t> ps, std::vector<size_t> pp)
        : Conv2dOp("Conv2dMaxPool", bn ? 7 : 3, kernels, strides, pads), epsilon_(eps), bn_(bn), relu_(relu),
          pool_kernels_(std::move(pk)), pool_strides_(std::move(ps)), pool_pads_(std::move(pp)) {}
    float getEpsilon() const { return epsilon_; }
    bool hasBatchNorm() const { return bn_; }
    bool hasRelu() const { return relu_; }
    std::vector<size_t> getPoolKernels() const { return pool_kernels_; }
    std::vector<size_t> getPoolStrides() const { return pool_strides_; }
    std::vector<size_t> getPoolPads() const { return pool_pads_; }
    // dims of the convolution's output for an input of `idims` and `oc` filters
    std::vector<size_t> convOutDims(const std::vector<size_t> &idims, size_t oc) const;
    void outTensorShapeGen(OpNode *node, size_t index, TensorShape *shape) override;
};

} // namespace op
} // namespace swc
#endif
