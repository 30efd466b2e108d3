// Tensor metadata of the SWC API: shape, dtype, layout and how the generated
// program initialises the buffer.  A Tensor owns no data; codegen assigns it an
// arena offset.  (Reference surface: src/tensor/tensor.h:19-179; 4-D tensors
// default to NHWC, :96-98.)
#ifndef SWC_TENSOR_H_
#define SWC_TENSOR_H_

#include <cassert>
#include <initializer_list>
#include <string>
#include <utility>
#include <vector>

#include "../common.h"

namespace swc {

class TensorShape {
    std::vector<size_t> dims_;

  public:
    explicit TensorShape(std::vector<size_t> *shape) : dims_(*shape) {}
    explicit TensorShape(const std::vector<size_t> &shape) : dims_(shape) {}
    TensorShape(const std::initializer_list<size_t> &shape) : dims_(shape) {}
    void destroy() {}
    int getNDim() const { return (int)dims_.size(); }
    size_t getDim(int idx) const { return dims_.at(idx); }
    const std::vector<size_t> &dims() const { return dims_; }
    size_t size() const {
        size_t n = 1;
        for (size_t d : dims_) n *= d;
        return n;
    }
    void setShape(const std::vector<size_t> &shape) { dims_ = shape; }
    // dims permuted so that result[i] = dims[shuffle[i]]
    TensorShape *getShuffledTensorShape(const std::vector<size_t> &shuffle) const {
        std::vector<size_t> out;
        for (size_t s : shuffle) out.push_back(dims_.at(s));
        return new TensorShape(out);
    }
};

class TensorInitInfo {
    std::string file_;
    float constant_{0};
    float filterSize_{3};
    size_t offset_{0};

  public:
    std::string getFilePath() const { return file_; }
    float getConstant() const { return constant_; }
    float getFilterSize() const { return filterSize_; }
    size_t getOffset() const { return offset_; }
    void setFilePath(std::string f) { file_ = std::move(f); }
    void setConstant(float c) { constant_ = c; }
    void setFilterSize(float f) { filterSize_ = f; }
    void setOffset(size_t o) { offset_ = o; }
};

class Tensor {
    DataType dataType_{DataType::Float_t};
    TensorShape *shape_{nullptr};
    mem_layout_t mem_layout_{layout_default};
    TensorInitType initType_{TensorInitType::NONE};
    TensorInitInfo initInfo_;
    int train_{0};

    void pickLayout(mem_layout_t layout) {
        mem_layout_ = (layout == layout_default && shape_ && shape_->getNDim() == 4) ? layout_nhwc : layout;
    }

  public:
    Tensor() = default;
    explicit Tensor(TensorShape *shape, DataType dtype = DataType::Float_t, mem_layout_t layout = layout_default)
        : dataType_(dtype), shape_(shape) {
        pickLayout(layout);
    }
    Tensor(const std::initializer_list<size_t> &shape, DataType dtype = DataType::Float_t,
           mem_layout_t layout = layout_default)
        : dataType_(dtype), shape_(new TensorShape(shape)) {
        pickLayout(layout);
    }
    void destroy() {}
    void reset(TensorShape *shape, DataType dtype = DataType::Float_t, mem_layout_t layout = layout_default) {
        shape_ = shape;
        dataType_ = dtype;
        pickLayout(layout);
    }
    Tensor *clone() const {
        Tensor *t = new Tensor(new TensorShape(shape_->dims()), dataType_, mem_layout_);
        t->initType_ = initType_;
        t->initInfo_ = initInfo_;
        t->train_ = train_;
        return t;
    }
    TensorShape *getShuffledTensorShape(const std::vector<size_t> &shuffle) const {
        return shape_->getShuffledTensorShape(shuffle);
    }
    std::vector<size_t> getShuffledDims(const std::vector<size_t> &shuffle) const {
        std::vector<size_t> out;
        for (size_t s : shuffle) out.push_back(getDim((int)s));
        return out;
    }
    DataType getDataType() const { return dataType_; }
    int getNDim() const { return shape_->getNDim(); }
    size_t getDim(int d) const { return shape_->getDim(d); }
    const std::vector<size_t> getDims() const { return shape_->dims(); }
    // rows = product of the first n dims, cols = product of the rest
    std::pair<size_t, size_t> viewAs2D(int n) const {
        size_t rows = 1, cols = 1;
        for (int i = 0; i < getNDim(); ++i) (i < n ? rows : cols) *= getDim(i);
        return {rows, cols};
    }
    void setTensorInit(TensorInitType type, float value = 0) {
        initType_ = type;
        if (type == TensorInitType::CONSTANT) initInfo_.setConstant(value);
        if (type == TensorInitType::XAVIER) initInfo_.setFilterSize(value);
    }
    void setTensorInit(TensorInitType type, std::string file, size_t offset = 0) {
        initType_ = type;
        initInfo_.setFilePath(std::move(file));
        initInfo_.setOffset(offset);
    }
    void setTensorInit(TensorInitType type, TensorInitInfo info) {
        initType_ = type;
        initInfo_ = std::move(info);
    }
    TensorInitType getTensorInitType() const { return initType_; }
    TensorInitInfo getTensorInitInfo() const { return initInfo_; }
    void setTraining(int t) { train_ = t; }
    int getTraining() const { return train_; }
    TensorShape *getTensorShape() const { return shape_; }
    size_t size() const { return shape_->size(); }
    size_t getSizeInBytes() const {
        switch (dataType_) {
        case DataType::Double_t: return size() * 8;
        case DataType::Int8_t: return size();
        default: return size() * 4;
        }
    }
    void setMemLayout(mem_layout_t l) { mem_layout_ = l; }
    mem_layout_t getMemLayout() const { return mem_layout_; }
    std::string getMemLayoutTag() const {
        switch (mem_layout_) {
        case layout_nchw: return "nchw";
        case layout_nhwc: return "nhwc";
        case layout_nc: return "nc";
        case layout_cn: return "cn";
        default: break;
        }
        switch (getNDim()) {
        case 1: return "x";
        case 2: return "xy";
        default: return "default";
        }
    }
};

} // namespace swc
#endif
