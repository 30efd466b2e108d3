// Per-node annotation the passes write and the code generators read: the op
// type name that selects an emitter, the lowering mark, the output mark that
// protects a node from dead-code elimination, and the DEVICE the node lives on
// (reference surface: src/pass/Label.h:17-67).
#ifndef SWC_LABEL_H_
#define SWC_LABEL_H_
#include <string>

#include "../common.h"

namespace swc {
class Label {
    std::string nodeName_, typeName_;
    int toLower_{0}, train_{0}, isOut_{0};
    TensorInitType initType_{TensorInitType::NONE};
    Device dev_;

  public:
    virtual ~Label() {}
    void destroy() {}
    void setNodeNameLabel(std::string s) { nodeName_ = std::move(s); }
    void setTypeNameLabel(std::string s) { typeName_ = std::move(s); }
    void setTensorInitTypeLabel(TensorInitType t) { initType_ = t; }
    void setDeviceLabel(Device d) { dev_ = d; }
    void setDeviceLabel(int rank, DeviceType type, int id) { dev_ = Device(rank, type, id); }
    void setLowerMark() { toLower_ = 1; }
    void clearLowerMark() { toLower_ = 0; }
    int getLowerMark() const { return toLower_; }
    void setTraining(int t) { train_ = t; }
    bool needTraining() const { return train_ == 1; }
    void setIsOut(int mark = 1) { isOut_ = mark; }
    int getIsOut() const { return isOut_; }
    std::string getNodeNameLabel() const { return nodeName_; }
    std::string getTypeNameLabel() const { return typeName_; }
    TensorInitType getTensorInitTypeLabel() const { return initType_; }
    Device getDeviceLabel() const { return dev_; }
};
} // namespace swc
#endif
