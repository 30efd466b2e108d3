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
    // what LabelingPass copies from the node
    struct Names {
        std::string node;   // the node's name at labeling time
        std::string type;   // op nodes: Op::getOpName(); a generator dispatches on this, so a pass may retarget an op by renaming it
    } names_;
    // marks: 0 / 1, kept as int because callers pass and compare ints
    struct Marks {
        int lower = 0;      // LoweringPass replaces the op by the nodes of Op::lowering()
        int train = 0;      // tensor nodes: the parameter is updated by the optimizer
        int out = 0;        // EliminationPass keeps the node and what it depends on
    } marks_;
    TensorInitType init_ = TensorInitType::NONE;   // tensor nodes: how the tensor gets its first value
    Device where_;                                 // arena and generator the node belongs to (default: host, rank 0)

  public:
    virtual ~Label() {}
    void destroy() {}

    // names
    void setNodeNameLabel(std::string s) { names_.node.swap(s); }
    std::string getNodeNameLabel() const { return names_.node; }
    void setTypeNameLabel(std::string s) { names_.type.swap(s); }
    std::string getTypeNameLabel() const { return names_.type; }

    // initialiser kind of a tensor node
    void setTensorInitTypeLabel(TensorInitType t) { init_ = t; }
    TensorInitType getTensorInitTypeLabel() const { return init_; }

    // placement: Device{rank, CPU|GPU, id}; DeviceMemoryLoweringPass sets GPU labels on what runs on the device
    void setDeviceLabel(Device d) { where_ = d; }
    void setDeviceLabel(int rank, DeviceType type, int id) { where_ = Device(rank, type, id); }
    Device getDeviceLabel() const { return where_; }

    // marks
    void setLowerMark() { marks_.lower = 1; }
    void clearLowerMark() { marks_.lower = 0; }
    int getLowerMark() const { return marks_.lower; }
    void setTraining(int t) { marks_.train = t; }
    bool needTraining() const { return marks_.train == 1; }
    void setIsOut(int mark = 1) { marks_.out = mark; }
    int getIsOut() const { return marks_.out; }
};
} // namespace swc
#endif
