// Container of the tensor/op DAG plus the derived views the passes and code
// generators use: inputs/outputs, topological levels, per-graph Config and
// device (reference surface: src/graphIR/IRGraph.h:26-200).
#ifndef SWC_IRGRAPH_H_
#define SWC_IRGRAPH_H_
#include <iostream>
#include <string>
#include <vector>

#include "../common.h"

namespace swc {
class TensorNode;
class OpNode;
class IRNode;

class IRGraph {
    std::vector<TensorNode *> tensors_;
    std::vector<OpNode *> ops_;
    std::vector<IRNode *> inNodes_, outNodes_, logicalOutNodes_;
    std::vector<std::vector<IRNode *>> levels_;
    std::vector<TensorNode *> displayNodes_;
    TensorNode *trainData_{nullptr}, *trainLabel_{nullptr};
    TensorNode *inferData_{nullptr}, *inferLabel_{nullptr};
    Config config_;
    Device dev_;

    template <typename V, typename N> static void eraseNode(V &vec, N *node, const char *what);

  public:
    IRGraph() {}
    ~IRGraph() {}

    TensorNode *getTensorNode(int i) const { return tensors_.at(i); }
    OpNode *getOpNode(int i) const { return ops_.at(i); }
    IRNode *getInNode(int i) const { return inNodes_.at(i); }
    IRNode *getOutNode(int i) const { return outNodes_.at(i); }
    int tensorNodeNum() const { return (int)tensors_.size(); }
    int opNodeNum() const { return (int)ops_.size(); }
    int inNodeNum() const { return (int)inNodes_.size(); }
    int outNodeNum() const { return (int)outNodes_.size(); }
    int topologyNum() const { return (int)levels_.size(); }
    int getNumInTopoLevel(int i) const { return (int)levels_.at(i).size(); }
    std::vector<IRNode *> getNodeInTopoLevel(int i) const { return levels_.at(i); }
    IRNode *getNodeInTopo(int i, int j) const { return levels_.at(i).at(j); }
    IRNode *getNodeByName(std::string name) const;

    template <typename... Ts> void pushTensorNode(Ts... nodes) { (tensors_.push_back(nodes), ...); }
    template <typename... Ts> void pushOpNode(Ts... nodes) { (ops_.push_back(nodes), ...); }
    template <typename... Ts> void delTensorNode(Ts... nodes) { (eraseNode(tensors_, nodes, "tensor"), ...); }
    template <typename... Ts> void delOpNode(Ts... nodes) { (eraseNode(ops_, nodes, "op"), ...); }
    template <typename... Ts> void pushInNode(Ts... nodes) { (inNodes_.push_back(nodes), ...); }
    template <typename... Ts> void pushOutNode(Ts... nodes) { (outNodes_.push_back(nodes), ...); }
    void clearOutNodes() {
        clearOutMark();
        outNodes_.clear();
    }

    // Nodes without parents / without children.
    void findInOut();
    // Levelises the DAG: level(n) = 1 + max level of its parents, inputs at 0.
    void updateTopology();
    // Fills in {0}-shaped (unset) output tensors from the ops' shape rules,
    // walking in topological order; also creates missing Tensor objects.
    void initTensorNodes();

    void setOutMark();          // marks outNodes_ (and display/logical outs) as graph outputs
    void setLogicalOutMark();
    void clearOutMark();

    void setDeviceLabel(Device dev);   // labels the graph and every node in it
    Device getDeviceLabel() const { return dev_; }

    void setTrainDataNodes(TensorNode *label, TensorNode *data) { trainLabel_ = label; trainData_ = data; }
    TensorNode *getTrainLabelNode() const { return trainLabel_; }
    TensorNode *getTrainDataNode() const { return trainData_; }
    void setInferDataNodes(TensorNode *label, TensorNode *data) { inferLabel_ = label; inferData_ = data; }
    TensorNode *getInferLabelNode() const { return inferLabel_; }
    TensorNode *getInferDataNode() const { return inferData_; }

    template <typename... Ts> void addDisplayTensorNodes(Ts... nodes) {
        (displayNodes_.push_back(nodes), ...);
        (logicalOutNodes_.push_back(nodes), ...);
    }
    std::vector<TensorNode *> getDisplayTensorNodes() const { return displayNodes_; }
    template <typename... Ts> void addLogicalOutNodes(Ts... nodes) { (logicalOutNodes_.push_back(nodes), ...); }
    std::vector<IRNode *> getLogicalOutNodes() const { return logicalOutNodes_; }

    void setConfig(Config c) { config_ = c; }
    Config getConfig() const { return config_; }

    // Structural copy: every node cloned (tensor metadata deep-copied), links,
    // in/out lists, config and device preserved.
    // Traffic between the ranks of a parallel program (reference: src/graphIR/IRGraph.h:165-170).  A program for one
    // device exchanges nothing.
    size_t getCommCost() const { return 0; }
    std::string getCommTrace() const { return ""; }
    IRGraph *clone() const;
    void copyTo(IRGraph *empty) const;   // the same copy into a graph the caller has made

    // The part of the graph between tensor `in` and tensor `out` moves into a nested graph behind a new SubGraph
    // op node (reference: src/graphIR/IRGraph.cpp:99-223): inside, `in`, `out` and every parameter the part reads
    // are represented by external mirror nodes of the same Tensor, joined to "<name>_sub" working copies by
    // Scatter nodes (run-once for parameters) and a Gather node; outside, the SubGraph node reads `in` and the
    // parameters and produces `out`.  Returns the node, or null if `out` does not depend on `in`.
    OpNode *extractSubGraph(TensorNode *in, TensorNode *out);
    // extractSubGraph, then `num` such SubGraph nodes side by side, each over 1/num of `in` along axis 0
    // (reference: src/graphIR/IRGraph.cpp:47-97; SLICE along axis 0 only, as there).
    bool buildSubGraphs(TensorNode *in, TensorNode *out, ParallelStrategy strategy, int axis = 0, int num = 2);
    // Code generation on one device: every SubGraph node is replaced by the nodes of its nested graph (nested
    // ones first), a mirror node becoming the outer node of the same Tensor, and every GPU label becomes device
    // `device` — the op sequence a generator that recursed into the nested graphs at the SubGraph node's place
    // (reference: src/codegen/Codegen.cpp:1035-1077) would emit.  Returns the number of nodes replaced.
    int inlineSubGraphs(int device = 0);
};

template <typename V, typename N> void IRGraph::eraseNode(V &vec, N *node, const char *what) {
    for (auto it = vec.begin(); it != vec.end(); ++it)
        if (static_cast<const void *>(*it) == static_cast<const void *>(node)) {
            vec.erase(it);
            return;
        }
    std::cout << "IRGraph: " << what << " node to delete not found" << std::endl;
}

} // namespace swc
#endif
