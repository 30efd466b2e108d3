// Node of the bipartite tensor/op DAG.  Parent order is operand order, child
// order is result order (reference surface: src/graphIR/IRNode.h:28-170).
#ifndef SWC_IRNODE_H_
#define SWC_IRNODE_H_
#include <algorithm>
#include <iostream>
#include <string>
#include <unordered_map>
#include <vector>

#include "../common.h"
#include "../pass/Label.h"

namespace swc {
class IRGraph;

class IRNode {
    std::vector<IRNode *> parents_, children_;
    std::string name_;
    NodeType nodeType_;
    int topologyId_{0};
    Label *label_;
    bool external_{false};

  public:
    IRNode(NodeType type, std::string name, IRNode *parent = nullptr)
        : name_(std::move(name)), nodeType_(type), label_(new Label()) {
        if (parent) exlinkUpperNode(parent);
    }
    virtual ~IRNode() {}

    template <typename... Ts> void pushParentNode(Ts... nodes) { (parents_.push_back(nodes), ...); }
    template <typename... Ts> void pushChildNode(Ts... nodes) { (children_.push_back(nodes), ...); }
    template <typename... Ts> void delParentNode(Ts... nodes) { (eraseFrom(parents_, nodes), ...); }
    template <typename... Ts> void delChildNode(Ts... nodes) { (eraseFrom(children_, nodes), ...); }
    // link: each argument becomes a parent of this node, in order
    template <typename... Ts> void exlinkUpperNode(Ts... uppers) { (linkOne(uppers), ...); }
    template <typename... Ts> void destroyUpperNode(Ts... uppers) { (unlinkOne(uppers), ...); }

    const std::vector<IRNode *> &getParentNodes() const { return parents_; }
    const std::vector<IRNode *> &getChildNodes() const { return children_; }
    std::vector<IRNode *> &getParentNodes() { return parents_; }
    std::vector<IRNode *> &getChildNodes() { return children_; }
    IRNode *getParentNode(int i) const { return parents_.at(i); }
    IRNode *getChildNode(int i) const { return children_.at(i); }
    const std::string name() const { return name_; }
    void setName(std::string n) { name_ = std::move(n); }
    int parentNum() const { return (int)parents_.size(); }
    int childNum() const { return (int)children_.size(); }
    int topologyId() const { return topologyId_; }
    void setTopologyId(int id) { topologyId_ = id; }
    NodeType nodeType() const { return nodeType_; }
    void setNodeType(NodeType t) { nodeType_ = t; }

    // `node` takes this node's place in every neighbour's operand/result list,
    // at the same position.
    void replaceUseKeepOrder(IRNode *node) {
        for (IRNode *p : parents_) {
            std::replace(p->children_.begin(), p->children_.end(), static_cast<IRNode *>(this), node);
            node->parents_.push_back(p);
        }
        for (IRNode *c : children_) {
            std::replace(c->parents_.begin(), c->parents_.end(), static_cast<IRNode *>(this), node);
            node->children_.push_back(c);
        }
        parents_.clear();
        children_.clear();
    }
    // every edge this -> spec_child becomes node -> spec_child (same operand slots)
    void replaceUseKeepOrder(IRNode *spec_child, IRNode *node) {
        const auto n = std::count(children_.begin(), children_.end(), spec_child);
        if (n == 0) return;
        children_.erase(std::remove(children_.begin(), children_.end(), spec_child), children_.end());
        std::replace(spec_child->parents_.begin(), spec_child->parents_.end(), static_cast<IRNode *>(this), node);
        for (auto i = n; i > 0; --i) node->children_.push_back(spec_child);
    }
    void replaceOutKeepOrder(IRNode *node, int n) {
        IRNode *old = children_.at(n);
        children_[n] = node;
        node->parents_.push_back(this);
        eraseFrom(old->parents_, this);
    }

    void setLabel(Label *l) { label_ = l; }
    Label *getLabel() const { return label_; }
    void setExternal(bool f) { external_ = f; }
    bool isExternal() const { return external_; }

    virtual IRNode *clone() const = 0;
    virtual IRNode *deepClone() const = 0;
    virtual void destroy() {}
    virtual void checkValid() {}

  private:
    static void eraseFrom(std::vector<IRNode *> &v, IRNode *n) {
        auto it = std::find(v.begin(), v.end(), n);
        if (it != v.end()) v.erase(it);
        else std::cout << "IRNode: link to " << n->name() << " not found" << std::endl;
    }
    void linkOne(IRNode *upper) {
        parents_.push_back(upper);
        upper->children_.push_back(this);
    }
    void unlinkOne(IRNode *upper) {
        eraseFrom(parents_, upper);
        eraseFrom(upper->children_, this);
    }
};
} // namespace swc
#endif
