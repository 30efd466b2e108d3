// Pass interface and FIFO pass manager (reference surface:
// src/pass/OptimizePass.h:15-24, src/pass/Optimizer.h:21-53).
#ifndef SWC_OPTIMIZEPASS_H_
#define SWC_OPTIMIZEPASS_H_
#include <iostream>
#include <queue>

#include "../graphIR/IRGraph.h"

namespace swc {
namespace pass {

class OptimizePass {
  protected:
    IRGraph *_graph;

  public:
    explicit OptimizePass(IRGraph *graph) : _graph(graph) {}
    virtual ~OptimizePass() {}
    void setGraph(IRGraph *graph) { _graph = graph; }
    virtual void run() {}
};

class PassManager {
    std::queue<OptimizePass *> queue_;

  public:
    void add(OptimizePass *p) { queue_.push(p); }
    void run() {
        for (; !queue_.empty(); queue_.pop()) queue_.front()->run();
    }
};

// labeling -> lowering -> labeling, the fixed pipeline user code may call directly
class Optimizer {
    IRGraph *_graph;

  public:
    explicit Optimizer(IRGraph *graph) : _graph(graph) {}
    void setGraph(IRGraph *graph) { _graph = graph; }
    void runOptimizer();
};

} // namespace pass
} // namespace swc
#endif
