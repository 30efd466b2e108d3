// Compile driver (reference surface: src/engine/Engine.h:17-43).
//
//   Engine e(graph); e.compile(); std::string code = e.genCode();
//
// compile() runs the inference pipeline on the graph in place; with
// Config::hip it ends with the fusion and device-memory lowering passes, and
// genCode() then instantiates HipCodegen (otherwise the CPU Codegen) unless a
// generator was injected with setCodegenerator().
#ifndef SWC_ENGINE_H_
#define SWC_ENGINE_H_
#include <string>

namespace swc {
namespace codegen {
class Codegen;
}
class IRGraph;

class Engine {
    IRGraph *graph_;
    codegen::Codegen *generator_{nullptr};

  public:
    Engine() = delete;
    explicit Engine(IRGraph *graph) : graph_(graph) {}
    virtual ~Engine() {}
    IRGraph *getGraph() { return graph_; }
    virtual void compile();
    void runInferPasses();
    void runTrainPasses();
    // HIP target only: fusion (if enabled) + device placement + renaming
    virtual void transformForHIP();
    std::string genCode();
    void setCodegenerator(codegen::Codegen *codegen) { generator_ = codegen; }
};
} // namespace swc
#endif
