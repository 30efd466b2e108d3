#include "Engine.h"

#include <cstdlib>

#include "../codegen/Codegen.h"
#include "../graphIR/IRGraph.h"
#include "../graphIR/OpNode.h"
#include "../graphIR/TensorNode.h"
#include "../pass/passes.h"

namespace swc {

using namespace pass;

void Engine::compile() {
    // SWC_TARGET=hip in the environment retargets a program that was written for the CPU target without touching
    // its source: the same as Config::hip = true in it
    if (const char *target = std::getenv("SWC_TARGET")) {
        if (std::string(target) == "hip") {
            Config retargeted = graph_->getConfig();
            retargeted.hip = true;
            graph_->setConfig(retargeted);
        }
    }
    const Config cfg = graph_->getConfig();
    if (cfg.mpi || cfg.mkldnn || cfg.cuda) {
        SWLOG_ERROR << "Engine: only the single-device pipelines (CPU or Config::hip) are part of this build" << std::endl;
        std::abort();
    }
    if (cfg.train_mode) runTrainPasses();
    else runInferPasses();
    if (cfg.hip) transformForHIP();
}

// autodiff on the graph itself, then labeling -> lowering -> labeling -> renaming -> elimination
// (reference order: src/engine/Engine.cpp:88-126).  The updated parameters are the graph's outputs; what
// leads to none of them or to a displayed tensor (the loss) is removed.
void Engine::runTrainPasses() {
    const Config cfg = graph_->getConfig();
    AutodiffPass autodiff(graph_);
    autodiff.getMethods(cfg.train_config.optimizer, cfg.train_config.lr, cfg.train_config.decay, cfg.train_config.momentum,
                        cfg.train_config.batch);
    autodiff.run();
    LabelingPass labeling(graph_);
    LoweringPass lowering(graph_);
    RenamingNodePass renaming(graph_);
    PassManager pm;
    pm.add(&labeling);
    pm.add(&lowering);
    pm.add(&labeling);
    pm.add(&renaming);
    pm.run();
    graph_->findInOut();
    graph_->updateTopology();
    graph_->clearOutMark();
    graph_->setLogicalOutMark();
    for (TensorNode *t : graph_->getDisplayTensorNodes()) t->getLabel()->setIsOut(1);
    EliminationPass elimination(graph_);
    elimination.run();
}

// labeling -> lowering -> labeling (new nodes) -> renaming, then refresh the
// derived views and mark the outputs (reference order: src/engine/Engine.cpp:61-86)
void Engine::runInferPasses() {
    LabelingPass labeling(graph_);
    LoweringPass lowering(graph_);
    RenamingNodePass renaming(graph_);
    PassManager pm;
    pm.add(&labeling);
    pm.add(&lowering);
    pm.add(&labeling);
    pm.add(&renaming);
    pm.run();
    graph_->findInOut();
    graph_->updateTopology();
    graph_->setOutMark();
}

void Engine::transformForHIP() {
    const Config cfg = graph_->getConfig();
    if (cfg.hip_fusion) {
        HipFusionPass fusion(graph_);
        fusion.run();
    }
    DeviceMemoryLoweringPass placement(graph_, cfg.hip_device);
    placement.run();
    LabelingPass labeling(graph_);
    labeling.run();
    graph_->findInOut();
    graph_->updateTopology();
}

std::string Engine::genCode() {
    Config cfg = graph_->getConfig();
    if (!generator_) generator_ = cfg.hip ? new codegen::HipCodegen(graph_, cfg) : new codegen::Codegen(graph_, cfg);
    return generator_->generate();
}

} // namespace swc
