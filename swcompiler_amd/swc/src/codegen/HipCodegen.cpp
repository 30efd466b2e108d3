// MI355X code generator: prints a host program that drives libswc_hip.
//
// Input is a graph that DeviceMemoryLoweringPass has placed: compute ops and
// their tensors carry a GPU label, Scatter/Gather nodes mark every transfer.
// The program owns two arenas — host (malloc) and device (swc_hip_malloc, every
// tensor on a 256-byte boundary) — uploads parameters once, then per iteration
// issues one asynchronous swc_hip_* call per op node on the library's single
// stream and synchronises only where a Gather brings a result back.
#include <array>
#include <cassert>
#include <cstdlib>
#include <iomanip>
#include <set>
#include <sstream>

#include "../graphIR/IRGraph.h"
#include "../graphIR/OpNode.h"
#include "../graphIR/TensorNode.h"
#include "../op/ops.h"
#include "Codegen.h"

namespace swc {
namespace codegen {

using namespace swc::op;

static Tensor *T(IRNode *n) { return static_cast<TensorNode *>(n)->getTensor(); }

void HipCodegen::initMakefileBuilder() {
    // SWC_HIP_ROOT = the checkout that holds include/swc_hip.h and swcompiler_amd/libswc_hip.so
    makefile_builder_.setCXXCompiler("/usr/bin/c++");
    makefile_builder_.addCXXFlag("-std=c++11");
    makefile_builder_.addCXXFlag("-O2");
    makefile_builder_.addIncDir("$(SWC_HIP_ROOT)/include");
    makefile_builder_.addLibDir("$(SWC_HIP_ROOT)/swcompiler_amd");
    makefile_builder_.addLib("swc_hip");
    makefile_builder_.addCXXSrc("Graph.cpp");
    swmakefile_builder_ = makefile_builder_;
}

void HipCodegen::emitHeader() {
    headerWriter_ << "// Graph.cpp -- generated from an IRGraph with " << graph_->tensorNodeNum() << " tensor nodes and "
                  << graph_->opNodeNum() << " op nodes (HIP target, " << device_.arch << ")\n";
    headerWriter_ << "#include <algorithm>\n#include <iostream>\n#include <random>\n#include <cstdlib>\n#include <cstdio>\n#include <cstring>\n#include <cmath>\n"
                  << "#include <sys/time.h>\n"
                  << "#include \"swc_host_utils.h\"\n#include \"swc_hip.h\"\n";
    if (config_.train_mode) headerWriter_ << "#include \"swc_snapshot.h\"\n";
    headerWriter_ << "#define SWC_HIP_CHECK(call) do { if ((call) != 0) { std::fprintf(stderr, \"%s:%d: %s\\n  %s\\n\", "
                     "__FILE__, __LINE__, #call, swc_hip_last_error()); std::exit(1); } } while (0)\n";
}

void HipCodegen::emitEnvInit() {
    writer_ << "SWC_HIP_CHECK(swc_hip_init(" << config_.hip_device << "));\n";
}

void HipCodegen::emitEnvFinalize() {
    writer_ << "SWC_HIP_CHECK(swc_hip_shutdown());\n";
    writer_ << "return 0;\n";
}

void HipCodegen::allocateMemAddr() {
    Codegen::allocateMemAddr();
    const uint64_t need = dev_allocator_map_.at(Device(0, DeviceType::GPU, config_.hip_device))->getMemAllocated();
    if (need > device_.hbmBytes) {
        SWLOG_ERROR << "graph needs " << need << " bytes of device memory, more than one MI355X holds" << std::endl;
        std::abort();
    }
}

// Some FC and convolution calls cut their work along K and keep partial results in a workspace: the program
// asks the library how much each of its calls needs and provides the maximum, so that no op allocates.
void HipCodegen::emitWorkspace() {
    std::vector<std::string> queries;
    for (int i = 0; i < graph_->opNodeNum(); ++i) {
        OpNode *op = graph_->getOpNode(i);
        if (op->getLabel()->getDeviceLabel().type != DeviceType::GPU) continue;   // (runable() counts its calls: not asked here)
        const std::string type = op->getOp()->getOpName();
        auto T = [&](int j) { return static_cast<TensorNode *>(op->getParentNode(j))->getTensor(); };
        std::ostringstream q;
        if (type == "MatrixMatrixMul" || type == "MatrixMatrixFCBias" || type == "MatrixMatrixFCBiasRelu" ||
            type == "MatrixMatrixFCBiasSoftmax") {
            Tensor *x = T(0), *w = T(1);
            q << "gpu0_ws_bytes = std::max(gpu0_ws_bytes, swc_hip_gemm_workspace_bytes(" << x->size() / w->getDim(0) << ", "
              << w->getDim(1) << ", " << w->getDim(0) << "));\n";
        } else if (type == "Conv2d" || type == "Conv2dWithActivation" || type == "Conv2dBatchNorm" || type == "Conv2dAdd") {
            auto *conv = static_cast<Conv2dOp *>(op->getOp());
            Tensor *y = static_cast<TensorNode *>(op->getChildNode(0))->getTensor();
            q << "{\n"
              << arrayDef("o", y->getDims()) << arrayDef("i", T(0)->getDims()) << arrayDef("f", T(1)->getDims())
              << arrayDef("k", conv->getKernels()) << arrayDef("s", conv->getStrides()) << arrayDef("p", conv->getPads())
              << "gpu0_ws_bytes = std::max(gpu0_ws_bytes, swc_hip_conv2d_workspace_bytes(o, i, f, k, s, p, "
              << conv->getGroup() << "));\n}\n";
        } else if (type == "Conv2dMaxPool") {
            auto *conv = static_cast<Conv2dMaxPoolOp *>(op->getOp());
            Tensor *y = static_cast<TensorNode *>(op->getChildNode(0))->getTensor();
            q << "{\n"
              << arrayDef("o", conv->convOutDims(T(0)->getDims(), T(1)->getDim(0))) << arrayDef("i", T(0)->getDims())
              << arrayDef("f", T(1)->getDims()) << arrayDef("k", conv->getKernels()) << arrayDef("s", conv->getStrides())
              << arrayDef("p", conv->getPads()) << arrayDef("po", y->getDims()) << arrayDef("pk", conv->getPoolKernels())
              << arrayDef("ps", conv->getPoolStrides()) << arrayDef("pp", conv->getPoolPads())
              << "gpu0_ws_bytes = std::max(gpu0_ws_bytes, swc_hip_conv2dFusedMaxpool_workspace_bytes(o, i, f, k, s, p, "
              << conv->getGroup() << ", po, pk, ps, pp));\n}\n";
        } else if (type == "Conv2dGrad") {   // parents: input, filter, outputGrad
            auto *conv = static_cast<Conv2dGradOp *>(op->getOp());
            q << "{\n"
              << arrayDef("o", T(2)->getDims()) << arrayDef("i", T(0)->getDims()) << arrayDef("f", T(1)->getDims())
              << arrayDef("k", conv->getKernels()) << arrayDef("s", conv->getStrides()) << arrayDef("p", conv->getPads())
              << "gpu0_ws_bytes = std::max(gpu0_ws_bytes, swc_hip_conv2dGrad_workspace_bytes(o, i, f, k, s, p, "
              << conv->getGroup() << "));\n}\n";
        } else if (type == "MatrixSoftmaxWithLoss") {
            q << "gpu0_ws_bytes = std::max(gpu0_ws_bytes, swc_hip_matrixSoftmaxWithLoss_workspace_bytes(" << T(0)->getDim(0)
              << ", " << T(0)->getDim(1) << "));\n";
        } else {
            continue;
        }
        queries.push_back(q.str());
    }
    has_workspace_ = !queries.empty();
    if (queries.empty()) return;
    writer_ << "size_t gpu0_ws_bytes = 0;\n";
    for (auto &q : queries) writer_ << q;
    writer_ << "void *gpu0_ws = gpu0_ws_bytes ? swc_hip_malloc(gpu0_ws_bytes) : nullptr;\n"
            << "if (gpu0_ws_bytes && !gpu0_ws) { std::fprintf(stderr, \"%s\\n\", swc_hip_last_error()); return 1; }\n"
            << "if (gpu0_ws) SWC_HIP_CHECK(swc_hip_set_workspace(gpu0_ws, gpu0_ws_bytes));\n";
}

void HipCodegen::emitMemAllocations() {
    emitWorkspace();   // ops never allocate: the program sizes the scratch memory of all its calls, gradients included
    for (auto &a : mem_allocators_) {
        if (!a->getMemAllocated()) continue;
        if (a->getDevice().type == DeviceType::CPU) {
            // page-locked: the per-iteration uploads and downloads run at the rate of the link
            writer_ << a->getBasePtrName() << " = (char*)swc_hip_host_malloc(" << a->getMemAllocated() << ");\n";
            writer_ << "if (!" << a->getBasePtrName() << ") { std::fprintf(stderr, \"%s\\n\", swc_hip_last_error()); "
                    << "return 1; }\n";
        } else {
            writer_ << a->getBasePtrName() << " = (char*)swc_hip_malloc(" << a->getMemAllocated() << ");\n";
            writer_ << "if (!" << a->getBasePtrName() << ") { std::fprintf(stderr, \"%s\\n\", swc_hip_last_error()); "
                    << "return 1; }\n";
        }
        // training: gradients start from zeros wherever a kernel leaves part of one unwritten (the bias
        // gradient of an FC layer, see BatchedReduceAdd) — what fresh pages give the CPU program
        if (config_.train_mode) {
            if (a->getDevice().type == DeviceType::CPU)
                writer_ << "std::memset(" << a->getBasePtrName() << ", 0, " << a->getMemAllocated() << ");\n";
            else
                writer_ << "SWC_HIP_CHECK(swc_hip_fill_f(reinterpret_cast<float*>(" << a->getBasePtrName() << "), 0.f, "
                        << a->getMemAllocated() / 4 << "));\n";
        }
    }
    writer_ << "\n";
}

// Host tensors are initialised as on the CPU target; a device tensor with an
// initialiser of its own (no host twin) is filled on the device; parameter
// uploads (run-once Scatter nodes) follow in graph order.
void HipCodegen::emitTensorInitializations() {
    std::vector<OpNode *> uploads;
    emitSnapshotRestoreBegin();
    for (TensorNode *tn : decl_order_) {
        Tensor *t = tn->getTensor();
        const std::string name = tensors_name_map_.at(t);
        const bool onGpu = tn->getLabel()->getDeviceLabel().type == DeviceType::GPU;
        const TensorInitInfo info = t->getTensorInitInfo();
        if (!onGpu) writer_ << restoreGuard(t);
        switch (t->getTensorInitType()) {
        case TensorInitType::PARENTOP:   // filled by its run-once producer, below
            break;
        case TensorInitType::CONSTANT:
        case TensorInitType::ZERO:
            if (!onGpu) {
                const float v = t->getTensorInitType() == TensorInitType::ZERO ? 0.f : info.getConstant();
                writer_ << "initTensorConstant(" << name << ", " << t->size() << ", " << v << ");\n";
            }
            break;   // device tensors: emitDeviceFills()
        case TensorInitType::XAVIER:
            assert(!onGpu);
            writer_ << "initTensorXavier(" << name << ", " << t->size() << ", " << info.getFilterSize() << ");\n";
            break;
        case TensorInitType::FILE:
            assert(!onGpu);
            writer_ << "load(" << name << ", " << t->size() << ", " << info.getOffset() << ", \"" << info.getFilePath()
                    << "\");\n";
            break;
        default:
            break;
        }
    }
    emitSnapshotRestoreEnd();
    emitDeviceFills();
    // every run-once op (parameter uploads), in topological order; runable() lets each through once
    for (int i = 0; i < graph_->topologyNum(); ++i)
        for (int j = 0; j < graph_->getNumInTopoLevel(i); ++j) {
            IRNode *node = graph_->getNodeInTopo(i, j);
            if (node->nodeType() == OP_NODE && static_cast<OpNode *>(node)->isRunOnce())
                uploads.push_back(static_cast<OpNode *>(node));
        }
    if (!uploads.empty()) writer_ << "// one-time parameter upload\n";
    for (OpNode *u : uploads) dispatchOpNode(u);
    writer_ << "\n";
}

// A device tensor with a constant initialiser of its own is filled on the device (the counters of an
// Accuracy node are the usual case).
void HipCodegen::emitDeviceFills() {
    for (TensorNode *tn : decl_order_) {
        Tensor *t = tn->getTensor();
        if (tn->getLabel()->getDeviceLabel().type != DeviceType::GPU) continue;
        const TensorInitType init = t->getTensorInitType();
        if (init != TensorInitType::CONSTANT && init != TensorInitType::ZERO) continue;
        const float v = init == TensorInitType::ZERO ? 0.f : t->getTensorInitInfo().getConstant();
        const std::string name = tensors_name_map_.at(t);
        if (t->getDataType() == DataType::Float_t)
            writer_ << "SWC_HIP_CHECK(swc_hip_fill_f(" << name << ", " << v << ", " << t->size() << "));\n";
        else if (t->getDataType() == DataType::Int32_t)
            writer_ << "SWC_HIP_CHECK(swc_hip_fill_i(" << name << ", " << static_cast<int>(v) << ", " << t->size()
                    << "));\n";
    }
}

// The host tensors a snapshot holds are the ones the CPU program would write, under the same names, so a
// snapshot of either program restores the other.  What the device has trained is downloaded into them first.
void HipCodegen::emitSaveSnapshot() {
    if (!config_.train_mode || !config_.train_config.snapshot) return;
    if (config_.benchmark) {
        writer_ << "// emitSaveSnapshot() disabled in benchmark mode\n";
        return;
    }
    writer_ << "\nif (iter % " << config_.train_config.snapshot << " == 0) {\n";
    writer_.indentInc();
    writer_ << "std::cout << \"iter = \" << iter << \", snapshot\\n\";\n";
    writer_ << "SnapshotNet net;\nnet.setIter(iter);\n";
    std::set<Tensor *> seen;
    for (TensorNode *tn : decl_order_) {
        Tensor *t = tn->getTensor();
        if (tn->getLabel()->getDeviceLabel().type != DeviceType::CPU || !inSnapshot(t) || !seen.insert(t).second) continue;
        const std::string name = tensors_name_map_.at(t);
        for (IRNode *c : tn->getChildNodes()) {
            if (c->nodeType() != OP_NODE) continue;
            auto *up = static_cast<OpNode *>(c);
            if (up->getOp()->getOpName() != "Scatter" || !up->isRunOnce() || up->childNum() != 1) continue;
            writer_ << "SWC_HIP_CHECK(swc_hip_d2h(" << name << ", " << nameOf(up->getChildNode(0)) << ", "
                    << t->getSizeInBytes() << "));\n";
            break;
        }
        writer_ << "addOp(net, \"" << name << "\", " << name << ", " << t->size() << ");\n";
    }
    writer_ << "std::string snapfile = \"snapshot_iter\" + std::to_string(iter) + \".model\";\n";
    writer_ << "if (!net.save(snapfile)) { std::cout << \"Error opening \" << snapfile << \"\\n\"; return 1; }\n";
    writer_ << "std::cout << \"save snapshot to \" << snapfile << \"\\n\";\n";
    writer_.indentDec();
    writer_ << "}\n";
}

void HipCodegen::emitDeferredGathers() {
    defer_output_gathers_ = false;
    if (!deferred_gathers_.empty()) writer_ << "// what the last batch left on the device\n";
    for (OpNode *g : deferred_gathers_) emitTransfer(g, false);
    deferred_gathers_.clear();
}

// The display tensors every Config::display iterations (reference: src/codegen/Codegen.cpp:815-854); one
// that lives on the device is downloaded there, into its host twin, and the twin is printed.
void HipCodegen::emitPrintGraphOutputs() {
    if (config_.train_mode && config_.benchmark) {
        writer_ << "// emitPrintGraphOutputs() disabled in benchmark mode\n";
        return;
    }
    writer_ << "\nif (iter % " << config_.display << " == 0) {\n";
    writer_.indentInc();
    writer_ << "std::cout << \"iterations \" << iter << \"\\n\";\n";
    for (TensorNode *tn : graph_->getDisplayTensorNodes()) {
        TensorNode *shown = tn;
        if (tn->getLabel()->getDeviceLabel().type == DeviceType::GPU) {
            OpNode *gather = nullptr;
            for (IRNode *c : tn->getChildNodes())
                if (c->nodeType() == OP_NODE && static_cast<OpNode *>(c)->getOp()->getOpName() == "Gather")
                    gather = static_cast<OpNode *>(c);
            if (!gather) {
                SWLOG_ERROR << "display tensor " << tn->name() << " lives on the device and has no Gather" << std::endl;
                std::abort();
            }
            emitTransfer(gather, false);
            shown = static_cast<TensorNode *>(gather->getChildNode(0));
        }
        Tensor *t = shown->getTensor();
        writer_ << "// " << tn->name() << "\n";
        writer_ << "printMatrix(" << tensors_name_map_.at(t) << ", " << t->getDim(0) << ", "
                << (t->getNDim() == 2 ? t->getDim(1) : 1) << ");\n";
    }
    writer_.indentDec();
    writer_ << "}\n";
}

void HipCodegen::emitExecute() {
    if (config_.use_dataloader && config_.hip_graph && deviceOpsAreContiguous()) {
        // The batch loop with the device ops of an iteration as one HIP graph: a pass over whatever the arena
        // holds (kernels configure themselves), the ops recorded once, and per batch the upload, one graph
        // launch, the download and the host ops.
        writer_ << "// warm-up pass and recording of the device ops\n{\n";
        writer_.indentInc();
        emitDeviceOpsOnly();
        writer_.indentDec();
        writer_ << "}\n";
        if (config_.train_mode) {
            // the warm-up pass has taken an optimizer step on whatever the arena held: parameters and momenta
            // are uploaded again
            writer_ << "// parameters and momenta as they were before the warm-up pass\n";
            for (int i = 0; i < graph_->topologyNum(); ++i)
                for (int j = 0; j < graph_->getNumInTopoLevel(i); ++j) {
                    IRNode *node = graph_->getNodeInTopo(i, j);
                    if (node->nodeType() != OP_NODE) continue;
                    auto *op = static_cast<OpNode *>(node);
                    if (op->isRunOnce() && op->getOp()->getOpName() == "Scatter") emitTransfer(op, true);
                }
        }
        emitDeviceFills();   // counters the warm-up pass has touched start again
        writer_ << "SWC_HIP_CHECK(swc_hip_sync());\n";
        writer_ << "void *swc_graph = NULL;\n";
        writer_ << "SWC_HIP_CHECK(swc_hip_graph_begin());\n{\n";
        writer_.indentInc();
        emitDeviceOpsOnly();
        writer_.indentDec();
        writer_ << "}\nSWC_HIP_CHECK(swc_hip_graph_end(&swc_graph));\n";
        defer_output_gathers_ = true;
        // per-batch uploads (the Scatter nodes that are not run-once), in emission order
        std::vector<OpNode *> uploads;
        for (int i = 0; i < graph_->topologyNum(); ++i)
            for (int j = 0; j < graph_->getNumInTopoLevel(i); ++j) {
                IRNode *node = graph_->getNodeInTopo(i, j);
                if (node->nodeType() != OP_NODE) continue;
                auto *op = static_cast<OpNode *>(node);
                if (!op->isRunOnce() && op->getOp()->getOpName() == "Scatter") uploads.push_back(op);
            }
        // With prefetching the loader overwrites its host buffers with batch i+1 as soon as the graph of batch i has
        // been launched.  A host op of the iteration, or a displayed tensor, that reads one of those buffers would see
        // the next batch: such a program keeps the plain loop.
        auto hostReadsLoaderBuffers = [&]() {
            Tensor *lt = T(loaderLabelNode()), *dt = T(loaderDataNode());
            for (int i = 0; i < graph_->topologyNum(); ++i)
                for (int j = 0; j < graph_->getNumInTopoLevel(i); ++j) {
                    IRNode *node = graph_->getNodeInTopo(i, j);
                    if (node->nodeType() != OP_NODE) continue;
                    auto *op = static_cast<OpNode *>(node);
                    const std::string type = op->getOp()->getOpName();
                    if (op->isRunOnce() || isDeviceComputeOp(op) || type == "Scatter" || type == "Gather") continue;
                    for (IRNode *p : op->getParentNodes())
                        if (p->nodeType() == TENSOR_NODE && (T(p) == lt || T(p) == dt)) return true;
                }
            if (config_.display > 0)
                for (TensorNode *tn : graph_->getDisplayTensorNodes())
                    if (tn->getTensor() == lt || tn->getTensor() == dt) return true;
            return false;
        };
        bool prefetch = config_.hip_prefetch && !uploads.empty();
        if (prefetch && hostReadsLoaderBuffers()) {
            prefetch = false;
            writer_ << "// (hip_prefetch: a host op or a displayed tensor reads the loader's host buffers: no prefetching)\n";
        }
        const std::string next = "loader.next(" + nameOf(loaderLabelNode()) + ", " + nameOf(loaderDataNode()) + ")";
        auto stageName = [&](OpNode *u) { return nameOf(u->getChildNode(0)) + "_stage"; };
        auto bytesOf = [&](OpNode *u) {
            return std::min(T(u->getParentNode(0))->getSizeInBytes(), T(u->getChildNode(0))->getSizeInBytes());
        };
        auto emitPrefetch = [&]() {   // the batch the loader has just produced starts its way to the staging buffers
            for (OpNode *u : uploads) {
                std::string src = nameOf(u->getParentNode(0));
                if (const size_t off = static_cast<ScatterOp *>(u->getOp())->getOffset()) src += " + " + std::to_string(off);
                writer_ << "SWC_HIP_CHECK(swc_hip_copy_h2d_async(" << stageName(u) << ", " << src << ", " << bytesOf(u)
                        << "));\n";
            }
        };
        if (prefetch) {
            // The loader reads batch i+1 and the copy stream uploads it into staging buffers while the device
            // computes batch i; a device-to-device copy hands a staged batch to the tensors the graph reads.
            writer_ << "// staging buffers: the next batch is uploaded while this one is computed\n";
            for (OpNode *u : uploads)
                writer_ << "void *" << stageName(u) << " = swc_hip_malloc(" << bytesOf(u) << ");\n"
                        << "if (!" << stageName(u) << ") { std::fprintf(stderr, \"%s\\n\", swc_hip_last_error()); return 1; }\n";
            writer_ << "bool swc_more = " << next << ";\n";
            writer_ << "if (swc_more) {\n";
            writer_.indentInc();
            emitPrefetch();
            writer_.indentDec();
            writer_ << "}\nwhile (swc_more) {\n";
            writer_.indentInc();
            writer_ << "SWC_HIP_CHECK(swc_hip_copy_sync());          // the batch has arrived; the host buffers are free\n";
            writer_ << "SWC_HIP_CHECK(swc_hip_ops_wait_copies());\n";
            for (OpNode *u : uploads)
                writer_ << "SWC_HIP_CHECK(swc_hip_d2d(" << nameOf(u->getChildNode(0)) << ", " << stageName(u) << ", "
                        << bytesOf(u) << "));\n";
            writer_ << "SWC_HIP_CHECK(swc_hip_copy_wait_ops());      // the next upload may overwrite the staging buffers after this\n";
        } else {
            writer_ << "while(" << next << ") {\n";
            writer_.indentInc();
        }
        bool launched = false;
        for (int i = 0; i < graph_->topologyNum(); ++i)
            for (int j = 0; j < graph_->getNumInTopoLevel(i); ++j) {
                IRNode *node = graph_->getNodeInTopo(i, j);
                if (node->nodeType() != OP_NODE) continue;
                auto *op = static_cast<OpNode *>(node);
                if (op->isRunOnce()) continue;
                if (isDeviceComputeOp(op)) {
                    if (!launched) {
                        writer_ << "SWC_HIP_CHECK(swc_hip_graph_launch(swc_graph));\n";
                        if (prefetch) {
                            writer_ << "swc_more = " << next << ";   // the next batch, while the device works on this one\n";
                            writer_ << "if (swc_more) {\n";
                            writer_.indentInc();
                            emitPrefetch();
                            writer_.indentDec();
                            writer_ << "}\n";
                        }
                    }
                    launched = true;
                    continue;
                }
                if (prefetch && op->getOp()->getOpName() == "Scatter") continue;   // done above
                writer_ << "// topology(" << i << ", " << j << "): " << op->name() << " : " << op->getOp()->getOpName()
                        << "\n";
                dispatchOpNode(op);
            }
        writer_ << "\niter++;\n";
        emitSaveSnapshot();
        if (config_.display > 0) emitPrintGraphOutputs();
        emitMaxItersBreak();
        writer_.indentDec();
        writer_ << "} //while\n";
        emitDeferredGathers();
        writer_ << "SWC_HIP_CHECK(swc_hip_sync());\n";
        if (prefetch)
            for (OpNode *u : uploads) writer_ << "SWC_HIP_CHECK(swc_hip_free(" << stageName(u) << "));\n";
        writer_ << "SWC_HIP_CHECK(swc_hip_graph_destroy(swc_graph));\n";
        return;
    }
    if (config_.use_dataloader) {
        // the batch loop of the CPU target; the per-iteration Scatter of the data
        // tensor and the Gather in front of each host op are ordinary op nodes
        defer_output_gathers_ = true;
        Codegen::emitExecute();
        emitDeferredGathers();
        writer_ << "SWC_HIP_CHECK(swc_hip_sync());\n";
        return;
    }
    if (config_.time_iters && config_.hip_graph) {
        // eager pass (kernels configure themselves, outputs reach the host), then the
        // device ops recorded once and replayed: one submission per iteration
        writer_ << "// eager pass\n";
        emitFuncCalls();
        writer_ << "SWC_HIP_CHECK(swc_hip_sync());\n";
        writer_ << "void *swc_graph = NULL;\n";
        writer_ << "SWC_HIP_CHECK(swc_hip_graph_begin());\n{\n";
        writer_.indentInc();
        emitDeviceOpsOnly();
        writer_.indentDec();
        writer_ << "}\nSWC_HIP_CHECK(swc_hip_graph_end(&swc_graph));\n";
        writer_ << "SWC_HIP_CHECK(swc_hip_graph_launch(swc_graph));\nSWC_HIP_CHECK(swc_hip_sync());\n";
        writer_ << "SWC_HIP_CHECK(swc_hip_timer_begin());\n";
        writer_ << "for (size_t swc_iter = 0; swc_iter < " << config_.time_iters << "; swc_iter++) {\n";
        writer_.indentInc();
        writer_ << "SWC_HIP_CHECK(swc_hip_graph_launch(swc_graph));\n";
        writer_.indentDec();
        writer_ << "}\n";
        writer_ << "SWC_HIP_CHECK(swc_hip_timer_end());\n";
        writer_ << "std::cout << \"swc_time_ms_per_iter \" << swc_hip_timer_elapsed_ms() / " << config_.time_iters
                << " << std::endl;\n";
        writer_ << "SWC_HIP_CHECK(swc_hip_graph_destroy(swc_graph));\n";
        return;
    }
    if (config_.time_iters) {
        // one untimed pass (first-touch, code load), then the timed loop
        writer_ << "// warm-up pass\n";
        emitFuncCalls();
        writer_ << "SWC_HIP_CHECK(swc_hip_sync());\n";
        writer_ << "SWC_HIP_CHECK(swc_hip_timer_begin());\n";
        writer_ << "for (size_t swc_iter = 0; swc_iter < " << config_.time_iters << "; swc_iter++) {\n";
        writer_.indentInc();
    }
    emitFuncCalls();
    if (config_.time_iters) {
        writer_.indentDec();
        writer_ << "}\n";
        writer_ << "SWC_HIP_CHECK(swc_hip_timer_end());\n";
        writer_ << "std::cout << \"swc_time_ms_per_iter \" << swc_hip_timer_elapsed_ms() / " << config_.time_iters
                << " << std::endl;\n";
    }
    writer_ << "SWC_HIP_CHECK(swc_hip_sync());\n";
}

// an op of the per-iteration part that runs on the device (not a transfer, not a host op)
bool HipCodegen::isDeviceComputeOp(OpNode *op) const {
    const std::string type = op->getOp()->getOpName();
    return !op->isRunOnce() && type != "Scatter" && type != "Gather" &&
           op->getLabel()->getDeviceLabel().type == DeviceType::GPU;
}

// In emission order, do all uploads come before the first device op and all downloads and host ops after the
// last?  Only then can the device ops of an iteration be replayed as one recorded graph.
bool HipCodegen::deviceOpsAreContiguous() const {
    int phase = 0;   // 0: before the device ops, 1: among them, 2: after
    for (int i = 0; i < graph_->topologyNum(); ++i)
        for (int j = 0; j < graph_->getNumInTopoLevel(i); ++j) {
            IRNode *node = graph_->getNodeInTopo(i, j);
            if (node->nodeType() != OP_NODE) continue;
            auto *op = static_cast<OpNode *>(node);
            if (op->isRunOnce()) continue;
            // (a download nobody on the host reads is not part of the batch loop's body: it is emitted where its
            // tensor is displayed and after the loop)
            if (config_.use_dataloader && op->getOp()->getOpName() == "Gather" && op->getChildNode(0)->childNum() == 0)
                continue;
            if (isDeviceComputeOp(op)) {
                if (phase == 2) return false;
                phase = 1;
            } else if (phase == 1) {
                phase = 2;
            }
        }
    return phase != 0;
}

void HipCodegen::emitDeviceOpsOnly() {
    for (int i = 0; i < graph_->topologyNum(); ++i)
        for (int j = 0; j < graph_->getNumInTopoLevel(i); ++j) {
            IRNode *node = graph_->getNodeInTopo(i, j);
            if (node->nodeType() != OP_NODE) continue;
            auto *op = static_cast<OpNode *>(node);
            if (isDeviceComputeOp(op)) emitHipCall(op);
        }
}

void HipCodegen::emitMemFree() {
    if (has_workspace_)
        writer_ << "SWC_HIP_CHECK(swc_hip_set_workspace(nullptr, 0));\n"
                << "if (gpu0_ws) SWC_HIP_CHECK(swc_hip_free(gpu0_ws));\n";
    for (auto &a : mem_allocators_) {
        if (!a->getMemAllocated()) continue;
        if (a->getDevice().type == DeviceType::CPU) writer_ << "SWC_HIP_CHECK(swc_hip_host_free(" << a->getBasePtrName() << "));\n";
        else writer_ << "SWC_HIP_CHECK(swc_hip_free(" << a->getBasePtrName() << "));\n";
    }
}

void HipCodegen::dispatchOpNode(OpNode *op) {
    if (!op->runable()) return;
    const std::string type = op->getOp()->getOpName();
    if (type == "Scatter") return emitTransfer(op, true);
    if (type == "Gather") {
        if (defer_output_gathers_ && op->getChildNode(0)->childNum() == 0) {
            if (std::find(deferred_gathers_.begin(), deferred_gathers_.end(), op) == deferred_gathers_.end())
                deferred_gathers_.push_back(op);
            writer_ << "// (no host op reads it: downloaded where it is displayed and after the loop)\n";
            return;
        }
        return emitTransfer(op, false);
    }
    if (op->getLabel()->getDeviceLabel().type == DeviceType::GPU) return emitHipCall(op);
    emitFuncCall(op);   // host-side ops: Debug
}

void HipCodegen::emitTransfer(OpNode *op, bool toDevice) {
    assert(op->parentNum() == 1 && op->childNum() == 1);
    Tensor *from = T(op->getParentNode(0));
    Tensor *to = T(op->getChildNode(0));
    const size_t bytes = std::min(from->getSizeInBytes(), to->getSizeInBytes());
    size_t offset = toDevice ? static_cast<ScatterOp *>(op->getOp())->getOffset()
                             : static_cast<GatherOp *>(op->getOp())->getOffset();
    // the offset (elements) applies to the host side
    std::string src = tensors_name_map_.at(from), dst = tensors_name_map_.at(to);
    if (offset) (toDevice ? src : dst) += " + " + std::to_string(offset);
    writer_ << "SWC_HIP_CHECK(" << (toDevice ? "swc_hip_h2d(" : "swc_hip_d2h(") << dst << ", " << src << ", " << bytes
            << "));\n";
}

// One libswc_hip call per GPU op node.  Argument lists are those of the CPU
// emitters (Codegen::emitFuncCall) with the swc_hip_ prefix; fused node types
// map to the fused entry points.
void HipCodegen::emitHipCall(OpNode *op) {
    const std::string type = op->getOp()->getOpName();
    const std::string nm = op->name();
    auto in = [&](int i) { return op->getParentNode(i); };
    auto out = [&](int i) { return op->getChildNode(i); };
    auto rowsCols = [](Tensor *t) {
        size_t cols = 1;
        for (int i = 1; i < t->getNDim(); ++i) cols *= t->getDim(i);
        return std::pair<size_t, size_t>(t->getDim(0), cols);
    };
    auto convArrays = [&](Conv2dOp *conv) {
        writer_ << arrayDef(nm + "_inDims", T(in(0))->getDims()) << arrayDef(nm + "_outDims", T(out(0))->getDims())
                << arrayDef(nm + "_filterDims", T(in(1))->getDims()) << arrayDef(nm + "_biasDims", T(in(2))->getDims())
                << arrayDef(nm + "_filterSizes", conv->getKernels()) << arrayDef(nm + "_strides", conv->getStrides())
                << arrayDef(nm + "_pads", conv->getPads());
    };
    auto convArgs = [&](Conv2dOp *conv) {
        std::ostringstream os;
        os << nameOf(out(0)) << ", " << nameOf(in(0)) << ", " << nameOf(in(1)) << ", " << nameOf(in(2)) << ", " << nm
           << "_outDims, " << nm << "_inDims, " << nm << "_filterDims, " << nm << "_biasDims, " << nm
           << "_filterSizes, " << nm << "_strides, " << nm << "_pads, " << conv->getGroup();
        return os.str();
    };

    if (type == "MatrixMatrixMul") {
        const size_t m = T(in(0))->getDim(0), k = T(in(1))->getDim(0), n = T(in(1))->getDim(1);
        writer_ << "SWC_HIP_CHECK(swc_hip_matrixMatrixMul_f(" << m << ", " << n << ", " << k << ", " << nameOf(in(0))
                << ", " << k << ", " << nameOf(in(1)) << ", " << n << ", " << nameOf(out(0)) << ", " << n << "));\n";
    } else if (type == "MatrixMatrixFCBias" || type == "MatrixMatrixFCBiasRelu") {
        auto rc = rowsCols(T(in(0)));   // rank > 2 inputs are read as [dim0, rest]
        const size_t k = T(in(1))->getDim(0), n = T(in(1))->getDim(1);
        assert(rc.second == k && "FC: flattened input width != weight rows");
        writer_ << "SWC_HIP_CHECK(swc_hip_matrixMatrixFCBias_f(" << rc.first << ", " << n << ", " << k << ", "
                << nameOf(in(0)) << ", " << k << ", " << nameOf(in(1)) << ", " << n << ", " << nameOf(in(2)) << ", "
                << nameOf(out(0)) << ", " << n << ", " << (type == "MatrixMatrixFCBiasRelu" ? 1 : 0) << "));\n";
    } else if (type == "MatrixMatrixFCBiasSoftmax") {
        auto rc = rowsCols(T(in(0)));
        const size_t k = T(in(1))->getDim(0), n = T(in(1))->getDim(1);
        assert(rc.second == k && "FC: flattened input width != weight rows");
        writer_ << "SWC_HIP_CHECK(swc_hip_matrixMatrixFCBiasSoftmax_f(" << rc.first << ", " << n << ", " << k << ", "
                << nameOf(in(0)) << ", " << k << ", " << nameOf(in(1)) << ", " << n << ", " << nameOf(in(2)) << ", "
                << nameOf(out(0)) << ", " << n << "));\n";
    } else if (type == "MatrixVectorAdd" || type == "BatchedAdd") {
        auto rc = rowsCols(T(in(0)));
        writer_ << "SWC_HIP_CHECK(swc_hip_batchedadd_f(" << nameOf(out(0)) << ", " << nameOf(in(0)) << ", "
                << nameOf(in(1)) << ", " << rc.first << ", " << rc.second << "));\n";
    } else if (type == "Reshape" || type == "TensorDescend" || type == "TensorAscend" || type == "Dropout") {
        writer_ << nameOf(out(0)) << " = " << nameOf(in(0)) << ";\n";
    } else if (type == "MatrixTanh" || type == "MatrixSoftmax") {
        const size_t m = T(in(0))->getDim(0), n = T(in(0))->getDim(1);
        writer_ << "SWC_HIP_CHECK(swc_hip_" << (type == "MatrixTanh" ? "matrixTanh_f(" : "matrixSoftmax_f(") << m << ", "
                << n << ", " << nameOf(in(0)) << ", " << n << ", " << nameOf(out(0)) << ", " << n << "));\n";
    } else if (type == "ElementAdd" || type == "ElementAddRelu") {
        writer_ << "SWC_HIP_CHECK(swc_hip_" << (type == "ElementAdd" ? "vecAdd_f(" : "vecAddRelu_f(")
                << T(in(0))->size() << ", " << nameOf(in(0)) << ", " << nameOf(in(1)) << ", " << nameOf(out(0))
                << "));\n";
    } else if (type == "Relu") {
        writer_ << "SWC_HIP_CHECK(swc_hip_relu_f(" << nameOf(in(0)) << ", " << nameOf(out(0)) << ", "
                << T(in(0))->size() << "));\n";
    } else if (type == "Conv2d") {
        auto *conv = static_cast<Conv2dOp *>(op->getOp());
        convArrays(conv);
        writer_ << "SWC_HIP_CHECK(swc_hip_conv2d_f(" << convArgs(conv) << "));\n";
    } else if (type == "Conv2dWithActivation") {
        auto *conv = static_cast<Conv2dWithActivationOp *>(op->getOp());
        if (conv->getActivationType() != SWC_ACTIVATION_RELU) {
            SWLOG_ERROR << "Conv2dWithActivation: only ReLU is implemented on the HIP target" << std::endl;
            std::abort();
        }
        convArrays(conv);
        writer_ << "SWC_HIP_CHECK(swc_hip_conv2dFused_f(" << convArgs(conv) << ", NULL, NULL, NULL, NULL, 0.f, 1));\n";
    } else if (type == "Conv2dBatchNorm") {
        // parents: input, filter, bias, bn scale, bn bias, bn mean, bn var
        auto *conv = static_cast<Conv2dBatchNormOp *>(op->getOp());
        convArrays(conv);
        writer_ << "SWC_HIP_CHECK(swc_hip_conv2dFused_f(" << convArgs(conv) << ", " << nameOf(in(5)) << ", "
                << nameOf(in(6)) << ", " << nameOf(in(3)) << ", " << nameOf(in(4)) << ", " << std::setprecision(12)
                << conv->getEpsilon() << ", " << (conv->hasRelu() ? 1 : 0) << "));\n";
    } else if (type == "Conv2dMaxPool") {
        // parents: input, filter, bias [, bn scale, bn bias, bn mean, bn var]; the child is the pooled tensor
        auto *conv = static_cast<Conv2dMaxPoolOp *>(op->getOp());
        writer_ << arrayDef(nm + "_inDims", T(in(0))->getDims())
                << arrayDef(nm + "_convDims", conv->convOutDims(T(in(0))->getDims(), T(in(1))->getDim(0)))
                << arrayDef(nm + "_outDims", T(out(0))->getDims()) << arrayDef(nm + "_filterDims", T(in(1))->getDims())
                << arrayDef(nm + "_biasDims", T(in(2))->getDims()) << arrayDef(nm + "_filterSizes", conv->getKernels())
                << arrayDef(nm + "_strides", conv->getStrides()) << arrayDef(nm + "_pads", conv->getPads())
                << arrayDef(nm + "_poolSizes", conv->getPoolKernels()) << arrayDef(nm + "_poolStrides", conv->getPoolStrides())
                << arrayDef(nm + "_poolPads", conv->getPoolPads());
        writer_ << "SWC_HIP_CHECK(swc_hip_conv2dFusedMaxpool_f(" << nameOf(out(0)) << ", " << nameOf(in(0)) << ", "
                << nameOf(in(1)) << ", " << nameOf(in(2)) << ", " << nm << "_convDims, " << nm << "_inDims, " << nm
                << "_filterDims, " << nm << "_biasDims, " << nm << "_filterSizes, " << nm << "_strides, " << nm << "_pads, "
                << conv->getGroup() << ", ";
        if (conv->hasBatchNorm())
            writer_ << nameOf(in(5)) << ", " << nameOf(in(6)) << ", " << nameOf(in(3)) << ", " << nameOf(in(4)) << ", "
                    << std::setprecision(12) << conv->getEpsilon();
        else
            writer_ << "NULL, NULL, NULL, NULL, 0.f";
        writer_ << ", " << (conv->hasRelu() ? 1 : 0) << ", " << nm << "_outDims, " << nm << "_poolSizes, " << nm
                << "_poolStrides, " << nm << "_poolPads));\n";
    } else if (type == "Conv2dAdd") {
        // parents: input, filter, bias, [bn scale, bn bias, bn mean, bn var,] the other summand
        auto *conv = static_cast<Conv2dAddOp *>(op->getOp());
        convArrays(conv);
        writer_ << "SWC_HIP_CHECK(swc_hip_conv2dFusedAdd_f(" << convArgs(conv) << ", ";
        if (conv->hasBatchNorm())
            writer_ << nameOf(in(5)) << ", " << nameOf(in(6)) << ", " << nameOf(in(3)) << ", " << nameOf(in(4)) << ", "
                    << std::setprecision(12) << conv->getEpsilon() << ", " << nameOf(in(7));
        else
            writer_ << "NULL, NULL, NULL, NULL, 0.f, " << nameOf(in(3));
        writer_ << ", " << (conv->hasRelu() ? 1 : 0) << "));\n";
    } else if (type == "BatchNormalization" || type == "BatchNormalizationRelu") {
        const bool relu = type == "BatchNormalizationRelu";
        const float eps = relu ? static_cast<BatchNormalizationReluOp *>(op->getOp())->getEpsilon()
                               : static_cast<BatchNormalizationOp *>(op->getOp())->getEpsilon();
        writer_ << arrayDef(nm + "_inDims", T(in(0))->getDims());
        writer_ << "SWC_HIP_CHECK(swc_hip_" << (relu ? "batchnormRelu_f(" : "batchnormalization_f(") << nameOf(out(0))
                << ", " << nameOf(in(0)) << ", " << nameOf(in(3)) << ", " << nameOf(in(4)) << ", " << nameOf(in(1))
                << ", " << nameOf(in(2)) << ", " << nm << "_inDims, " << std::setprecision(12) << eps << "));\n";
    } else if (type == "BatchNormReluMaxPool") {   // parents as BatchNormalization: in, scale, bias, mean, var
        auto *bp = static_cast<BatchNormReluMaxPoolOp *>(op->getOp());
        writer_ << arrayDef(nm + "_inDims", T(in(0))->getDims()) << arrayDef(nm + "_outDims", T(out(0))->getDims())
                << arrayDef(nm + "_filterSizes", bp->getKernels()) << arrayDef(nm + "_strides", bp->getStrides())
                << arrayDef(nm + "_pads", bp->getPads());
        writer_ << "SWC_HIP_CHECK(swc_hip_batchnormReluMaxpool_f(" << nameOf(out(0)) << ", " << nameOf(in(0)) << ", "
                << nameOf(in(3)) << ", " << nameOf(in(4)) << ", " << nameOf(in(1)) << ", " << nameOf(in(2)) << ", " << nm
                << "_inDims, " << std::setprecision(12) << bp->getEpsilon() << ", " << nm << "_outDims, " << nm
                << "_filterSizes, " << nm << "_strides, " << nm << "_pads));\n";
    } else if (type == "MaxPool") {
        auto *pool = static_cast<MaxPoolOp *>(op->getOp());
        writer_ << arrayDef(nm + "_inDims", T(in(0))->getDims()) << arrayDef(nm + "_outDims", T(out(0))->getDims())
                << arrayDef(nm + "_filterSizes", pool->getKernels()) << arrayDef(nm + "_strides", pool->getStrides())
                << arrayDef(nm + "_pads", pool->getPads());
        writer_ << "SWC_HIP_CHECK(swc_hip_maxpool_f(" << nameOf(in(0)) << ", " << nameOf(out(0)) << ", " << nm
                << "_inDims, " << nm << "_outDims, " << nm << "_filterSizes, " << nm << "_strides, " << nm
                << "_pads));\n";
    } else if (type == "AveragePool") {
        auto *pool = static_cast<AvgPoolOp *>(op->getOp());
        writer_ << arrayDef(nm + "_inDims", T(in(0))->getDims()) << arrayDef(nm + "_outDims", T(out(0))->getDims())
                << arrayDef(nm + "_filterSizes", pool->getKernels()) << arrayDef(nm + "_strides", pool->getStrides())
                << arrayDef(nm + "_pads", pool->getPads());
        writer_ << "SWC_HIP_CHECK(swc_hip_avgpool_f(" << nameOf(in(0)) << ", " << nameOf(out(0)) << ", " << nm
                << "_inDims, " << nm << "_outDims, " << nm << "_filterSizes, " << nm << "_strides, " << nm
                << "_pads));\n";
    } else if (type == "Transpose") {
        auto *tr = static_cast<TransposeOp *>(op->getOp());
        const int nd = T(in(0))->getNDim();
        if ((nd != 2 && nd != 4) || (int)tr->getShuffle().size() != nd) {
            SWLOG_ERROR << "Transpose " << nm << ": only 2-D and 4-D tensors with a full shuffle" << std::endl;
            std::abort();
        }
        writer_ << arrayDef(nm + "_inDims", T(in(0))->getDims()) << arrayDef(nm + "_outDims", T(out(0))->getDims())
                << arrayDef(nm + "_shuffle", tr->getShuffle());
        writer_ << "SWC_HIP_CHECK(swc_hip_" << (nd == 2 ? "transpose2d_f(" : "transpose4d_f(") << nameOf(in(0)) << ", "
                << nameOf(out(0)) << ", " << nm << "_inDims, " << nm << "_outDims, " << nm << "_shuffle));\n";
    } else if (type == "ArgMax") {
        const int topK = static_cast<ArgMaxOp *>(op->getOp())->getTopK();
        writer_ << "SWC_HIP_CHECK(swc_hip_argMax_i(" << nameOf(in(0)) << ", " << nameOf(out(0)) << ", "
                << T(in(0))->getDim(0) << ", " << T(in(0))->getDim(1) << ", " << topK << "));\n";
    } else if (type == "BatchedReduceAdd") {
        const auto rc = T(in(0))->viewAs2D(T(in(0))->getNDim() - 1);
        if (rc.first > T(out(0))->size()) {   // one sum per ROW goes into the result (kernels.h:554-563): it must hold them
            SWLOG_ERROR << "BatchedReduceAdd " << nm << ": " << rc.first << " rows into a result of " << T(out(0))->size()
                        << " elements — the reference's kernel would write past it (mini-batch larger than the layer)" << std::endl;
            std::abort();
        }
        writer_ << "SWC_HIP_CHECK(swc_hip_batchedreduceadd_f(" << nameOf(out(0)) << ", " << nameOf(in(0)) << ", " << rc.first
                << ", " << rc.second << "));\n";
    } else if (type == "ReluGrad") {
        writer_ << "SWC_HIP_CHECK(swc_hip_reluGrad_f(" << nameOf(out(0)) << ", " << nameOf(in(0)) << ", " << nameOf(in(1))
                << ", " << T(in(0))->size() << "));\n";
    } else if (type == "MatrixTanhGrad") {
        const size_t m = T(in(0))->getDim(0), n = T(in(0))->getDim(1);
        writer_ << "SWC_HIP_CHECK(swc_hip_matrixTanhGrad_f(" << m << ", " << n << ", " << nameOf(out(0)) << ", " << n << ", "
                << nameOf(in(1)) << ", " << n << ", " << nameOf(in(2)) << ", " << n << "));\n";
    } else if (type == "MaxPoolGrad") {
        auto *pool = static_cast<MaxPoolGradOp *>(op->getOp());
        writer_ << arrayDef(nm + "_inDims", T(in(0))->getDims()) << arrayDef(nm + "_outDims", T(in(1))->getDims())
                << arrayDef(nm + "_filterSizes", pool->getKernels()) << arrayDef(nm + "_strides", pool->getStrides())
                << arrayDef(nm + "_pads", pool->getPads());
        writer_ << "SWC_HIP_CHECK(swc_hip_maxpoolGrad_f(" << nameOf(out(0)) << ", " << nameOf(in(2)) << ", " << nameOf(in(0))
                << ", " << nm << "_inDims, " << nm << "_outDims, " << nm << "_filterSizes, " << nm << "_strides, " << nm
                << "_pads));\n";
    } else if (type == "Conv2dGrad") {
        auto *conv = static_cast<Conv2dGradOp *>(op->getOp());
        writer_ << arrayDef(nm + "_inDims", T(in(0))->getDims()) << arrayDef(nm + "_outDims", T(in(2))->getDims())
                << arrayDef(nm + "_filterDims", T(in(1))->getDims()) << arrayDef(nm + "_biasDims", T(out(2))->getDims())
                << arrayDef(nm + "_filterSizes", conv->getKernels()) << arrayDef(nm + "_strides", conv->getStrides())
                << arrayDef(nm + "_pads", conv->getPads());
        writer_ << "SWC_HIP_CHECK(swc_hip_conv2dGrad_f(" << nameOf(out(0)) << ", " << nameOf(out(1)) << ", " << nameOf(out(2))
                << ", " << nameOf(in(2)) << ", " << nameOf(in(0)) << ", " << nameOf(in(1)) << ", " << nm << "_outDims, "
                << nm << "_inDims, " << nm << "_filterDims, " << nm << "_biasDims, " << nm << "_filterSizes, " << nm
                << "_strides, " << nm << "_pads, " << conv->getGroup() << "));\n";
    } else if (type == "MatrixSoftmaxWithLoss") {
        const size_t m = T(in(0))->getDim(0), n = T(in(0))->getDim(1);
        writer_ << "SWC_HIP_CHECK(swc_hip_matrixSoftmaxWithLoss_f(" << m << ", " << n << ", " << nameOf(in(0)) << ", " << n
                << ", " << nameOf(out(0)) << ", " << n << ", " << nameOf(in(1)) << ", " << nameOf(out(1)) << "));\n";
    } else if (type == "MatrixSoftmaxWithLossGrad") {
        const size_t m = T(in(1))->getDim(0), n = T(in(1))->getDim(1);
        writer_ << "SWC_HIP_CHECK(swc_hip_matrixSoftmaxWithLossGrad_f(" << m << ", " << n << ", " << nameOf(out(0)) << ", " << n
                << ", " << nameOf(in(1)) << ", " << n << ", " << nameOf(in(0)) << "));\n";
    } else if (type == "MatrixSoftmaxGrad") {
        const size_t m = T(in(0))->getDim(0), n = T(in(0))->getDim(1);
        writer_ << "SWC_HIP_CHECK(swc_hip_matrixSoftmaxGrad_f(" << m << ", " << n << ", " << nameOf(out(0)) << ", " << n
                << ", " << nameOf(in(2)) << ", " << n << ", " << nameOf(in(1)) << "));\n";
    } else if (type == "SGD") {
        auto *sgd = static_cast<SGDOp *>(op->getOp());
        writer_ << "SWC_HIP_CHECK(swc_hip_sgd_f(" << T(in(0))->size() << ", " << nameOf(in(0)) << ", " << nameOf(in(0)) << ", "
                << nameOf(in(1)) << ", " << nameOf(in(2)) << ", " << sgd->getLR() << ", " << sgd->getDecay() << ", "
                << sgd->getMomentum() << ", " << sgd->getBatch() << "));\n";
    } else if (type == "Accuracy") {
        writer_ << "SWC_HIP_CHECK(swc_hip_accuracy_i(" << nameOf(in(0)) << ", " << nameOf(in(1)) << ", " << nameOf(out(0))
                << ", " << T(in(0))->getDim(0) << ", " << T(in(0))->getDim(1) << "));\n";
    } else {
        SWLOG_ERROR << "no HIP emitter for op type " << type << " (node " << nm << ")" << std::endl;
        std::abort();
    }
}

} // namespace codegen
} // namespace swc
