// CPU code generator and the machinery shared with the HIP target.
#include "Codegen.h"

#include "../pass/passes.h"

#include <cassert>
#include <cstdlib>
#include <fstream>
#include <iomanip>
#include <set>

#include "../graphIR/IRGraph.h"
#include "../graphIR/OpNode.h"
#include "../graphIR/TensorNode.h"
#include "../op/ops.h"

namespace swc {
namespace codegen {

using namespace swc::op;

// ------------------------------------------------------------------ helpers
uint64_t MemoryAllocator::allocate(Tensor *t, uint64_t bytes) {
    const uint64_t start = (used_ + alignment_ - 1) / alignment_ * alignment_;
    if (start + bytes > capacity_) {
        SWLOG_ERROR << "arena " << base_ << " exhausted: need " << start + bytes << " of " << capacity_ << std::endl;
        std::abort();
    }
    offsets_[t] = start;
    used_ = start + bytes;
    return start;
}

std::string MakefileBuilder::generate() const {
    std::ostringstream os;
    os << "all: " << target_ << "\n";
    os << "CXX := " << cxx_ << "\n";
    os << "CXXFLAGS :=";
    for (auto &f : flags_) os << " " << f;
    for (auto &d : incs_) os << " -I" << d;
    os << "\nLDFLAGS :=";
    for (auto &d : libDirs_) os << " -L" << d << " -Wl,-rpath," << d;
    for (auto &l : libs_) os << " -l" << l;
    os << "\n" << target_ << ":";
    for (auto &s : srcs_) os << " " << s;
    os << "\n\t$(CXX) $(CXXFLAGS) $^ $(LDFLAGS) -o $@\n";
    os << "run: " << target_ << "\n\t" << runCmd_ << "\n";
    os << "clean:\n\trm -f " << target_ << "\n";
    return os.str();
}

static std::string deviceTag(const Device &d) {
    return (d.type == DeviceType::GPU ? "gpu" : "cpu") + std::to_string(d.id);
}

// [d0, d1*d2*...]
static std::pair<size_t, size_t> rowsCols(const std::vector<size_t> &dims) {
    size_t cols = 1;
    for (size_t i = 1; i < dims.size(); ++i) cols *= dims[i];
    return {dims.empty() ? 0 : dims[0], cols};
}

std::string Codegen::arrayDef(const std::string &name, const std::vector<size_t> &v) {
    std::ostringstream os;
    os << "const size_t " << name << "[] = {";
    for (size_t i = 0; i < v.size(); ++i) os << (i ? ", " : "") << v[i];
    os << "};\n";
    return os.str();
}

std::string Codegen::getTypeString(Tensor *t) const {
    switch (t->getDataType()) {
    case DataType::Double_t: return "double";
    case DataType::Int8_t: return "char";
    case DataType::Int32_t: return "int";
    default: return "float";
    }
}

static Tensor *T(IRNode *n) { return static_cast<TensorNode *>(n)->getTensor(); }

std::string Codegen::nameOf(IRNode *tensorNode) { return tensors_name_map_.at(T(tensorNode)); }

std::string Codegen::UniqueName(std::string name) {
    for (char &c : name)
        if (c == '/' || c == '.' || c == '-') c = '_';
    auto it = names_map_.find(name);
    if (it == names_map_.end()) {
        names_map_[name] = 0;
        return name;
    }
    std::string u;
    do u = name + std::to_string(++it->second);
    while (names_map_.count(u));
    names_map_[u] = 0;
    return u;
}

// ------------------------------------------------------------------- set-up
Codegen::Codegen(IRGraph *graph) : graph_(graph) {
    config_ = graph->getConfig();
    trainAsBatchLoop();
}
Codegen::Codegen(IRGraph *graph, Config &config) : graph_(graph), config_(config) { trainAsBatchLoop(); }

// A training program is the batch loop of the inference generator over the training records (reference:
// src/codegen/Codegen.cpp:952-1019: the same `while(loader.next(label, data))` with the gradient and optimizer
// calls inside): the training settings are carried over into the fields that loop reads.
void Codegen::trainAsBatchLoop() {
    if (!config_.train_mode) return;
    config_.use_dataloader = true;
    config_.dataloader_src = config_.train_config.train_data_file;
    config_.label_bytes = config_.train_config.label_bytes;
    config_.data_bytes = config_.train_config.data_bytes;
    config_.dataloader_samples = config_.train_config.train_data_samples;
    config_.display = config_.train_config.display;
}
TensorNode *Codegen::loaderLabelNode() const {
    return config_.train_mode ? graph_->getTrainLabelNode() : graph_->getInferLabelNode();
}
TensorNode *Codegen::loaderDataNode() const {
    return config_.train_mode ? graph_->getTrainDataNode() : graph_->getInferDataNode();
}

void Codegen::codeGenInit() {
    mem_allocators_.clear();
    dev_allocator_map_.clear();
    tensors_name_map_.clear();
    tensors_offset_map_.clear();
    decl_order_.clear();
    names_map_.clear();
    headerWriter_.clear();
    writer_.clear();
    // one arena per device that can appear in a label
    for (Device d : {Device(0, DeviceType::CPU, 0), Device(0, DeviceType::GPU, config_.hip_device)}) {
        const uint64_t align = d.type == DeviceType::GPU ? devices::HipDevice().arenaAlignment : 64;
        auto a = std::make_shared<MemoryAllocator>(d, deviceTag(d) + "_baseptr", UINT64_MAX, align);
        mem_allocators_.push_back(a);
        dev_allocator_map_[d] = a.get();
    }
    makefile_builder_ = MakefileBuilder();
    swmakefile_builder_ = MakefileBuilder();
    initMakefileBuilder();
}

void Codegen::initMakefileBuilder() {
    // the reference's generated Makefile: g++ -std=c++11 -O2 (src/codegen/MakefileBuilder.h:34)
    makefile_builder_.setCXXCompiler("/usr/bin/c++");
    makefile_builder_.addCXXFlag("-std=c++11");
    makefile_builder_.addCXXFlag("-O2");
    makefile_builder_.addIncDir("/usr/local/include");
    if (config_.train_mode) makefile_builder_.addIncDir("$(SWC_HIP_ROOT)/include");   // swc_snapshot.h (header-only)
    makefile_builder_.addCXXSrc("Graph.cpp");
    swmakefile_builder_.setCXXCompiler("mpiCC");
    swmakefile_builder_.addCXXFlag("-O2");
}

void Codegen::emitHeader() {
    headerWriter_ << "// Graph.cpp -- generated from an IRGraph with " << graph_->tensorNodeNum() << " tensor nodes and "
                  << graph_->opNodeNum() << " op nodes (CPU target)\n";
    headerWriter_ << "#include <iostream>\n#include <random>\n#include <cstdlib>\n#include <cmath>\n"
                  << "#include <sys/time.h>\n#include <sys/types.h>\n"
                  << "#include \"utils/image.h\"\n#include \"utils/kernels.h\"\n";
    if (config_.use_dataloader) headerWriter_ << "#include \"utils/DataLoader.h\"\n";
    if (config_.train_mode) headerWriter_ << "#include \"swc_snapshot.h\"\n";
}

void Codegen::emitEnvInit() {
    if (config_.cuda || config_.mkldnn || config_.mpi) {
        SWLOG_ERROR << "the cuda / mkldnn / mpi targets are not part of this build; use Config::hip" << std::endl;
        std::abort();
    }
}
void Codegen::emitEnvFinalize() { writer_ << "return 0;\n"; }

// ------------------------------------------------------------------ driver
std::string Codegen::generate() {
    // Nested graphs (SubGraph nodes: the reference's route to a GPU, test/cuda/testGPUInfer.cpp, whose generator
    // recurses into them, src/codegen/Codegen.cpp:1035-1077) are emitted in place of their node; on this one-device
    // target every GPU they name is device Config::hip_device.
    graph_->inlineSubGraphs(config_.hip_device);
    // A program written for the reference's CUDA route (Config::cuda on a plain Codegen) or for the CPU, run with
    // SWC_TARGET=hip or Config::hip: the hand-placed part keeps its Scatter/Gather nodes, what was left on the host
    // is placed on the device as Engine::compile would, and the HIP generator writes the program.
    if (!isHipGenerator()) {
        const char *target = std::getenv("SWC_TARGET");
        if (config_.hip || (target && std::string(target) == "hip")) {
            Config cfg = config_;
            cfg.hip = true;
            cfg.cuda = cfg.cuda_stream = cfg.cublas = false;
            graph_->setConfig(cfg);
            pass::DeviceMemoryLoweringPass place(graph_, cfg.hip_device);
            place.run();
            HipCodegen hip(graph_, cfg);
            return hip.generate();
        }
    }
    codeGenInit();
    emitHeader();
    headerWriter_ << "using namespace std;\n";
    writer_ << "#define TIME_MS(a,b)     (1000.0*((b).tv_sec-(a).tv_sec)+0.001*((b).tv_usec-(a).tv_usec))\n";
    writer_ << "\nint main(int argc, char** argv) {\n";
    writer_.indentInc();
    writer_ << "struct timeval ts,te;\n(void)ts; (void)te; (void)argc; (void)argv;\n";
    if (config_.train_mode)   // (the reference defines the same flag with gflags, src/codegen/Codegen.h:44-48)
        writer_ << "const std::string FLAGS_snapshot = swcFlagString(argc, argv, \"snapshot\");\n";
    emitEnvInit();
    writer_ << "\n// variable declaration and initiation\n";
    emitMemAllocs();
    writer_ << "\n// call op routine functions\n";
    emitExecute();
    emitOutputDump();
    writer_ << "\n// free memory\n";
    emitMemFree();
    emitEnvFinalize();
    writer_.indentDec();
    writer_ << "}\n";

    const std::string code = headerWriter_.get_code() + writer_.get_code();
    std::ofstream("Graph.cpp") << code;
    std::ofstream("G_Makefile") << makefile_builder_.generate();
    swmakefile_builder_.addCXXSrc("Graph.cpp");
    std::ofstream("SW_Makefile") << swmakefile_builder_.generate();
    return code;
}

void Codegen::emitMemAllocs() {
    allocateMemAddr();
    emitVarDeclarations();
    emitMemAllocations();
    emitTensorAddresses();
    if (config_.use_dataloader) emitInferDataLoaderInit();
    emitTensorInitializations();
}

static std::string bracedDims(const std::vector<size_t> &dims) {
    std::ostringstream os;
    os << "{";
    for (size_t i = 0; i < dims.size(); ++i) os << (i ? ", " : "") << dims[i];
    os << "}";
    return os.str();
}

// Reference: src/codegen/Codegen.cpp:930-951.  One epoch over
// Config::dataloader_samples records of Config::dataloader_src, mini-batch =
// dim 0 of the label tensor.
void Codegen::emitInferDataLoaderInit() {
    TensorNode *label = loaderLabelNode();
    TensorNode *data = loaderDataNode();
    if (!label || !data) {
        SWLOG_ERROR << "the batch loop needs IRGraph::setInferDataNodes(label, data) (training: setTrainDataNodes)" << std::endl;
        std::abort();
    }
    auto proto = [](BytesProto p) { return p == ONE_BYTE_AS_INT ? "ONE_BYTE_AS_INT" : "FOUR_BYTES_AS_FLOAT"; };
    writer_ << "std::string dataloader_infer_source = \"" << config_.dataloader_src << "\";\n";
    writer_ << "DataLoader loader(dataloader_infer_source, " << proto(config_.label_bytes) << ", "
            << proto(config_.data_bytes) << ", " << (config_.train_mode ? config_.train_config.max_epoch : 1) << ", "
            << config_.dataloader_samples << ", " << bracedDims(label->getDims())
            << ", " << bracedDims(data->getDims()) << ");\n";
    writer_ << "size_t iter = 0;\n\n";
}

// TrainingConfig::max_iters > 0 ends the loop early (the reference's ParallelCodegen does the same,
// src/codegen/ParallelCodegen.cpp:156-157; its single-process loop runs until the epochs are used up).
void Codegen::emitMaxItersBreak() {
    if (config_.train_mode && config_.train_config.max_iters > 0)
        writer_ << "if (iter >= " << config_.train_config.max_iters << ") break;\n";
}

// Reference: src/codegen/Codegen.cpp:815-854.
void Codegen::emitPrintGraphOutputs() {
    if (config_.train_mode && config_.benchmark) {   // reference: src/codegen/Codegen.cpp:1009-1015
        writer_ << "// emitPrintGraphOutputs() disabled in benchmark mode\n";
        return;
    }
    writer_ << "\nif (iter % " << config_.display << " == 0) {\n";
    writer_.indentInc();
    writer_ << "std::cout << \"iterations \" << iter << \"\\n\";\n";
    for (TensorNode *tn : graph_->getDisplayTensorNodes()) {
        Tensor *t = tn->getTensor();
        writer_ << "// " << tn->name() << "\n";
        writer_ << "printMatrix(" << tensors_name_map_.at(t) << ", " << t->getDim(0) << ", "
                << (t->getNDim() == 2 ? t->getDim(1) : 1) << ");\n";
    }
    writer_.indentDec();
    writer_ << "}\n";
}

// Every distinct Tensor gets a name and an offset in the arena of its label's
// device, in topological order.  The output of a Reshape shares its input's
// storage.
void Codegen::allocateMemAddr() {
    for (int i = 0; i < graph_->topologyNum(); ++i)
        for (int j = 0; j < graph_->getNumInTopoLevel(i); ++j) {
            IRNode *node = graph_->getNodeInTopo(i, j);
            if (node->nodeType() != TENSOR_NODE) continue;
            auto *tn = static_cast<TensorNode *>(node);
            Tensor *t = tn->getTensor();
            if (tensors_name_map_.count(t)) continue;
            const Device dev = tn->getLabel()->getDeviceLabel();
            auto it = dev_allocator_map_.find(dev);
            if (it == dev_allocator_map_.end()) {
                SWLOG_ERROR << "no arena for the device of tensor " << tn->name() << std::endl;
                std::abort();
            }
            MemoryAllocator *arena = it->second;
            uint64_t off;
            IRNode *producer = tn->parentNum() ? tn->getParentNode(0) : nullptr;
            const std::string made = producer ? static_cast<OpNode *>(producer)->getOp()->getOpName() : "";
            if ((made == "Reshape" || made == "TensorDescend" || made == "TensorAscend") &&
                tensors_offset_map_.count(T(producer->getParentNode(0))) &&
                producer->getParentNode(0)->getLabel()->getDeviceLabel() == dev) {
                off = tensors_offset_map_.at(T(producer->getParentNode(0))).second;
                arena->alias(t, off);
            } else {
                off = arena->allocate(t, t->getSizeInBytes());
            }
            tensors_name_map_[t] = UniqueName(tn->name());
            tensors_offset_map_[t] = {arena->getBasePtrName(), off};
            decl_order_.push_back(tn);
        }
}

void Codegen::emitVarDeclarations() {
    for (auto &a : mem_allocators_)
        if (a->getMemAllocated()) writer_ << "char *" << a->getBasePtrName() << ";\n";
    for (TensorNode *tn : decl_order_)
        writer_ << getTypeString(tn->getTensor()) << " *" << tensors_name_map_.at(tn->getTensor()) << ";\n";
    writer_ << "\n";
}

void Codegen::emitMemAllocations() {
    for (auto &a : mem_allocators_) {
        if (!a->getMemAllocated()) continue;
        if (a->getDevice().type != DeviceType::CPU) {
            SWLOG_ERROR << "the CPU generator met a GPU-labelled tensor; use HipCodegen (Config::hip)" << std::endl;
            std::abort();
        }
        // (training: zeroed, as the fresh pages of the reference's malloc are — part of a bias gradient is never written)
        if (config_.train_mode) writer_ << a->getBasePtrName() << " = (char*)calloc(" << a->getMemAllocated() << ", 1);\n";
        else writer_ << a->getBasePtrName() << " = (char*)malloc(" << a->getMemAllocated() << ");\n";
    }
    writer_ << "\n";
}

void Codegen::emitTensorAddresses() {
    for (TensorNode *tn : decl_order_) {
        Tensor *t = tn->getTensor();
        const auto &where = tensors_offset_map_.at(t);
        writer_ << tensors_name_map_.at(t) << " = reinterpret_cast<" << getTypeString(t) << "*>(" << where.first
                << " + " << where.second << ");\n";
    }
    writer_ << "\n";
}

void Codegen::emitTensorInitializations() {
    emitSnapshotRestoreBegin();
    for (TensorNode *tn : decl_order_) {
        Tensor *t = tn->getTensor();
        const std::string name = tensors_name_map_.at(t);
        const TensorInitInfo info = t->getTensorInitInfo();
        writer_ << restoreGuard(t);
        switch (t->getTensorInitType()) {
        case TensorInitType::XAVIER:
            writer_ << "initTensorXavier(" << name << ", " << t->size() << ", " << info.getFilterSize() << ");\n";
            break;
        case TensorInitType::CONSTANT:
            writer_ << "initTensorConstant(" << name << ", " << t->size() << ", " << info.getConstant() << ");\n";
            break;
        case TensorInitType::ZERO:
            writer_ << "initTensorZero(" << name << ", " << t->size() << ");\n";
            break;
        case TensorInitType::FILE:
            writer_ << "load(" << name << ", " << t->size() << ", " << info.getOffset() << ", \"" << info.getFilePath()
                    << "\");\n";
            break;
        case TensorInitType::PARENTOP:
            dispatchOpNode(static_cast<OpNode *>(tn->getParentNode(0)));
            break;
        default:
            break;
        }
    }
    emitSnapshotRestoreEnd();
    writer_ << "\n";
}

bool Codegen::inSnapshot(Tensor *t) const {
    if (!config_.train_mode || t->getDataType() != DataType::Float_t) return false;
    const TensorInitType init = t->getTensorInitType();
    return init == TensorInitType::XAVIER || init == TensorInitType::CONSTANT || init == TensorInitType::ZERO;
}

std::string Codegen::restoreGuard(Tensor *t) const {
    if (!inSnapshot(t)) return "";
    const std::string name = tensors_name_map_.at(t);
    return "if (!swc_restored || !loadFromSnapShot(swc_snapshot, \"" + name + "\", " + name + ", " +
           std::to_string(t->size()) + ")) ";
}

void Codegen::emitSnapshotRestoreBegin() {
    if (!config_.train_mode) return;
    writer_ << "SnapshotNet swc_snapshot;\nconst bool swc_restored = FLAGS_snapshot.size() > 0;\n";
    writer_ << "if (swc_restored) {\n";
    writer_.indentInc();
    writer_ << "std::cout << \"restoring from snapshot \" << FLAGS_snapshot << std::endl;\n";
    writer_ << "if (!swc_snapshot.parse(FLAGS_snapshot)) { std::cout << \"Error loading \" << FLAGS_snapshot << \"\\n\"; "
            << "return 1; }\n";
    writer_.indentDec();
    writer_ << "}\n";
}

void Codegen::emitSnapshotRestoreEnd() {
    if (!config_.train_mode) return;
    writer_ << "if (swc_restored) {\n";
    writer_.indentInc();
    writer_ << "size_t snap_iter = getIterFromSnapShot(swc_snapshot);\nloader.shift(snap_iter);\niter = snap_iter;\n";
    writer_ << "std::cout << \"snapshot iter= \" << snap_iter << std::endl;\n";
    writer_.indentDec();
    writer_ << "}\n";
}

void Codegen::emitSaveSnapshot() {
    if (!config_.train_mode || !config_.train_config.snapshot) return;
    if (config_.benchmark) {   // reference: src/codegen/Codegen.cpp:1001-1007
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
        if (!inSnapshot(t) || !seen.insert(t).second) continue;
        const std::string name = tensors_name_map_.at(t);
        writer_ << "addOp(net, \"" << name << "\", " << name << ", " << t->size() << ");\n";
    }
    writer_ << "std::string snapfile = \"snapshot_iter\" + std::to_string(iter) + \".model\";\n";
    writer_ << "if (!net.save(snapfile)) { std::cout << \"Error opening \" << snapfile << \"\\n\"; return 1; }\n";
    writer_ << "std::cout << \"save snapshot to \" << snapfile << \"\\n\";\n";
    writer_.indentDec();
    writer_ << "}\n";
}

void Codegen::emitExecute() {
    if (config_.use_dataloader) {   // reference: src/codegen/Codegen.cpp:979-993, 1020-1030
        writer_ << "while(loader.next(" << nameOf(loaderLabelNode()) << ", " << nameOf(loaderDataNode()) << ")) {\n";
        writer_.indentInc();
        emitFuncCalls();
        writer_ << "\niter++;\n";
        emitSaveSnapshot();
        if (config_.display > 0) emitPrintGraphOutputs();
        emitMaxItersBreak();
        writer_.indentDec();
        writer_ << "} //while\n";
        return;
    }
    if (config_.time_iters) {
        writer_ << "gettimeofday(&ts, NULL);\n";
        writer_ << "for (size_t swc_iter = 0; swc_iter < " << config_.time_iters << "; swc_iter++) {\n";
        writer_.indentInc();
    }
    emitFuncCalls();
    if (config_.time_iters) {
        writer_.indentDec();
        writer_ << "}\n";
        writer_ << "gettimeofday(&te, NULL);\n";
        writer_ << "std::cout << \"swc_time_ms_per_iter \" << TIME_MS(ts, te) / " << config_.time_iters
                << " << std::endl;\n";
    }
}

void Codegen::emitFuncCalls() {
    for (int i = 0; i < graph_->topologyNum(); ++i)
        for (int j = 0; j < graph_->getNumInTopoLevel(i); ++j) {
            IRNode *node = graph_->getNodeInTopo(i, j);
            if (node->nodeType() != OP_NODE) continue;
            auto *op = static_cast<OpNode *>(node);
            if (op->isRunOnce()) continue;   // emitted with the initialisations
            writer_ << "// topology(" << i << ", " << j << "): " << op->name() << " : " << op->getOp()->getOpName()
                    << "\n";
            dispatchOpNode(op);
        }
}

void Codegen::dispatchOpNode(OpNode *op) {
    if (!op->runable()) return;
    if (op->getLabel()->getDeviceLabel().type != DeviceType::CPU) {
        SWLOG_ERROR << "op " << op->name() << " is labelled for a GPU; the CPU generator cannot emit it" << std::endl;
        std::abort();
    }
    emitFuncCall(op);
}

void Codegen::emitMemFree() {
    for (auto &a : mem_allocators_)
        if (a->getMemAllocated() && a->getDevice().type == DeviceType::CPU)
            writer_ << "free(" << a->getBasePtrName() << ");\n";
}

// Writes every output-marked tensor that lives on the host to "<name>.bin" (a Tensor named by several nodes —
// a parameter and its updated self — is an output if any of them is marked).
void Codegen::emitOutputDump() {
    if (!config_.dump_outputs) return;
    writer_ << "\n// dump graph outputs\n";
    std::set<Tensor *> marked;
    for (int i = 0; i < graph_->tensorNodeNum(); ++i) {
        TensorNode *tn = graph_->getTensorNode(i);
        if (tn->getLabel()->getIsOut() && tn->getLabel()->getDeviceLabel().type == DeviceType::CPU) marked.insert(tn->getTensor());
    }
    for (TensorNode *tn : decl_order_) {
        Tensor *t = tn->getTensor();
        if (!marked.count(t)) continue;
        writer_ << "store(" << tensors_name_map_.at(t) << ", " << t->size() << ", \"" << tensors_name_map_.at(t)
                << ".bin\");\n";
    }
}

// ------------------------------------------------------------ CPU emitters
// One call per op node: the kernel name and argument order of the reference's
// generator for the same op type (file:line of the reference given per case).
void Codegen::emitFuncCall(OpNode *op) {
    const std::string type = op->getOp()->getOpName();
    const std::string nm = op->name();
    auto in = [&](int i) { return op->getParentNode(i); };
    auto out = [&](int i) { return op->getChildNode(i); };

    if (type == "MatrixMatrixMul") {   // Codegen.cpp:1334-1337
        const size_t m = T(in(0))->getDim(0), k = T(in(1))->getDim(0), n = T(in(1))->getDim(1);
        writer_ << "matrixMatrixMul_f(" << m << ", " << n << ", " << k << ", " << nameOf(in(0)) << ", " << k << ", "
                << nameOf(in(1)) << ", " << n << ", " << nameOf(out(0)) << ", " << n << ");\n";
    } else if (type == "MatrixVectorAdd" || type == "BatchedAdd") {   // Codegen.cpp:1513-1515
        auto rc = rowsCols(T(in(0))->getDims());
        assert(rc.second == T(in(1))->size() && "bias length != row length");
        writer_ << "batchedadd_f(" << nameOf(out(0)) << ", " << nameOf(in(0)) << ", " << nameOf(in(1)) << ", "
                << rc.first << ", " << rc.second << ");\n";
    } else if (type == "Reshape" || type == "TensorDescend" || type == "TensorAscend" || type == "Dropout") {   // Codegen.cpp:1480-1485 (pointer alias)
        writer_ << nameOf(out(0)) << " = " << nameOf(in(0)) << ";\n";
    } else if (type == "MatrixTanh") {   // Codegen.cpp:2293-2295
        const size_t m = T(in(0))->getDim(0), n = T(in(0))->getDim(1);
        writer_ << "matrixTanh_f(" << m << ", " << n << ", " << nameOf(in(0)) << ", " << n << ", " << nameOf(out(0))
                << ", " << n << ");\n";
    } else if (type == "MatrixSoftmax") {   // Codegen.cpp:2352-2354
        const size_t m = T(in(0))->getDim(0), n = T(in(0))->getDim(1);
        writer_ << "matrixSoftmax_f(" << m << ", " << n << ", " << nameOf(in(0)) << ", " << n << ", "
                << nameOf(out(0)) << ", " << n << ");\n";
    } else if (type == "ElementAdd") {   // Codegen.cpp:1608-1610
        writer_ << "vecAdd_f(" << T(in(0))->size() << ", " << nameOf(in(0)) << ", " << nameOf(in(1)) << ", "
                << nameOf(out(0)) << ");\n";
    } else if (type == "Relu") {   // Codegen.cpp:2134-2135
        writer_ << "relu_f(" << nameOf(in(0)) << ", " << nameOf(out(0)) << ", " << T(in(0))->size() << ");\n";
    } else if (type == "Conv2d") {   // Codegen.cpp:1761-1782
        auto *conv = static_cast<Conv2dOp *>(op->getOp());
        writer_ << arrayDef(nm + "_inDims", T(in(0))->getDims()) << arrayDef(nm + "_outDims", T(out(0))->getDims())
                << arrayDef(nm + "_filterDims", T(in(1))->getDims()) << arrayDef(nm + "_biasDims", T(in(2))->getDims())
                << arrayDef(nm + "_filterSizes", conv->getKernels()) << arrayDef(nm + "_strides", conv->getStrides())
                << arrayDef(nm + "_pads", conv->getPads());
        writer_ << "conv2d_f(" << nameOf(out(0)) << ", " << nameOf(in(0)) << ", " << nameOf(in(1)) << ", "
                << nameOf(in(2)) << ", " << nm << "_outDims, " << nm << "_inDims, " << nm << "_filterDims, " << nm
                << "_biasDims, " << nm << "_filterSizes, " << nm << "_strides, " << nm << "_pads, "
                << conv->getGroup() << ");\n";
    } else if (type == "BatchNormalization") {   // Codegen.cpp:1832-1837,1907-1915: parents in, scale, bias, mean, var
        const float eps = static_cast<BatchNormalizationOp *>(op->getOp())->getEpsilon();
        writer_ << arrayDef(nm + "_inDims", T(in(0))->getDims());
        writer_ << "batchnormalization_f(" << nameOf(out(0)) << ", " << nameOf(in(0)) << ", " << nameOf(in(3)) << ", "
                << nameOf(in(4)) << ", " << nameOf(in(1)) << ", " << nameOf(in(2)) << ", " << nm << "_inDims, "
                << std::setprecision(12) << eps << ");\n";
    } else if (type == "MaxPool") {   // Codegen.cpp:2020-2037
        auto *pool = static_cast<MaxPoolOp *>(op->getOp());
        writer_ << arrayDef(nm + "_inDims", T(in(0))->getDims()) << arrayDef(nm + "_outDims", T(out(0))->getDims())
                << arrayDef(nm + "_filterSizes", pool->getKernels()) << arrayDef(nm + "_strides", pool->getStrides())
                << arrayDef(nm + "_pads", pool->getPads());
        writer_ << "maxpool_f(" << nameOf(in(0)) << ", " << nameOf(out(0)) << ", " << nm << "_inDims, " << nm
                << "_outDims, " << nm << "_filterSizes, " << nm << "_strides, " << nm << "_pads);\n";
    } else if (type == "AveragePool") {   // Codegen.cpp:2020-2044
        auto *pool = static_cast<AvgPoolOp *>(op->getOp());
        writer_ << arrayDef(nm + "_inDims", T(in(0))->getDims()) << arrayDef(nm + "_outDims", T(out(0))->getDims())
                << arrayDef(nm + "_filterSizes", pool->getKernels()) << arrayDef(nm + "_strides", pool->getStrides())
                << arrayDef(nm + "_pads", pool->getPads());
        writer_ << "avgpool_f(" << nameOf(in(0)) << ", " << nameOf(out(0)) << ", " << nm << "_inDims, " << nm
                << "_outDims, " << nm << "_filterSizes, " << nm << "_strides, " << nm << "_pads);\n";
    } else if (type == "Transpose") {   // Codegen.cpp:2255-2284 (which hard-codes the shuffle {1,0}; the op's own is used here)
        auto *tr = static_cast<TransposeOp *>(op->getOp());
        const int nd = T(in(0))->getNDim();
        if ((nd != 2 && nd != 4) || (int)tr->getShuffle().size() != nd) {
            SWLOG_ERROR << "Transpose " << nm << ": only 2-D and 4-D tensors with a full shuffle" << std::endl;
            std::abort();
        }
        writer_ << arrayDef(nm + "_inDims", T(in(0))->getDims()) << arrayDef(nm + "_outDims", T(out(0))->getDims())
                << arrayDef(nm + "_shuffle", tr->getShuffle());
        writer_ << (nd == 2 ? "transpose2d_f(" : "transpose4d_f(") << nameOf(in(0)) << ", " << nameOf(out(0)) << ", "
                << nm << "_inDims, " << nm << "_outDims, " << nm << "_shuffle);\n";
    } else if (type == "ArgMax") {   // Codegen.cpp:2372-2385
        const int topK = static_cast<ArgMaxOp *>(op->getOp())->getTopK();
        writer_ << "argMax_i(" << nameOf(in(0)) << ", " << nameOf(out(0)) << ", " << T(in(0))->getDim(0) << ", "
                << T(in(0))->getDim(1) << ", " << topK << ");\n";
    } else if (type == "Accuracy") {   // Codegen.cpp:2387-2398
        writer_ << "accuracy_i(" << nameOf(in(0)) << ", " << nameOf(in(1)) << ", " << nameOf(out(0)) << ", "
                << T(in(0))->getDim(0) << ", " << T(in(0))->getDim(1) << ");\n";
    } else if (type == "BatchedReduceAdd") {   // Codegen.cpp:1517-1531
        const auto rc = T(in(0))->viewAs2D(T(in(0))->getNDim() - 1);
        if (rc.first > T(out(0))->size()) {   // one sum per ROW goes into the result (kernels.h:554-563): it must hold them
            SWLOG_ERROR << "BatchedReduceAdd " << nm << ": " << rc.first << " rows into a result of " << T(out(0))->size()
                        << " elements — the reference's kernel would write past it (mini-batch larger than the layer)" << std::endl;
            std::abort();
        }
        writer_ << "batchedreduceadd_f(" << nameOf(out(0)) << ", " << nameOf(in(0)) << ", " << rc.first << ", " << rc.second
                << ");\n";
    } else if (type == "ReluGrad") {   // Codegen.cpp:2138-2148: parents input, outputGrad
        writer_ << "reluGrad_f(" << nameOf(out(0)) << ", " << nameOf(in(0)) << ", " << nameOf(in(1)) << ", "
                << T(in(0))->size() << ");\n";
    } else if (type == "MatrixTanhGrad") {   // Codegen.cpp:2414-2427: parents input, output, outputGrad
        const size_t m = T(in(0))->getDim(0), n = T(in(0))->getDim(1);
        writer_ << "matrixTanhGrad_f(" << m << ", " << n << ", " << nameOf(out(0)) << ", " << n << ", " << nameOf(in(1))
                << ", " << n << ", " << nameOf(in(2)) << ", " << n << ");\n";
    } else if (type == "MaxPoolGrad") {   // Codegen.cpp:2047-2079: parents input, output, outputGrad
        auto *pool = static_cast<MaxPoolGradOp *>(op->getOp());
        writer_ << arrayDef(nm + "_inDims", T(in(0))->getDims()) << arrayDef(nm + "_outDims", T(in(1))->getDims())
                << arrayDef(nm + "_filterSizes", pool->getKernels()) << arrayDef(nm + "_strides", pool->getStrides())
                << arrayDef(nm + "_pads", pool->getPads());
        writer_ << "maxpoolGrad_f(" << nameOf(out(0)) << ", " << nameOf(in(2)) << ", " << nameOf(in(0)) << ", " << nm
                << "_inDims, " << nm << "_outDims, " << nm << "_filterSizes, " << nm << "_strides, " << nm << "_pads);\n";
    } else if (type == "Conv2dGrad") {   // Codegen.cpp:1785-1830: parents input, filter, outputGrad
        auto *conv = static_cast<Conv2dGradOp *>(op->getOp());
        writer_ << arrayDef(nm + "_inDims", T(in(0))->getDims()) << arrayDef(nm + "_outDims", T(in(2))->getDims())
                << arrayDef(nm + "_filterDims", T(in(1))->getDims()) << arrayDef(nm + "_biasDims", T(out(2))->getDims())
                << arrayDef(nm + "_filterSizes", conv->getKernels()) << arrayDef(nm + "_strides", conv->getStrides())
                << arrayDef(nm + "_pads", conv->getPads());
        writer_ << "conv2dGrad_f(" << nameOf(out(0)) << ", " << nameOf(out(1)) << ", " << nameOf(out(2)) << ", "
                << nameOf(in(2)) << ", " << nameOf(in(0)) << ", " << nameOf(in(1)) << ", " << nm << "_outDims, " << nm
                << "_inDims, " << nm << "_filterDims, " << nm << "_biasDims, " << nm << "_filterSizes, " << nm
                << "_strides, " << nm << "_pads, " << conv->getGroup() << ");\n";
    } else if (type == "MatrixSoftmaxWithLoss") {   // Codegen.cpp:2357-2370: parents logits, label -> prob, loss
        const size_t m = T(in(0))->getDim(0), n = T(in(0))->getDim(1);
        writer_ << "matrixSoftmaxWithLoss_f(" << m << ", " << n << ", " << nameOf(in(0)) << ", " << n << ", "
                << nameOf(out(0)) << ", " << n << ", " << nameOf(in(1)) << ", " << nameOf(out(1)) << ");\n";
    } else if (type == "MatrixSoftmaxWithLossGrad") {   // Codegen.cpp:2446-2465: parents label, prob
        const size_t m = T(in(1))->getDim(0), n = T(in(1))->getDim(1);
        writer_ << "matrixSoftmaxWithLossGrad_f(" << m << ", " << n << ", " << nameOf(out(0)) << ", " << n << ", "
                << nameOf(in(1)) << ", " << n << ", " << nameOf(in(0)) << ");\n";
    } else if (type == "MatrixSoftmaxGrad") {   // Codegen.cpp:2429-2444: parents input, label, output(, outputGrad)
        const size_t m = T(in(0))->getDim(0), n = T(in(0))->getDim(1);
        writer_ << "matrixSoftmaxGrad_f(" << m << ", " << n << ", " << nameOf(out(0)) << ", " << n << ", "
                << nameOf(in(2)) << ", " << n << ", " << nameOf(in(1)) << ");\n";
    } else if (type == "SGD") {   // Codegen.cpp:2468-2489: parents parameter, gradient, momentum; in place
        auto *sgd = static_cast<SGDOp *>(op->getOp());
        writer_ << "sgd_f(" << T(in(0))->size() << ", " << nameOf(in(0)) << ", " << nameOf(in(0)) << ", " << nameOf(in(1))
                << ", " << nameOf(in(2)) << ", " << sgd->getLR() << ", " << sgd->getDecay() << ", " << sgd->getMomentum()
                << ", " << sgd->getBatch() << ");\n";
    } else if (type == "Debug") {   // Codegen.cpp:2401-2412
        Tensor *a = T(in(0));
        writer_ << "printMatrix(" << nameOf(in(0)) << ", " << a->getDim(0) << ", "
                << (a->getNDim() == 2 ? a->getDim(1) : 1) << ");\n";
        if (op->childNum()) writer_ << nameOf(out(0)) << " = " << nameOf(in(0)) << ";\n";
    } else {
        SWLOG_ERROR << "no CPU emitter for op type " << type << " (node " << nm << ")" << std::endl;
        std::abort();
    }
}

} // namespace codegen
} // namespace swc
