// Code generators: print a C++ host program for an IRGraph.
//
//   Codegen      the CPU target.  Emits, per op node in topological order, the
//                call into the reference's kernel header that the reference's
//                generator emits (same function names, same argument order;
//                src/codegen/Codegen.cpp:1171-2494, non-MKLDNN branches), so
//                the program builds against `utils/image.h` + `utils/kernels.h`.
//   HipCodegen   the MI355X target.  Walks a graph the DeviceMemoryLoweringPass
//                has placed, emits swc_hip_* calls (include/swc_hip.h) on one
//                256-byte-aligned device arena, h2d/d2h at Scatter/Gather nodes.
// The emit phases are virtual in the order generate() calls them, the same
// override surface as the reference's Codegen (src/codegen/Codegen.h:51-151).
#ifndef SWC_CODEGEN_H_
#define SWC_CODEGEN_H_
#include <cstdint>
#include <map>
#include <memory>
#include <set>
#include <sstream>
#include <string>
#include <unordered_map>
#include <vector>

#include "../common.h"
#include "../devices/HipDevice.h"

namespace swc {
class IRGraph;
class TensorNode;
class OpNode;
class Tensor;
class IRNode;

namespace codegen {

// Indentation-aware string sink (reference: src/codegen/CodeWriter.h).
class CodeWriter {
    std::ostringstream out_;
    int indent_{0};
    bool lineStart_{true};

  public:
    void indentInc() { ++indent_; }
    void indentDec() { if (indent_ > 0) --indent_; }
    template <typename T> CodeWriter &operator<<(const T &v) {
        std::ostringstream tmp;
        tmp << v;
        write(tmp.str());
        return *this;
    }
    std::string get_code() const { return out_.str(); }
    void clear() { out_.str(""); lineStart_ = true; }

  private:
    void write(const std::string &s) {
        for (char c : s) {
            if (lineStart_ && c != '\n') out_ << std::string((size_t)indent_ * 4, ' ');
            out_ << c;
            lineStart_ = (c == '\n');
        }
    }
};

// Bump allocator over one arena (reference: src/codegen/MemoryAllocator.h:21-49,
// which packs with no alignment).  Offsets are rounded up to `alignment`.
class MemoryAllocator {
    Device dev_;
    std::string base_;
    uint64_t capacity_, used_{0}, alignment_;
    std::map<Tensor *, uint64_t> offsets_;

  public:
    MemoryAllocator(Device dev, std::string basePtrName, uint64_t capacity = UINT64_MAX, uint64_t alignment = 1)
        : dev_(dev), base_(std::move(basePtrName)), capacity_(capacity), alignment_(alignment ? alignment : 1) {}
    uint64_t allocate(Tensor *t, uint64_t bytes);
    void alias(Tensor *t, uint64_t offset) { offsets_[t] = offset; }
    bool has(Tensor *t) const { return offsets_.count(t) != 0; }
    uint64_t offsetOf(Tensor *t) const { return offsets_.at(t); }
    uint64_t getMemAllocated() const { return used_; }
    uint64_t getCapacity() const { return capacity_; }
    std::string getBasePtrName() const { return base_; }
    Device getDevice() const { return dev_; }
    void setBasePtrName(std::string n) { base_ = std::move(n); }
    void clear() { used_ = 0; offsets_.clear(); }
};

// Makefile text for the generated program (reference: src/codegen/MakefileBuilder.h).
class MakefileBuilder {
    std::string cxx_{"/usr/bin/c++"}, target_{"net.bin"}, runCmd_{"./net.bin"};
    std::vector<std::string> flags_, incs_, libDirs_, libs_, srcs_;

  public:
    void setCXXCompiler(std::string c) { cxx_ = std::move(c); }
    void addCXXFlag(std::string f) { flags_.push_back(std::move(f)); }
    void addIncDir(std::string d) { incs_.push_back(std::move(d)); }
    void addLibDir(std::string d) { libDirs_.push_back(std::move(d)); }
    void addLib(std::string l) { libs_.push_back(std::move(l)); }
    void addCXXSrc(std::string s) { srcs_.push_back(std::move(s)); }
    void setTarget(std::string t) { target_ = std::move(t); }
    void setRunCmd(std::string c) { runCmd_ = std::move(c); }
    std::string generate() const;
};

class Codegen {
  public:
    Codegen() : graph_(nullptr) {}
    explicit Codegen(IRGraph *graph);
    Codegen(IRGraph *graph, Config &config);
    virtual ~Codegen() {}

    // Prints the program, writes ./Graph.cpp, ./G_Makefile and ./SW_Makefile,
    // returns the source text.
    std::string generate();
    virtual bool isHipGenerator() const { return false; }

    virtual void initMakefileBuilder();
    virtual void emitHeader();
    virtual void emitEnvInit();
    virtual void emitEnvFinalize();
    virtual void allocateMemAddr();
    virtual void emitVarDeclarations();
    virtual void emitMemAllocations();
    virtual void emitTensorAddresses();
    virtual void emitTensorInitializations();
    virtual void emitExecute();
    virtual void emitFuncCalls();
    virtual void emitMemFree();
    virtual void emitDataLoaderInit() {}          // (the training loader is emitInferDataLoaderInit over the training records)
    void emitMaxItersBreak();
    void trainAsBatchLoop();                       // Config::train_mode: the training settings become the batch loop's
    TensorNode *loaderLabelNode() const;           // what loader.next fills: the training or the inference pair
    TensorNode *loaderDataNode() const;
    virtual void emitInferDataLoaderInit();        // `DataLoader loader(...)` + iteration counter
    virtual void emitPrintGraphOutputs();          // every Config::display iterations: the display tensors
    // Snapshots of a training program (reference: src/codegen/Codegen.cpp:659-812).  Every
    // TrainingConfig::snapshot iterations the tensors that start from an initialiser (Xavier, constant, zero:
    // parameters and momenta) and the iteration count go to snapshot_iter<N>.model; a program started with
    // --snapshot=<file> takes those tensors and the count from the file and moves the loader on accordingly.
    virtual void emitSaveSnapshot();
    void emitSnapshotRestoreBegin();               // parses the file named by the flag, if any
    void emitSnapshotRestoreEnd();                 // iteration count and loader position
    bool inSnapshot(Tensor *t) const;              // float tensor with an initialiser of its own, training program
    std::string restoreGuard(Tensor *t) const;     // prefix of such a tensor's initialiser call: restore, else initialise

    void codeGenInit();
    void emitMemAllocs();
    std::string UniqueName(std::string name);

  protected:
    // one op node -> its call; CPU emitters here, overridden by the HIP target
    virtual void dispatchOpNode(OpNode *op);
    void emitFuncCall(OpNode *op);
    void emitOutputDump();
    std::string getTypeString(Tensor *t) const;
    std::string nameOf(IRNode *tensorNode);
    static std::string arrayDef(const std::string &name, const std::vector<size_t> &values);

    CodeWriter headerWriter_, writer_;
    MakefileBuilder makefile_builder_, swmakefile_builder_;
    IRGraph *graph_;
    Config config_;
    std::unordered_map<std::string, int> names_map_;
    std::vector<std::shared_ptr<MemoryAllocator>> mem_allocators_;
    std::map<Tensor *, std::string> tensors_name_map_;
    std::map<Tensor *, std::pair<std::string, uint64_t>> tensors_offset_map_;
    std::unordered_map<Device, MemoryAllocator *> dev_allocator_map_;
    std::vector<TensorNode *> decl_order_;   // tensors in first-seen topological order
};

class HipCodegen : public Codegen {
    devices::HipDevice device_;
    bool has_workspace_ = false;   // the program holds a workspace for its FC calls
    // Inside the batch loop a download nobody on the host reads (a graph output, a counter that is only
    // displayed) is not emitted per iteration: it is held here and emitted where it is shown and once after
    // the loop, so the device runs one batch while the loader reads the next.
    bool defer_output_gathers_ = false;
    std::vector<OpNode *> deferred_gathers_;

  public:
    HipCodegen(IRGraph *graph, Config &config) : Codegen(graph, config) {}
    bool isHipGenerator() const override { return true; }
    void initMakefileBuilder() override;
    void emitHeader() override;
    void emitEnvInit() override;
    void emitEnvFinalize() override;
    void allocateMemAddr() override;
    void emitMemAllocations() override;
    void emitWorkspace();
    bool isDeviceComputeOp(OpNode *op) const;
    bool deviceOpsAreContiguous() const;
    void emitTensorInitializations() override;
    void emitExecute() override;
    void emitMemFree() override;
    void emitPrintGraphOutputs() override;
    void emitSaveSnapshot() override;   // the trained copies live on the device: they are downloaded into their host tensors first

  protected:
    void emitDeviceFills();        // constant initialisers of device tensors that have no host twin
    void emitDeferredGathers();
    void dispatchOpNode(OpNode *op) override;
    void emitHipCall(OpNode *op);
    void emitTransfer(OpNode *op, bool toDevice);
    void emitDeviceOpsOnly();   // the op sequence without transfers and host ops (what a HIP graph records)
};

} // namespace codegen
} // namespace swc
#endif
