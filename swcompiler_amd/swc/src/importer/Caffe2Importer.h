// Builds an IRGraph from a Caffe2 model: `predict_net` (the operators) and
// `init_net` (the weights, as GivenTensorFill / ConstantFill operators).
// Same constructor and behaviour as the reference's importer
// (src/importer/Caffe2Importer.h:32-74, Caffe2Importer.cpp:119-563):
//   * the caller defines the data tensor(s) in NHWC and passes them in `udef_nodes`;
//   * Conv weights arrive as [oC,iC,kh,kw] and get a Transpose(NCHW2NHWC) node;
//   * FC weights arrive as [out,in] and get a Transpose({1,0}); a 4-D FC input
//     is transposed back to NCHW first, so that its flattened order is the one
//     the weights were trained with;
//   * SpatialBN, Relu, Sum, MaxPool, AveragePool, Softmax, Dropout map to the
//     ops of the same meaning; an operator that writes its own input shares
//     the input's Tensor (in place);
//   * weight values are written to raw fp32 files (FILE initialisers).
//
// The reference parses the files with libprotobuf and generated classes; this
// one reads the protobuf wire format (and the text format of `.pbtxt` files)
// directly — only the fields of NetDef / OperatorDef / Argument the importer
// uses (caffe2.proto:152-166, 208-268, 270-309) — so it needs no library.
#ifndef SWC_CAFFE2IMPORTER_H_
#define SWC_CAFFE2IMPORTER_H_
#include <cstdint>
#include <string>
#include <unordered_map>
#include <vector>

#include "../graphIR/IRGraph.h"

namespace swc {

class TensorNode;
class OpNode;

namespace caffe2 {
struct Argument {
    std::string name, s;
    float f = 0.f;
    int64_t i = 0;
    bool has_f = false, has_i = false, has_s = false;
    std::vector<float> floats;
    std::vector<int64_t> ints;
    std::vector<std::string> strings;
};
struct OperatorDef {
    std::vector<std::string> input, output;
    std::string name, type;
    std::vector<Argument> arg;
    const Argument *find(const std::string &argName) const {
        for (const Argument &a : arg)
            if (a.name == argName) return &a;
        return nullptr;
    }
};
struct NetDef {
    std::string name;
    std::vector<OperatorDef> op;
    std::vector<std::string> external_input, external_output;
};
// binary (.pb) or text (.pbtxt) by file name; false with a message in `error` if the file cannot be read or parsed
bool loadNetDef(const std::string &path, NetDef &net, std::string &error);
} // namespace caffe2

class Caffe2Importer {
    IRGraph *graph_;
    std::string weightDir_;
    std::unordered_map<std::string, TensorNode *> name_tNode_map_;
    std::unordered_map<std::string, OpNode *> name_opNode_map_;
    std::unordered_map<std::string, int> op_names_;

    void loadNetwork(const caffe2::NetDef &net);
    void loadTensors(const caffe2::NetDef &tensors);
    void loadOp(const caffe2::OperatorDef &op);
    void loadTensor(const caffe2::OperatorDef &op);
    TensorNode *blob(const caffe2::OperatorDef &op, int inputIdx) const;
    TensorNode *result(const caffe2::OperatorDef &op, TensorNode *like, OpNode *producer,
                       const std::vector<size_t> *dims = nullptr);
    std::string uniqueOpName(const std::string &type);

  public:
    // weightDir: where the raw fp32 files of the GivenTensorFill values go (created if missing; the reference
    // uses /tmp/SW)
    Caffe2Importer(IRGraph *g, const std::string &netProtoFile, const std::string &tensorProtoFile,
                   std::vector<TensorNode *> &udef_nodes, const std::string &weightDir = "/tmp/SW");

    static const std::vector<std::string> &supportedOps();
};

} // namespace swc
#endif
