// Caffe2 model -> IRGraph (see Caffe2Importer.h).  Reference behaviour:
// src/importer/Caffe2Importer.cpp:119-563.
#include "Caffe2Importer.h"

#include <algorithm>
#include <cctype>
#include <cerrno>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <fstream>
#include <iostream>
#include <iterator>
#include <sys/stat.h>

#include "../SWLOG.h"
#include "../common.h"
#include "../graphIR/OpNode.h"
#include "../graphIR/TensorNode.h"
#include "../op/ops.h"
#include "../tensor/tensor.h"

namespace swc {
namespace caffe2 {
namespace {

// ------------------------------------------------------ protobuf wire format
// A message is a sequence of (tag, value): tag = field number << 3 | wire type; wire types 0 varint,
// 1 fixed 64-bit, 2 length-delimited (strings, sub-messages, packed repeated scalars), 5 fixed 32-bit.
struct Wire {
    const uint8_t *p, *end;
    bool ok = true;

    bool done() const { return !ok || p >= end; }
    uint64_t varint() {
        uint64_t v = 0;
        for (int shift = 0; shift < 64 && p < end; shift += 7) {
            const uint8_t b = *p++;
            v |= (uint64_t)(b & 0x7f) << shift;
            if (!(b & 0x80)) return v;
        }
        ok = false;
        return 0;
    }
    template <typename T> T fixed() {
        T v{};
        if ((size_t)(end - p) < sizeof(T)) {
            ok = false;
            return v;
        }
        std::memcpy(&v, p, sizeof(T));   // little-endian on the wire and on the host
        p += sizeof(T);
        return v;
    }
    Wire sub() {
        const uint64_t n = varint();
        if (!ok || n > (uint64_t)(end - p)) {
            ok = false;
            return Wire{p, p};
        }
        Wire w{p, p + n};
        p += n;
        return w;
    }
    std::string str() {
        Wire w = sub();
        return std::string(reinterpret_cast<const char *>(w.p), w.end - w.p);
    }
    void skip(uint32_t wireType) {
        switch (wireType) {
        case 0: (void)varint(); break;
        case 1: (void)fixed<uint64_t>(); break;
        case 2: (void)sub(); break;
        case 5: (void)fixed<uint32_t>(); break;
        default: ok = false;   // groups (3, 4) do not occur in these messages
        }
    }
};

bool parseArgument(Wire w, Argument &a) {
    while (!w.done()) {
        const uint64_t tag = w.varint();
        const uint32_t field = (uint32_t)(tag >> 3), wt = (uint32_t)(tag & 7);
        if (field == 1 && wt == 2) a.name = w.str();
        else if (field == 2 && wt == 5) a.f = w.fixed<float>(), a.has_f = true;
        else if (field == 3 && wt == 0) a.i = (int64_t)w.varint(), a.has_i = true;
        else if (field == 4 && wt == 2) a.s = w.str(), a.has_s = true;
        else if (field == 5 && wt == 5) a.floats.push_back(w.fixed<float>());
        else if (field == 5 && wt == 2) {   // packed
            Wire pk = w.sub();
            a.floats.reserve(a.floats.size() + (pk.end - pk.p) / 4);
            while (!pk.done()) a.floats.push_back(pk.fixed<float>());
            w.ok &= pk.ok;
        } else if (field == 6 && wt == 0) a.ints.push_back((int64_t)w.varint());
        else if (field == 6 && wt == 2) {
            Wire pk = w.sub();
            while (!pk.done()) a.ints.push_back((int64_t)pk.varint());
            w.ok &= pk.ok;
        } else if (field == 7 && wt == 2) a.strings.push_back(w.str());
        else w.skip(wt);
    }
    return w.ok;
}

bool parseOperator(Wire w, OperatorDef &op) {
    while (!w.done()) {
        const uint64_t tag = w.varint();
        const uint32_t field = (uint32_t)(tag >> 3), wt = (uint32_t)(tag & 7);
        if (field == 1 && wt == 2) op.input.push_back(w.str());
        else if (field == 2 && wt == 2) op.output.push_back(w.str());
        else if (field == 3 && wt == 2) op.name = w.str();
        else if (field == 4 && wt == 2) op.type = w.str();
        else if (field == 5 && wt == 2) {
            op.arg.emplace_back();
            if (!parseArgument(w.sub(), op.arg.back())) return false;
        } else w.skip(wt);
    }
    return w.ok;
}

bool parseNet(Wire w, NetDef &net) {
    while (!w.done()) {
        const uint64_t tag = w.varint();
        const uint32_t field = (uint32_t)(tag >> 3), wt = (uint32_t)(tag & 7);
        if (field == 1 && wt == 2) net.name = w.str();
        else if (field == 2 && wt == 2) {
            net.op.emplace_back();
            if (!parseOperator(w.sub(), net.op.back())) return false;
        } else if (field == 7 && wt == 2) net.external_input.push_back(w.str());
        else if (field == 8 && wt == 2) net.external_output.push_back(w.str());
        else w.skip(wt);
    }
    return w.ok;
}

// -------------------------------------------------------- protobuf text format
// `name: value` and `name { ... }` (also `name: { ... }`), `#` comments, quoted strings with C escapes.
struct Text {
    const char *p, *end;
    std::string error;

    void space() {
        while (p < end) {
            if (std::isspace((unsigned char)*p)) ++p;
            else if (*p == '#') while (p < end && *p != '\n') ++p;
            else break;
        }
    }
    bool fail(const std::string &what) {
        if (error.empty()) error = what;
        return false;
    }
    bool ident(std::string &out) {
        space();
        const char *b = p;
        while (p < end && (std::isalnum((unsigned char)*p) || *p == '_')) ++p;
        out.assign(b, p);
        return !out.empty() || fail("field name expected");
    }
    bool eat(char c) {
        space();
        if (p < end && *p == c) return ++p, true;
        return false;
    }
    bool quoted(std::string &out) {
        space();
        out.clear();
        bool any = false;
        while (p < end && (*p == '"' || *p == '\'')) {   // adjacent literals concatenate
            const char q = *p++;
            any = true;
            while (p < end && *p != q) {
                char c = *p++;
                if (c == '\\' && p < end) {
                    c = *p++;
                    switch (c) {
                    case 'n': c = '\n'; break;
                    case 't': c = '\t'; break;
                    case 'r': c = '\r'; break;
                    case '0': case '1': case '2': case '3': case '4': case '5': case '6': case '7': {
                        int v = c - '0';
                        for (int k = 0; k < 2 && p < end && *p >= '0' && *p <= '7'; ++k) v = v * 8 + (*p++ - '0');
                        c = (char)v;
                        break;
                    }
                    default: break;   // \\ \" \' and anything else: the character itself
                    }
                }
                out.push_back(c);
            }
            if (p >= end) return fail("unterminated string");
            ++p;
            space();
        }
        return any || fail("string expected");
    }
    bool number(std::string &out) {
        space();
        const char *b = p;
        while (p < end && (std::isalnum((unsigned char)*p) || *p == '.' || *p == '-' || *p == '+')) ++p;
        out.assign(b, p);
        return !out.empty() || fail("number expected");
    }
    bool skipValue() {   // a field this importer does not use
        if (eat(':')) {
            space();
            if (p < end && (*p == '"' || *p == '\'')) {
                std::string s;
                return quoted(s);
            }
            if (p < end && *p == '{') return skipValue();
            std::string n;
            return number(n);
        }
        if (!eat('{')) return fail("':' or '{' expected");
        for (;;) {
            if (eat('}')) return true;
            std::string name;
            if (!ident(name) || !skipValue()) return false;
        }
    }
    // `{` of a sub-message, with or without a colon in front
    bool open() {
        (void)eat(':');
        return eat('{') || fail("'{' expected");
    }
};

bool textArgument(Text &t, Argument &a) {
    if (!t.open()) return false;
    for (;;) {
        if (t.eat('}')) return true;
        std::string name, v;
        if (!t.ident(name)) return false;
        if (name == "name" || name == "s" || name == "strings") {
            if (!t.eat(':') || !t.quoted(v)) return t.fail("string value expected after " + name);
            if (name == "name") a.name = v;
            else if (name == "s") a.s = v, a.has_s = true;
            else a.strings.push_back(v);
        } else if (name == "f" || name == "floats" || name == "i" || name == "ints") {
            if (!t.eat(':') || !t.number(v)) return t.fail("number expected after " + name);
            if (name == "f") a.f = std::strtof(v.c_str(), nullptr), a.has_f = true;
            else if (name == "floats") a.floats.push_back(std::strtof(v.c_str(), nullptr));
            else if (name == "i") a.i = std::strtoll(v.c_str(), nullptr, 10), a.has_i = true;
            else a.ints.push_back(std::strtoll(v.c_str(), nullptr, 10));
        } else if (!t.skipValue()) return false;
    }
}

bool textOperator(Text &t, OperatorDef &op) {
    if (!t.open()) return false;
    for (;;) {
        if (t.eat('}')) return true;
        std::string name, v;
        if (!t.ident(name)) return false;
        if (name == "input" || name == "output" || name == "name" || name == "type") {
            if (!t.eat(':') || !t.quoted(v)) return t.fail("string value expected after " + name);
            if (name == "input") op.input.push_back(v);
            else if (name == "output") op.output.push_back(v);
            else if (name == "name") op.name = v;
            else op.type = v;
        } else if (name == "arg") {
            op.arg.emplace_back();
            if (!textArgument(t, op.arg.back())) return false;
        } else if (!t.skipValue()) return false;
    }
}

bool textNet(Text &t, NetDef &net) {
    for (;;) {
        t.space();
        if (t.p >= t.end) return true;
        std::string name, v;
        if (!t.ident(name)) return false;
        if (name == "name" || name == "external_input" || name == "external_output") {
            if (!t.eat(':') || !t.quoted(v)) return t.fail("string value expected after " + name);
            if (name == "name") net.name = v;
            else if (name == "external_input") net.external_input.push_back(v);
            else net.external_output.push_back(v);
        } else if (name == "op") {
            net.op.emplace_back();
            if (!textOperator(t, net.op.back())) return false;
        } else if (!t.skipValue()) return false;
    }
}

} // namespace

bool loadNetDef(const std::string &path, NetDef &net, std::string &error) {
    std::ifstream f(path, std::ios::in | std::ios::binary);
    if (!f) {
        error = "cannot open " + path;
        return false;
    }
    const std::string bytes((std::istreambuf_iterator<char>(f)), std::istreambuf_iterator<char>());
    if (path.find(".pbtxt") != std::string::npos) {   // the reference's rule (Caffe2Importer.cpp:152)
        Text t{bytes.data(), bytes.data() + bytes.size(), ""};
        if (!textNet(t, net)) {
            error = path + ": " + t.error;
            return false;
        }
        return true;
    }
    const auto *b = reinterpret_cast<const uint8_t *>(bytes.data());
    if (!parseNet(Wire{b, b + bytes.size()}, net)) {
        error = path + ": not a serialized NetDef";
        return false;
    }
    return true;
}

} // namespace caffe2

// ------------------------------------------------------------------ importer
using namespace swc::op;

namespace {

[[noreturn]] void die(const std::string &what) {
    SWLOG_ERROR << "Caffe2Importer: " << what << std::endl;
    std::exit(EXIT_FAILURE);
}

// pad | pad_t,l,b,r | pads: {top, left, bottom, right}   (Caffe2Importer.cpp:35-57)
std::vector<size_t> padsOf(const caffe2::OperatorDef &op) {
    if (auto *a = op.find("pad")) return std::vector<size_t>(4, (size_t)a->i);
    if (op.find("pad_t")) {
        std::vector<size_t> p;
        for (const char *n : {"pad_t", "pad_l", "pad_b", "pad_r"}) p.push_back(op.find(n) ? (size_t)op.find(n)->i : 0);
        return p;
    }
    if (auto *a = op.find("pads")) {
        std::vector<size_t> p(a->ints.begin(), a->ints.end());
        if (p.size() != 4) die(op.type + ": `pads` needs four values");
        return p;
    }
    return {0, 0, 0, 0};
}

// kernel | kernel_h,kernel_w | kernels; {0,0} if none is given (Caffe2Importer.cpp:60-70 reads `kernel` only)
std::vector<size_t> pairOf(const caffe2::OperatorDef &op, const char *one, const char *h, const char *w, const char *list,
                           size_t fallback) {
    if (auto *a = op.find(one)) return {(size_t)a->i, (size_t)a->i};
    if (op.find(h) && op.find(w)) return {(size_t)op.find(h)->i, (size_t)op.find(w)->i};
    if (auto *a = op.find(list))
        if (a->ints.size() == 2) return {(size_t)a->ints[0], (size_t)a->ints[1]};
    return {fallback, fallback};
}

// (in + pad_begin + pad_end - k) / s + 1   (Caffe2Importer.cpp:79-91)
std::vector<size_t> outHW(const std::string &who, size_t ih, size_t iw, const std::vector<size_t> &k,
                          const std::vector<size_t> &s, const std::vector<size_t> &p) {
    if (!k[0] || !k[1] || !s[0] || !s[1]) die(who + ": kernel and stride must be positive");
    if (ih + p[0] + p[2] < k[0] || iw + p[1] + p[3] < k[1]) die(who + ": window larger than the padded input");
    return {(ih + p[0] + p[2] - k[0]) / s[0] + 1, (iw + p[1] + p[3] - k[1]) / s[1] + 1};
}

std::string fileNameOf(const std::string &blob) {
    std::string s = blob;
    for (char &c : s)
        if (!(std::isalnum((unsigned char)c) || c == '_')) c = '_';
    return s;
}

} // namespace

const std::vector<std::string> &Caffe2Importer::supportedOps() {
    static const std::vector<std::string> ops = {"Conv", "SpatialBN", "Relu",    "Sum",    "MaxPool",
                                                 "AveragePool", "FC",  "Softmax", "Dropout"};
    return ops;
}

Caffe2Importer::Caffe2Importer(IRGraph *g, const std::string &netProtoFile, const std::string &tensorProtoFile,
                               std::vector<TensorNode *> &udef_nodes, const std::string &weightDir)
    : graph_(g), weightDir_(weightDir) {
    for (TensorNode *t : udef_nodes) {
        graph_->pushTensorNode(t);
        name_tNode_map_[t->name()] = t;
    }
    if (mkdir(weightDir_.c_str(), 0777) != 0 && errno != EEXIST) die("cannot create directory " + weightDir_);

    caffe2::NetDef tensors, network;
    std::string error;
    if (!caffe2::loadNetDef(netProtoFile, network, error)) die(error);
    if (!caffe2::loadNetDef(tensorProtoFile, tensors, error)) die(error);
    loadTensors(tensors);   // the weights first: the operators look their shapes up
    loadNetwork(network);
}

void Caffe2Importer::loadTensors(const caffe2::NetDef &tensors) {
    for (const caffe2::OperatorDef &op : tensors.op) loadTensor(op);
}

void Caffe2Importer::loadNetwork(const caffe2::NetDef &net) {
    if (!net.name.empty()) std::clog << "[INFO] loading network " << net.name << std::endl;
    for (const caffe2::OperatorDef &op : net.op) loadOp(op);
}

// One weight blob.  GivenTensorFill: shape + values, written to a raw fp32 file that the generated program loads;
// ConstantFill: shape + value (0 if absent).  A name the caller has defined already is left alone.
// (Caffe2Importer.cpp:474-563)
void Caffe2Importer::loadTensor(const caffe2::OperatorDef &op) {
    if (op.output.empty()) return;
    auto shapeOf = [&]() {
        const caffe2::Argument *a = op.find("shape");
        if (!a) die(op.type + " of " + op.output[0] + " has no shape");
        return std::vector<size_t>(a->ints.begin(), a->ints.end());
    };
    Tensor *tensor = nullptr;
    if (op.type == "GivenTensorFill") {
        const std::vector<size_t> shape = shapeOf();
        const caffe2::Argument *values = op.find("values");
        tensor = new Tensor(new TensorShape(shape));
        if (!values || values->floats.size() != tensor->size())
            die("GivenTensorFill of " + op.output[0] + ": " + std::to_string(values ? values->floats.size() : 0) +
                " values for a shape of " + std::to_string(tensor->size()) + " elements");
        const std::string path = weightDir_ + "/" + fileNameOf(op.output[0]) + ".bin";
        FILE *f = std::fopen(path.c_str(), "wb");
        if (!f || std::fwrite(values->floats.data(), sizeof(float), values->floats.size(), f) != values->floats.size())
            die("cannot write " + path);
        std::fclose(f);
        tensor->setTensorInit(TensorInitType::FILE, path);
    } else if (op.type == "ConstantFill") {
        tensor = new Tensor(new TensorShape(shapeOf()));
        const caffe2::Argument *v = op.find("value");
        tensor->setTensorInit(TensorInitType::CONSTANT, v && v->has_f ? v->f : 0.f);
    } else {
        die("initialiser " + op.type + " of " + op.output[0] + " is not supported (GivenTensorFill, ConstantFill)");
    }
    for (const std::string &name : op.output) {
        if (name_tNode_map_.count(name)) continue;
        auto *node = new TensorNode(name, tensor);
        graph_->pushTensorNode(node);
        name_tNode_map_[name] = node;
    }
}

TensorNode *Caffe2Importer::blob(const caffe2::OperatorDef &op, int inputIdx) const {
    if (inputIdx >= (int)op.input.size()) die(op.type + ": input " + std::to_string(inputIdx) + " is missing");
    auto it = name_tNode_map_.find(op.input[inputIdx]);
    if (it == name_tNode_map_.end())
        die(op.type + ": blob " + op.input[inputIdx] + " is neither defined by the caller nor produced before it is used");
    return it->second;
}

// The tensor node of op.output(0), produced by `producer`.  With `dims` it gets a tensor of that shape; without,
// one shaped like `like` — or, when an operator writes a blob that exists already (Relu and Sum in place),
// that blob's Tensor itself, so both nodes name one buffer (Caffe2Importer.cpp:291-301).
TensorNode *Caffe2Importer::result(const caffe2::OperatorDef &op, TensorNode *like, OpNode *producer,
                                   const std::vector<size_t> *dims) {
    if (op.output.empty()) die(op.type + ": no output");
    const std::string &name = op.output[0];
    TensorNode *node;
    if (dims) node = new TensorNode(name, new Tensor(new TensorShape(*dims)), producer);
    else if (like == nullptr) node = new TensorNode(name, name_tNode_map_.at(name)->getTensor(), producer);
    else node = new TensorNode(name, new Tensor(new TensorShape(like->getDims())), producer);
    name_tNode_map_[name] = node;   // later operators read the newest producer of the name
    graph_->pushTensorNode(node);
    return node;
}

std::string Caffe2Importer::uniqueOpName(const std::string &type) {
    std::string base = type;
    std::transform(base.begin(), base.end(), base.begin(), [](unsigned char c) { return std::tolower(c); });
    const int n = op_names_[base]++;
    return n ? base + std::to_string(n) : base;
}

// (Caffe2Importer.cpp:176-467)
void Caffe2Importer::loadOp(const caffe2::OperatorDef &op) {
    const auto &ok = supportedOps();
    if (std::find(ok.begin(), ok.end(), op.type) == ok.end()) die("unsupported Caffe2 operator " + op.type);
    const std::string opName = uniqueOpName(op.type);
    if (const caffe2::Argument *order = op.find("order"))
        if (order->has_s && order->s != "NCHW") die(op.type + ": only models stored in NCHW order are supported");
    OpNode *opNode = nullptr;

    if (op.type == "Conv") {
        TensorNode *data = blob(op, 0), *weight = blob(op, 1);
        if (data->getTensor()->getNDim() != 4 || weight->getTensor()->getNDim() != 4) die("Conv: 4-D data and weights expected");
        if (const caffe2::Argument *grp = op.find("group"))
            if (grp->i != 1) die("Conv with group = " + std::to_string(grp->i) + " is not supported");
        const std::vector<size_t> in = data->getDims(), wd = weight->getDims();   // weights: [oC, iC, kh, kw]
        std::vector<size_t> kernels = pairOf(op, "kernel", "kernel_h", "kernel_w", "kernels", 0);
        if (!kernels[0]) kernels = {wd[2], wd[3]};
        std::vector<size_t> strides = pairOf(op, "stride", "stride_h", "stride_w", "strides", 1);
        std::vector<size_t> pads = padsOf(op);
        if (wd[1] != in[3]) die("Conv " + op.output[0] + ": weights expect " + std::to_string(wd[1]) + " channels, data has " + std::to_string(in[3]));

        TensorNode *bias;
        if (op.input.size() >= 3) {
            bias = blob(op, 2);
        } else {   // the kernels always add a bias (the reference leaves this one uninitialised)
            bias = new TensorNode(opName + "_bias", new Tensor(new TensorShape({wd[0]})));
            bias->getTensor()->setTensorInit(TensorInitType::CONSTANT, 0.f);
            graph_->pushTensorNode(bias);
        }
        // [oC,iC,kh,kw] -> [oC,kh,kw,iC]
        weight->getTensor()->setMemLayout(layout_nchw);
        auto *trans = new OpNode("op_" + weight->name() + "_T", new TransposeOp(NCHW2NHWC));
        trans->exlinkUpperNode(weight);
        auto *wT = new TensorNode(weight->name() + "_T",
                                  new Tensor(weight->getTensor()->getShuffledTensorShape(NCHW2NHWC), weight->getTensor()->getDataType(), layout_nhwc),
                                  trans);
        graph_->pushOpNode(trans);
        graph_->pushTensorNode(wT);

        opNode = new OpNode(opName, new Conv2dOp(kernels, strides, pads));
        opNode->exlinkUpperNode(data, wT, bias);
        const std::vector<size_t> hw = outHW("Conv " + op.output[0], in[1], in[2], kernels, strides, pads);
        const std::vector<size_t> out = {in[0], hw[0], hw[1], wd[0]};
        result(op, data, opNode, &out);
    } else if (op.type == "SpatialBN") {
        if (op.input.size() != 5) die("SpatialBN needs 5 inputs");
        const caffe2::Argument *eps = op.find("epsilon");
        opNode = new OpNode(opName, new BatchNormalizationOp(eps && eps->has_f ? eps->f : 1e-5f));
        TensorNode *data = blob(op, 0);
        opNode->exlinkUpperNode(data, blob(op, 1), blob(op, 2), blob(op, 3), blob(op, 4));   // scale, bias, mean, var
        const std::vector<size_t> out = data->getDims();
        result(op, data, opNode, &out);
    } else if (op.type == "Relu") {
        opNode = new OpNode(opName, new ReluOp());
        TensorNode *in = blob(op, 0);
        opNode->exlinkUpperNode(in);
        result(op, name_tNode_map_.count(op.output.empty() ? "" : op.output[0]) ? nullptr : in, opNode);
    } else if (op.type == "Sum") {
        if (op.input.size() != 2) die("Sum of " + std::to_string(op.input.size()) + " blobs: only two are supported");
        opNode = new OpNode(opName, new ElementAddOp());
        TensorNode *lhs = blob(op, 0), *rhs = blob(op, 1);
        if (lhs->getDims() != rhs->getDims()) die("Sum " + op.output[0] + ": shapes differ");
        opNode->exlinkUpperNode(lhs, rhs);
        result(op, name_tNode_map_.count(op.output.empty() ? "" : op.output[0]) ? nullptr : lhs, opNode);
    } else if (op.type == "MaxPool" || op.type == "AveragePool") {
        TensorNode *in = blob(op, 0);
        if (in->getTensor()->getNDim() != 4) die(op.type + ": 4-D input expected");
        const std::vector<size_t> id = in->getDims();
        std::vector<size_t> kernels = pairOf(op, "kernel", "kernel_h", "kernel_w", "kernels", 0);
        std::vector<size_t> strides = pairOf(op, "stride", "stride_h", "stride_w", "strides", 1);
        std::vector<size_t> pads = padsOf(op);
        if (const caffe2::Argument *gp = op.find("global_pooling"))
            if (gp->i) kernels = {id[1], id[2]};
        Op *pool = op.type == "MaxPool" ? static_cast<Op *>(new MaxPoolOp(kernels, strides, pads))
                                        : static_cast<Op *>(new AvgPoolOp(kernels, strides, pads));
        opNode = new OpNode(opName, pool);
        opNode->exlinkUpperNode(in);
        const std::vector<size_t> hw = outHW(op.type + " " + op.output[0], id[1], id[2], kernels, strides, pads);
        const std::vector<size_t> out = {id[0], hw[0], hw[1], id[3]};
        result(op, in, opNode, &out);
    } else if (op.type == "FC") {
        if (op.input.size() != 3) die("FC needs data, weights and bias");
        TensorNode *in = blob(op, 0), *weight = blob(op, 1), *bias = blob(op, 2);
        if (weight->getTensor()->getNDim() != 2) die("FC: 2-D weights expected");
        // [out,in] -> [in,out]
        auto *trans = new OpNode("op_" + weight->name() + "_T", new TransposeOp({1, 0}));
        trans->exlinkUpperNode(weight);
        auto *wT = new TensorNode(weight->name() + "_T", new Tensor(weight->getTensor()->getShuffledTensorShape({1, 0})), trans);
        graph_->pushOpNode(trans);
        graph_->pushTensorNode(wT);

        opNode = new OpNode(opName, new MatrixMatrixFCBiasOp());
        if (in->getTensor()->getNDim() == 4) {   // NHWC activations back to the order the weights were trained with
            auto *transIn = new OpNode("op_" + in->name() + "_T", new TransposeOp(NHWC2NCHW));
            transIn->exlinkUpperNode(in);
            auto *inT = new TensorNode(in->name() + "_T",
                                       new Tensor(in->getTensor()->getShuffledTensorShape(NHWC2NCHW), in->getTensor()->getDataType(), layout_nchw),
                                       transIn);
            graph_->pushOpNode(transIn);
            graph_->pushTensorNode(inT);
            opNode->exlinkUpperNode(inT, wT, bias);
        } else {
            opNode->exlinkUpperNode(in, wT, bias);
        }
        const std::vector<size_t> id = in->getDims(), wd = wT->getDims();
        size_t flat = 1;
        for (size_t i = 1; i < id.size(); ++i) flat *= id[i];
        if (flat != wd[0])
            die("FC " + op.output[0] + ": flattened input has " + std::to_string(flat) + " columns, weights have " + std::to_string(wd[0]) + " rows");
        const std::vector<size_t> out = {id[0], wd[1]};
        result(op, in, opNode, &out);
    } else if (op.type == "Softmax") {
        TensorNode *in = blob(op, 0);
        opNode = new OpNode(opName, new MatrixSoftmaxOp());
        opNode->exlinkUpperNode(in);
        const std::vector<size_t> out = in->getDims();
        result(op, in, opNode, &out);
    } else if (op.type == "Dropout") {
        TensorNode *in = blob(op, 0);
        const caffe2::Argument *ratio = op.find("ratio");
        auto *mask = new TensorNode(opName + "_mask", new Tensor(new TensorShape(in->getDims())));
        opNode = new OpNode(opName, new DropoutOp(ratio && ratio->has_f ? ratio->f : 0.5f));
        opNode->exlinkUpperNode(in, mask);
        graph_->pushTensorNode(mask);
        const std::vector<size_t> out = in->getDims();
        result(op, in, opNode, &out);
    }
    name_opNode_map_[opName] = opNode;
    graph_->pushOpNode(opNode);
}

} // namespace swc
