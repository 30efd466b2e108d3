#include "dotGen.h"

#include <cstdlib>
#include <fstream>
#include <unordered_map>

#include "../graphIR/IRGraph.h"
#include "../graphIR/OpNode.h"
#include "../graphIR/TensorNode.h"
#include "../op/Op.h"

namespace swc {

void dotGen(IRGraph *graph, std::string file) {
    std::ofstream os(file);
    os << "digraph IRGraph {\n  rankdir=TB;\n";
    std::unordered_map<const IRNode *, std::string> id;
    for (int i = 0; i < graph->tensorNodeNum(); ++i) {
        TensorNode *t = graph->getTensorNode(i);
        id[t] = "t" + std::to_string(i);
        os << "  " << id[t] << " [shape=box, label=\"" << t->name() << "\\n[";
        const std::vector<size_t> dims = t->getDims();
        for (size_t d = 0; d < dims.size(); ++d) os << (d ? "," : "") << dims[d];
        os << "]\"" << (t->getTraining() ? ", style=filled, fillcolor=lightgrey" : "") << "];\n";
    }
    for (int i = 0; i < graph->opNodeNum(); ++i) {
        OpNode *o = graph->getOpNode(i);
        id[o] = "o" + std::to_string(i);
        os << "  " << id[o] << " [shape=ellipse, label=\"" << o->name() << "\\n" << o->getOp()->getOpName() << "\"];\n";
    }
    auto edges = [&](IRNode *n) {
        for (IRNode *c : n->getChildNodes())
            if (id.count(c)) os << "  " << id[n] << " -> " << id[c] << ";\n";
    };
    for (int i = 0; i < graph->tensorNodeNum(); ++i) edges(graph->getTensorNode(i));
    for (int i = 0; i < graph->opNodeNum(); ++i) edges(graph->getOpNode(i));
    os << "}\n";
}

void svgGen(IRGraph *graph, std::string file) {
    dotGen(graph, file);
    const std::string cmd = "command -v dot >/dev/null 2>&1 && dot -Tsvg '" + file + "' -o '" + file + ".svg'";
    if (std::system(cmd.c_str()) != 0) { /* no Graphviz here: the .dot file is what there is */ }
}

} // namespace swc
