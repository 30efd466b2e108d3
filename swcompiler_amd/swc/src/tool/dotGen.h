// Writes an IRGraph as a Graphviz file (reference: src/tool/dotGen.h:18-19, dotGen.cpp): tensor nodes as boxes
// with their shapes, op nodes as ellipses with their op types, one edge per link.  dotGen leaves `file`; svgGen
// also asks the `dot` program for "<file>.svg" if there is one on the PATH.
//
// The file holds one `digraph IRGraph`: a box per tensor node labelled "<name>\n[d0,d1,...]" (grey when the tensor
// is marked for training), an ellipse per op node labelled "<name>\n<op type>", and an edge for every
// parent -> child link, tensors first, then ops, in the order the graph holds them.  Render it with
// `dot -Tpng IRGraph.dot -o IRGraph.png`; nothing in the library depends on Graphviz being installed.
#ifndef SWC_DOTGEN_H_
#define SWC_DOTGEN_H_
#include <string>

namespace swc {
class IRGraph;
void dotGen(IRGraph *graph, std::string file = "IRGraph.dot");
void svgGen(IRGraph *graph, std::string file = "IRGraph.dot");
} // namespace swc
#endif
