// Writes an IRGraph as a Graphviz file (reference: src/tool/dotGen.h:18-19, dotGen.cpp): tensor nodes as boxes
// with their shapes, op nodes as ellipses with their op types, one edge per link.  dotGen leaves `file`; svgGen
// also asks the `dot` program for "<file>.svg" if there is one on the PATH.
#ifndef SWC_DOTGEN_H_
#define SWC_DOTGEN_H_
#include <string>

namespace swc {
class IRGraph;
void dotGen(IRGraph *graph, std::string file = "IRGraph.dot");
void svgGen(IRGraph *graph, std::string file = "IRGraph.dot");
} // namespace swc
#endif
