// Umbrella header of the SWC graph-compiler API: `#include "SWC.h"`, then
// `using namespace swc; using namespace swc::op;` as in the reference's
// programs (reference: include/SWC.h:11-43).
#ifndef SWC_H_
#define SWC_H_

#include <string>
#include <utility>
#include <vector>

#include "../src/SWLOG.h"
#include "../src/common.h"

#include "../src/tensor/tensor.h"
#include "../src/op/Op.h"
#include "../src/op/ops.h"

#include "../src/graphIR/IRGraph.h"
#include "../src/graphIR/IRNode.h"
#include "../src/graphIR/OpNode.h"
#include "../src/graphIR/TensorNode.h"

#include "../src/SWDSL.h"

#include "../src/pass/Label.h"
#include "../src/pass/OptimizePass.h"
#include "../src/pass/passes.h"

#include "../src/diff/AutoDiff.h"
#include "../src/tool/dotGen.h"
#include "../src/devices/HipDevice.h"
#include "../src/codegen/Codegen.h"
#include "../src/importer/Caffe2Importer.h"
#include "../src/engine/Engine.h"

#endif
