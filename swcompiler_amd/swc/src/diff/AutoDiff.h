// The training graph of an inference graph as a free function, for programs that
// run their passes by hand (reference: src/diff/AutoDiff.h:21, AutoDiff.cpp:27-184).
#ifndef SWC_AUTODIFF_H_
#define SWC_AUTODIFF_H_
#include "../common.h"

namespace swc {
class IRGraph;

// A copy of `graph` with the gradient ops and the SGD updates of the trained parameters added (AutodiffPass on
// the copy, SGD with the profile's lr / decay / momentum / batch).  Nodes keep their names, so getNodeByName finds
// them in the copy.
IRGraph *getTrainNet(IRGraph *graph, TrainingConfig &profile);
} // namespace swc
#endif
