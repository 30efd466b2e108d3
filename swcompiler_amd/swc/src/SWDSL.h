// Graph-building shorthand of the SWC API.  The macro names and the variables
// they introduce (`x`, `x_Tensor`, `x_Op`) are what user programs rely on
// (reference: src/SWDSL.h:24-120).
#ifndef SWC_SWDSL_H_
#define SWC_SWDSL_H_

namespace swc {
namespace dsl {
template <typename OpT, typename... A> inline OpNode *makeOpNode(const char *name, OpT *&opOut, A &&... args) {
    opOut = new OpT(std::forward<A>(args)...);
    return new OpNode(name, opOut);
}
} // namespace dsl
} // namespace swc

// TENSOR(x, 8, 784): TensorNode *x with Tensor *x_Tensor of that shape
#define TENSOR(name, args...)                                                                      \
    swc::Tensor *name##_Tensor = new swc::Tensor(new swc::TensorShape(std::vector<size_t>{args})); \
    swc::TensorNode *name = new swc::TensorNode(#name, name##_Tensor)

#define INIT(name, type, args) name##_Tensor->setTensorInit(type, args)

// OP(fc0, MatrixMatrixFCBiasOp): OpNode *fc0 with MatrixMatrixFCBiasOp *fc0_Op
#define OP(name, method)                                                                           \
    method *name##_Op = nullptr;                                                                   \
    swc::OpNode *name = swc::dsl::makeOpNode<method>(#name, name##_Op)

// DYOP(conv0, Conv2dOp, kernels, strides, pads): like OP with constructor arguments
#define DYOP(name, method, para...)                                                                \
    method *name##_Op = nullptr;                                                                   \
    swc::OpNode *name = swc::dsl::makeOpNode<method>(#name, name##_Op, para)

#define LINKPARENT(self, parent...) self->pushParentNode(parent)
#define LINKCHILD(self, child...) self->pushChildNode(child)
#define LINKUPPER(self, upperNode...) self->exlinkUpperNode(upperNode)
#define DESTROYUPPER(self, upperNode...) self->destroyUpperNode(upperNode)

#define G(name) swc::IRGraph *name = new swc::IRGraph()
#define GpT(name, tensorNodes...) name->pushTensorNode(tensorNodes)
#define GpO(name, OpNodes...) name->pushOpNode(OpNodes)
#define GdT(name, tensorNodes...) name->delTensorNode(tensorNodes)
#define GdO(name, OpNodes...) name->delOpNode(OpNodes)

// marks nodes as graph outputs so that EliminationPass keeps them
#define SETOUT(graph, nodes...)                                                                    \
    graph->pushOutNode(nodes);                                                                     \
    graph->setOutMark()

#define CHECKT(t) SWLOG_INFO << (t)->toString() << " topo " << (t)->topologyId() << std::endl
#define CHECKO(o) SWLOG_INFO << (o)->toString() << " topo " << (o)->topologyId() << std::endl
// TRAIN(net, "sgd", lr, decay, momentum, batch): declares the graph `net_train`, a copy of `net` with the gradient
// ops and the optimizer updates added (reference: src/SWDSL.h:106-111)
#define TRAIN(graph, parameters...)                                                                \
    swc::pass::AutodiffPass auto_diff_path(graph);                                                 \
    auto_diff_path.getMethods(parameters);                                                         \
    auto_diff_path.show();                                                                         \
    G(graph##_train);                                                                              \
    auto_diff_path.run(graph##_train)

#define CHECKG(g)                                                                                  \
    for (int i_ = 0; i_ < (g)->tensorNodeNum(); i_++) CHECKT((g)->getTensorNode(i_));              \
    for (int i_ = 0; i_ < (g)->opNodeNum(); i_++) CHECKO((g)->getOpNode(i_))

#endif
