// Exports the reference's own CPU kernels behind C symbols, for checking the
// oracle restatement (swc_oracle.cpp) and for timing the reference CPU path.
//
// TEST INFRASTRUCTURE ONLY.  This translation unit contains no kernel code of
// its own: it includes the reference header where it lies (the include path is
// given on the compiler command line by oracle/Makefile, REF_ROOT) and
// forwards to it.  The header has no includes of its own and expects the ones
// the reference's generated program puts before it (Codegen.cpp:234-260).
#include <algorithm>
#include <cmath>
#include <cstdlib>
#include <fstream>
#include <iostream>
#include <random>
#include <string>
#include <vector>
#include <sys/types.h>
using namespace std;

#include "src/codegen/utils/kernels.h"

extern "C" {
void ref_matrixMatrixMul_f(int m, int n, int k, const float *a, int lda,
                           const float *b, int ldb, float *c, int ldc) {
    matrixMatrixMul_f(m, n, k, a, lda, b, ldb, c, ldc);
}
void ref_matrixTanh_f(int m, int n, const float *a, int lda, float *b, int ldb) {
    matrixTanh_f(m, n, a, lda, b, ldb);
}
void ref_matrixSoftmax_f(int m, int n, const float *a, int lda, float *b, int ldb) {
    matrixSoftmax_f(m, n, a, lda, b, ldb);
}
void ref_conv2d_f(float *o, const float *i, const float *f, const float *b,
                  const size_t *od, const size_t *id, const size_t *fd,
                  const size_t *bd, const size_t *k, const size_t *s,
                  const size_t *p, size_t group) {
    conv2d_f(o, i, f, b, od, id, fd, bd, k, s, p, group);
}
void ref_maxpool_f(const float *i, float *o, const size_t *id, const size_t *od,
                   const size_t *k, const size_t *s, const size_t *p) {
    maxpool_f(i, o, id, od, k, s, p);
}
// the reference records the chosen tap only inside the gradient kernel
void ref_maxpoolGrad_f(float *ig, const float *og, const float *i,
                       const size_t *id, const size_t *od, const size_t *k,
                       const size_t *s, const size_t *p) {
    maxpoolGrad_f(ig, og, i, id, od, k, s, p);
}
void ref_avgpool_f(const float *i, float *o, const size_t *id, const size_t *od,
                   const size_t *k, const size_t *s, const size_t *p) {
    avgpool_f(i, o, id, od, k, s, p);
}
void ref_transpose4d_f(const float *i, float *o, const size_t *id, const size_t *od, const size_t *sh) {
    transpose4d_f(i, o, id, od, sh);
}
void ref_transpose2d_f(const float *i, float *o, const size_t *id, const size_t *od, const size_t *sh) {
    transpose2d_f(i, o, id, od, sh);
}
void ref_batchnormalization_f(float *o, const float *i, const float *mean,
                              const float *var, const float *scale,
                              const float *bias, const size_t *id, float eps) {
    batchnormalization_f(o, i, mean, var, scale, bias, id, eps);
}
void ref_batchedadd_f(float *d, const float *b, const float *s, size_t ns, size_t ss) {
    batchedadd_f(d, b, s, ns, ss);
}
void ref_relu_f(const float *s, float *d, size_t n) { relu_f(s, d, n); }
void ref_vecAdd_f(int n, float *a, float *b, float *c) { vecAdd_f(n, a, b, c); }
void ref_argMax_i(const float *in, int *idx, int m, int n, int k) {
    argMax_i(in, idx, m, n, k);
}
void ref_accuracy_i(const int *pred, const int *label, int *accum, int m, int n) { accuracy_i(pred, label, accum, m, n); }
void ref_matrixTrans_f(int m, int n, const float *a, int lda, float *b, int ldb) { matrixTrans_f(m, n, a, lda, b, ldb); }
void ref_matrixTanhGrad_f(int m, int n, float *a, int lda, const float *b, int ldb, const float *c, int ldc) {
    matrixTanhGrad_f(m, n, a, lda, b, ldb, c, ldc);
}
void ref_matrixSoftmaxWithLoss_f(int m, int n, const float *a, int lda, float *b, int ldb, const int *sel, float *loss) {
    matrixSoftmaxWithLoss_f(m, n, a, lda, b, ldb, sel, loss);
}
void ref_matrixSoftmaxGrad_f(int m, int n, float *a, int lda, const float *b, int ldb, const int *sel) {
    matrixSoftmaxGrad_f(m, n, a, lda, b, ldb, sel);
}
void ref_matrixSoftmaxWithLossGrad_f(int m, int n, float *a, int lda, const float *b, int ldb, const int *sel) {
    matrixSoftmaxWithLossGrad_f(m, n, a, lda, b, ldb, sel);
}
void ref_conv2dGrad_f(float *ig, float *fg, float *bg, const float *og, const float *i, const float *f,
                      const size_t *od, const size_t *id, const size_t *fd, const size_t *bd, const size_t *k,
                      const size_t *s, const size_t *p, size_t group) {
    conv2dGrad_f(ig, fg, bg, og, i, f, od, id, fd, bd, k, s, p, group);
}
void ref_batchedreduceadd_f(float *d, const float *b, size_t ns, size_t ss) { batchedreduceadd_f(d, b, ns, ss); }
void ref_sgd_f(size_t size, float *out, float *w, float *dw, float *mom, float lr, float decay, float momentum,
               size_t batch) {
    sgd_f(size, out, w, dw, mom, lr, decay, momentum, batch);
}
void ref_reluGrad_f(float *sg, const float *s, const float *dg, size_t n) { reluGrad_f(sg, s, dg, n); }
}
