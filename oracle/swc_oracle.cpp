// CPU oracle for the SWCompiler inference kernels and the training kernels next to them.
//
// THIS FILE IS TEST INFRASTRUCTURE.  It is the checker that the HIP kernels are
// compared against; it is never linked into, loaded by or called from the
// shipped library.  Only tests/, __graft_entry__.smoke() and bench.py's
// cpu_baseline leg may use it.
//
// Every function restates the arithmetic of one kernel of the reference's
// generated-code support header (src/codegen/utils/kernels.h) such that each
// output element sees exactly the same sequence of IEEE-754 operations as in
// the reference; loops are reordered for cache locality only where that does
// not change the per-element operation order.  Build without FMA contraction
// (see oracle/Makefile: -ffp-contract=off, no -ffast-math) or results drift.
//
// Pinning status (what proves this file equals the reference):
//   * every function below is compared bit-for-bit with the reference header
//     itself, compiled from /root/reference into oracle/_ref/libswc_ref.so,
//     on seeded inputs (tests/test_oracle_vs_ref.py, tests/test_oracle_training.py,
//     skipped when the reference tree is absent);
//   * the outputs of that reference build are committed as fixtures under
//     tests/golden/ and checked on every run (tests/test_oracle_golden.py);
//   * the MNIST-8 known answer of the reference's test inputs and closed-form
//     / invariant checks (tests/test_oracle_math.py); each gradient kernel is
//     checked as the derivative of its forward kernel by differences in float64
//     (tests/test_oracle_training.py).
//   No function here is "parity unpinned".

#include <cmath>
#include <cstddef>
#include <cstdint>
#include <cstring>
#include <sys/types.h>
#include <utility>
#include <vector>
#include <algorithm>

namespace {

struct Dims4 {
    size_t d0, d1, d2, d3;
    explicit Dims4(const size_t *p) : d0(p[0]), d1(p[1]), d2(p[2]), d3(p[3]) {}
    // row-major flat index, kernels.h:154-158
    size_t at(size_t a, size_t b, size_t c, size_t d) const {
        return ((a * d1 + b) * d2 + c) * d3 + d;
    }
};

} // namespace

extern "C" {

// kernels.h:41-56.  C[i,j] starts at 0.f and receives fl(A[i,p]*B[p,j]) for
// p = 0..k-1 in order, each product rounded to fp32 before the fp32 add.
// The reference iterates p,j,i; here i,p,j — per element the order over p is
// the same, so the bits are the same.
void oracle_matrixMatrixMul_f(int m, int n, int k, const float *a, int lda,
                              const float *b, int ldb, float *c, int ldc) {
    for (int i = 0; i < m; ++i) {
        float *crow = c + (size_t)i * ldc;
        for (int j = 0; j < n; ++j) crow[j] = 0.f;
        const float *arow = a + (size_t)i * lda;
        for (int p = 0; p < k; ++p) {
            const float av = arow[p];
            const float *brow = b + (size_t)p * ldb;
            for (int j = 0; j < n; ++j) crow[j] += av * brow[j];
        }
    }
}

// kernels.h:58-64.  All fp32: 1 - 2/(expf(2x)+1).
void oracle_matrixTanh_f(int m, int n, const float *a, int lda, float *b,
                         int ldb) {
    for (int i = 0; i < m; ++i)
        for (int j = 0; j < n; ++j) {
            float e = expf(a[(size_t)i * lda + j] * 2);
            b[(size_t)i * ldb + j] = 1 - 2 / (e + 1);
        }
}

// kernels.h:88-103.  Row max via std::max starting from element 0 (so a NaN
// in a later column is ignored and a NaN in column 0 sticks), expf of the
// shifted value, sequential fp32 sum left to right, true division.
void oracle_matrixSoftmax_f(int m, int n, const float *a, int lda, float *b,
                            int ldb) {
    for (int i = 0; i < m; ++i) {
        const float *x = a + (size_t)i * lda;
        float *y = b + (size_t)i * ldb;
        float mx = x[0];
        for (int j = 0; j < n; ++j) mx = (mx < x[j]) ? x[j] : mx;
        float total = 0;
        for (int j = 0; j < n; ++j) {
            y[j] = expf(x[j] - mx);
            total += y[j];
        }
        for (int j = 0; j < n; ++j) y[j] = y[j] / total;
    }
}

// kernels.h:163-243 (conv2d_set_bias + conv2d_f), NHWC input, [oC,kH,kW,iC]
// filter.  Each output starts at bias[co] and then receives the in-bounds taps
// in (kx, ky, ci) order, product rounded to fp32 then added in fp32.  Only
// pads[0] (top) and pads[1] (left) take part in the index arithmetic.  The
// reference adds g*inCG to the last filter axis for group g; kept literally.
void oracle_conv2d_f(float *output, const float *input, const float *filter,
                     const float *bias, const size_t *odims,
                     const size_t *idims, const size_t *fdims,
                     const size_t * /*bdims*/, const size_t *kernels,
                     const size_t *strides, const size_t *pads, size_t group) {
    const Dims4 O(odims), I(idims), F(fdims);
    const size_t cin_g = I.d3 / group, cout_g = O.d3 / group;
    const ssize_t kh = kernels[0], kw = kernels[1];
    const ssize_t sh = strides[0], sw = strides[1];
    const ssize_t pt = pads[0], pl = pads[1];
    for (size_t n = 0; n < I.d0; ++n)
        for (size_t ox = 0; ox < O.d1; ++ox)
            for (size_t oy = 0; oy < O.d2; ++oy)
                for (size_t co = 0; co < O.d3; ++co) {
                    const size_t g = co / cout_g;
                    float acc = bias[co];
                    for (ssize_t kx = 0; kx < kh; ++kx) {
                        const ssize_t ix = (ssize_t)ox * sh - pt + kx;
                        if (ix < 0 || ix >= (ssize_t)I.d1) continue;
                        for (ssize_t ky = 0; ky < kw; ++ky) {
                            const ssize_t iy = (ssize_t)oy * sw - pl + ky;
                            if (iy < 0 || iy >= (ssize_t)I.d2) continue;
                            const float *ip =
                                input + I.at(n, ix, iy, g * cin_g);
                            const float *fp =
                                filter + F.at(co, kx, ky, g * cin_g);
                            for (size_t ci = 0; ci < cin_g; ++ci)
                                acc += ip[ci] * fp[ci];
                        }
                    }
                    output[O.at(n, ox, oy, co)] = acc;
                }
}

// kernels.h:323-377 (values) and the index bookkeeping of kernels.h:407-436.
// The first in-bounds tap initialises the running maximum; a later tap
// replaces it only when strictly greater (NaN never replaces; a NaN first tap
// is never replaced).  A window with no in-bounds tap yields 0.
// argmax (may be null) receives the flat NHWC input index of the chosen tap,
// or -1 for an empty window.
void oracle_maxpool_argmax_f(const float *input, float *output, int32_t *argmax,
                             const size_t *idims, const size_t *odims,
                             const size_t *kernels, const size_t *strides,
                             const size_t *pads) {
    const Dims4 I(idims), O(odims);
    const ssize_t kh = kernels[0], kw = kernels[1];
    const ssize_t sh = strides[0], sw = strides[1];
    const ssize_t pt = pads[0], pl = pads[1];
    for (size_t n = 0; n < I.d0; ++n)
        for (size_t ox = 0; ox < O.d1; ++ox)
            for (size_t oy = 0; oy < O.d2; ++oy)
                for (size_t c = 0; c < I.d3; ++c) {
                    bool have = false;
                    float best = 0;
                    int64_t where = -1;
                    for (ssize_t kx = 0; kx < kh; ++kx) {
                        const ssize_t ix = (ssize_t)ox * sh - pt + kx;
                        if (ix < 0 || ix >= (ssize_t)I.d1) continue;
                        for (ssize_t ky = 0; ky < kw; ++ky) {
                            const ssize_t iy = (ssize_t)oy * sw - pl + ky;
                            if (iy < 0 || iy >= (ssize_t)I.d2) continue;
                            const size_t idx = I.at(n, ix, iy, c);
                            const float v = input[idx];
                            if (!have || v > best) {
                                best = v;
                                where = (int64_t)idx;
                                have = true;
                            }
                        }
                    }
                    const size_t o = O.at(n, ox, oy, c);
                    output[o] = best;
                    if (argmax) argmax[o] = (int32_t)where;
                }
}

void oracle_maxpool_f(const float *input, float *output, const size_t *idims,
                      const size_t *odims, const size_t *kernels,
                      const size_t *strides, const size_t *pads) {
    oracle_maxpool_argmax_f(input, output, nullptr, idims, odims, kernels,
                            strides, pads);
}

// kernels.h:444-493.  Sum of the in-bounds taps in (kx, ky) order, fp32, divided
// by kernel_h*kernel_w whatever the number of in-bounds taps (so padded borders
// are averaged as if the padding were zeros).
void oracle_avgpool_f(const float *input, float *output, const size_t *idims,
                      const size_t *odims, const size_t *kernels,
                      const size_t *strides, const size_t *pads) {
    const Dims4 I(idims), O(odims);
    const ssize_t kh = kernels[0], kw = kernels[1];
    const ssize_t sh = strides[0], sw = strides[1];
    const ssize_t pt = pads[0], pl = pads[1];
    const float count = (float)(kernels[0] * kernels[1]);
    for (size_t n = 0; n < I.d0; ++n)
        for (size_t ox = 0; ox < O.d1; ++ox)
            for (size_t oy = 0; oy < O.d2; ++oy)
                for (size_t c = 0; c < I.d3; ++c) {
                    float sum = 0;
                    for (ssize_t kx = 0; kx < kh; ++kx) {
                        const ssize_t ix = (ssize_t)ox * sh - pt + kx;
                        if (ix < 0 || ix >= (ssize_t)I.d1) continue;
                        for (ssize_t ky = 0; ky < kw; ++ky) {
                            const ssize_t iy = (ssize_t)oy * sw - pl + ky;
                            if (iy < 0 || iy >= (ssize_t)I.d2) continue;
                            sum += input[I.at(n, ix, iy, c)];
                        }
                    }
                    output[O.at(n, ox, oy, c)] = sum / count;
                }
}

// kernels.h:519-540.  out[idx[shuffle[0]], idx[shuffle[1]], ...] = in[idx]:
// output axis a is input axis shuffle[a].
void oracle_transpose4d_f(const float *input, float *output, const size_t *idims,
                          const size_t *odims, const size_t *shuffle) {
    const Dims4 I(idims), O(odims);
    size_t idx[4];
    for (idx[0] = 0; idx[0] < I.d0; ++idx[0])
        for (idx[1] = 0; idx[1] < I.d1; ++idx[1])
            for (idx[2] = 0; idx[2] < I.d2; ++idx[2])
                for (idx[3] = 0; idx[3] < I.d3; ++idx[3])
                    output[O.at(idx[shuffle[0]], idx[shuffle[1]], idx[shuffle[2]], idx[shuffle[3]])] =
                        input[I.at(idx[0], idx[1], idx[2], idx[3])];
}

void oracle_transpose2d_f(const float *input, float *output, const size_t *idims,
                          const size_t *odims, const size_t *shuffle) {
    size_t idx[2];
    for (idx[0] = 0; idx[0] < idims[0]; ++idx[0])
        for (idx[1] = 0; idx[1] < idims[1]; ++idx[1])
            output[idx[shuffle[0]] * odims[1] + idx[shuffle[1]]] = input[idx[0] * idims[1] + idx[1]];
}

// kernels.h:496-517.  var[c]+epsilon is an fp32 add; std::pow(float,double)
// promotes, so everything after it is double arithmetic, rounded to fp32 once
// on the store: ((in-mean) -> double) * pow(.) * scale + bias.
void oracle_batchnormalization_f(float *output, const float *input,
                                 const float *mean, const float *var,
                                 const float *scale, const float *bias,
                                 const size_t *idims, float epsilon) {
    const size_t C = idims[3];
    const size_t rows = idims[0] * idims[1] * idims[2];
    std::vector<double> rs(C);
    for (size_t c = 0; c < C; ++c) {
        const float ve = var[c] + epsilon;
        rs[c] = std::pow((double)ve, -0.5);
    }
    for (size_t r = 0; r < rows; ++r) {
        const float *x = input + r * C;
        float *y = output + r * C;
        for (size_t c = 0; c < C; ++c) {
            const float centred = x[c] - mean[c];
            y[c] = (float)((double)centred * rs[c] * (double)scale[c] +
                           (double)bias[c]);
        }
    }
}

// kernels.h:542-552.
void oracle_batchedadd_f(float *dest, const float *batch, const float *slice,
                         size_t numSlice, size_t sliceSize) {
    for (size_t r = 0; r < numSlice; ++r)
        for (size_t j = 0; j < sliceSize; ++j)
            dest[r * sliceSize + j] = batch[r * sliceSize + j] + slice[j];
}

// kernels.h:575-580.  (x > 0) ? x : 0 — so -0.0 -> +0.0 and NaN -> 0.
void oracle_relu_f(const float *src, float *dest, size_t size) {
    for (size_t i = 0; i < size; ++i) dest[i] = (src[i] > 0) ? src[i] : 0;
}

// kernels.h:592-596.
void oracle_vecAdd_f(int size, const float *a, const float *b, float *c) {
    for (int i = 0; i < size; ++i) c[i] = a[i] + b[i];
}

// kernels.h:601-613.  Top-k column indices per row, ordered by descending
// (value, index) pairs: equal values list the larger index first.
void oracle_argMax_i(const float *input, int *idx, int m, int n, int top_k) {
    std::vector<int> order(n);
    for (int i = 0; i < m; ++i) {
        const float *row = input + (size_t)i * n;
        for (int j = 0; j < n; ++j) order[j] = j;
        std::stable_sort(order.begin(), order.end(), [row](int p, int q) {
            if (row[p] > row[q]) return true;
            if (row[q] > row[p]) return false;
            return p > q;
        });
        for (int j = 0; j < top_k; ++j) idx[(size_t)i * top_k + j] = order[j];
    }
}

// kernels.h:615-627.  Each of the m rows adds one to accum_cnt[1], and one to accum_cnt[0] when its
// label is among its n predictions (first match ends the search of the row).
void oracle_accuracy_i(const int *pred, const int *label, int *accum_cnt, int m, int n) {
    for (int row = 0; row < m; ++row) {
        accum_cnt[1] += 1;
        const int *p = pred + (size_t)row * n;
        if (std::find(p, p + n, label[row]) != p + n) accum_cnt[0] += 1;
    }
}

// image.h:13-33: raw little-endian fp32 file, `offset` counted in elements.
// Returns the number of elements copied, or -1 if the file cannot be read.
long oracle_load_f(float *data, size_t size, size_t offset, const char *path);


// ---------------------------------------------------------------- training
// The kernels a generated TRAINING program calls next to the inference ones
// (Codegen.cpp:1518-1531, 1785-1830, 2047-2079, 2138-2148, 2357-2465, 2466-2489).

// kernels.h:68-76.  B[n,m] = A[m,n]^T.
void oracle_matrixTrans_f(int m, int n, const float *a, int lda, float *b, int ldb) {
    for (int i = 0; i < n; ++i)
        for (int j = 0; j < m; ++j) b[(size_t)i * ldb + j] = a[(size_t)j * lda + i];
}

// kernels.h:79-86.  A = (1 - B*B) * C with B the tanh output and C the incoming
// gradient: fl(fl(1 - fl(B*B)) * C).
void oracle_matrixTanhGrad_f(int m, int n, float *a, int lda, const float *b, int ldb, const float *c, int ldc) {
    for (int i = 0; i < m; ++i)
        for (int j = 0; j < n; ++j) {
            const float bb = b[(size_t)i * ldb + j];
            a[(size_t)i * lda + j] = (1 - bb * bb) * c[(size_t)i * ldc + j];
        }
}

// kernels.h:105-129.  Row softmax as matrixSoftmax_f plus the mean
// cross-entropy: loss = (1/m) * sum_i [ logf(sum_i * expf(max_i)) - A(i, selected[i]) ],
// accumulated over rows in order in fp32.
void oracle_matrixSoftmaxWithLoss_f(int m, int n, const float *a, int lda, float *b, int ldb, const int *selected,
                                    float *loss) {
    *loss = 0;
    for (int i = 0; i < m; ++i) {
        const float *arow = a + (size_t)i * lda;
        float *brow = b + (size_t)i * ldb;
        float max_ = arow[0];
        for (int j = 0; j < n; ++j) max_ = std::max(max_, arow[j]);
        float sum = 0;
        for (int j = 0; j < n; ++j) {
            brow[j] = expf(arow[j] - max_);
            sum += brow[j];
        }
        for (int j = 0; j < n; ++j) brow[j] = brow[j] / sum;
        *loss += logf(sum * expf(max_)) - arow[selected[i]];
    }
    *loss /= m;
}

// kernels.h:133-151 (matrixSoftmaxGrad_f and matrixSoftmaxWithLossGrad_f are the
// same loop).  A = B - onehot(selected).
void oracle_matrixSoftmaxGrad_f(int m, int n, float *a, int lda, const float *b, int ldb, const int *selected) {
    for (int i = 0; i < m; ++i)
        for (int j = 0; j < n; ++j) {
            const float delta = (selected[i] == j);
            a[(size_t)i * lda + j] = b[(size_t)i * ldb + j] - delta;
        }
}

// kernels.h:245-319.  All three gradients start at zero and are accumulated in
// fp32 in the loop order n, g, co, kx, ky, ox, oy, ci; the bias gradient takes
// outputG once per output element, at tap (0,0) and after the bounds test — so an
// output pixel whose first tap lies in the padding does not contribute (with
// padding this is not the full bias gradient; it is what the reference computes).
// Loop order is kept as in
// the reference: the per-element operation order of inputG and filterG depends on it.
void oracle_conv2dGrad_f(float *inputG, float *filterG, float *biasG, const float *outputG, const float *input,
                         const float *filter, const size_t *odims, const size_t *idims, const size_t *fdims,
                         const size_t *bdims, const size_t *kernels, const size_t *strides, const size_t *pads,
                         size_t group) {
    (void)bdims;
    const Dims4 od(odims), id(idims), fd(fdims);
    const size_t batch = id.d0, inC = id.d3, oC = od.d3;
    const size_t inCG = inC / group, oCG = oC / group;
    const size_t kh = kernels[0], kw = kernels[1], sh = strides[0], sw = strides[1], pt = pads[0], pl = pads[1];
    std::fill(inputG, inputG + id.d0 * id.d1 * id.d2 * id.d3, 0.f);
    std::fill(filterG, filterG + fd.d0 * fd.d1 * fd.d2 * fd.d3, 0.f);
    std::fill(biasG, biasG + oC, 0.f);
    for (size_t n = 0; n < batch; ++n)
        for (size_t g = 0; g < group; ++g)
            for (size_t co = g * oCG; co < (g + 1) * oCG; ++co)
                for (size_t kx = 0; kx < kh; ++kx)
                    for (size_t ky = 0; ky < kw; ++ky) {
                        const size_t fbase = fd.at(co, kx, ky, g * inCG);
                        for (size_t ox = 0; ox < od.d1; ++ox)
                            for (size_t oy = 0; oy < od.d2; ++oy) {
                                const ssize_t ix = (ssize_t)ox * sh - pt + kx;
                                const ssize_t iy = (ssize_t)oy * sw - pl + ky;
                                if (ix < 0 || ix >= (ssize_t)id.d1 || iy < 0 || iy >= (ssize_t)id.d2) continue;
                                const size_t ibase = id.at(n, ix, iy, g * inCG);
                                const float og = outputG[od.at(n, ox, oy, co)];
                                for (size_t ci = 0; ci < inCG; ++ci) {
                                    inputG[ibase + ci] += filter[fbase + ci] * og;
                                    filterG[fbase + ci] += input[ibase + ci] * og;
                                }
                                if (kx == 0 && ky == 0) biasG[co] += og;
                            }
                    }
}

// kernels.h:380-442.  inputG starts at zero; every output element adds its
// gradient to the input element its window selected (first maximum in scan
// order; a window with no in-bounds tap selects element (0,0) of the image, as
// the reference's uninitialised max_ix/max_iy = 0 do), in (n, ox, oy, c) order.
void oracle_maxpoolGrad_f(float *inputG, const float *outputG, const float *input, const size_t *idims,
                          const size_t *odims, const size_t *kernels, const size_t *strides, const size_t *pads) {
    const Dims4 id(idims), od(odims);
    const size_t kh = kernels[0], kw = kernels[1], sh = strides[0], sw = strides[1];
    std::fill(inputG, inputG + id.d0 * id.d1 * id.d2 * id.d3, 0.f);
    for (size_t n = 0; n < id.d0; ++n)
        for (size_t ox = 0; ox < od.d1; ++ox)
            for (size_t oy = 0; oy < od.d2; ++oy)
                for (size_t c = 0; c < id.d3; ++c) {
                    const ssize_t ixb = (ssize_t)(ox * sh) - (ssize_t)pads[0];
                    const ssize_t iyb = (ssize_t)(oy * sw) - (ssize_t)pads[1];
                    bool uninit = true;
                    float mx = 0;
                    size_t mix = 0, miy = 0;
                    for (size_t kx = 0; kx < kh; ++kx)
                        for (size_t ky = 0; ky < kw; ++ky) {
                            const ssize_t ix = ixb + (ssize_t)kx, iy = iyb + (ssize_t)ky;
                            if (ix < 0 || ix >= (ssize_t)id.d1 || iy < 0 || iy >= (ssize_t)id.d2) continue;
                            const float v = input[id.at(n, ix, iy, c)];
                            if (uninit || v > mx) {
                                mx = v;
                                mix = ix;
                                miy = iy;
                                uninit = false;
                            }
                        }
                    inputG[id.at(n, mix, miy, c)] += outputG[od.at(n, ox, oy, c)];
                }
}

// kernels.h:554-563.  dest[n] = sum of slice n (sliceSize consecutive floats), in
// order, in fp32 — a sum per ROW of the [numSlice, sliceSize] matrix, numSlice results.
void oracle_batchedreduceadd_f(float *dest, const float *batch, size_t numSlice, size_t sliceSize) {
    for (size_t n = 0; n < numSlice; ++n) {
        float sum = 0;
        for (size_t i = 0; i < sliceSize; ++i) sum += batch[n * sliceSize + i];
        dest[n] = sum;
    }
}

// kernels.h:565-573.  neglr = -lr / batch (fp32);
// negDelta = fl(fl(fl(fl(w*decay) + dw) * neglr) + fl(mom*momentum)); mom = negDelta; out += negDelta.
void oracle_sgd_f(size_t size, float *out, float *w, float *dw, float *dw_mom, float lr, float decay, float momentum,
                  size_t batch) {
    const float neglr = -lr / batch;
    for (size_t i = 0; i < size; ++i) {
        const float negDelta = (w[i] * decay + dw[i]) * neglr + dw_mom[i] * momentum;
        dw_mom[i] = negDelta;
        out[i] += negDelta;
    }
}

// kernels.h:586-590.  srcGrad = (src > 0) ? destGrad : 0.
void oracle_reluGrad_f(float *srcGrad, const float *src, const float *destGrad, size_t size) {
    for (size_t i = 0; i < size; ++i) srcGrad[i] = (src[i] > 0) ? destGrad[i] : 0;
}

} // extern "C"

#include <cstdio>
extern "C" long oracle_load_f(float *data, size_t size, size_t offset,
                              const char *path) {
    FILE *f = std::fopen(path, "rb");
    if (!f) return -1;
    if (std::fseek(f, (long)(offset * sizeof(float)), SEEK_SET) != 0) {
        std::fclose(f);
        return -1;
    }
    size_t got = std::fread(data, sizeof(float), size, f);
    std::fclose(f);
    return got == size ? (long)got : -1;
}
