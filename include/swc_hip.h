/*
 * swc_hip.h — C ABI of libswc_hip, the MI355X (gfx950) runtime that generated
 * SWCompiler host programs call.
 *
 * The reference has no runtime library: its generated Graph.cpp calls C
 * functions of a header copied next to it (src/codegen/utils/kernels.h) on
 * host memory.  Each op entry point below takes the SAME argument list, in the
 * same order and with the same meaning, as the CPU function the reference's
 * code generator emits for that op (file:line given per function), so that a
 * generated call site differs only by the `swc_hip_` prefix.  Differences:
 *   - every data pointer is a DEVICE pointer (from swc_hip_malloc, or any HIP
 *     device allocation, e.g. a torch tensor's data_ptr());
 *   - the small `const size_t*` shape arrays (dims, kernels, strides, pads) stay
 *     HOST pointers, read before the call returns;
 *   - every function returns 0 on success and a non-zero SWC_HIP_E* code on
 *     failure, with a message kept for swc_hip_last_error().  (The reference's
 *     convention is "ignore or exit", src/codegen/utils/image.h:17-20.)
 *   - ops are asynchronous on one in-order HIP stream per process (the
 *     reference's CUDA path uses one stream per GPU,
 *     src/codegen/Codegen.cpp:166-172); call swc_hip_sync() before reading
 *     results on the host.  swc_hip_d2h synchronises by itself.
 * Nothing here allocates device memory except swc_hip_malloc: an op that needs
 * scratch memory (swc_hip_conv2dGrad_f, swc_hip_matrixSoftmaxWithLoss_f, and the
 * FC/GEMM and convolution entry points for shapes they cut along K) takes it
 * from the workspace the caller sized with the swc_hip_*_workspace_bytes queries
 * and handed over with swc_hip_set_workspace, and fails with SWC_HIP_EINVAL when
 * there is none or it is too small.  (A harness may opt in to a buffer the
 * library allocates and grows by itself: swc_hip_enable_auto_workspace.)
 * Layouts are the reference's: 4-D activations NHWC, conv filters
 * [oC, kH, kW, iC], matrices row-major.  All data is fp32.
 */
#ifndef SWC_HIP_H_
#define SWC_HIP_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

enum {
    SWC_HIP_OK = 0,
    SWC_HIP_EINVAL = 1,      /* bad argument (null pointer, negative size, shape mismatch) */
    SWC_HIP_EUNSUPPORTED = 2,/* valid in the reference but not implemented here (e.g. group != 1) */
    SWC_HIP_ERUNTIME = 3,    /* a HIP call failed; message holds hipGetErrorString */
    SWC_HIP_ENOTINIT = 4     /* swc_hip_init has not succeeded in this process */
};

/* ---- runtime: replaces the cudaSetDevice/cudaMalloc/cudaMemcpy/cudaFree and
 * stream set-up lines the reference prints (src/codegen/Codegen.cpp:154-172,
 * 504-521, 1134-1169, 2499-2526). ---- */
int swc_hip_init(int device);                 /* idempotent; selects device, creates the stream */
int swc_hip_shutdown(void);                   /* destroys the stream; outstanding allocations stay valid */
void *swc_hip_malloc(size_t bytes);           /* 256-byte aligned device memory, NULL on failure */
int swc_hip_free(void *dptr);
/* Page-locked host memory for buffers that are uploaded or downloaded every
 * iteration (the host arena of a generated program, where the reference's
 * generated code calls malloc, src/codegen/Codegen.cpp:504-511): copies from
 * and to it run at the full rate of the link, without the staging copy pageable
 * memory costs. */
void *swc_hip_host_malloc(size_t bytes);      /* NULL on failure */
int swc_hip_host_free(void *hptr);
int swc_hip_h2d(void *dst_dev, const void *src_host, size_t bytes); /* ordered after prior ops, returns when done */
int swc_hip_d2h(void *dst_host, const void *src_dev, size_t bytes); /* ordered after prior ops, returns when done */
int swc_hip_d2d(void *dst_dev, const void *src_dev, size_t bytes);  /* async on the stream */
/* No counterpart in the reference (its one stream per GPU carries copies and
 * kernels alike, src/codegen/Codegen.cpp:166-172, 1142-1168).  Uploads on a second
 * stream of the library, so that the next batch travels while the ops work on
 * this one:
 *   swc_hip_copy_h2d_async  enqueues a copy from page-locked host memory
 *                           (swc_hip_host_malloc) on the copy stream and returns;
 *   swc_hip_copy_wait_ops   copies enqueued from now on start only after every op
 *                           issued so far (the buffer they overwrite is free then);
 *   swc_hip_ops_wait_copies ops issued from now on start only after every copy
 *                           enqueued so far (on the device; the host does not wait);
 *   swc_hip_copy_sync       the host waits for the copy stream (the host buffer of
 *                           a copy may be written again).
 * Both streams have the default priority. */
int swc_hip_copy_h2d_async(void *dst_dev, const void *src_host, size_t bytes);
int swc_hip_copy_wait_ops(void);
int swc_hip_ops_wait_copies(void);
int swc_hip_copy_sync(void);
int swc_hip_fill_f(float *dst_dev, float value, size_t count);      /* initTensorConstant/Zero, kernels.h:23-29 */
int swc_hip_fill_i(int *dst_dev, int value, size_t count);          /* the same for an Int32 tensor (counters) */
int swc_hip_sync(void);
/* No counterpart in the reference (its kernels need no scratch memory).
 * Scratch device memory for the ops that need some (FC/GEMM and convolution
 * calls that are cut along K or run on padded copies: swc_hip_gemm_workspace_bytes,
 * swc_hip_conv2d_workspace_bytes; conv2dGrad_f: swc_hip_conv2dGrad_workspace_bytes;
 * matrixSoftmaxWithLoss_f: swc_hip_matrixSoftmaxWithLoss_workspace_bytes).  A
 * generated program allocates the maximum over its calls once and passes it
 * here; an op that finds no workspace, or one too small, fails with
 * SWC_HIP_EINVAL and a message naming the query.  dptr NULL, bytes 0: no
 * workspace.  The buffer is shared by all ops on the stream.  Not while a graph
 * is being recorded. */
int swc_hip_set_workspace(void *dptr, size_t bytes);
/* No counterpart in the reference.  enable != 0: an op that needs more scratch
 * memory than the current workspace holds lets the library allocate (and later
 * grow) a buffer of its own instead of failing — for test and bench harnesses
 * that call ops of many shapes; a generated program never needs it.  The
 * library's buffer is not replaced while a graph is being recorded, nor while an
 * executable graph recorded on it is still alive (the call that would need it
 * fails instead, and so does swc_hip_set_workspace). */
int swc_hip_enable_auto_workspace(int enable);
/* No counterpart in the reference.  Workspace a matrixMatrixMul_f /
 * matrixMatrixFCBias_f call of this shape uses on the initialised device (0 for
 * most shapes: only products with few output tiles and a K of hundreds are
 * split over K, and only on operands the direct-to-LDS kernels take — rows on
 * 16-byte boundaries; for others the call needs none and the figure is an upper
 * bound).  A generated program takes the maximum over its calls and provides
 * that much with swc_hip_set_workspace. */
size_t swc_hip_gemm_workspace_bytes(int m, int n, int k);
/* The same for a conv2d_f / conv2dFused_f call of these shapes (arguments as in
 * swc_hip_conv2d_f, tensors assumed 16-byte aligned): the output tiles that are
 * left over after every CU has had its share of whole tiles are cut along K and
 * their partial sums kept here; a layer whose input-channel count is no multiple
 * of 4 (and that is too large for the direct first-layer kernel) is computed on
 * zero-padded copies of input and filter, which live here too, and so does the
 * filter copy of a call with more than one group.  The size queries do not see
 * the pointers: each answers for whichever alignment of the operands (on
 * 16-byte boundaries or not) needs the most. */
size_t swc_hip_conv2d_workspace_bytes(const size_t *odims, const size_t *idims, const size_t *fdims,
                                      const size_t *kernels, const size_t *strides, const size_t *pads,
                                      size_t group);
/* The same for a conv2dGrad_f call (arguments as there): the turned filter, the
 * transposed output gradient, padded operand copies and the partial sums of the
 * filter and bias gradients. */
size_t swc_hip_conv2dGrad_workspace_bytes(const size_t *odims, const size_t *idims, const size_t *fdims,
                                          const size_t *kernels, const size_t *strides, const size_t *pads,
                                          size_t group);
/* The same for a matrixSoftmaxWithLoss_f call over m rows of n (the rows' loss terms). */
size_t swc_hip_matrixSoftmaxWithLoss_workspace_bytes(int m, int n);
const char *swc_hip_last_error(void);         /* message of the last failure on this thread ("" if none) */
/* Name of the kernel variant the last FC/GEMM or convolution call on this thread dispatched to, with its
 * template arguments (e.g. "gemm_dma2<2,4,4,2,false,8>"; "" before the first such call): lets a harness check
 * that the kernel it reports on is the one that ran. */
const char *swc_hip_last_kernel(void);
/* The SWC_HIP_* environment variables (test and tuning switches that force kernel variants; none is part of the
 * contract) are read once, by swc_hip_init; no op reads the environment.  A test process that changes them calls
 * this to have them read again — not while a graph is being recorded.  No counterpart in the reference. */
int swc_hip_reload_switches(void);
void *swc_hip_stream(void);                   /* the hipStream_t ops are launched on */
int swc_hip_set_stream(void *hip_stream);     /* launch on a caller-owned stream (NULL: back to the library's own) */
const char *swc_hip_device_name(void);        /* gcnArchName of the selected device */
int swc_hip_device_cus(void);                 /* its compute units (what the split plans divide work over); 0 before init */

/* Event timing on the library's stream, for harnesses: begin/end bracket a
 * region; elapsed returns milliseconds of the last closed region. */
int swc_hip_timer_begin(void);
int swc_hip_timer_end(void);                  /* records the end event and waits for it */
float swc_hip_timer_elapsed_ms(void);
/* Numbered events (slots 0..4095) recorded on the current stream, so a harness
 * can time individual kernels inside a longer timed region. elapsed waits for
 * `second` and returns milliseconds, or a negative value on error. */
int swc_hip_event_record(int slot);
float swc_hip_event_elapsed_ms(int first, int second);

/* HIP graphs: the ops issued between begin and end are recorded instead of run;
 * launch replays them with a single submission (the launch-bound small graphs —
 * batch-8 MLP, LeNet — spend most of their time between kernels otherwise).
 * Run the sequence once eagerly first (kernels configure themselves on first
 * use).  h2d/d2h/sync and the timers must not be called while capturing.  The
 * recorded launches keep the pointers and shapes they were issued with. */
int swc_hip_graph_begin(void);
int swc_hip_graph_end(void **graph_out);      /* returns an executable graph handle */
int swc_hip_graph_launch(void *graph);        /* async on the stream */
int swc_hip_graph_destroy(void *graph);

/* ---- ops: same arguments as the reference's CPU kernels ---- */

/* kernels.h:41-56; emitted at Codegen.cpp:1334-1337 with lda=k, ldb=n, ldc=n.
 * C[m,n] = A[m,k] * B[k,n], row-major, leading dimensions in elements. */
int swc_hip_matrixMatrixMul_f(int m, int n, int k, const float *a, int lda,
                              const float *b, int ldb, float *c, int ldc);

/* kernels.h:542-552; emitted at Codegen.cpp:1513-1515.
 * dest[r,j] = batch[r,j] + slice[j]. dest may alias batch. */
int swc_hip_batchedadd_f(float *dest, const float *batch, const float *slice,
                         size_t numSlice, size_t sliceSize);

/* kernels.h:575-580; Codegen.cpp:2134-2135. dest = (src > 0) ? src : 0, bit-exact
 * (-0 -> +0, NaN -> 0). dest may alias src. */
int swc_hip_relu_f(const float *src, float *dest, size_t size);

/* kernels.h:592-596; Codegen.cpp:1608-1610. c = a + b. c may alias a or b. */
int swc_hip_vecAdd_f(int size, const float *a, const float *b, float *c);

/* kernels.h:177-243; Codegen.cpp:1777-1782.  NHWC input idims[4], filter
 * fdims = {oC,kH,kW,iC}, bias bdims = {oC}, output odims[4]; pads = {t,l,b,r} of
 * which only t and l enter the index arithmetic (as in the reference).
 * out = bias + sum over in-bounds taps.  group > 1 as the reference indexes it:
 * the filter keeps all iC channels per tap, and output channel co of group g
 * reads channels [g*iC/group, (g+1)*iC/group) of input and filter only (computed
 * as one group over a filter copy with the other channels zeroed, so a non-finite
 * input value in another group's channels reaches the output as NaN).  The
 * gradient entry point takes group 1 only. */
int swc_hip_conv2d_f(float *output, const float *input, const float *filter,
                     const float *bias, const size_t *odims, const size_t *idims,
                     const size_t *fdims, const size_t *bdims,
                     const size_t *kernels, const size_t *strides,
                     const size_t *pads, size_t group);

/* kernels.h:496-517; Codegen.cpp:1910-1915.  NHWC, per-channel parameters,
 * out = (in-mean)*pow(var+eps,-0.5)*scale+bias evaluated in double. */
int swc_hip_batchnormalization_f(float *output, const float *input,
                                 const float *mean, const float *var,
                                 const float *scale, const float *bias,
                                 const size_t *idims, float epsilon);

/* kernels.h:323-377; Codegen.cpp:2033-2037.  NHWC window max, first maximum
 * in (kx,ky) scan order wins, out-of-bounds taps skipped, bit-exact. */
int swc_hip_maxpool_f(const float *input, float *output, const size_t *idims,
                      const size_t *odims, const size_t *kernels,
                      const size_t *strides, const size_t *pads);

/* Same values as swc_hip_maxpool_f plus the flat NHWC input index of the
 * chosen tap (-1 for a window with no in-bounds tap): the bookkeeping the
 * reference keeps only inside maxpoolGrad_f (kernels.h:407-436). */
int swc_hip_maxpool_argmax_f(const float *input, float *output, int32_t *argmax,
                             const size_t *idims, const size_t *odims,
                             const size_t *kernels, const size_t *strides,
                             const size_t *pads);

/* kernels.h:444-493; Codegen.cpp:2038-2044.  NHWC window average: fp32 sum of the
 * in-bounds taps in scan order divided by kh*kw (padding counts as zeros), bit-exact. */
int swc_hip_avgpool_f(const float *input, float *output, const size_t *idims,
                      const size_t *odims, const size_t *kernels,
                      const size_t *strides, const size_t *pads);

/* kernels.h:519-540; Codegen.cpp:2255-2284.  Axis permutation: output axis a is
 * input axis shuffle[a], odims[a] = idims[shuffle[a]]; 4 resp. 2 entries per array.
 * output must not alias input. */
int swc_hip_transpose4d_f(const float *input, float *output, const size_t *idims,
                          const size_t *odims, const size_t *shuffle);
int swc_hip_transpose2d_f(const float *input, float *output, const size_t *idims,
                          const size_t *odims, const size_t *shuffle);

/* kernels.h:88-103; Codegen.cpp:2352-2354.  Row softmax of A[m,n]. b may alias a. */
int swc_hip_matrixSoftmax_f(int m, int n, const float *a, int lda, float *b,
                            int ldb);

/* kernels.h:58-64; Codegen.cpp:2286-2296 (MatrixTanh). b = 1 - 2/(exp(2a)+1). */
int swc_hip_matrixTanh_f(int m, int n, const float *a, int lda, float *b,
                         int ldb);

/* kernels.h:601-613; Codegen.cpp:2372-2385 (ArgMax op).  idx[m,top_k] = columns of the top_k largest
 * values of each row, ties listing the larger column first. top_k <= 8. */
int swc_hip_argMax_i(const float *input, int *idx, int m, int n, int top_k);

/* kernels.h:615-627; Codegen.cpp:2387-2398 (Accuracy op).  For each of the m rows: accum_cnt[1] += 1, and
 * accum_cnt[0] += 1 when label[row] is among the row's n predictions pred[row, 0..n).  The counters
 * accumulate over calls; all three pointers are device memory. */
int swc_hip_accuracy_i(const int *pred, const int *label, int *accum_cnt, int m, int n);

/* ---- training kernels: same arguments as the reference's; `selected` and `loss`
 * are device pointers like every other data pointer ---- */

/* kernels.h:68-76 (the generator emits transpose2d_f for MatrixTranspose, Codegen.cpp:2220-2284; matrixTrans_f is
 * the hand-written form of the same operation with leading dimensions).  b[n,m] = a[m,n]^T. */
int swc_hip_matrixTrans_f(int m, int n, const float *a, int lda, float *b, int ldb);

/* kernels.h:79-86; Codegen.cpp:2414-2427.  a = (1 - b*b) * c: b the tanh output,
 * c the gradient arriving at it, a the gradient of the tanh input.  Bit-exact. */
int swc_hip_matrixTanhGrad_f(int m, int n, float *a, int lda, const float *b, int ldb,
                             const float *c, int ldc);

/* kernels.h:105-129; Codegen.cpp:2357-2370.  b = row softmax of a (as
 * matrixSoftmax_f); *loss = mean over rows of logf(sum*expf(max)) - a[row, selected[row]].
 * b may alias a. */
int swc_hip_matrixSoftmaxWithLoss_f(int m, int n, const float *a, int lda, float *b, int ldb,
                                    const int *selected, float *loss);

/* kernels.h:133-151; Codegen.cpp:2429-2465.  a = b - onehot(selected): the
 * gradient of the SUM (not the mean) of the rows' losses.  Bit-exact. */
int swc_hip_matrixSoftmaxGrad_f(int m, int n, float *a, int lda, const float *b, int ldb,
                                const int *selected);
int swc_hip_matrixSoftmaxWithLossGrad_f(int m, int n, float *a, int lda, const float *b, int ldb,
                                        const int *selected);

/* kernels.h:245-319; Codegen.cpp:1785-1830.  Gradients of conv2d_f with respect to
 * input, filter and bias from the gradient of its output; all three are
 * overwritten.  biasG follows the reference literally: an output pixel whose
 * first tap (0,0) lies in the padding does not contribute.  group must be 1. */
int swc_hip_conv2dGrad_f(float *inputG, float *filterG, float *biasG, const float *outputG,
                         const float *input, const float *filter, const size_t *odims,
                         const size_t *idims, const size_t *fdims, const size_t *bdims,
                         const size_t *kernels, const size_t *strides, const size_t *pads,
                         size_t group);

/* kernels.h:380-442; Codegen.cpp:2047-2079.  inputG = 0, then every output
 * element adds its gradient to the input element its window selected (first
 * maximum in scan order), in the reference's accumulation order: bit-exact,
 * also for overlapping windows. */
int swc_hip_maxpoolGrad_f(float *inputG, const float *outputG, const float *input,
                          const size_t *idims, const size_t *odims, const size_t *kernels,
                          const size_t *strides, const size_t *pads);

/* kernels.h:554-563; Codegen.cpp:1517-1531.  dest[s] = sum of slice s (sliceSize
 * consecutive floats of batch) added in order in fp32 — one result per ROW of the
 * [numSlice, sliceSize] matrix, exactly as the reference computes it (its call
 * site passes a dest of sliceSize floats; dest must hold numSlice).  Bit-exact. */
int swc_hip_batchedreduceadd_f(float *dest, const float *batch, size_t numSlice, size_t sliceSize);

/* kernels.h:565-573; Codegen.cpp:2468-2489.  neglr = -lr/batch;
 * d = (w*decay + dw)*neglr + dw_mom*momentum; dw_mom = d; out += d.  out may be w.  Bit-exact. */
int swc_hip_sgd_f(size_t size, float *out, float *w, float *dw, float *dw_mom, float lr,
                  float decay, float momentum, size_t batch);

/* kernels.h:586-590; Codegen.cpp:2138-2148.  srcGrad = (src > 0) ? destGrad : 0.  Bit-exact. */
int swc_hip_reluGrad_f(float *srcGrad, const float *src, const float *destGrad, size_t size);

/* ---- fused ops: what the HIP target emits when the graph allows.  Each equals
 * the named sequence of reference kernels. ---- */

/* MatrixMatrixFCBias kept un-lowered (the reference lowers it to
 * matrixMatrixMul_f + batchedadd_f, src/op/dlOp/dlOpEinsum.cpp:154-237):
 * C = A*B + bias[n], then ReLU if relu != 0. bias may be NULL (no bias). */
int swc_hip_matrixMatrixFCBias_f(int m, int n, int k, const float *a, int lda,
                                 const float *b, int ldb, const float *bias,
                                 float *c, int ldc, int relu);

/* No counterpart in the reference, whose kernels need no scratch memory at all.
 * For callers that cannot allocate device memory or have it allocated on their
 * behalf — code under HIP graph capture, tight serving loops, harnesses that
 * forbid hipMalloc: swc_hip_matrixMatrixFCBias_f (same arguments, same kernels,
 * bit-identical result) with the partial tiles of a product cut along K kept in
 * a fixed array of SWC_HIP_NOALLOC_SCRATCH_BYTES inside the library's device
 * code instead of the workspace.  It never calls hipMalloc/hipFree and ignores
 * swc_hip_set_workspace.  A product whose partial tiles
 * (swc_hip_gemm_workspace_bytes) exceed the array is refused with
 * SWC_HIP_EINVAL before anything is launched.  All calls on one GPU share the
 * one array (nothing in it needs to start at zero: every partial tile is
 * written in full before it is read), so calls that overlap on one GPU — two
 * streams, two host threads — race; calls on the library's single in-order
 * stream do not. */
#define SWC_HIP_NOALLOC_SCRATCH_BYTES (16u << 20)
int swc_hip_matrixMatrixFCBias_noalloc_f(int m, int n, int k, const float *a, int lda,
                                         const float *b, int ldb, const float *bias,
                                         float *c, int ldc, int relu);

/* MatrixMatrixFCBias followed by MatrixSoftmax (the classifier head of every
 * MLP/LeNet graph): c = softmax over each row of A*B + bias, i.e. the result of
 * matrixMatrixMul_f + batchedadd_f + matrixSoftmax_f (kernels.h:41-56, 542-552,
 * 88-103).  One launch when n <= 16 (the workgroup that computes 16 rows also
 * normalises them); otherwise the two kernels in sequence. */
int swc_hip_matrixMatrixFCBiasSoftmax_f(int m, int n, int k, const float *a, int lda,
                                        const float *b, int ldb, const float *bias,
                                        float *c, int ldc);

/* vecAdd_f followed by relu_f. */
int swc_hip_vecAddRelu_f(int size, const float *a, const float *b, float *c);

/* batchnormalization_f followed by relu_f. */
int swc_hip_batchnormRelu_f(float *output, const float *input, const float *mean,
                            const float *var, const float *scale,
                            const float *bias, const size_t *idims,
                            float epsilon);

/* batchnormalization_f, relu_f, then maxpool_f over the result (output has the
 * pooled shape odims). */
int swc_hip_batchnormReluMaxpool_f(float *output, const float *input,
                                   const float *mean, const float *var,
                                   const float *scale, const float *bias,
                                   const size_t *idims, float epsilon,
                                   const size_t *odims, const size_t *kernels,
                                   const size_t *strides, const size_t *pads);

/* conv2d_f, then optionally batchnormalization_f (when bn_mean != NULL; all four
 * bn_* pointers must then be given), then optionally relu_f. */
int swc_hip_conv2dFused_f(float *output, const float *input, const float *filter,
                          const float *bias, const size_t *odims,
                          const size_t *idims, const size_t *fdims,
                          const size_t *bdims, const size_t *kernels,
                          const size_t *strides, const size_t *pads,
                          size_t group, const float *bn_mean,
                          const float *bn_var, const float *bn_scale,
                          const float *bn_bias, float epsilon, int relu);

/* The same with a second summand before the ReLU: conv2d_f, optionally
 * batchnormalization_f, then vecAdd_f with `residual` (a tensor of the output's
 * shape: the other branch of a residual block; NULL: none; it may be the output
 * itself), then optionally relu_f. */
int swc_hip_conv2dFusedAdd_f(float *output, const float *input, const float *filter,
                             const float *bias, const size_t *odims,
                             const size_t *idims, const size_t *fdims,
                             const size_t *bdims, const size_t *kernels,
                             const size_t *strides, const size_t *pads,
                             size_t group, const float *bn_mean,
                             const float *bn_var, const float *bn_scale,
                             const float *bn_bias, float epsilon,
                             const float *residual, int relu);

/* swc_hip_conv2dFused_f followed by maxpool_f (kernels.h:343-383) over its
 * result, in one call: conv2d_f (kernels.h:177-243), optionally
 * batchnormalization_f, optionally relu_f, then the pooling.  `cdims` are the
 * convolution's output dims [N,OH,OW,oC] (that tensor is never stored), `pdims`
 * the pooled output's [N,PH,PW,oC] = `output`.  For 2x2 windows with stride 2
 * and no padding over even OH and OW the convolution kernel takes the maximum
 * in its epilogue — the same bits as the two calls in sequence, one launch and
 * the convolution's output neither written nor read back; any other pooling
 * runs the two steps with the intermediate tensor in the workspace.
 * Workspace: swc_hip_conv2dFusedMaxpool_workspace_bytes. */
int swc_hip_conv2dFusedMaxpool_f(float *output, const float *input, const float *filter,
                                 const float *bias, const size_t *cdims,
                                 const size_t *idims, const size_t *fdims,
                                 const size_t *bdims, const size_t *kernels,
                                 const size_t *strides, const size_t *pads,
                                 size_t group, const float *bn_mean,
                                 const float *bn_var, const float *bn_scale,
                                 const float *bn_bias, float epsilon, int relu,
                                 const size_t *pdims, const size_t *pool_kernels,
                                 const size_t *pool_strides, const size_t *pool_pads);
size_t swc_hip_conv2dFusedMaxpool_workspace_bytes(const size_t *cdims, const size_t *idims,
                                                  const size_t *fdims, const size_t *kernels,
                                                  const size_t *strides, const size_t *pads,
                                                  size_t group, const size_t *pdims,
                                                  const size_t *pool_kernels,
                                                  const size_t *pool_strides,
                                                  const size_t *pool_pads);

#ifdef __cplusplus
}
#endif
#endif /* SWC_HIP_H_ */
