/*
 * saga_hip.h - C ABI of the MI355X (gfx950) kernel library behind Saga's "hip" engine.
 *
 * Every entry point enqueues work on the given HIP stream and returns immediately.
 * Plain pointers and sizes only: no C++ types, no exceptions, no torch types.
 * Return value: 0 on success, a negative SAGA_HIP_E* code for a rejected argument,
 * or a positive hipError_t from the runtime.
 *
 * Each declaration cites the reference code whose role it takes (paths relative to
 * the reference tree).  The callers in the reference design are the exec() methods
 * of the backend's operation objects (src/cuda/cuda_dnn.cpp, cuda_optimizer.cpp).
 */
#ifndef SAGA_HIP_H
#define SAGA_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* A hipStream_t, passed opaque so that C callers need no HIP headers. */
typedef void *saga_stream_t;

/* Element types; values equal saga::Tensor::DataType (saga.hpp:161-168). */
enum SagaDType {
    SAGA_U8 = 0,
    SAGA_HALF = 1,
    SAGA_FLOAT = 2,
    SAGA_INT64 = 3,
    SAGA_I32 = 4,
    SAGA_I16 = 5
};

enum SagaError {
    SAGA_HIP_OK = 0,
    SAGA_HIP_EINVAL = -1,       /* malformed argument (null pointer, negative size ...) */
    SAGA_HIP_ESHAPE = -2,       /* operand shapes do not agree */
    SAGA_HIP_EUNSUPPORTED = -3, /* valid but not implemented (dtype / layout combination) */
    SAGA_HIP_EWORKSPACE = -4,   /* workspace missing or too small */
    SAGA_HIP_ETOOLARGE = -5     /* operand beyond the fixed scratch of an entry point that allocates nothing */
};

/*
 * A tensor as the kernels see it: logical dims are always (N, C, H, W) (rank-2 tensors
 * use H = W = 1) and the strides, in elements, carry the physical layout: NCHW, NHWC,
 * or a channel slice of a wider tensor (how concat is realised).
 * Takes the role of cudnnTensorDescriptor_t + device pointer (src/cuda/cuda_tensor.cpp:560-583).
 */
typedef struct SagaTensorView {
    void *ptr;
    int32_t dims[4];
    int64_t strides[4];
    int32_t dtype; /* enum SagaDType */
} SagaTensorView;

/* Square pad / stride / dilation as in src/cuda/cuda_dnn.cpp:227-235. */
typedef struct SagaConvParams {
    int32_t pad;
    int32_t stride;
    int32_t dilation;
    int32_t group;
} SagaConvParams;

/* Flags returned to the host by the optimizer; layout of CudaAux (src/cuda/cuda_aux.hpp:5-10). */
typedef struct SagaAux {
    uint32_t range;
    uint32_t inf;
    uint32_t nan;
    uint32_t anomaly;
} SagaAux;

enum SagaConvKind { SAGA_CONV_FWD = 0, SAGA_CONV_BWD_DATA = 1, SAGA_CONV_BWD_FILTER = 2 };
enum SagaActMode { SAGA_ACT_RELU = 0, SAGA_ACT_SIGMOID = 1, SAGA_ACT_TANH = 2, SAGA_ACT_SWISH = 3, SAGA_ACT_LEAKYRELU = 4 };
enum SagaPoolMode { SAGA_POOL_MAX = 0, SAGA_POOL_AVG = 1 };

/* Epilogue / fusion flags for the batch-norm entry points. */
enum SagaBnFlags {
    SAGA_BN_RELU = 1, /* y = relu(bn(x) [+ z]) ; backward masks dy by y > 0 */
    SAGA_BN_ADD = 2   /* z is added before the activation; backward also emits dz */
};

const char *saga_hip_error_string(int code);

/* Library / device bring-up; returns the number of compute units of `device` in *cus (may be NULL). */
int saga_hip_init(int device, int *cus);

/* ---- convolution: cudnnConvolutionForward / BackwardData / BackwardFilter
 *      (src/cuda/cuda_dnn.cpp:338-347, :467-476, :419-428).  Cross-correlation.
 *      w has logical dims (K, C/group, R, S); for NHWC programs it is stored K,R,S,C
 *      (strides say so).  out = alpha * conv + beta * out.
 *      Transposed convolution is the same three calls with roles exchanged
 *      (src/cuda/cuda_dnn.cpp:542-574). */
size_t saga_hip_conv2d_workspace_size(int kind, const SagaTensorView *x, const SagaTensorView *w,
                                      const SagaTensorView *y, const SagaConvParams *p);
int saga_hip_conv2d_fwd(const SagaTensorView *x, const SagaTensorView *w, const SagaTensorView *y,
                        const SagaConvParams *p, float alpha, float beta, void *workspace, size_t ws_bytes,
                        saga_stream_t stream);
int saga_hip_conv2d_bwd_data(const SagaTensorView *dy, const SagaTensorView *w, const SagaTensorView *dx,
                             const SagaConvParams *p, float alpha, float beta, void *workspace, size_t ws_bytes,
                             saga_stream_t stream);
int saga_hip_conv2d_bwd_filter(const SagaTensorView *x, const SagaTensorView *dy, const SagaTensorView *dw,
                               const SagaConvParams *p, float alpha, float beta, void *workspace,
                               size_t ws_bytes, saga_stream_t stream);

/* ---- backward data with the filter transposed ahead of time.  No counterpart in the reference (cuDNN
 *      keeps filter handling inside cudnnConvolutionBackwardData, src/cuda/cuda_dnn.cpp:447-493).
 *      The fp16 channels-last path of saga_hip_conv2d_bwd_data first copies the K,R,S,C filter to
 *      C,R,S,K in its workspace - one small launch per layer and step.  A caller that owns a buffer
 *      per layer can instead transpose every filter of a network in ONE launch
 *      (saga_hip_filter_transpose_batched, after the optimizer changed the weights) and hand the copy
 *      in.  saga_hip_conv2d_bwd_data_wt_bytes: size of that copy, 0 when this convolution would not
 *      take the path (use saga_hip_conv2d_bwd_data).  jobs_device: array in device memory; first_block
 *      of job j = sum of saga_hip_filter_transpose_blocks over the jobs before it, total_blocks the sum
 *      over all.  saga_hip_conv2d_bwd_data_wt with wt == NULL is saga_hip_conv2d_bwd_data. */
typedef struct SagaFilterTransposeJob {
    const void *w; /* K,R,S,C fp16, dense */
    void *wt;      /* C,R,S,K fp16, dense, 16-byte aligned */
    int32_t K, C, RS, first_block;
} SagaFilterTransposeJob;
size_t saga_hip_conv2d_bwd_data_wt_bytes(const SagaTensorView *dy, const SagaTensorView *w, const SagaTensorView *dx,
                                         const SagaConvParams *p);
int saga_hip_filter_transpose_blocks(const SagaTensorView *w);
int saga_hip_filter_transpose_batched(const SagaFilterTransposeJob *jobs_device, int njobs, int total_blocks,
                                      saga_stream_t stream);
int saga_hip_conv2d_bwd_data_wt(const SagaTensorView *dy, const SagaTensorView *w, const void *wt, const SagaTensorView *dx,
                                const SagaConvParams *p, float alpha, float beta, void *workspace, size_t ws_bytes,
                                saga_stream_t stream);

/* ---- convolution forward that also leaves, for a batch normalisation that consumes y, the
 *      per-channel sum and sum of squares of y as partial[rows][K][2] (one row per block of
 *      output pixels; *partial_rows receives the count).  The reference runs
 *      cudnnConvolutionForward (src/cuda/cuda_dnn.cpp:207-221) and then
 *      cudnnBatchNormalizationForwardTrainingEx (:1717-1741), which reads y once more for these
 *      sums; here they fall out of the convolution's epilogue.  beta is 0.  Returns
 *      SAGA_HIP_EUNSUPPORTED (nothing written to y) when the fp16 channels-last MFMA path does
 *      not cover the problem: run saga_hip_conv2d_fwd and saga_hip_bn_train_fwd instead.
 *      _size: bytes `partial` must hold (0: never supported for these operands). */
size_t saga_hip_conv2d_fwd_bnstats_size(const SagaTensorView *x, const SagaTensorView *w, const SagaTensorView *y,
                                        const SagaConvParams *p);
int saga_hip_conv2d_fwd_bnstats(const SagaTensorView *x, const SagaTensorView *w, const SagaTensorView *y,
                                const SagaConvParams *p, float alpha, void *workspace, size_t ws_bytes,
                                float *partial, size_t partial_bytes, int *partial_rows, saga_stream_t stream);

/* ---- convolution forward with the batch-norm INFERENCE that follows it (and that norm's optional
 *      residual add and relu) applied in the epilogue: y = act(s*(conv(x,w) - m)/sqrt(v+eps) + b (+ z)).
 *      The reference runs cudnnConvolutionForward (src/cuda/cuda_dnn.cpp:207-221) and
 *      cudnnBatchNormalizationForwardInference (:1641-1651) as two passes over the tensor; here the
 *      convolution's output never reaches memory un-normalised (and is not rounded to fp16 in
 *      between).  Returns SAGA_HIP_EUNSUPPORTED, with nothing written, outside the fp16
 *      channels-last MFMA path: run saga_hip_conv2d_fwd and saga_hip_bn_infer instead. */
int saga_hip_conv2d_fwd_bn_infer(const SagaTensorView *x, const SagaTensorView *w, const SagaTensorView *y,
                                 const SagaTensorView *z, const SagaConvParams *p, const float *s, const float *b,
                                 const float *m, const float *v, float eps, int flags, void *workspace,
                                 size_t ws_bytes, saga_stream_t stream);

/* ---- backward data of the convolution that consumes a batch norm's (+ relu) output, with the first pass
 *      of that norm's backward done in the epilogue.  The reference runs cudnnConvolutionBackwardData
 *      (src/cuda/cuda_dnn.cpp:467-476) and then cudnnBatchNormalizationBackwardEx (:2138-2163), whose first
 *      pass reads the gradient and the norm's input again for two per-channel sums.  Here dx - which is
 *      the gradient of the norm's result y = act(bn(link->x)) - is stored already masked by y > 0
 *      (link->flags & SAGA_BN_RELU; the mask is recomputed from link->x with the forward's own expression)
 *      and link->partial[link->partial_rows][C][2] receives, per block of pixels and channel, the sums of
 *      the masked gradient and of masked gradient * (x - save_mean).  saga_hip_bn_bwd_linked then finishes
 *      the norm's backward from dx and those sums.  This launch must be the only writer of dx that the
 *      norm sees after it (beta != 0 accumulates onto earlier writers as usual).  wt: the transposed filter
 *      of saga_hip_conv2d_bwd_data_wt, or NULL.  Returns SAGA_HIP_EUNSUPPORTED, with nothing written to dx,
 *      outside the fp16 channels-last MFMA path (C % 8 == 0, stride 1, 2 or 4, dilation 1): run
 *      saga_hip_conv2d_bwd_data(_wt) and saga_hip_bn_bwd_ex instead.  _size: bytes link->partial must
 *      hold (0: never supported for these operands). */
typedef struct SagaBnBwdLink {
    const SagaTensorView *x;  /* the norm's input: dims of dx, fp16 channels-last, not dx itself */
    const float *s, *b;       /* scale and bias; read only with SAGA_BN_RELU */
    const float *save_mean, *save_invstd;
    int32_t flags;            /* SAGA_BN_RELU or 0 */
    int32_t partial_rows;     /* out */
    float *partial;
    size_t partial_bytes;
} SagaBnBwdLink;
size_t saga_hip_conv2d_bwd_data_bnbwd_size(const SagaTensorView *dy, const SagaTensorView *w, const SagaTensorView *dx,
                                           const SagaConvParams *p);
int saga_hip_conv2d_bwd_data_bnbwd(const SagaTensorView *dy, const SagaTensorView *w, const void *wt,
                                   const SagaTensorView *dx, const SagaConvParams *p, float alpha, float beta,
                                   void *workspace, size_t ws_bytes, SagaBnBwdLink *link, saga_stream_t stream);

/* y[n,c,:,:] += b[c] : cudnnAddTensor of a {1,C,1,1} bias (src/cuda/cuda_dnn.cpp:39-68). b is fp32 or y's type. */
int saga_hip_bias_add(const SagaTensorView *y, const SagaTensorView *b, saga_stream_t stream);
/* db[c] = beta*db + sum_{n,h,w} dy : cudnnConvolutionBackwardBias (src/cuda/cuda_dnn.cpp:378-385). */
size_t saga_hip_bias_bwd_workspace_size(const SagaTensorView *dy);
int saga_hip_bias_bwd(const SagaTensorView *dy, const SagaTensorView *db, float beta, void *workspace, size_t ws_bytes,
                      saga_stream_t stream);

/* saga_hip_bias_bwd for callers that cannot allocate (code under HIP graph capture, serving loops and harnesses
 * that forbid hipMalloc and so cannot provide a workspace).  No counterpart in the reference.  Same result as
 * saga_hip_bias_bwd; the partial sums of the two-pass reduction live in a fixed array of
 * SAGA_HIP_BIAS_BWD_NOALLOC_MAX_BYTES of device memory that every GPU the library runs on holds until the
 * process ends.  Returns SAGA_HIP_ETOOLARGE, with nothing written, when saga_hip_bias_bwd_workspace_size(dy)
 * exceeds that (channels-last tensors of more than 2048 channels once they have 2^20 elements).  The
 * device the stream belongs to must be current (SAGA_HIP_EINVAL when the stream reports another device).
 * saga_hip_init(device) resolves the array's address; without it the first call on a device does, which loads
 * the code object - runtime work that must not happen under stream capture, so a first call made while the
 * stream is capturing returns SAGA_HIP_EINVAL: call saga_hip_init(device) before capturing.  All calls on one
 * GPU share the array: calls that overlap on one GPU (two streams, two threads) race; calls in stream order do
 * not. */
#define SAGA_HIP_BIAS_BWD_NOALLOC_MAX_BYTES (4u << 20)
int saga_hip_bias_bwd_noalloc(const SagaTensorView *dy, const SagaTensorView *db, float beta, saga_stream_t stream);

/* ---- GEMM: cublasSgemm / cublasHgemm as used by the fc node (src/cuda/cuda_dnn.cpp:1001-1025).
 *      Row-major: C[M,N] = alpha * op(A) * op(B) + beta * C, op(A) is MxK, op(B) is KxN;
 *      trans flag set means the matrix is stored transposed (A as KxM, B as NxK).
 *      fp16 operands accumulate in fp32. */
int saga_hip_gemm(int transA, int transB, int M, int N, int K, float alpha, const void *A, int lda, const void *B,
                  int ldb, float beta, void *C, int ldc, int dtype, saga_stream_t stream);

/* ---- batch normalisation (spatial, per channel; s,b,m,v and saved statistics are fp32 [C]).
 *      infer: cudnnBatchNormalizationForwardInference (src/cuda/cuda_dnn.cpp:1641-1651);
 *      train: ...ForwardTraining / ForwardTrainingEx with BN, BN_ACTIVATION, BN_ADD_ACTIVATION
 *             (src/cuda/cuda_dnn.cpp:1689-1709, :2041-2069);
 *      bwd:   ...Backward / BackwardEx (src/cuda/cuda_dnn.cpp:1754-1766, :2138-2163).
 *      z / dz may be NULL unless SAGA_BN_ADD is set.  save_invstd holds 1/sqrt(var+eps).
 *      Running variance is updated with the unbiased batch variance. */
int saga_hip_bn_infer(const SagaTensorView *x, const SagaTensorView *z, const SagaTensorView *y, const float *s,
                      const float *b, const float *m, const float *v, float eps, int flags, saga_stream_t stream);
size_t saga_hip_bn_workspace_size(const SagaTensorView *x);
int saga_hip_bn_train_fwd(const SagaTensorView *x, const SagaTensorView *z, const SagaTensorView *y,
                          const float *s, const float *b, float *run_m, float *run_v, float *save_mean,
                          float *save_invstd, float eps, float expavg, int flags, void *workspace,
                          size_t ws_bytes, saga_stream_t stream);
/* training forward from per-channel partial sums of x that already exist (the output of
 * saga_hip_conv2d_fwd_bnstats): finalises the statistics and normalises, without the pass
 * over x that computes them.  workspace: 2*C floats.  Channels-last tensors only.
 * relu_mask (may be NULL; fp16 with C % 8 == 0 and SAGA_BN_RELU only): rows*C/8 bytes, bit j of byte
 * [row][c/8] set where y[row][c - c%8 + j] > 0 - the role of cuDNN's reserve space for the fused
 * add + relu operation (src/cuda/cuda_dnn.cpp:2095-2136); saga_hip_bn_bwd_ex reads it in place of y.
 * y NULL (then z and relu_mask NULL too): only the statistics are finalised - save_mean, save_invstd, the
 * running statistics - and the workspace receives scale[c] = s*invstd and shift[c] = b - mean*scale (2*C
 * floats), for a consumer that normalises on the fly (saga_hip_maxpool_fwd_codes_bn). */
int saga_hip_bn_train_fwd_partials(const SagaTensorView *x, const SagaTensorView *z, const SagaTensorView *y,
                                   const float *s, const float *b, float *run_m, float *run_v, float *save_mean,
                                   float *save_invstd, float eps, float expavg, int flags, const float *partial,
                                   int partial_rows, uint8_t *relu_mask, void *workspace, size_t ws_bytes,
                                   saga_stream_t stream);
int saga_hip_bn_bwd(const SagaTensorView *x, const SagaTensorView *y, const SagaTensorView *dy,
                    const SagaTensorView *dx, const SagaTensorView *dz, const float *s, const float *save_mean,
                    const float *save_invstd, float *ds, float *db, float beta_dx, float beta_dz, float beta_p,
                    int flags, void *workspace, size_t ws_bytes, saga_stream_t stream);

/* bwd with the bias b at hand, as cudnnBatchNormalizationBackwardEx receives it
 * (src/cuda/cuda_dnn.cpp:2138-2163): for SAGA_BN_RELU without SAGA_BN_ADD on channels-last tensors
 * the relu mask is recomputed from x (the forward's own expression, rounded as it was stored)
 * and y may be NULL - one tensor less to read in each of the two passes.  b NULL: as saga_hip_bn_bwd.
 * relu_mask (may be NULL): the bytes saga_hip_bn_train_fwd_partials left; where the masked gradient goes
 * to dz first (SAGA_BN_ADD, beta_dz == 0, fp16 channels-last) they replace the read of y. */
int saga_hip_bn_bwd_ex(const SagaTensorView *x, const SagaTensorView *y, const SagaTensorView *dy,
                       const SagaTensorView *dx, const SagaTensorView *dz, const float *s, const float *b,
                       const float *save_mean, const float *save_invstd, float *ds, float *db, float beta_dx,
                       float beta_dz, float beta_p, int flags, const uint8_t *relu_mask, void *workspace,
                       size_t ws_bytes, saga_stream_t stream);

/* second half of cudnnBatchNormalizationBackwardEx (src/cuda/cuda_dnn.cpp:2138-2163) for a norm whose
 * first pass saga_hip_conv2d_bwd_data_bnbwd performed: g is the masked gradient that launch stored,
 * partial[partial_rows][C][2] its sums.  Writes ds, db (beta_p as in saga_hip_bn_bwd) and
 * dx = s*invstd*(g - db/M - (x - mean)*invstd*ds/M) + beta_dx*dx.  fp16 or fp32 channels-last tensors.
 * workspace: saga_hip_bn_workspace_size(x). */
int saga_hip_bn_bwd_linked(const SagaTensorView *x, const SagaTensorView *g, const SagaTensorView *dx, const float *s,
                           const float *save_mean, const float *save_invstd, float *ds, float *db, float beta_dx,
                           float beta_p, const float *partial, int partial_rows, void *workspace, size_t ws_bytes,
                           saga_stream_t stream);

/* ---- activations: cudnnActivationForward / Backward (src/cuda/cuda_dnn.cpp:631-638, :668-676),
 *      leaky relu kernel (src/cuda/cuda_kernels.cu:478-495).  y = act(x) + beta*y ; dx = dy*act'(x) + beta*dx. */
int saga_hip_act_fwd(int mode, float alpha, const SagaTensorView *x, const SagaTensorView *y, float beta,
                     saga_stream_t stream);
int saga_hip_act_bwd(int mode, float alpha, const SagaTensorView *x, const SagaTensorView *y,
                     const SagaTensorView *dy, const SagaTensorView *dx, float beta, saga_stream_t stream);

/* ---- pooling: cudnnPoolingForward / Backward, MAX and AVERAGE_COUNT_INCLUDE_PADDING
 *      (src/cuda/cuda_dnn.cpp:820-836, :858-866).  idx (optional, I32, dims of y) receives the
 *      flat h*W+w position of each window's maximum, first maximum in scan order. */
int saga_hip_pool_fwd(int mode, const SagaTensorView *x, const SagaTensorView *y, const SagaTensorView *idx,
                      int size, int pad, int stride, saga_stream_t stream);
int saga_hip_pool_bwd(int mode, const SagaTensorView *x, const SagaTensorView *y, const SagaTensorView *dy,
                      const SagaTensorView *dx, int size, int pad, int stride, float beta, saga_stream_t stream);
/* Max pooling for training that remembers where each maximum came from.  No single counterpart in the
 * reference: cudnnPoolingBackward re-derives the maximum from x and y (src/cuda/cuda_dnn.cpp:873-899); here
 * the forward pass leaves one byte per output element (window position r*size + s of the first maximum,
 * dense N,P,Q,C order, 8-byte aligned buffer of N*C*P*Q bytes) and the backward pass reads only those and
 * dy - same result, less than half the traffic.  Channels-last tensors with whole 16-byte channel vectors,
 * size 2 or 3; SAGA_HIP_EUNSUPPORTED otherwise (use saga_hip_pool_fwd / saga_hip_pool_bwd).
 * Zeros of both signs tie (the first one is the maximum, as under a float comparison) and the first NaN of a
 * window is its maximum.  For fp16 tensors with 3x3 windows, stride 2 and padding 1 (also through
 * saga_hip_pool_fwd without idx, and in the _bn form below) a pooled -0 is stored as +0 and a pooled NaN as a
 * quiet NaN of positive sign, whatever the input's sign and payload were. */
int saga_hip_maxpool_fwd_codes(const SagaTensorView *x, const SagaTensorView *y, uint8_t *codes, int size, int pad,
                               int stride, saga_stream_t stream);
/* The same on the OUTPUT of a batch norm (+ relu) that is never written: x is the norm's input and every window
 * position holds act(x*scale[c] + shift[c]) rounded to the tensor's type, exactly what
 * saga_hip_bn_train_fwd_partials would have stored (scale_shift: the 2*C floats that call leaves when its y is
 * NULL).  The reference runs cudnnBatchNormalizationForwardTrainingEx and cudnnPoolingForward one after the
 * other (src/cuda/cuda_dnn.cpp:2095-2136, :820-836); fused, the normalised tensor - the largest activation of a
 * ResNet stem - is neither written nor read.  flags: SAGA_BN_RELU or 0. */
int saga_hip_maxpool_fwd_codes_bn(const SagaTensorView *x, const SagaTensorView *y, uint8_t *codes, int size, int pad,
                                  int stride, const float *scale_shift, int flags, saga_stream_t stream);

/* Backward of that pair in one: cudnnPoolingBackward followed by cudnnBatchNormalizationBackwardEx
 * (src/cuda/cuda_dnn.cpp:873-899, :2138-2163) without the tensor between them.  dp is the gradient of the POOLED
 * output, codes the bytes the forward left, x the norm's input; both passes of the norm's backward gather their
 * gradient from dp through the codes (rounded to the tensor's type as the pooling's backward would have stored
 * it, masked by the relu recomputed from x when flags has SAGA_BN_RELU - b is then required).  Writes ds, db
 * (beta_p) and dx = s*invstd*(g - db/M - (x - mean)*invstd*ds/M) + beta_dx*dx.  3x3 windows at stride 2 on
 * channels-last tensors with whole 16-byte channel vectors; SAGA_HIP_EUNSUPPORTED otherwise (the size query
 * returns 0 then). */
size_t saga_hip_bn_bwd_pooled_workspace_size(const SagaTensorView *x, const SagaTensorView *dp, int size, int pad,
                                             int stride);
int saga_hip_bn_bwd_pooled(const SagaTensorView *x, const SagaTensorView *dp, const uint8_t *codes,
                           const SagaTensorView *dx, const float *s, const float *b, const float *save_mean,
                           const float *save_invstd, float *ds, float *db, float beta_dx, float beta_p, int flags,
                           int size, int pad, int stride, void *workspace, size_t ws_bytes, saga_stream_t stream);
int saga_hip_maxpool_bwd_codes(const uint8_t *codes, const SagaTensorView *dy, const SagaTensorView *dx, int size,
                               int pad, int stride, float beta, saga_stream_t stream);

/* y = a + b : cudnnOpTensor ADD (src/cuda/cuda_dnn.cpp:1866-1875). */
int saga_hip_add(const SagaTensorView *a, const SagaTensorView *b, const SagaTensorView *y, saga_stream_t stream);
/* dst = alpha*src + beta*dst : cudnnTransformTensor (src/cuda/cuda_dnn.cpp:72-99); also layout conversion. */
int saga_hip_axpby(const SagaTensorView *src, const SagaTensorView *dst, float alpha, float beta,
                   saga_stream_t stream);
/* dst = (float)src * scale : convert kernels (src/cuda/cuda_kernels.cu:102-151). */
int saga_hip_convert(const SagaTensorView *src, const SagaTensorView *dst, float scale, saga_stream_t stream);
/* softmax over C at every (n,h,w): cudnnSoftmaxForward ACCURATE / MODE_CHANNEL (src/cuda/cuda_dnn.cpp:1937-1945). */
int saga_hip_softmax(const SagaTensorView *x, const SagaTensorView *y, saga_stream_t stream);

/* y[n,c,h,w] = bilinear sample of x[n,c] at theta[n] (2x3, row major, fp32 [N,2,3] on the device) applied to
 * the normalised output coordinate; samples outside x count as zero.  Forward only.
 * cudnnSpatialTfGridGeneratorForward + cudnnSpatialTfSamplerForward, CUDNN_SAMPLER_BILINEAR
 * (src/cuda/cuda_dnn.cpp:2372-2425). */
int saga_hip_spatial_transform(const SagaTensorView *x, const float *theta, const SagaTensorView *y,
                               saga_stream_t stream);

/* ---- dropout: cudnnDropoutForward / cudnnDropoutBackward (src/cuda/cuda_dnn.cpp:1486-1574).
 *      y = x * keep / (1 - prob), dx = beta*dx + dy * keep / (1 - prob), keep ~ Bernoulli(1 - prob).
 *      keep is a pure function of (seed, offset, logical N,C,H,W index of the element): the backward pass
 *      recomputes the mask from the key the forward pass used, nothing is stored (cuDNN keeps it in a
 *      reserve space).  cuDNN's generator is closed, so masks differ from the reference's; the rule does not. */
int saga_hip_dropout_fwd(const SagaTensorView *x, const SagaTensorView *y, float prob, uint64_t seed, uint64_t offset,
                         saga_stream_t stream);
int saga_hip_dropout_bwd(const SagaTensorView *dy, const SagaTensorView *dx, float prob, uint64_t seed, uint64_t offset,
                         float beta, saga_stream_t stream);

/* ---- classifier head: catclassifier_fwd / catclassifier_bwd (src/cuda/cuda_kernels.cu:11-96).
 *      x is [N,C] with contiguous rows; pred/labels are int32 [N]; loss fp32 [N] (may be NULL). */
int saga_hip_catclassifier_fwd(const SagaTensorView *x, int32_t *pred, saga_stream_t stream);
int saga_hip_catclassifier_bwd(const SagaTensorView *x, const SagaTensorView *dx, const int32_t *pred,
                               const int32_t *labels, float *loss, float scale, saga_stream_t stream);

/* ---- L2 loss: loss_bwd_* (src/cuda/cuda_kernels.cu:396-473, called from CudaLossBwd,
 *      src/cuda/cuda_dnn.cpp:1394-1458).  Per sample n over its c elements: v = x - target,
 *      dx = v * scale, mmss[n] = {min(0, min v), max(0, max v), mean v, mean v^2} (fp32 [N][4]); the zeros
 *      in min / max are the reference's (its block reduction pads with zeros).  x, dx: fp16 or fp32,
 *      target: fp32, or fp16 with fp16 x.  The forward pass of the node is a copy (saga_hip_convert).
 * ---- tensor statistics: tensor_stats_* (src/cuda/cuda_kernels.cu:313-383, the "stats" node):
 *      out4 = {min(0, min), max(0, max), mean, variance} over all elements of x. */
int saga_hip_loss_bwd(const SagaTensorView *x, const SagaTensorView *target, const SagaTensorView *dx, float *mmss,
                      float scale, saga_stream_t stream);
size_t saga_hip_tensor_stats_workspace_size(void);
int saga_hip_tensor_stats(const SagaTensorView *x, float *out4, void *workspace, size_t ws_bytes, saga_stream_t stream);

/* ---- optimizer: adam_float / adam_mixed (src/cuda/cuda_kernels.cu:159-250).
 *      b1t = 1/(1-0.9^t), b2t = 1/(1-0.999^t) are computed by the caller (src/cuda/cuda_optimizer.cpp:79-80).
 *      aux points to a SagaAux in device-visible memory. */
int saga_hip_adam_f32(size_t n, float *w, const float *g, float *m, float *v, float b1t, float b2t, float lr,
                      float lambda, SagaAux *aux, saga_stream_t stream);
int saga_hip_adam_mixed(size_t n, float alpha, void *w_half, const void *g_half, float *m, float *v, float *c,
                        float b1t, float b2t, float lr, float lambda, SagaAux *aux, saga_stream_t stream);

/* Fills `bytes` bytes with the byte `value` using a kernel (safe inside captured graphs). */
int saga_hip_fill(void *ptr, int value, size_t bytes, saga_stream_t stream);

#ifdef __cplusplus
}
#endif
#endif /* SAGA_HIP_H */
