// Internal interfaces between the convolution dispatcher and its kernel families.
#pragma once
#include "common.hpp"

struct ConvGeom {
    int N, C, H, W;    // input (x / dx)
    int K, R, S;       // filters
    int P, Q;          // output (y / dy)
    int pad, stride, dil, group;
};

// Direct (non-MFMA) kernels: any dtype in {half, float}, any strides, groups, dilation.
int conv_direct_fwd(const SagaTensorView *x, const SagaTensorView *w, const SagaTensorView *y, const ConvGeom &g,
                    float alpha, float beta, hipStream_t st);
int conv_direct_bwd_data(const SagaTensorView *dy, const SagaTensorView *w, const SagaTensorView *dx,
                         const ConvGeom &g, float alpha, float beta, hipStream_t st);
int conv_direct_bwd_filter(const SagaTensorView *x, const SagaTensorView *dy, const SagaTensorView *dw,
                           const ConvGeom &g, float alpha, float beta, hipStream_t st);

// MFMA implicit-GEMM kernels (fp16, channels-last).  Each returns SAGA_HIP_EUNSUPPORTED when the
// problem is outside what it covers, and the dispatcher falls back to the direct kernels.
size_t conv_mfma_workspace(int kind, const SagaTensorView *x, const SagaTensorView *w, const SagaTensorView *y,
                           const ConvGeom &g);
// stats (optional): receives per block row and output channel the sum and the sum of squares of
// the stored outputs, [*stats_rows][K][2] floats; needs beta == 0 and conv_mfma_stats_floats(g) floats
size_t conv_mfma_stats_floats(const ConvGeom &g);
// batch-norm inference (+ residual + relu) folded into the forward epilogue
struct ConvBnFold {
    const float *s, *b, *m, *v;
    float eps;
    int flags;
    const SagaTensorView *z;
};
int conv_mfma_fwd(const SagaTensorView *x, const SagaTensorView *w, const SagaTensorView *y, const ConvGeom &g,
                  float alpha, float beta, void *ws, size_t ws_bytes, hipStream_t st, float *stats = nullptr,
                  size_t stats_floats = 0, int *stats_rows = nullptr, const ConvBnFold *bn = nullptr);
// backward data whose result dx is the gradient of a batch norm's (+ relu) output, with that norm's first
// backward pass done in the epilogue: dx is stored masked by the relu and partial[*partial_rows][C][2]
// receives sum(dx) and sum(dx * (x - mean)) per block row and channel.  EUNSUPPORTED (nothing written)
// outside the pipelined kernel with 16-byte channel vectors.
struct ConvBnBwdLink {
    const SagaTensorView *x;               // the norm's input, dims of dx
    const float *mean, *invstd, *s, *b;    // invstd, s, b only for relu
    int relu;
    float *partial;
    size_t partial_floats;                 // at least conv_mfma_bnbwd_floats(g)
    int *partial_rows;
};
size_t conv_mfma_bnbwd_floats(const ConvGeom &g);
int conv_mfma_bwd_data(const SagaTensorView *dy, const SagaTensorView *w, const SagaTensorView *dx,
                       const ConvGeom &g, float alpha, float beta, void *ws, size_t ws_bytes, hipStream_t st,
                       const void *wt_ready = nullptr, const ConvBnBwdLink *link = nullptr);
bool conv_mfma_bwd_data_ok(const SagaTensorView *dy, const SagaTensorView *w, const SagaTensorView *dx, const ConvGeom &g);
bool conv_mfma_bnbwd_link_ok(const SagaTensorView *dy, const SagaTensorView *w, const SagaTensorView *dx, const ConvGeom &g);
int conv_mfma_transpose_blocks(int K, int C, int RS);
int conv_mfma_transpose_batched(const SagaFilterTransposeJob *jobs, int njobs, int total_blocks, hipStream_t st);
int conv_mfma_bwd_filter(const SagaTensorView *x, const SagaTensorView *dy, const SagaTensorView *dw,
                         const ConvGeom &g, float alpha, float beta, void *ws, size_t ws_bytes, hipStream_t st);

// fp32 MFMA implicit-GEMM kernels (any strides, groups == 1); SAGA_HIP_EUNSUPPORTED otherwise.
size_t conv_f32_workspace(int kind, const SagaTensorView *x, const SagaTensorView *w, const SagaTensorView *y,
                          const ConvGeom &g);
int conv_f32_fwd(const SagaTensorView *x, const SagaTensorView *w, const SagaTensorView *y, const ConvGeom &g, float alpha,
                 float beta, void *ws, size_t ws_bytes, hipStream_t st);
int conv_f32_bwd_data(const SagaTensorView *dy, const SagaTensorView *w, const SagaTensorView *dx, const ConvGeom &g,
                      float alpha, float beta, void *ws, size_t ws_bytes, hipStream_t st);
int conv_f32_bwd_filter(const SagaTensorView *x, const SagaTensorView *dy, const SagaTensorView *dw, const ConvGeom &g,
                        float alpha, float beta, void *ws, size_t ws_bytes, hipStream_t st);
