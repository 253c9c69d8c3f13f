// Convolution entry points: argument checking, geometry, and the choice between the MFMA
// implicit-GEMM kernels and the direct fallback.
#include "conv.hpp"

#include <stdlib.h>

namespace {

// 0 when the padded input is smaller than the dilated filter (C's division would truncate a negative
// numerator toward zero and report one output position)
static int conv_dim(int in, int k, int pad, int stride, int dil)
{
    const int span = in + 2 * pad - ((k - 1) * dil + 1);
    return span < 0 ? 0 : 1 + span / stride;
}

// x: (N,C,H,W)  w: (K,C/group,R,S)  y: (N,K,P,Q)
static int geometry(const SagaTensorView *x, const SagaTensorView *w, const SagaTensorView *y, const SagaConvParams *p,
                    ConvGeom *g)
{
    if(!valid_view(x) || !valid_view(w) || !valid_view(y) || !p)
        return SAGA_HIP_EINVAL;
    if(p->stride < 1 || p->pad < 0 || p->dilation < 1 || p->group < 1)
        return SAGA_HIP_EINVAL;
    g->N = x->dims[0]; g->C = x->dims[1]; g->H = x->dims[2]; g->W = x->dims[3];
    g->K = w->dims[0]; g->R = w->dims[2]; g->S = w->dims[3];
    g->pad = p->pad; g->stride = p->stride; g->dil = p->dilation; g->group = p->group;
    g->P = conv_dim(g->H, g->R, g->pad, g->stride, g->dil);
    g->Q = conv_dim(g->W, g->S, g->pad, g->stride, g->dil);
    if(g->C % g->group || g->K % g->group || w->dims[1] != g->C / g->group)
        return SAGA_HIP_ESHAPE;
    if(y->dims[0] != g->N || y->dims[1] != g->K || y->dims[2] != g->P || y->dims[3] != g->Q || g->P < 1 || g->Q < 1)
        return SAGA_HIP_ESHAPE;
    if(x->dtype != w->dtype || x->dtype != y->dtype || (x->dtype != SAGA_HALF && x->dtype != SAGA_FLOAT))
        return SAGA_HIP_EUNSUPPORTED;
    return 0;
}

static bool force_direct()
{
    static int v = -1;
    if(v < 0) {
        const char *e = getenv("SAGA_HIP_FORCE_DIRECT");
        v = (e && *e && *e != '0') ? 1 : 0;
    }
    return v == 1;
}

} // namespace

extern "C" {

size_t saga_hip_conv2d_workspace_size(int kind, const SagaTensorView *x, const SagaTensorView *w,
                                      const SagaTensorView *y, const SagaConvParams *p)
{
    ConvGeom g;
    if(geometry(x, w, y, p, &g))
        return 0;
    return std::max(conv_mfma_workspace(kind, x, w, y, g), conv_f32_workspace(kind, x, w, y, g));
}

int saga_hip_conv2d_fwd(const SagaTensorView *x, const SagaTensorView *w, const SagaTensorView *y,
                        const SagaConvParams *p, float alpha, float beta, void *workspace, size_t ws_bytes,
                        saga_stream_t stream)
{
    ConvGeom g;
    int r = geometry(x, w, y, p, &g);
    if(r)
        return r;
    if(!force_direct()) {
        r = conv_mfma_fwd(x, w, y, g, alpha, beta, workspace, ws_bytes, as_stream(stream));
        if(r != SAGA_HIP_EUNSUPPORTED)
            return r;
        r = conv_f32_fwd(x, w, y, g, alpha, beta, workspace, ws_bytes, as_stream(stream));
        if(r != SAGA_HIP_EUNSUPPORTED)
            return r;
    }
    return conv_direct_fwd(x, w, y, g, alpha, beta, as_stream(stream));
}

size_t saga_hip_conv2d_fwd_bnstats_size(const SagaTensorView *x, const SagaTensorView *w, const SagaTensorView *y,
                                        const SagaConvParams *p)
{
    ConvGeom g;
    if(geometry(x, w, y, p, &g) || x->dtype != SAGA_HALF || force_direct())
        return 0;
    return conv_mfma_stats_floats(g) * sizeof(float);
}

int saga_hip_conv2d_fwd_bnstats(const SagaTensorView *x, const SagaTensorView *w, const SagaTensorView *y,
                                const SagaConvParams *p, float alpha, void *workspace, size_t ws_bytes,
                                float *partial, size_t partial_bytes, int *partial_rows, saga_stream_t stream)
{
    ConvGeom g;
    int r = geometry(x, w, y, p, &g);
    if(r)
        return r;
    if(!partial || !partial_rows)
        return SAGA_HIP_EINVAL;
    if(force_direct())
        return SAGA_HIP_EUNSUPPORTED;
    return conv_mfma_fwd(x, w, y, g, alpha, 0.0f, workspace, ws_bytes, as_stream(stream), partial,
                         partial_bytes / sizeof(float), partial_rows);
}

int saga_hip_conv2d_fwd_bn_infer(const SagaTensorView *x, const SagaTensorView *w, const SagaTensorView *y,
                                 const SagaTensorView *z, const SagaConvParams *p, const float *s, const float *b,
                                 const float *m, const float *v, float eps, int flags, void *workspace,
                                 size_t ws_bytes, saga_stream_t stream)
{
    ConvGeom g;
    int r = geometry(x, w, y, p, &g);
    if(r)
        return r;
    if(!s || !b || !m || !v || ((flags & SAGA_BN_ADD) && !z))
        return SAGA_HIP_EINVAL;
    if(force_direct())
        return SAGA_HIP_EUNSUPPORTED;
    const ConvBnFold bn = {s, b, m, v, eps, flags, z};
    return conv_mfma_fwd(x, w, y, g, 1.0f, 0.0f, workspace, ws_bytes, as_stream(stream), nullptr, 0, nullptr, &bn);
}

int saga_hip_conv2d_bwd_data(const SagaTensorView *dy, const SagaTensorView *w, const SagaTensorView *dx,
                             const SagaConvParams *p, float alpha, float beta, void *workspace, size_t ws_bytes,
                             saga_stream_t stream)
{
    ConvGeom g;
    int r = geometry(dx, w, dy, p, &g);
    if(r)
        return r;
    if(!force_direct()) {
        r = conv_mfma_bwd_data(dy, w, dx, g, alpha, beta, workspace, ws_bytes, as_stream(stream));
        if(r != SAGA_HIP_EUNSUPPORTED)
            return r;
        r = conv_f32_bwd_data(dy, w, dx, g, alpha, beta, workspace, ws_bytes, as_stream(stream));
        if(r != SAGA_HIP_EUNSUPPORTED)
            return r;
    }
    return conv_direct_bwd_data(dy, w, dx, g, alpha, beta, as_stream(stream));
}

size_t saga_hip_conv2d_bwd_data_wt_bytes(const SagaTensorView *dy, const SagaTensorView *w, const SagaTensorView *dx,
                                         const SagaConvParams *p)
{
    ConvGeom g;
    if(geometry(dx, w, dy, p, &g) || force_direct() || !conv_mfma_bwd_data_ok(dy, w, dx, g))
        return 0;
    return (size_t)g.K * g.C * g.R * g.S * 2;
}

int saga_hip_filter_transpose_blocks(const SagaTensorView *w)
{
    if(!valid_view(w))
        return 0;
    return conv_mfma_transpose_blocks(w->dims[0], w->dims[1], w->dims[2] * w->dims[3]);
}

int saga_hip_filter_transpose_batched(const SagaFilterTransposeJob *jobs_device, int njobs, int total_blocks,
                                      saga_stream_t stream)
{
    if(!jobs_device || njobs < 1 || total_blocks < 1)
        return SAGA_HIP_EINVAL;
    return conv_mfma_transpose_batched(jobs_device, njobs, total_blocks, as_stream(stream));
}

int saga_hip_conv2d_bwd_data_wt(const SagaTensorView *dy, const SagaTensorView *w, const void *wt, const SagaTensorView *dx,
                                const SagaConvParams *p, float alpha, float beta, void *workspace, size_t ws_bytes,
                                saga_stream_t stream)
{
    if(!wt)
        return saga_hip_conv2d_bwd_data(dy, w, dx, p, alpha, beta, workspace, ws_bytes, stream);
    ConvGeom g;
    int r = geometry(dx, w, dy, p, &g);
    if(r)
        return r;
    if(force_direct() || !conv_mfma_bwd_data_ok(dy, w, dx, g))
        return SAGA_HIP_EUNSUPPORTED; // only the path saga_hip_conv2d_bwd_data_wt_bytes answered for takes wt
    return conv_mfma_bwd_data(dy, w, dx, g, alpha, beta, workspace, ws_bytes, as_stream(stream), wt);
}

size_t saga_hip_conv2d_bwd_data_bnbwd_size(const SagaTensorView *dy, const SagaTensorView *w, const SagaTensorView *dx,
                                           const SagaConvParams *p)
{
    ConvGeom g;
    if(geometry(dx, w, dy, p, &g) || force_direct() || !conv_mfma_bnbwd_link_ok(dy, w, dx, g))
        return 0;
    return conv_mfma_bnbwd_floats(g) * sizeof(float);
}

int saga_hip_conv2d_bwd_data_bnbwd(const SagaTensorView *dy, const SagaTensorView *w, const void *wt,
                                   const SagaTensorView *dx, const SagaConvParams *p, float alpha, float beta,
                                   void *workspace, size_t ws_bytes, SagaBnBwdLink *link, saga_stream_t stream)
{
    if(!link || !valid_view(link->x) || !link->save_mean || !link->partial)
        return SAGA_HIP_EINVAL;
    if((link->flags & ~SAGA_BN_RELU) || ((link->flags & SAGA_BN_RELU) && (!link->s || !link->b || !link->save_invstd)))
        return SAGA_HIP_EINVAL;
    ConvGeom g;
    int r = geometry(dx, w, dy, p, &g);
    if(r)
        return r;
    if(force_direct() || !conv_mfma_bwd_data_ok(dy, w, dx, g))
        return SAGA_HIP_EUNSUPPORTED;
    int rows = 0;
    const ConvBnBwdLink l = {link->x, link->save_mean, link->save_invstd, link->s, link->b, link->flags & SAGA_BN_RELU,
                             link->partial, link->partial_bytes / sizeof(float), &rows};
    r = conv_mfma_bwd_data(dy, w, dx, g, alpha, beta, workspace, ws_bytes, as_stream(stream), wt, &l);
    if(r == 0)
        link->partial_rows = rows;
    return r;
}

int saga_hip_conv2d_bwd_filter(const SagaTensorView *x, const SagaTensorView *dy, const SagaTensorView *dw,
                               const SagaConvParams *p, float alpha, float beta, void *workspace,
                               size_t ws_bytes, saga_stream_t stream)
{
    ConvGeom g;
    int r = geometry(x, dw, dy, p, &g);
    if(r)
        return r;
    if(!force_direct()) {
        r = conv_mfma_bwd_filter(x, dy, dw, g, alpha, beta, workspace, ws_bytes, as_stream(stream));
        if(r != SAGA_HIP_EUNSUPPORTED)
            return r;
        r = conv_f32_bwd_filter(x, dy, dw, g, alpha, beta, workspace, ws_bytes, as_stream(stream));
        if(r != SAGA_HIP_EUNSUPPORTED)
            return r;
    }
    return conv_direct_bwd_filter(x, dy, dw, g, alpha, beta, as_stream(stream));
}

} // extern "C"
