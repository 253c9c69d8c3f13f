// Direct convolution kernels: the general fallback for shapes, layouts and dtypes the MFMA
// implicit-GEMM kernels do not cover (odd channel counts, groups, dilation, fp32, NCHW).
// One output element per lane, fp32 accumulation, addresses from the 4-D strides.
#include "conv.hpp"

namespace {

struct G {
    int N, C, H, W, K, R, S, P, Q, pad, stride, dil, group;
};

template <typename T>
__global__ void __launch_bounds__(256)
    direct_fwd(DView x, DView w, DView y, G g, float alpha, float beta, int cl, int64_t total)
{
    const int Cg = g.C / g.group, Kg = g.K / g.group;
    for(int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < total; i += (int64_t)gridDim.x * blockDim.x) {
        int n, k, p, q;
        int64_t t = i;
        if(cl) {
            k = (int)(t % g.K); t /= g.K;
            q = (int)(t % g.Q); t /= g.Q;
            p = (int)(t % g.P); n = (int)(t / g.P);
        } else {
            q = (int)(t % g.Q); t /= g.Q;
            p = (int)(t % g.P); t /= g.P;
            k = (int)(t % g.K); n = (int)(t / g.K);
        }
        const int grp = k / Kg;
        float acc = 0;
        for(int r = 0; r < g.R; r++) {
            const int h = p * g.stride - g.pad + r * g.dil;
            if(h < 0 || h >= g.H)
                continue;
            for(int s = 0; s < g.S; s++) {
                const int ww = q * g.stride - g.pad + s * g.dil;
                if(ww < 0 || ww >= g.W)
                    continue;
                const T *xp = (const T *)x.ptr + n * x.s[0] + (int64_t)(grp * Cg) * x.s[1] + h * x.s[2] + ww * x.s[3];
                const T *wp = (const T *)w.ptr + k * w.s[0] + r * w.s[2] + s * w.s[3];
                for(int c = 0; c < Cg; c++)
                    acc += (float)xp[c * x.s[1]] * (float)wp[c * w.s[1]];
            }
        }
        T *o = (T *)y.ptr + n * y.s[0] + k * y.s[1] + p * y.s[2] + q * y.s[3];
        const float v = alpha * acc;
        *o = (T)(beta != 0.0f ? v + beta * (float)*o : v);
    }
}

template <typename T>
__global__ void __launch_bounds__(256)
    direct_bwd_data(DView dy, DView w, DView dx, G g, float alpha, float beta, int cl, int64_t total)
{
    const int Cg = g.C / g.group, Kg = g.K / g.group;
    for(int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < total; i += (int64_t)gridDim.x * blockDim.x) {
        int n, c, h, ww;
        int64_t t = i;
        if(cl) {
            c = (int)(t % g.C); t /= g.C;
            ww = (int)(t % g.W); t /= g.W;
            h = (int)(t % g.H); n = (int)(t / g.H);
        } else {
            ww = (int)(t % g.W); t /= g.W;
            h = (int)(t % g.H); t /= g.H;
            c = (int)(t % g.C); n = (int)(t / g.C);
        }
        const int grp = c / Cg, cl_ = c % Cg;
        float acc = 0;
        for(int r = 0; r < g.R; r++) {
            const int tp = h + g.pad - r * g.dil;
            if(tp < 0 || tp % g.stride)
                continue;
            const int p = tp / g.stride;
            if(p >= g.P)
                continue;
            for(int s = 0; s < g.S; s++) {
                const int tq = ww + g.pad - s * g.dil;
                if(tq < 0 || tq % g.stride)
                    continue;
                const int q = tq / g.stride;
                if(q >= g.Q)
                    continue;
                const T *gp = (const T *)dy.ptr + n * dy.s[0] + (int64_t)(grp * Kg) * dy.s[1] + p * dy.s[2] + q * dy.s[3];
                const T *wp = (const T *)w.ptr + (int64_t)(grp * Kg) * w.s[0] + cl_ * w.s[1] + r * w.s[2] + s * w.s[3];
                for(int k = 0; k < Kg; k++)
                    acc += (float)gp[k * dy.s[1]] * (float)wp[k * w.s[0]];
            }
        }
        T *o = (T *)dx.ptr + n * dx.s[0] + c * dx.s[1] + h * dx.s[2] + ww * dx.s[3];
        const float v = alpha * acc;
        *o = (T)(beta != 0.0f ? v + beta * (float)*o : v);
    }
}

// One block per filter tap (k, c, r, s); lanes stride over (n, p, q) and reduce.
template <typename T>
__global__ void __launch_bounds__(256) direct_bwd_filter(DView x, DView dy, DView dw, G g, float alpha, float beta)
{
    __shared__ float red[4];
    const int Cg = g.C / g.group, Kg = g.K / g.group;
    int64_t t = blockIdx.x;
    const int s = (int)(t % g.S); t /= g.S;
    const int r = (int)(t % g.R); t /= g.R;
    const int c = (int)(t % Cg);
    const int k = (int)(t / Cg);
    const int grp = k / Kg;
    const int64_t M = (int64_t)g.N * g.P * g.Q;
    float acc = 0;
    for(int64_t m = threadIdx.x; m < M; m += 256) {
        const int q = (int)(m % g.Q);
        const int p = (int)((m / g.Q) % g.P);
        const int n = (int)(m / ((int64_t)g.Q * g.P));
        const int h = p * g.stride - g.pad + r * g.dil, ww = q * g.stride - g.pad + s * g.dil;
        if(h < 0 || h >= g.H || ww < 0 || ww >= g.W)
            continue;
        acc += (float)((const T *)dy.ptr)[n * dy.s[0] + k * dy.s[1] + p * dy.s[2] + q * dy.s[3]] *
               (float)((const T *)x.ptr)[n * x.s[0] + (int64_t)(grp * Cg + c) * x.s[1] + h * x.s[2] + ww * x.s[3]];
    }
    acc = wave_sum(acc);
    if((threadIdx.x & 63) == 0)
        red[threadIdx.x >> 6] = acc;
    __syncthreads();
    if(threadIdx.x == 0) {
        const float v = alpha * (red[0] + red[1] + red[2] + red[3]);
        T *o = (T *)dw.ptr + k * dw.s[0] + c * dw.s[1] + r * dw.s[2] + s * dw.s[3];
        *o = (T)(beta != 0.0f ? v + beta * (float)*o : v);
    }
}

static G mk(const ConvGeom &g) { return G{g.N, g.C, g.H, g.W, g.K, g.R, g.S, g.P, g.Q, g.pad, g.stride, g.dil, g.group}; }
static int is_cl(const SagaTensorView *v) { return (v->dims[1] == 1 || v->strides[1] == 1) ? 1 : 0; }

} // namespace

int conv_direct_fwd(const SagaTensorView *x, const SagaTensorView *w, const SagaTensorView *y, const ConvGeom &g,
                    float alpha, float beta, hipStream_t st)
{
    const int64_t total = view_elements(y);
    const int grid = grid_for(total, 256, 256 * 64);
    if(x->dtype == SAGA_HALF)
        direct_fwd<half_t><<<grid, 256, 0, st>>>(dview(x), dview(w), dview(y), mk(g), alpha, beta, is_cl(y), total);
    else
        direct_fwd<float><<<grid, 256, 0, st>>>(dview(x), dview(w), dview(y), mk(g), alpha, beta, is_cl(y), total);
    SAGA_CHECK_LAUNCH();
    return 0;
}

int conv_direct_bwd_data(const SagaTensorView *dy, const SagaTensorView *w, const SagaTensorView *dx,
                         const ConvGeom &g, float alpha, float beta, hipStream_t st)
{
    const int64_t total = view_elements(dx);
    const int grid = grid_for(total, 256, 256 * 64);
    if(dx->dtype == SAGA_HALF)
        direct_bwd_data<half_t><<<grid, 256, 0, st>>>(dview(dy), dview(w), dview(dx), mk(g), alpha, beta, is_cl(dx), total);
    else
        direct_bwd_data<float><<<grid, 256, 0, st>>>(dview(dy), dview(w), dview(dx), mk(g), alpha, beta, is_cl(dx), total);
    SAGA_CHECK_LAUNCH();
    return 0;
}

int conv_direct_bwd_filter(const SagaTensorView *x, const SagaTensorView *dy, const SagaTensorView *dw,
                           const ConvGeom &g, float alpha, float beta, hipStream_t st)
{
    const int64_t blocks = view_elements(dw);
    if(blocks > 0x7fffffff)
        return SAGA_HIP_EUNSUPPORTED;
    if(x->dtype == SAGA_HALF)
        direct_bwd_filter<half_t><<<(int)blocks, 256, 0, st>>>(dview(x), dview(dy), dview(dw), mk(g), alpha, beta);
    else
        direct_bwd_filter<float><<<(int)blocks, 256, 0, st>>>(dview(x), dview(dy), dview(dw), mk(g), alpha, beta);
    SAGA_CHECK_LAUNCH();
    return 0;
}
