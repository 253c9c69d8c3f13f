// Adam weight update, fp32 and mixed precision (fp16 weights/gradients, fp32 moments and
// master copy).  28 bytes of HBM traffic per element and a handful of flops: the kernels
// move 4 elements per lane per access (16-byte fp32 vectors, 8-byte fp16 vectors) over one
// contiguous arena, grid-stride, so every wavefront streams whole cache lines.
#include "common.hpp"

namespace {

constexpr float ADAM_B1 = 0.9f;
constexpr float ADAM_B2 = 0.999f;
constexpr float ADAM_EPS = 1e-8f;

__device__ __forceinline__ bool adam_step(float dw, float &m, float &v, float &w, float b1t, float b2t, float lr,
                                          float lambda)
{
    m = ADAM_B1 * m + (1.0f - ADAM_B1) * dw;
    v = ADAM_B2 * v + (1.0f - ADAM_B2) * dw * dw;
    const float m_hat = m * b1t;
    const float v_hat = v * b2t;
    w = w - lr * m_hat * (1.0f / sqrtf(v_hat + ADAM_EPS)) - lr * lambda * w;
    return true;
}

__global__ void __launch_bounds__(256)
    adam_f32_k(size_t n, float *__restrict__ w, const float *__restrict__ g, float *__restrict__ mv,
               float *__restrict__ vv, float b1t, float b2t, float lr, float lambda, SagaAux *aux)
{
    const size_t nvec = n / 4;
    const size_t stride = (size_t)gridDim.x * blockDim.x;
    bool saw_nan = false, saw_inf = false;
    for(size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < nvec; i += stride) {
        float4_t gw = ((const float4_t *)g)[i];
        float4_t ww = ((float4_t *)w)[i], mm = ((float4_t *)mv)[i], vx = ((float4_t *)vv)[i];
#pragma unroll
        for(int j = 0; j < 4; j++) {
            const float dw = gw[j];
            if(!isfinite(dw)) {
                if(dw != dw)
                    saw_nan = true;
                else
                    saw_inf = true;
                continue;
            }
            float m = mm[j], v = vx[j], wj = ww[j];
            adam_step(dw, m, v, wj, b1t, b2t, lr, lambda);
            mm[j] = m;
            vx[j] = v;
            ww[j] = wj;
        }
        ((float4_t *)w)[i] = ww;
        ((float4_t *)mv)[i] = mm;
        ((float4_t *)vv)[i] = vx;
    }
    for(size_t i = nvec * 4 + (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += stride) {
        const float dw = g[i];
        if(!isfinite(dw)) {
            if(dw != dw)
                saw_nan = true;
            else
                saw_inf = true;
            continue;
        }
        adam_step(dw, mv[i], vv[i], w[i], b1t, b2t, lr, lambda);
    }
    if(saw_nan)
        aux->nan = 1;
    if(saw_inf)
        aux->inf = 1;
}

__global__ void __launch_bounds__(256)
    adam_mixed_k(size_t n, float alpha, half_t *__restrict__ w, const half_t *__restrict__ g, float *__restrict__ mv,
                 float *__restrict__ vv, float *__restrict__ cv, float b1t, float b2t, float lr, float lambda,
                 SagaAux *aux)
{
    const size_t nvec = n / 4;
    const size_t stride = (size_t)gridDim.x * blockDim.x;
    bool saw_nan = false, saw_inf = false, saw_range = false;
    for(size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < nvec; i += stride) {
        const half4_t gh = ((const half4_t *)g)[i];
        half4_t wh = ((half4_t *)w)[i];
        // (the moments and the fp32 master weights are touched once per step: non-temporal, so that they do not push
        // what the next step reads first out of the last-level cache)
        float4_t mm = __builtin_nontemporal_load((const float4_t *)mv + i), vx = __builtin_nontemporal_load((const float4_t *)vv + i),
                 cc = __builtin_nontemporal_load((const float4_t *)cv + i);
#pragma unroll
        for(int j = 0; j < 4; j++) {
            const half_t gj = gh[j];
            const uint16_t u = __builtin_bit_cast(uint16_t, gj);
            if((u & 0x7800) == 0x7800) {
                saw_range = true;
                if((u & 0x7c00) == 0x7c00) {
                    if(u & 0x3ff)
                        saw_nan = true;
                    else
                        saw_inf = true;
                    continue;
                }
            }
            const float dw = (float)gj * alpha;
            float m = mm[j], v = vx[j], wj = cc[j];
            adam_step(dw, m, v, wj, b1t, b2t, lr, lambda);
            mm[j] = m;
            vx[j] = v;
            cc[j] = wj;
            wh[j] = (half_t)wj;
        }
        ((half4_t *)w)[i] = wh;
        __builtin_nontemporal_store(mm, (float4_t *)mv + i);
        __builtin_nontemporal_store(vx, (float4_t *)vv + i);
        __builtin_nontemporal_store(cc, (float4_t *)cv + i);
    }
    for(size_t i = nvec * 4 + (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += stride) {
        const half_t gj = g[i];
        const uint16_t u = __builtin_bit_cast(uint16_t, gj);
        if((u & 0x7800) == 0x7800) {
            saw_range = true;
            if((u & 0x7c00) == 0x7c00) {
                if(u & 0x3ff)
                    saw_nan = true;
                else
                    saw_inf = true;
                continue;
            }
        }
        float wj = cv[i];
        adam_step((float)gj * alpha, mv[i], vv[i], wj, b1t, b2t, lr, lambda);
        cv[i] = wj;
        w[i] = (half_t)wj;
    }
    if(saw_range)
        aux->range = 1;
    if(saw_nan)
        aux->nan = 1;
    if(saw_inf)
        aux->inf = 1;
}

} // namespace

extern "C" {

int saga_hip_adam_f32(size_t n, float *w, const float *g, float *m, float *v, float b1t, float b2t, float lr,
                      float lambda, SagaAux *aux, saga_stream_t stream)
{
    if(!w || !g || !m || !v || !aux)
        return SAGA_HIP_EINVAL;
    if(n == 0)
        return 0;
    if(!aligned16(w) || !aligned16(g) || !aligned16(m) || !aligned16(v))
        return SAGA_HIP_EUNSUPPORTED;
    // one 16-byte vector per lane and as many blocks as that takes: dispatched in order, the blocks sweep the
    // arena front to back, which this GPU's memory system serves faster than a grid-stride walk
    adam_f32_k<<<grid_for((int64_t)(n / 4 + 1), 256, 1 << 24), 256, 0, as_stream(stream)>>>(n, w, g, m, v, b1t, b2t, lr,
                                                                                         lambda, aux);
    SAGA_CHECK_LAUNCH();
    return 0;
}

int saga_hip_adam_mixed(size_t n, float alpha, void *w_half, const void *g_half, float *m, float *v, float *c,
                        float b1t, float b2t, float lr, float lambda, SagaAux *aux, saga_stream_t stream)
{
    if(!w_half || !g_half || !m || !v || !c || !aux)
        return SAGA_HIP_EINVAL;
    if(n == 0)
        return 0;
    if(((uintptr_t)w_half & 7) || ((uintptr_t)g_half & 7) || !aligned16(m) || !aligned16(v) || !aligned16(c))
        return SAGA_HIP_EUNSUPPORTED;
    adam_mixed_k<<<grid_for((int64_t)(n / 4 + 1), 256, 1 << 24), 256, 0, as_stream(stream)>>>(
        n, alpha, (half_t *)w_half, (const half_t *)g_half, m, v, c, b1t, b2t, lr, lambda, aux);
    SAGA_CHECK_LAUNCH();
    return 0;
}

} // extern "C"
