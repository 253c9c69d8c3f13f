// Classifier head: arg-max labels, softmax cross-entropy gradient + per-sample loss, and the
// per-position channel softmax.  One wavefront per sample: lanes stride over the classes with
// coalesced loads and combine with cross-lane reductions.
#include "common.hpp"

namespace {

// First maximum from the left under strict '>' (NaN never wins unless it is element 0).
template <typename T>
__global__ void __launch_bounds__(256) catclassifier_fwd_k(const T *__restrict__ x, int64_t pitch, int32_t *pred, int N, int C)
{
    const int lane = threadIdx.x & 63;
    const int i = blockIdx.x * 4 + (threadIdx.x >> 6);
    if(i >= N)
        return;
    const T *xi = x + (int64_t)i * pitch;
    const float x0 = (float)xi[0];
    float best = -INFINITY;
    int bi = 0x7fffffff;
    for(int j = lane; j < C; j += 64) {
        const float v = (float)xi[j];
        if(v > best || (v == best && j < bi)) {
            best = v;
            bi = j;
        }
    }
#pragma unroll
    for(int o = 32; o > 0; o >>= 1) {
        const float ov = __shfl_xor(best, o, 64);
        const int oi = __shfl_xor(bi, o, 64);
        if(ov > best || (ov == best && oi < bi)) {
            best = ov;
            bi = oi;
        }
    }
    if(lane == 0) {
        int label = (bi == 0x7fffffff) ? 0 : bi;
        if(x0 != x0)
            label = 0; // a NaN in front is never beaten
        pred[i] = label;
    }
}

__device__ __forceinline__ double wave_sum_d(double v)
{
#pragma unroll
    for(int o = 32; o > 0; o >>= 1)
        v += __shfl_xor(v, o, 64);
    return v;
}

template <typename T>
__global__ void __launch_bounds__(256)
    catclassifier_bwd_k(const T *__restrict__ x, int64_t px, T *__restrict__ dx, int64_t pdx, const int32_t *pred,
                        const int32_t *labels, float *loss, int N, int C, float scale)
{
    const int lane = threadIdx.x & 63;
    const int i = blockIdx.x * 4 + (threadIdx.x >> 6);
    if(i >= N)
        return;
    const T *xi = x + (int64_t)i * px;
    T *di = dx + (int64_t)i * pdx;
    int pj = pred[i];
    if(pj < 0 || pj >= C)
        pj = 0;
    const double mx = (double)(float)xi[pj];
    double sum = 0;
    for(int j = lane; j < C; j += 64)
        sum += exp((double)(float)xi[j] - mx);
    sum = wave_sum_d(sum);
    const double offset = mx + log(sum);
    const int label = labels[i];
    for(int j = lane; j < C; j += 64) {
        const double p = exp((double)(float)xi[j] - offset);
        if(j == label) {
            di[j] = (T)(float)((p - 1.0) * scale);
            if(loss)
                loss[i] = (float)-log(p);
        } else {
            di[j] = (T)(float)(p * scale);
        }
    }
}

template <typename T>
__global__ void __launch_bounds__(256) softmax_k(DView x, DView y, int64_t total)
{
    const int C = x.d[1], H = x.d[2], W = x.d[3];
    for(int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < total; i += (int64_t)gridDim.x * blockDim.x) {
        const int w = (int)(i % W);
        const int h = (int)((i / W) % H);
        const int n = (int)(i / ((int64_t)W * H));
        const T *xp = (const T *)x.ptr + n * x.s[0] + h * x.s[2] + w * x.s[3];
        T *yp = (T *)y.ptr + n * y.s[0] + h * y.s[2] + w * y.s[3];
        float mx = -INFINITY;
        for(int c = 0; c < C; c++)
            mx = fmaxf(mx, (float)xp[c * x.s[1]]);
        float sum = 0;
        for(int c = 0; c < C; c++)
            sum += __expf((float)xp[c * x.s[1]] - mx);
        const float inv = 1.0f / sum;
        for(int c = 0; c < C; c++)
            yp[c * y.s[1]] = (T)(__expf((float)xp[c * x.s[1]] - mx) * inv);
    }
}

} // namespace

extern "C" {

int saga_hip_catclassifier_fwd(const SagaTensorView *x, int32_t *pred, saga_stream_t stream)
{
    if(!valid_view(x) || !pred)
        return SAGA_HIP_EINVAL;
    if(x->dims[2] != 1 || x->dims[3] != 1)
        return SAGA_HIP_ESHAPE;
    if(x->dims[1] > 1 && x->strides[1] != 1)
        return SAGA_HIP_EUNSUPPORTED;
    const int N = x->dims[0], C = x->dims[1];
    const int64_t pitch = N > 1 ? x->strides[0] : C;
    hipStream_t st = as_stream(stream);
    if(x->dtype == SAGA_HALF)
        catclassifier_fwd_k<half_t><<<(N + 3) / 4, 256, 0, st>>>((const half_t *)x->ptr, pitch, pred, N, C);
    else if(x->dtype == SAGA_FLOAT)
        catclassifier_fwd_k<float><<<(N + 3) / 4, 256, 0, st>>>((const float *)x->ptr, pitch, pred, N, C);
    else
        return SAGA_HIP_EUNSUPPORTED;
    SAGA_CHECK_LAUNCH();
    return 0;
}

int saga_hip_catclassifier_bwd(const SagaTensorView *x, const SagaTensorView *dx, const int32_t *pred,
                               const int32_t *labels, float *loss, float scale, saga_stream_t stream)
{
    if(!valid_view(x) || !valid_view(dx) || !pred || !labels)
        return SAGA_HIP_EINVAL;
    if(!same_dims(x, dx) || x->dims[2] != 1 || x->dims[3] != 1)
        return SAGA_HIP_ESHAPE;
    if(x->dtype != dx->dtype || (x->dims[1] > 1 && (x->strides[1] != 1 || dx->strides[1] != 1)))
        return SAGA_HIP_EUNSUPPORTED;
    const int N = x->dims[0], C = x->dims[1];
    const int64_t px = N > 1 ? x->strides[0] : C, pdx = N > 1 ? dx->strides[0] : C;
    hipStream_t st = as_stream(stream);
    if(x->dtype == SAGA_HALF)
        catclassifier_bwd_k<half_t><<<(N + 3) / 4, 256, 0, st>>>((const half_t *)x->ptr, px, (half_t *)dx->ptr, pdx,
                                                                 pred, labels, loss, N, C, scale);
    else if(x->dtype == SAGA_FLOAT)
        catclassifier_bwd_k<float><<<(N + 3) / 4, 256, 0, st>>>((const float *)x->ptr, px, (float *)dx->ptr, pdx, pred,
                                                                labels, loss, N, C, scale);
    else
        return SAGA_HIP_EUNSUPPORTED;
    SAGA_CHECK_LAUNCH();
    return 0;
}

int saga_hip_softmax(const SagaTensorView *x, const SagaTensorView *y, saga_stream_t stream)
{
    if(!valid_view(x) || !valid_view(y))
        return SAGA_HIP_EINVAL;
    if(!same_dims(x, y))
        return SAGA_HIP_ESHAPE;
    if(x->dtype != y->dtype)
        return SAGA_HIP_EUNSUPPORTED;
    const int64_t total = (int64_t)x->dims[0] * x->dims[2] * x->dims[3];
    const int g = grid_for(total, 256, 256 * 32);
    hipStream_t st = as_stream(stream);
    if(x->dtype == SAGA_HALF)
        softmax_k<half_t><<<g, 256, 0, st>>>(dview(x), dview(y), total);
    else if(x->dtype == SAGA_FLOAT)
        softmax_k<float><<<g, 256, 0, st>>>(dview(x), dview(y), total);
    else
        return SAGA_HIP_EUNSUPPORTED;
    SAGA_CHECK_LAUNCH();
    return 0;
}

} // extern "C"
