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

// ---------------------------------------------------------------- L2 loss and tensor statistics
//
// Both report {min, max, mean, second moment or variance} the way the reference's kernels do
// (src/cuda/cuda_kernels.cu:252-430): its block reduction pads the last stage with zeros, so the reported
// minimum is min(0, smallest value) and the maximum max(0, largest value).

struct Stat4 {
    float mn, mx;
    double s, ss;
};

__device__ __forceinline__ Stat4 block_stat4(Stat4 v)
{
    __shared__ Stat4 red[4];
#pragma unroll
    for(int o = 32; o > 0; o >>= 1) {
        v.mn = fminf(v.mn, __shfl_xor(v.mn, o, 64));
        v.mx = fmaxf(v.mx, __shfl_xor(v.mx, o, 64));
        v.s += __shfl_xor(v.s, o, 64);
        v.ss += __shfl_xor(v.ss, o, 64);
    }
    if((threadIdx.x & 63) == 0)
        red[threadIdx.x >> 6] = v;
    __syncthreads();
    Stat4 r = red[0];
    for(int w = 1; w < 4; w++) {
        r.mn = fminf(r.mn, red[w].mn);
        r.mx = fmaxf(r.mx, red[w].mx);
        r.s += red[w].s;
        r.ss += red[w].ss;
    }
    return r;
}

// element e (row-major over C,H,W) of sample n
__device__ __forceinline__ int64_t sample_off(const DView &v, int n, int64_t e)
{
    const int w = (int)(e % v.d[3]);
    e /= v.d[3];
    const int h = (int)(e % v.d[2]);
    const int c = (int)(e / v.d[2]);
    return n * v.s[0] + c * v.s[1] + h * v.s[2] + w * v.s[3];
}

// one block per sample: v = x - target, dx = v * scale, mmss[n] = {min(0,v), max(0,v), mean v, mean v^2}
template <typename T, typename TT>
__global__ void __launch_bounds__(256) loss_bwd_k(DView x, DView target, DView dx, float *__restrict__ mmss, float scale)
{
    const int n = blockIdx.x;
    const int64_t c = (int64_t)x.d[1] * x.d[2] * x.d[3];
    Stat4 a = {0.0f, 0.0f, 0.0, 0.0};
    for(int64_t e = threadIdx.x; e < c; e += 256) {
        const float v = (float)((const T *)x.ptr)[sample_off(x, n, e)] - (float)((const TT *)target.ptr)[sample_off(target, n, e)];
        ((T *)dx.ptr)[sample_off(dx, n, e)] = (T)(v * scale);
        a.mn = fminf(a.mn, v);
        a.mx = fmaxf(a.mx, v);
        a.s += v;
        a.ss += (double)v * v;
    }
    a = block_stat4(a);
    if(threadIdx.x == 0) {
        mmss[n * 4 + 0] = a.mn;
        mmss[n * 4 + 1] = a.mx;
        mmss[n * 4 + 2] = (float)(a.s / (double)c);
        mmss[n * 4 + 3] = (float)(a.ss / (double)c);
    }
}

// partial[b] = statistics of the elements block b strides over (logical order, any strides)
template <typename T> __global__ void __launch_bounds__(256) stats_partial_k(DView x, int64_t total, Stat4 *__restrict__ partial)
{
    const int64_t per = (int64_t)x.d[1] * x.d[2] * x.d[3];
    Stat4 a = {0.0f, 0.0f, 0.0, 0.0};
    for(int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < total; i += (int64_t)gridDim.x * 256) {
        const float v = (float)((const T *)x.ptr)[sample_off(x, (int)(i / per), i % per)];
        a.mn = fminf(a.mn, v);
        a.mx = fmaxf(a.mx, v);
        a.s += v;
        a.ss += (double)v * v;
    }
    a = block_stat4(a);
    if(threadIdx.x == 0)
        partial[blockIdx.x] = a;
}

__global__ void __launch_bounds__(64) stats_final_k(const Stat4 *__restrict__ partial, int blocks, double n, float *__restrict__ out)
{
    if(threadIdx.x != 0)
        return;
    Stat4 r = partial[0];
    for(int b = 1; b < blocks; b++) { // fixed order: the same result every run
        r.mn = fminf(r.mn, partial[b].mn);
        r.mx = fmaxf(r.mx, partial[b].mx);
        r.s += partial[b].s;
        r.ss += partial[b].ss;
    }
    out[0] = r.mn;
    out[1] = r.mx;
    out[2] = (float)(r.s / n);
    out[3] = (float)((r.ss - r.s * r.s / n) / n);
}

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

int saga_hip_loss_bwd(const SagaTensorView *x, const SagaTensorView *target, const SagaTensorView *dx, float *mmss,
                      float scale, saga_stream_t stream)
{
    if(!valid_view(x) || !valid_view(target) || !valid_view(dx) || !mmss)
        return SAGA_HIP_EINVAL;
    if(!same_dims(x, target) || !same_dims(x, dx))
        return SAGA_HIP_ESHAPE;
    if(x->dtype != dx->dtype)
        return SAGA_HIP_EUNSUPPORTED;
    hipStream_t st = as_stream(stream);
    const int N = x->dims[0];
    if(x->dtype == SAGA_HALF && target->dtype == SAGA_FLOAT)
        loss_bwd_k<half_t, float><<<N, 256, 0, st>>>(dview(x), dview(target), dview(dx), mmss, scale);
    else if(x->dtype == SAGA_HALF && target->dtype == SAGA_HALF)
        loss_bwd_k<half_t, half_t><<<N, 256, 0, st>>>(dview(x), dview(target), dview(dx), mmss, scale);
    else if(x->dtype == SAGA_FLOAT && target->dtype == SAGA_FLOAT)
        loss_bwd_k<float, float><<<N, 256, 0, st>>>(dview(x), dview(target), dview(dx), mmss, scale);
    else
        return SAGA_HIP_EUNSUPPORTED; // the combinations of the reference (src/cuda/cuda_dnn.cpp:1415-1440)
    SAGA_CHECK_LAUNCH();
    return 0;
}

size_t saga_hip_tensor_stats_workspace_size(void) { return 256 * sizeof(Stat4); }

int saga_hip_tensor_stats(const SagaTensorView *x, float *out4, void *workspace, size_t ws_bytes, saga_stream_t stream)
{
    if(!valid_view(x) || !out4)
        return SAGA_HIP_EINVAL;
    if(!workspace || ws_bytes < saga_hip_tensor_stats_workspace_size() || ((uintptr_t)workspace & 7))
        return SAGA_HIP_EWORKSPACE;
    const int64_t total = view_elements(x);
    const int blocks = grid_for(total, 256 * 16, 256);
    hipStream_t st = as_stream(stream);
    if(x->dtype == SAGA_HALF)
        stats_partial_k<half_t><<<blocks, 256, 0, st>>>(dview(x), total, (Stat4 *)workspace);
    else if(x->dtype == SAGA_FLOAT)
        stats_partial_k<float><<<blocks, 256, 0, st>>>(dview(x), total, (Stat4 *)workspace);
    else
        return SAGA_HIP_EUNSUPPORTED;
    stats_final_k<<<1, 64, 0, st>>>((const Stat4 *)workspace, blocks, (double)total, out4);
    SAGA_CHECK_LAUNCH();
    return 0;
}

} // extern "C"
