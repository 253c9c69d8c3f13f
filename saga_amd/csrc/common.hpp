// Shared device/host helpers of the gfx950 kernel library.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "saga_hip.h"

typedef _Float16 half_t;
typedef _Float16 half2_t __attribute__((ext_vector_type(2)));
typedef _Float16 half4_t __attribute__((ext_vector_type(4)));
typedef _Float16 half8_t __attribute__((ext_vector_type(8)));
typedef float float4_t __attribute__((ext_vector_type(4)));
typedef float float16_t __attribute__((ext_vector_type(16)));

#define SAGA_WAVE 64

#define SAGA_CHECK_LAUNCH()                  \
    do {                                     \
        hipError_t e__ = hipGetLastError();  \
        if(e__ != hipSuccess)                \
            return (int)e__;                 \
    } while(0)

static inline hipStream_t as_stream(saga_stream_t s) { return (hipStream_t)s; }

static inline size_t dtype_size(int dt)
{
    switch(dt) {
    case SAGA_U8: return 1;
    case SAGA_HALF: return 2;
    case SAGA_FLOAT: return 4;
    case SAGA_INT64: return 8;
    case SAGA_I32: return 4;
    case SAGA_I16: return 2;
    }
    return 0;
}

static inline bool same_dims(const SagaTensorView *a, const SagaTensorView *b)
{
    for(int i = 0; i < 4; i++)
        if(a->dims[i] != b->dims[i])
            return false;
    return true;
}

static inline bool valid_view(const SagaTensorView *v)
{
    if(!v || !v->ptr)
        return false;
    for(int i = 0; i < 4; i++)
        if(v->dims[i] < 1)
            return false;
    return dtype_size(v->dtype) != 0;
}

static inline int64_t view_elements(const SagaTensorView *v)
{
    return (int64_t)v->dims[0] * v->dims[1] * v->dims[2] * v->dims[3];
}

// Channels-last with a row pitch: element (n,c,h,w) at ((n*H+h)*W+w)*pitch + c.
// pitch > C describes a channel slice of a wider NHWC tensor.
struct CLInfo {
    int64_t rows; // N*H*W
    int C;
    int64_t pitch;
};

static inline bool as_channels_last(const SagaTensorView *v, CLInfo *o)
{
    const int N = v->dims[0], C = v->dims[1], H = v->dims[2], W = v->dims[3];
    if(C > 1 && v->strides[1] != 1)
        return false;
    int64_t pitch = W > 1 ? v->strides[3] : (H > 1 ? v->strides[2] : (N > 1 ? v->strides[0] : C));
    if(pitch < C)
        return false;
    if(W > 1 && v->strides[3] != pitch)
        return false;
    if(H > 1 && v->strides[2] != (int64_t)W * pitch)
        return false;
    if(N > 1 && v->strides[0] != (int64_t)H * W * pitch)
        return false;
    o->rows = (int64_t)N * H * W;
    o->C = C;
    o->pitch = pitch;
    return true;
}

// Channels-first: element (n,c,h,w) at n*npitch + (c*H+h)*W + w.
struct CFInfo {
    int N, C;
    int64_t HW;
    int64_t npitch;
};

static inline bool as_channels_first(const SagaTensorView *v, CFInfo *o)
{
    const int N = v->dims[0], C = v->dims[1], H = v->dims[2], W = v->dims[3];
    if(W > 1 && v->strides[3] != 1)
        return false;
    if(H > 1 && v->strides[2] != W)
        return false;
    if(C > 1 && v->strides[1] != (int64_t)H * W)
        return false;
    int64_t np = N > 1 ? v->strides[0] : (int64_t)C * H * W;
    if(np < (int64_t)C * H * W)
        return false;
    o->N = N;
    o->C = C;
    o->HW = (int64_t)H * W;
    o->npitch = np;
    return true;
}

static inline bool aligned16(const void *p) { return (((uintptr_t)p) & 15) == 0; }

// Device-side POD copy of a view (kernel argument).
struct DView {
    char *ptr;
    int d[4];
    int64_t s[4];
};

static inline DView dview(const SagaTensorView *v)
{
    DView r;
    r.ptr = (char *)v->ptr;
    for(int i = 0; i < 4; i++) {
        r.d[i] = v->dims[i];
        r.s[i] = v->strides[i];
    }
    return r;
}

template <typename T> __device__ __forceinline__ float ld(const T *p) { return (float)*p; }
template <typename T> __device__ __forceinline__ void st(T *p, float v) { *p = (T)v; }

__device__ __forceinline__ float wave_sum(float v)
{
#pragma unroll
    for(int o = 32; o > 0; o >>= 1)
        v += __shfl_xor(v, o, 64);
    return v;
}

__device__ __forceinline__ float wave_max(float v)
{
#pragma unroll
    for(int o = 32; o > 0; o >>= 1)
        v = fmaxf(v, __shfl_xor(v, o, 64));
    return v;
}

static inline int grid_for(int64_t work, int block, int cap = 256 * 64)
{
    int64_t g = (work + block - 1) / block;
    if(g < 1)
        g = 1;
    if(g > cap)
        g = cap;
    return (int)g;
}

// bn.hip: the per-channel step between the two passes of a batch norm's backward (bn_bwd_finalize), for kernels
// in other files that produce the partial sums [rows][C][2] themselves
int bn_launch_bwd_finalize(const float *partial, int rows, const float *s, const float *save_invstd, float *ds, float *db,
                           float *coef, double M, int C, float beta_p, hipStream_t st);

