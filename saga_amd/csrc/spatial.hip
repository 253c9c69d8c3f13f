// Spatial transformer: affine sampling grid + bilinear sampler in one pass.
//
// Replaces cudnnSpatialTfGridGeneratorForward + cudnnSpatialTfSamplerForward as the reference
// calls them (src/cuda/cuda_dnn.cpp:2372-2425): for every output pixel (h, w) the normalised
// target coordinate (xt, yt) in [-1, 1] (-1 and 1 are the centres of the first and last pixel)
// goes through the sample's 2x3 matrix theta to a source coordinate (xs, ys) in the same
// normalisation over the input; the output is the bilinear mix of the four input pixels around
// it, pixels outside the input counting as zero.  The reference writes the grid to memory
// between the two calls; here it stays in registers.  Forward only (so is the reference).
#include "common.hpp"

namespace {

template <typename T>
__global__ void __launch_bounds__(256) spatial_transform_k(DView x, const float *__restrict__ theta, DView y, int64_t total)
{
    const int C = y.d[1], OH = y.d[2], OW = y.d[3];
    const int IH = x.d[2], IW = x.d[3];
    const float sx = OW > 1 ? 2.0f / (float)(OW - 1) : 0.0f, sy = OH > 1 ? 2.0f / (float)(OH - 1) : 0.0f;
    for(int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < total; i += (int64_t)gridDim.x * blockDim.x) {
        const int w = (int)(i % OW);
        const int h = (int)((i / OW) % OH);
        const int n = (int)(i / ((int64_t)OW * OH));
        const float *t = theta + (int64_t)n * 6;
        const float xt = -1.0f + sx * (float)w, yt = -1.0f + sy * (float)h;
        const float xs = t[0] * xt + t[1] * yt + t[2];
        const float ys = t[3] * xt + t[4] * yt + t[5];
        const float px = (xs + 1.0f) * 0.5f * (float)(IW - 1);
        const float py = (ys + 1.0f) * 0.5f * (float)(IH - 1);
        const float fx0 = floorf(px), fy0 = floorf(py);
        const float ax = px - fx0, ay = py - fy0;
        // far outside coordinates are clamped before the conversion to int (all four taps miss)
        const int x0 = (int)fminf(fmaxf(fx0, -2.0f), (float)IW), y0 = (int)fminf(fmaxf(fy0, -2.0f), (float)IH);
        const int x1 = x0 + 1, y1 = y0 + 1;
        const bool vx0 = x0 >= 0 && x0 < IW, vx1 = x1 >= 0 && x1 < IW;
        const bool vy0 = y0 >= 0 && y0 < IH, vy1 = y1 >= 0 && y1 < IH;
        const float w00 = (1.0f - ax) * (1.0f - ay), w01 = ax * (1.0f - ay), w10 = (1.0f - ax) * ay, w11 = ax * ay;
        const T *xn = (const T *)x.ptr + n * x.s[0];
        T *yp = (T *)y.ptr + n * y.s[0] + h * y.s[2] + w * y.s[3];
        for(int c = 0; c < C; c++) {
            const T *xc = xn + c * x.s[1];
            float v = 0.0f;
            if(vy0 && vx0)
                v += w00 * (float)xc[y0 * x.s[2] + x0 * x.s[3]];
            if(vy0 && vx1)
                v += w01 * (float)xc[y0 * x.s[2] + x1 * x.s[3]];
            if(vy1 && vx0)
                v += w10 * (float)xc[y1 * x.s[2] + x0 * x.s[3]];
            if(vy1 && vx1)
                v += w11 * (float)xc[y1 * x.s[2] + x1 * x.s[3]];
            yp[c * y.s[1]] = (T)v;
        }
    }
}

} // namespace

extern "C" int saga_hip_spatial_transform(const SagaTensorView *x, const float *theta, const SagaTensorView *y,
                                          saga_stream_t stream)
{
    if(!valid_view(x) || !valid_view(y) || !theta)
        return SAGA_HIP_EINVAL;
    if(x->dims[0] != y->dims[0] || x->dims[1] != y->dims[1])
        return SAGA_HIP_ESHAPE;
    if(x->dtype != y->dtype)
        return SAGA_HIP_EUNSUPPORTED;
    const int64_t total = (int64_t)y->dims[0] * y->dims[2] * y->dims[3];
    const int g = grid_for(total, 256, 256 * 64);
    hipStream_t st = as_stream(stream);
    if(x->dtype == SAGA_HALF)
        spatial_transform_k<half_t><<<g, 256, 0, st>>>(dview(x), theta, dview(y), total);
    else if(x->dtype == SAGA_FLOAT)
        spatial_transform_k<float><<<g, 256, 0, st>>>(dview(x), theta, dview(y), total);
    else
        return SAGA_HIP_EUNSUPPORTED;
    SAGA_CHECK_LAUNCH();
    return 0;
}
