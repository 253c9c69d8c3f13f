/*
 * CPU oracle for the Saga compute path.  TEST INFRASTRUCTURE ONLY.
 *
 * This file restates, in plain C, the arithmetic that the reference obtains from
 * cuDNN / cuBLAS and from its own CUDA kernels.  It is the checker for the HIP
 * backend: only tests/, __graft_entry__.smoke() and the cpu_baseline leg of
 * bench.py may load it.  Nothing in saga_amd/ links, loads or calls it.
 *
 * Conventions: every tensor is fp32, contiguous, in LOGICAL order (N,C,H,W or
 * N,C); the callers (tests) permute to and from the device layout.  Sums run in
 * double so that the oracle is more accurate than either fp32 or fp16 device
 * code; outputs are rounded to fp32 once.
 *
 * Pinning status (what fixes each function besides this restatement):
 *   so_conv2d_fwd, so_bias_add     reference vectors test/test_ops.cpp:31-215, test_resnode
 *   so_conv2d_bwd_data             reference vectors test/test_resnode.cpp:104-134
 *   so_conv2d_bwd_filter           adjoint identity <conv(x,w),dy> = <w,bwd_filter(x,dy)>, torch-CPU
 *   so_conv2d_* with dilation > 1  torch-CPU double conv2d and its autograd, dilation 2 and 3, with stride and groups
 *   so_bias_bwd                    closed form (plain sum)
 *   so_fc_*                        reference vectors test/test_ops.cpp:286-386 (fwd); adjoint (bwd)
 *   so_bn_infer                    reference vectors test/test_ops.cpp:438-470
 *   so_bn_train_fwd, so_bn_bwd     reference vectors test/test_resnode.cpp (y, dx); finite differences
 *                                  running mean/var update: cuDNN-documented rule, parity unpinned
 *   so_relu_*                      reference vectors test_ops.cpp:24-28, test_resnode
 *   so_maxpool_*, so_avgpool_*     reference vectors test_ops.cpp:218-283 (fwd); brute force + sum
 *                                  conservation (bwd); max-pool tie break = first index, parity unpinned
 *   so_catclassifier_*             in-tree kernel src/cuda/cuda_kernels.cu:11-64 is the spec; closed forms
 *   so_adam_*                      in-tree kernel src/cuda/cuda_kernels.cu:159-230 is the spec; t=1 closed form;
 *                                  t > 1, weight decay and the fp16 skip / flag rules against a numpy restatement
 *                                  of the kernel over several steps (tests/test_oracle_net.py)
 *   so_softmax                     closed form, rows sum to one
 *   so_loss_bwd, so_tensor_stats   in-tree kernels src/cuda/cuda_kernels.cu:252-473 are the spec (incl. the zeros their
 *                                  block reduction feeds into min / max); hand-computed case + numpy closed forms
 *   so_spatial_transform           cuDNN's spatial transformer is third-party code outside the reference tree and
 *                                  the reference holds no vectors for it; restated from cuDNN's published rule
 *                                  (normalised coordinates, -1 / 1 = centres of the border pixels, zeros outside)
 *                                  and pinned against torch's affine_grid + grid_sample(align_corners=True) on
 *                                  the CPU, identity = copy, and the closed form for resizing a linear ramp
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

#define IDX4(n, c, h, w, C, H, W) ((((size_t)(n) * (C) + (c)) * (H) + (h)) * (W) + (w))

/* ---------------------------------------------------------------- fp16 <-> fp32 */

/* IEEE binary16 -> binary32 (exact). */
float so_half_to_float(uint16_t h)
{
    uint32_t sign = (uint32_t)(h & 0x8000u) << 16;
    uint32_t exp = (h >> 10) & 0x1f;
    uint32_t man = h & 0x3ff;
    uint32_t bits;
    if(exp == 0) {
        if(man == 0) {
            bits = sign;
        } else {
            int e = -1;
            do {
                man <<= 1;
                e++;
            } while(!(man & 0x400));
            man &= 0x3ff;
            bits = sign | ((uint32_t)(127 - 15 - e) << 23) | (man << 13);
        }
    } else if(exp == 31) {
        bits = sign | 0x7f800000u | (man << 13);
    } else {
        bits = sign | ((exp + 127 - 15) << 23) | (man << 13);
    }
    float f;
    memcpy(&f, &bits, 4);
    return f;
}

/* binary32 -> binary16, round to nearest even (what the device conversion does). */
uint16_t so_float_to_half(float f)
{
    uint32_t x;
    memcpy(&x, &f, 4);
    uint32_t sign = (x >> 16) & 0x8000u;
    uint32_t exp = (x >> 23) & 0xff;
    uint32_t man = x & 0x7fffffu;
    if(exp == 0xff)
        return (uint16_t)(sign | 0x7c00u | (man ? (0x200u | (man >> 13)) : 0));
    int e = (int)exp - 127 + 15;
    if(e >= 31)
        return (uint16_t)(sign | 0x7c00u);
    if(e <= 0) {
        if(e < -10)
            return (uint16_t)sign;
        man |= 0x800000u;
        int shift = 14 - e;
        uint32_t half_man = man >> shift;
        uint32_t rem = man & ((1u << shift) - 1);
        uint32_t halfway = 1u << (shift - 1);
        if(rem > halfway || (rem == halfway && (half_man & 1)))
            half_man++;
        return (uint16_t)(sign | half_man);
    }
    uint32_t half = sign | ((uint32_t)e << 10) | (man >> 13);
    uint32_t rem = man & 0x1fffu;
    if(rem > 0x1000u || (rem == 0x1000u && (half & 1)))
        half++;
    return (uint16_t)half;
}

void so_round_to_half(float *x, size_t n)
{
    for(size_t i = 0; i < n; i++)
        x[i] = so_half_to_float(so_float_to_half(x[i]));
}

/* ---------------------------------------------------------------- convolution */

static int conv_out(int in, int k, int pad, int stride, int dil)
{
    return 1 + (in + 2 * pad - ((k - 1) * dil + 1)) / stride; /* src/node.cpp:72-76 */
}

/*
 * y[n,k,p,q] = beta*y + sum_{c,r,s} x[n, g*Cg+c, p*st-pad+r*dil, q*st-pad+s*dil] * w[k,c,r,s]
 * Cross-correlation, square stride/pad (src/cuda/cuda_dnn.cpp:227-235, :338-347).
 * w dims [K, C/group, R, S] (src/node.cpp:99-110).
 */
void so_conv2d_fwd(const float *x, const float *w, float *y, int N, int C, int H, int W, int K, int R, int S,
                   int pad, int stride, int dil, int group, float beta)
{
    const int P = conv_out(H, R, pad, stride, dil), Q = conv_out(W, S, pad, stride, dil);
    const int Cg = C / group, Kg = K / group;
#pragma omp parallel for collapse(2) schedule(static)
    for(int n = 0; n < N; n++) {
        for(int k = 0; k < K; k++) {
            double *acc = (double *)calloc((size_t)P * Q, sizeof(double));
            const int g = k / Kg;
            for(int c = 0; c < Cg; c++) {
                const float *xc = x + IDX4(n, g * Cg + c, 0, 0, C, H, W);
                for(int r = 0; r < R; r++) {
                    for(int s = 0; s < S; s++) {
                        const double wv = w[(((size_t)k * Cg + c) * R + r) * S + s];
                        for(int p = 0; p < P; p++) {
                            const int h = p * stride - pad + r * dil;
                            if(h < 0 || h >= H)
                                continue;
                            const float *xr = xc + (size_t)h * W;
                            double *ar = acc + (size_t)p * Q;
                            int q0 = 0, q1 = Q;
                            /* valid q: 0 <= q*stride - pad + s*dil < W */
                            const int off = s * dil - pad;
                            while(q0 < Q && q0 * stride + off < 0)
                                q0++;
                            while(q1 > q0 && (q1 - 1) * stride + off >= W)
                                q1--;
                            for(int q = q0; q < q1; q++)
                                ar[q] += wv * xr[q * stride + off];
                        }
                    }
                }
            }
            float *yo = y + IDX4(n, k, 0, 0, K, P, Q);
            for(int i = 0; i < P * Q; i++)
                yo[i] = (float)(acc[i] + (beta != 0.0f ? (double)beta * yo[i] : 0.0));
            free(acc);
        }
    }
}

/*
 * dx[n,c,h,w] = beta*dx + sum_{k,r,s : h = p*st-pad+r*dil, w = q*st-pad+s*dil} dy[n,k,p,q] * w[k,c,r,s]
 * (src/cuda/cuda_dnn.cpp:467-476).  N,C,H,W describe dx; dy is [N,K,P,Q].
 */
void so_conv2d_bwd_data(const float *dy, const float *w, float *dx, int N, int C, int H, int W, int K, int R,
                        int S, int pad, int stride, int dil, int group, float beta)
{
    const int P = conv_out(H, R, pad, stride, dil), Q = conv_out(W, S, pad, stride, dil);
    const int Cg = C / group, Kg = K / group;
#pragma omp parallel for collapse(2) schedule(static)
    for(int n = 0; n < N; n++) {
        for(int c = 0; c < C; c++) {
            double *acc = (double *)calloc((size_t)H * W, sizeof(double));
            const int g = c / Cg, cl = c % Cg;
            for(int kk = 0; kk < Kg; kk++) {
                const int k = g * Kg + kk;
                const float *dyk = dy + IDX4(n, k, 0, 0, K, P, Q);
                for(int r = 0; r < R; r++) {
                    for(int s = 0; s < S; s++) {
                        const double wv = w[(((size_t)k * Cg + cl) * R + r) * S + s];
                        for(int p = 0; p < P; p++) {
                            const int h = p * stride - pad + r * dil;
                            if(h < 0 || h >= H)
                                continue;
                            for(int q = 0; q < Q; q++) {
                                const int ww = q * stride - pad + s * dil;
                                if(ww < 0 || ww >= W)
                                    continue;
                                acc[(size_t)h * W + ww] += wv * dyk[(size_t)p * Q + q];
                            }
                        }
                    }
                }
            }
            float *o = dx + IDX4(n, c, 0, 0, C, H, W);
            for(int i = 0; i < H * W; i++)
                o[i] = (float)(acc[i] + (beta != 0.0f ? (double)beta * o[i] : 0.0));
            free(acc);
        }
    }
}

/*
 * dw[k,c,r,s] = beta*dw + sum_{n,p,q} dy[n,k,p,q] * x[n, g*Cg+c, p*st-pad+r*dil, q*st-pad+s*dil]
 * (src/cuda/cuda_dnn.cpp:419-428).
 */
void so_conv2d_bwd_filter(const float *x, const float *dy, float *dw, int N, int C, int H, int W, int K, int R,
                          int S, int pad, int stride, int dil, int group, float beta)
{
    const int P = conv_out(H, R, pad, stride, dil), Q = conv_out(W, S, pad, stride, dil);
    const int Cg = C / group, Kg = K / group;
#pragma omp parallel for collapse(2) schedule(static)
    for(int k = 0; k < K; k++) {
        for(int c = 0; c < Cg; c++) {
            const int g = k / Kg;
            for(int r = 0; r < R; r++) {
                for(int s = 0; s < S; s++) {
                    double acc = 0;
                    for(int n = 0; n < N; n++) {
                        const float *xc = x + IDX4(n, g * Cg + c, 0, 0, C, H, W);
                        const float *dyk = dy + IDX4(n, k, 0, 0, K, P, Q);
                        for(int p = 0; p < P; p++) {
                            const int h = p * stride - pad + r * dil;
                            if(h < 0 || h >= H)
                                continue;
                            for(int q = 0; q < Q; q++) {
                                const int ww = q * stride - pad + s * dil;
                                if(ww < 0 || ww >= W)
                                    continue;
                                acc += (double)dyk[(size_t)p * Q + q] * xc[(size_t)h * W + ww];
                            }
                        }
                    }
                    float *o = dw + (((size_t)k * Cg + c) * R + r) * S + s;
                    *o = (float)(acc + (beta != 0.0f ? (double)beta * *o : 0.0));
                }
            }
        }
    }
}

/* y[n,k,:,:] += b[k]   (cudnnAddTensor of a {1,K,1,1} bias, src/cuda/cuda_dnn.cpp:39-68, :518-519) */
void so_bias_add(float *y, const float *b, int N, int K, int HW)
{
    for(int n = 0; n < N; n++)
        for(int k = 0; k < K; k++) {
            float *o = y + ((size_t)n * K + k) * HW;
            for(int i = 0; i < HW; i++)
                o[i] += b[k];
        }
}

/* db[k] = beta*db + sum_{n,p,q} dy[n,k,p,q]   (src/cuda/cuda_dnn.cpp:378-385) */
void so_bias_bwd(const float *dy, float *db, int N, int K, int HW, float beta)
{
    for(int k = 0; k < K; k++) {
        double acc = 0;
        for(int n = 0; n < N; n++) {
            const float *o = dy + ((size_t)n * K + k) * HW;
            for(int i = 0; i < HW; i++)
                acc += o[i];
        }
        db[k] = (float)(acc + (beta != 0.0f ? (double)beta * db[k] : 0.0));
    }
}

/* ---------------------------------------------------------------- fully connected */

/*
 * y[b,o] = beta*y + sum_i x[b,i] * (transW ? w[o,i] : w[i,o])
 * (src/cuda/cuda_dnn.cpp:1058-1066: column-major GEMM m=out n=batch k=in.)
 */
void so_fc_fwd(const float *x, const float *w, float *y, int B, int In, int Out, int transW, float beta)
{
#pragma omp parallel for schedule(static)
    for(int b = 0; b < B; b++)
        for(int o = 0; o < Out; o++) {
            double acc = 0;
            for(int i = 0; i < In; i++)
                acc += (double)x[(size_t)b * In + i] * (transW ? w[(size_t)o * In + i] : w[(size_t)i * Out + o]);
            float *yo = y + (size_t)b * Out + o;
            *yo = (float)(acc + (beta != 0.0f ? (double)beta * *yo : 0.0));
        }
}

/* dw = beta*dw + x^T dy, stored [In,Out] or (transW) [Out,In]  (src/cuda/cuda_dnn.cpp:1081-1099) */
void so_fc_bwd_w(const float *x, const float *dy, float *dw, int B, int In, int Out, int transW, float beta)
{
#pragma omp parallel for schedule(static)
    for(int i = 0; i < In; i++)
        for(int o = 0; o < Out; o++) {
            double acc = 0;
            for(int b = 0; b < B; b++)
                acc += (double)x[(size_t)b * In + i] * dy[(size_t)b * Out + o];
            float *d = transW ? dw + (size_t)o * In + i : dw + (size_t)i * Out + o;
            *d = (float)(acc + (beta != 0.0f ? (double)beta * *d : 0.0));
        }
}

/* dx[b,i] = beta*dx + sum_o dy[b,o] * W(i,o)   (src/cuda/cuda_dnn.cpp:1116-1126) */
void so_fc_bwd_x(const float *dy, const float *w, float *dx, int B, int In, int Out, int transW, float beta)
{
#pragma omp parallel for schedule(static)
    for(int b = 0; b < B; b++)
        for(int i = 0; i < In; i++) {
            double acc = 0;
            for(int o = 0; o < Out; o++)
                acc += (double)dy[(size_t)b * Out + o] * (transW ? w[(size_t)o * In + i] : w[(size_t)i * Out + o]);
            float *d = dx + (size_t)b * In + i;
            *d = (float)(acc + (beta != 0.0f ? (double)beta * *d : 0.0));
        }
}

/* ---------------------------------------------------------------- batch normalisation */

/* y = s*(x-m)/sqrt(v+eps) + b per channel  (cudnnBatchNormalizationForwardInference SPATIAL,
 * src/cuda/cuda_dnn.cpp:1641-1651) */
void so_bn_infer(const float *x, const float *s, const float *b, const float *m, const float *v, float *y, int N,
                 int C, int HW, float eps)
{
    for(int n = 0; n < N; n++)
        for(int c = 0; c < C; c++) {
            const double inv = 1.0 / sqrt((double)v[c] + eps);
            const float *xi = x + ((size_t)n * C + c) * HW;
            float *yo = y + ((size_t)n * C + c) * HW;
            for(int i = 0; i < HW; i++)
                yo[i] = (float)((double)s[c] * ((double)xi[i] - m[c]) * inv + b[c]);
        }
}

/*
 * Training forward (cudnnBatchNormalizationForwardTraining SPATIAL, src/cuda/cuda_dnn.cpp:1689-1709):
 * mean / biased variance over N*H*W, y = s*(x-mean)*invstd + b; saves mean and invstd;
 * running m,v <- (1-f)*old + f*new, with the UNBIASED variance for v (cuDNN's documented rule).
 */
void so_bn_train_fwd(const float *x, const float *s, const float *b, float *run_m, float *run_v, float *y,
                     float *save_mean, float *save_invstd, int N, int C, int HW, float eps, float expavg)
{
    const double M = (double)N * HW;
#pragma omp parallel for schedule(static)
    for(int c = 0; c < C; c++) {
        double sum = 0;
        for(int n = 0; n < N; n++) {
            const float *xi = x + ((size_t)n * C + c) * HW;
            for(int i = 0; i < HW; i++)
                sum += xi[i];
        }
        const double mean = sum / M;
        double var = 0;
        for(int n = 0; n < N; n++) {
            const float *xi = x + ((size_t)n * C + c) * HW;
            for(int i = 0; i < HW; i++) {
                const double d = xi[i] - mean;
                var += d * d;
            }
        }
        var /= M;
        const double inv = 1.0 / sqrt(var + eps);
        for(int n = 0; n < N; n++) {
            const float *xi = x + ((size_t)n * C + c) * HW;
            float *yo = y + ((size_t)n * C + c) * HW;
            for(int i = 0; i < HW; i++)
                yo[i] = (float)((double)s[c] * (xi[i] - mean) * inv + b[c]);
        }
        if(save_mean)
            save_mean[c] = (float)mean;
        if(save_invstd)
            save_invstd[c] = (float)inv;
        if(run_m)
            run_m[c] = (float)((1.0 - expavg) * run_m[c] + expavg * mean);
        if(run_v) {
            const double unbiased = M > 1 ? var * M / (M - 1.0) : var;
            run_v[c] = (float)((1.0 - expavg) * run_v[c] + expavg * unbiased);
        }
    }
}

/*
 * Backward (cudnnBatchNormalizationBackward, src/cuda/cuda_dnn.cpp:1754-1766):
 * xhat=(x-mean)*invstd; db=sum dy; ds=sum dy*xhat; dx = s*invstd/M*(M*dy - db - xhat*ds).
 * dx accumulates with beta_dx, ds/db with beta_p.
 */
void so_bn_bwd(const float *x, const float *dy, const float *s, const float *save_mean, const float *save_invstd,
               float *dx, float *ds, float *db, int N, int C, int HW, float beta_dx, float beta_p)
{
    const double M = (double)N * HW;
#pragma omp parallel for schedule(static)
    for(int c = 0; c < C; c++) {
        const double mean = save_mean[c], inv = save_invstd[c];
        double sdy = 0, sdyx = 0;
        for(int n = 0; n < N; n++) {
            const float *xi = x + ((size_t)n * C + c) * HW;
            const float *gi = dy + ((size_t)n * C + c) * HW;
            for(int i = 0; i < HW; i++) {
                sdy += gi[i];
                sdyx += (double)gi[i] * (xi[i] - mean) * inv;
            }
        }
        for(int n = 0; n < N; n++) {
            const float *xi = x + ((size_t)n * C + c) * HW;
            const float *gi = dy + ((size_t)n * C + c) * HW;
            float *o = dx + ((size_t)n * C + c) * HW;
            for(int i = 0; i < HW; i++) {
                const double xh = (xi[i] - mean) * inv;
                const double v = (double)s[c] * inv / M * (M * gi[i] - sdy - xh * sdyx);
                o[i] = (float)(v + (beta_dx != 0.0f ? (double)beta_dx * o[i] : 0.0));
            }
        }
        ds[c] = (float)(sdyx + (beta_p != 0.0f ? (double)beta_p * ds[c] : 0.0));
        db[c] = (float)(sdy + (beta_p != 0.0f ? (double)beta_p * db[c] : 0.0));
    }
}

/* ---------------------------------------------------------------- activations */

/* mode: 0 relu, 1 sigmoid, 2 tanh, 3 swish (beta 1), 4 leakyrelu(alpha)
 * (cudnnActivationForward, src/cuda/cuda_dnn.cpp:610-756; leaky relu src/cuda/cuda_kernels.cu:478-487).
 * relu propagates NaN (CUDNN_PROPAGATE_NAN). */
void so_act_fwd(const float *x, float *y, size_t n, int mode, float alpha)
{
    for(size_t i = 0; i < n; i++) {
        const double v = x[i];
        double r;
        switch(mode) {
        case 0:
            r = (v != v) ? v : (v > 0 ? v : 0);
            break;
        case 1:
            r = 1.0 / (1.0 + exp(-v));
            break;
        case 2:
            r = tanh(v);
            break;
        case 3:
            r = v / (1.0 + exp(-v));
            break;
        default:
            r = v > 0 ? v : v * alpha;
            break;
        }
        y[i] = (float)r;
    }
}

/* dx = beta*dx + dy * f'(x)  (cudnnActivationBackward(y,dy,x -> dx), src/cuda/cuda_dnn.cpp:668-676) */
void so_act_bwd(const float *x, const float *y, const float *dy, float *dx, size_t n, int mode, float alpha,
                float beta)
{
    for(size_t i = 0; i < n; i++) {
        const double v = x[i];
        double d;
        switch(mode) {
        case 0:
            d = v > 0 ? 1.0 : 0.0;
            break;
        case 1:
            d = (double)y[i] * (1.0 - y[i]);
            break;
        case 2:
            d = 1.0 - (double)y[i] * y[i];
            break;
        case 3: {
            const double sg = 1.0 / (1.0 + exp(-v));
            d = sg + v * sg * (1.0 - sg);
            break;
        }
        default:
            d = v > 0 ? 1.0 : alpha;
            break;
        }
        dx[i] = (float)(d * dy[i] + (beta != 0.0f ? (double)beta * dx[i] : 0.0));
    }
}

/* ---------------------------------------------------------------- pooling */

static int pool_out(int in, int k, int pad, int stride)
{
    return 1 + (in + 2 * pad - k) / stride; /* src/node.cpp:187-188 */
}

/*
 * Max pooling, padding acts as -inf, NaN propagates (cudnnPoolingForward MAX, PROPAGATE_NAN,
 * src/cuda/cuda_dnn.cpp:820-836).  idx (optional) receives the flat h*W+w index of the first
 * maximum in window scan order (rows, then columns) - the tie break this oracle defines.
 */
void so_maxpool_fwd(const float *x, float *y, int32_t *idx, int N, int C, int H, int W, int k, int pad, int stride)
{
    const int P = pool_out(H, k, pad, stride), Q = pool_out(W, k, pad, stride);
#pragma omp parallel for schedule(static)
    for(int nc = 0; nc < N * C; nc++) {
        const float *xi = x + (size_t)nc * H * W;
        for(int p = 0; p < P; p++)
            for(int q = 0; q < Q; q++) {
                float best = -INFINITY;
                int bi = -1;
                int isnan_ = 0;
                for(int r = 0; r < k; r++) {
                    const int h = p * stride - pad + r;
                    if(h < 0 || h >= H)
                        continue;
                    for(int s = 0; s < k; s++) {
                        const int w = q * stride - pad + s;
                        if(w < 0 || w >= W)
                            continue;
                        const float v = xi[(size_t)h * W + w];
                        if(v != v && !isnan_) {
                            isnan_ = 1;
                            best = v;
                            bi = h * W + w;
                        }
                        if(!isnan_ && (bi < 0 || v > best)) {
                            best = v;
                            bi = h * W + w;
                        }
                    }
                }
                y[(size_t)nc * P * Q + (size_t)p * Q + q] = best;
                if(idx)
                    idx[(size_t)nc * P * Q + (size_t)p * Q + q] = bi;
            }
    }
}

/* dx = beta*dx + scatter of dy to the arg-max position of each window (first index wins). */
void so_maxpool_bwd(const float *x, const float *dy, float *dx, int N, int C, int H, int W, int k, int pad,
                    int stride, float beta)
{
    const int P = pool_out(H, k, pad, stride), Q = pool_out(W, k, pad, stride);
    int32_t *idx = (int32_t *)malloc(sizeof(int32_t) * (size_t)N * C * P * Q);
    float *y = (float *)malloc(sizeof(float) * (size_t)N * C * P * Q);
    so_maxpool_fwd(x, y, idx, N, C, H, W, k, pad, stride);
#pragma omp parallel for schedule(static)
    for(int nc = 0; nc < N * C; nc++) {
        double *acc = (double *)calloc((size_t)H * W, sizeof(double));
        for(int i = 0; i < P * Q; i++) {
            const int t = idx[(size_t)nc * P * Q + i];
            if(t >= 0)
                acc[t] += dy[(size_t)nc * P * Q + i];
        }
        float *o = dx + (size_t)nc * H * W;
        for(int i = 0; i < H * W; i++)
            o[i] = (float)(acc[i] + (beta != 0.0f ? (double)beta * o[i] : 0.0));
        free(acc);
    }
    free(idx);
    free(y);
}

/* Average pooling, divisor always k*k (CUDNN_POOLING_AVERAGE_COUNT_INCLUDE_PADDING, src/cuda/cuda_dnn.cpp:923) */
void so_avgpool_fwd(const float *x, float *y, int N, int C, int H, int W, int k, int pad, int stride)
{
    const int P = pool_out(H, k, pad, stride), Q = pool_out(W, k, pad, stride);
#pragma omp parallel for schedule(static)
    for(int nc = 0; nc < N * C; nc++) {
        const float *xi = x + (size_t)nc * H * W;
        for(int p = 0; p < P; p++)
            for(int q = 0; q < Q; q++) {
                double acc = 0;
                for(int r = 0; r < k; r++) {
                    const int h = p * stride - pad + r;
                    if(h < 0 || h >= H)
                        continue;
                    for(int s = 0; s < k; s++) {
                        const int w = q * stride - pad + s;
                        if(w < 0 || w >= W)
                            continue;
                        acc += xi[(size_t)h * W + w];
                    }
                }
                y[(size_t)nc * P * Q + (size_t)p * Q + q] = (float)(acc / ((double)k * k));
            }
    }
}

void so_avgpool_bwd(const float *dy, float *dx, int N, int C, int H, int W, int k, int pad, int stride, float beta)
{
    const int P = pool_out(H, k, pad, stride), Q = pool_out(W, k, pad, stride);
#pragma omp parallel for schedule(static)
    for(int nc = 0; nc < N * C; nc++) {
        double *acc = (double *)calloc((size_t)H * W, sizeof(double));
        for(int p = 0; p < P; p++)
            for(int q = 0; q < Q; q++) {
                const double g = dy[(size_t)nc * P * Q + (size_t)p * Q + q] / ((double)k * k);
                for(int r = 0; r < k; r++) {
                    const int h = p * stride - pad + r;
                    if(h < 0 || h >= H)
                        continue;
                    for(int s = 0; s < k; s++) {
                        const int w = q * stride - pad + s;
                        if(w < 0 || w >= W)
                            continue;
                        acc[(size_t)h * W + w] += g;
                    }
                }
            }
        float *o = dx + (size_t)nc * H * W;
        for(int i = 0; i < H * W; i++)
            o[i] = (float)(acc[i] + (beta != 0.0f ? (double)beta * o[i] : 0.0));
        free(acc);
    }
}

/* ---------------------------------------------------------------- spatial transformer */

/* affine grid + bilinear sampler, zeros outside (cudnnSpatialTfGridGeneratorForward +
 * cudnnSpatialTfSamplerForward as called at src/cuda/cuda_dnn.cpp:2407-2416); theta is [N,2,3] */
void so_spatial_transform(const float *x, const float *theta, float *y, int N, int C, int IH, int IW, int OH, int OW)
{
    for(int n = 0; n < N; n++) {
        const float *t = theta + (size_t)n * 6;
        for(int h = 0; h < OH; h++)
            for(int w = 0; w < OW; w++) {
                const double xt = OW > 1 ? -1.0 + 2.0 * w / (OW - 1) : -1.0;
                const double yt = OH > 1 ? -1.0 + 2.0 * h / (OH - 1) : -1.0;
                const double xs = t[0] * xt + t[1] * yt + t[2];
                const double ys = t[3] * xt + t[4] * yt + t[5];
                const double px = (xs + 1.0) * 0.5 * (IW - 1), py = (ys + 1.0) * 0.5 * (IH - 1);
                const double fx = floor(px), fy = floor(py);
                const double ax = px - fx, ay = py - fy;
                for(int c = 0; c < C; c++) {
                    double v = 0;
                    for(int dy = 0; dy < 2; dy++)
                        for(int dx = 0; dx < 2; dx++) {
                            const double yy = fy + dy, xx = fx + dx;
                            if(yy < 0 || yy >= IH || xx < 0 || xx >= IW)
                                continue;
                            v += (dx ? ax : 1.0 - ax) * (dy ? ay : 1.0 - ay) * x[IDX4(n, c, (int)yy, (int)xx, C, IH, IW)];
                        }
                    y[IDX4(n, c, h, w, C, OH, OW)] = (float)v;
                }
            }
    }
}

/* ---------------------------------------------------------------- softmax / classifier */

/* softmax over C for every (n, spatial) position, max-subtracted
 * (CUDNN_SOFTMAX_ACCURATE, MODE_CHANNEL, src/cuda/cuda_dnn.cpp:1941-1944) */
/* L2 loss backward (reference: deviceLossReduction + loss_bwd_*, src/cuda/cuda_kernels.cu:396-473): per
 * sample v = x - target, dx = v * scale; mmss = {min, max, sum / c, sum of squares / c}.  The reference feeds
 * its per-thread SUMS into the min / max lanes and pads the last reduction stage with zeros
 * (blockReduceStats, :273-290); with its launch shape (one element per thread) that is min(0, min v) and
 * max(0, max v). */
void so_loss_bwd(const float *x, const float *target, float *dx, float *mmss, int N, int c, float scale)
{
    for(int n = 0; n < N; n++) {
        double s = 0, ss = 0;
        float mn = 0.0f, mx = 0.0f;
        for(int e = 0; e < c; e++) {
            const float v = x[(size_t)n * c + e] - target[(size_t)n * c + e];
            dx[(size_t)n * c + e] = v * scale;
            if(v < mn)
                mn = v;
            if(v > mx)
                mx = v;
            s += v;
            ss += (double)v * v;
        }
        mmss[n * 4 + 0] = mn;
        mmss[n * 4 + 1] = mx;
        mmss[n * 4 + 2] = (float)(s / c);
        mmss[n * 4 + 3] = (float)(ss / c);
    }
}

/* the "stats" node (reference: deviceReduceStats + compute_mean_stddev, src/cuda/cuda_kernels.cu:313-383):
 * {min(0, min), max(0, max), mean, (sum of squares - sum^2 / n) / n} */
void so_tensor_stats(const float *x, float *out4, size_t n)
{
    double s = 0, ss = 0;
    float mn = 0.0f, mx = 0.0f;
    for(size_t i = 0; i < n; i++) {
        const float v = x[i];
        if(v < mn)
            mn = v;
        if(v > mx)
            mx = v;
        s += v;
        ss += (double)v * v;
    }
    out4[0] = mn;
    out4[1] = mx;
    out4[2] = (float)(s / (double)n);
    out4[3] = (float)((ss - s * s / (double)n) / (double)n);
}

void so_softmax(const float *x, float *y, int N, int C, int HW)
{
    for(int n = 0; n < N; n++)
        for(int i = 0; i < HW; i++) {
            const float *xi = x + (size_t)n * C * HW + i;
            float *yo = y + (size_t)n * C * HW + i;
            double mx = -INFINITY;
            for(int c = 0; c < C; c++)
                if(xi[(size_t)c * HW] > mx)
                    mx = xi[(size_t)c * HW];
            double sum = 0;
            for(int c = 0; c < C; c++)
                sum += exp(xi[(size_t)c * HW] - mx);
            for(int c = 0; c < C; c++)
                yo[(size_t)c * HW] = (float)(exp(xi[(size_t)c * HW] - mx) / sum);
        }
}

/* label[i] = first index of the maximum, strict '>' (src/cuda/cuda_kernels.cu:11-31) */
void so_catclassifier_fwd(const float *x, int32_t *y, int N, int C)
{
    for(int i = 0; i < N; i++) {
        const float *xi = x + (size_t)i * C;
        int32_t label = 0;
        float best = xi[0];
        for(int j = 1; j < C; j++)
            if(xi[j] > best) {
                best = xi[j];
                label = j;
            }
        y[i] = label;
    }
}

/*
 * src/cuda/cuda_kernels.cu:33-64: max = x[pred]; lse = max + log(sum exp(x-max)); p = exp(x-lse);
 * dx[j] = (p - [j==label]) * scale; loss[i] = -log p[label].  All in double.
 */
void so_catclassifier_bwd(const float *x, float *dx, const int32_t *pred, const int32_t *label, float *loss,
                          int N, int C, float scale)
{
    for(int i = 0; i < N; i++) {
        const float *xi = x + (size_t)i * C;
        float *di = dx + (size_t)i * C;
        const double mx = xi[pred[i]];
        double sum = 0;
        for(int j = 0; j < C; j++)
            sum += exp((double)xi[j] - mx);
        const double offset = mx + log(sum);
        for(int j = 0; j < C; j++) {
            const double p = exp((double)xi[j] - offset);
            if(label[i] == j) {
                di[j] = (float)((p - 1.0) * scale);
                if(loss)
                    loss[i] = (float)-log(p);
            } else {
                di[j] = (float)(p * scale);
            }
        }
    }
}

/* ---------------------------------------------------------------- Adam */

#define SO_ADAM_B1 0.9f   /* src/cuda/cuda_kernels.hpp:54 */
#define SO_ADAM_B2 0.999f /* src/cuda/cuda_kernels.hpp:55 */
#define SO_ADAM_EPS 1e-8f /* src/cuda/cuda_kernels.cu:157 */

/*
 * fp32 Adam, src/cuda/cuda_kernels.cu:159-189.  b1t = 1/(1-b1^t), b2t = 1/(1-b2^t)
 * (src/cuda/cuda_optimizer.cpp:79-80).  Non-finite gradients skip the element and raise a flag:
 * flags[0]=range, flags[1]=inf, flags[2]=nan (src/cuda/cuda_aux.hpp:5-10).
 * Arithmetic is fp32, as on the device; the update uses rsqrt(v_hat + eps).
 */
void so_adam_f32(float *w, const float *g, float *m, float *v, size_t n, float b1t, float b2t, float lr,
                 float lambda, uint32_t *flags)
{
    for(size_t i = 0; i < n; i++) {
        const float dw = g[i];
        if(!isfinite(dw)) {
            if(isnan(dw))
                flags[2] = 1;
            else
                flags[1] = 1;
            continue;
        }
        const float mi = m[i] = SO_ADAM_B1 * m[i] + (1.0f - SO_ADAM_B1) * dw;
        const float vi = v[i] = SO_ADAM_B2 * v[i] + (1.0f - SO_ADAM_B2) * dw * dw;
        const float m_hat = mi * b1t;
        const float v_hat = vi * b2t;
        float wi = w[i];
        wi = wi - lr * m_hat * (float)(1.0 / sqrt((double)(v_hat + SO_ADAM_EPS))) - lr * lambda * wi;
        w[i] = wi;
    }
}

/*
 * Mixed precision Adam, src/cuda/cuda_kernels.cu:191-230: fp16 weights/gradients, fp32 m, v and
 * master copy c.  Gradient bits with exponent >= 0x1e raise `range`; all-ones exponent raises
 * inf/nan and skips the element.  g = half(g) * alpha with alpha = 1/loss_scale.
 */
void so_adam_mixed(uint16_t *w, const uint16_t *g, float *m, float *v, float *c, size_t n, float alpha, float b1t,
                   float b2t, float lr, float lambda, uint32_t *flags)
{
    for(size_t i = 0; i < n; i++) {
        const uint16_t u = g[i];
        if((u & 0x7800) == 0x7800) {
            flags[0] = 1;
            if((u & 0x7c00) == 0x7c00) {
                if(u & 0x3ff)
                    flags[2] = 1;
                else
                    flags[1] = 1;
                continue;
            }
        }
        const float dw = so_half_to_float(u) * alpha;
        const float mi = SO_ADAM_B1 * m[i] + (1.0f - SO_ADAM_B1) * dw;
        const float vi = SO_ADAM_B2 * v[i] + (1.0f - SO_ADAM_B2) * dw * dw;
        const float m_hat = mi * b1t;
        const float v_hat = vi * b2t;
        float wi = c[i];
        wi = wi - lr * m_hat * (float)(1.0 / sqrt((double)(v_hat + SO_ADAM_EPS))) - lr * lambda * wi;
        m[i] = mi;
        v[i] = vi;
        c[i] = wi;
        w[i] = so_float_to_half(wi);
    }
}

/* ---------------------------------------------------------------- elementwise helpers */

/* y = x0 + x1 (cudnnOpTensor ADD, src/cuda/cuda_dnn.cpp:1866-1875) */
void so_add(const float *a, const float *b, float *y, size_t n)
{
    for(size_t i = 0; i < n; i++)
        y[i] = a[i] + b[i];
}

/* dst = beta*dst + src (cudnnTransformTensor used for sum backward, src/cuda/cuda_dnn.cpp:72-99) */
void so_axpby(const float *src, float *dst, size_t n, float beta)
{
    for(size_t i = 0; i < n; i++)
        dst[i] = src[i] + (beta != 0.0f ? beta * dst[i] : 0.0f);
}

/* dst = (float)src * scale for u8 sources (src/cuda/cuda_kernels.cu:102-111) */
void so_convert_u8(const uint8_t *src, float *dst, size_t n, float scale)
{
    for(size_t i = 0; i < n; i++)
        dst[i] = (float)src[i] * scale;
}
