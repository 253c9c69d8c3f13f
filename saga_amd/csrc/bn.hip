// Batch normalisation for gfx950: inference, training forward (with optional fused
// residual add + relu) and backward.  Everything here is HBM-bound.
//
// Channels-last tensors are walked as rows of C contiguous channels: a 256-thread block is
// shaped (CVB channel-vectors) x (RB rows); lanes along x read consecutive 16-byte vectors so
// each wavefront touches whole rows, and every thread keeps its channel's parameters in
// registers for all the rows it visits.  Per-channel sums are reduced thread -> LDS ->
// per-block partials in the workspace -> one small finalize kernel, so the data is read
// exactly twice in training forward (statistics, then normalise) and backward.
//
// Statistics are accumulated on values shifted by the channel's first element, which removes
// the cancellation in E[x^2] - E[x]^2 when |mean| >> stddev.
#include "common.hpp"

#include <stdlib.h>

namespace {

template <typename T, int VN> struct VecT;
template <> struct VecT<half_t, 8> { typedef half8_t type; };
template <> struct VecT<float, 4> { typedef float4_t type; };
template <> struct VecT<half_t, 1> { typedef half_t type; };
template <> struct VecT<float, 1> { typedef float type; };

template <typename T, int VN, bool NT = true> struct Ld {
    typedef typename VecT<T, VN>::type V;
    static __device__ __forceinline__ void load(const T *p, float (&o)[VN])
    {
        if constexpr(VN == 1) {
            o[0] = (float)*p;
        } else {
            // (non-temporal, like the stores below: these kernels read every tensor once; 9.18 -> 8.99 ms for the
            // batch-norm kernels of a ResNet-50 training step)
            const V v = NT ? __builtin_nontemporal_load((const V *)p) : *(const V *)p;
#pragma unroll
            for(int j = 0; j < VN; j++)
                o[j] = (float)v[j];
        }
    }
    static __device__ __forceinline__ V raw(const T *p) { return NT ? __builtin_nontemporal_load((const V *)p) : *(const V *)p; }
    static __device__ __forceinline__ float at(const V &v, int j)
    {
        if constexpr(VN == 1)
            return (float)v;
        else
            return (float)v[j];
    }
    static __device__ __forceinline__ void store(T *p, const float (&o)[VN])
    {
        if constexpr(VN == 1) {
            *p = (T)o[0];
        } else {
            V v;
#pragma unroll
            for(int j = 0; j < VN; j++)
                v[j] = (T)o[j];
            // non-temporal: what these kernels write is a stream that the next operation reads whole; with the hint
            // the batch-norm kernels of a ResNet-50 training step take 9.06 ms instead of 9.23, and the convolutions
            // that read the results take what they took
            __builtin_nontemporal_store(v, (V *)p);
        }
    }
};

struct Shape {
    int cvb;  // channel vectors per block (power of two <= 64)
    int rb;   // rows per block = 256 / cvb
    int gy;   // blocks along channels
    int gx;   // blocks along rows of the kernels that leave one partial row per block
    int gxa;  // blocks along rows of the kernels that only stream (no partials: as many as there are batches)
};

static int env_int(const char *name, int dflt)
{
    const char *e = getenv(name);
    return e && *e ? atoi(e) : dflt;
}

// backward: the statistics pass leaves fewer partial rows (measured on MI355X inside the ResNet-50 step: 512
// blocks of contiguous row runs beat 2048 by 3 %), and the apply pass that follows uses the same small grid
static Shape plan(int64_t rows, int cvec, bool backward = false)
{
    Shape s;
    s.cvb = 1;
    while(s.cvb < cvec && s.cvb < 64)
        s.cvb <<= 1;
    s.rb = 256 / s.cvb;
    s.gy = (cvec + s.cvb - 1) / s.cvb;
    // SAGA_HIP_BN_STATS_BLOCKS / SAGA_HIP_BN_APPLY_GROUPS: experiment knobs (blocks of a reducing kernel over the
    // whole tensor; row groups per block of a streaming kernel)
    static const int fwd_blocks = env_int("SAGA_HIP_BN_STATS_BLOCKS", 2048);
    static const int bwd_blocks = env_int("SAGA_HIP_BN_BWD_BLOCKS", 512);
    const int stats_blocks = backward ? bwd_blocks : fwd_blocks;
    static const int apply_groups = env_int("SAGA_HIP_BN_APPLY_GROUPS", 4);
    int64_t want = (rows + (int64_t)s.rb * 4 - 1) / ((int64_t)s.rb * 4);
    int cap = stats_blocks / s.gy;
    if(cap < 1)
        cap = 1;
    if(want > cap)
        want = cap;
    if(want < 1)
        want = 1;
    s.gx = (int)want;
    int64_t wa = (rows + (int64_t)s.rb * apply_groups - 1) / ((int64_t)s.rb * apply_groups);
    if(wa > 65535)
        wa = 65535;
    if(wa < 1)
        wa = 1;
    s.gxa = (int)wa;
    return s;
}

// ---------------------------------------------------------------- channels-last kernels

// Rows of a block.  Either a block owns a CONTIGUOUS run of row groups (rb rows each) and walks it in order, so
// that the batch of rows it has in flight is one contiguous piece of memory and the blocks, dispatched in order,
// sweep the tensor front to back; or (cvb < 0) the grid-stride walk, where the rows of a batch lie a whole grid
// apart.  On tensors that come from HBM the first order is much faster (a plain copy moves 5.4 - 6 TB/s that way
// and 4.1 - 4.5 TB/s grid-strided; batch-norm backward on 411 MB tensors 367 us against 494 us).  Inside a
// training step part of the data is still in the last-level cache and the picture is mixed - measured per kernel
// on the ResNet-50 b256 step: the backward statistics pass gains 5 % from contiguous runs with 512 blocks, the
// two apply passes lose 2 - 7 % - hence the default of gridstride_mask().  r0 = first row of this thread,
// rend = end of the block's run, stride = distance of a thread's consecutive rows.
struct RowRun {
    int64_t r0, rend, stride;
};
__device__ __forceinline__ RowRun row_run(int64_t rows, int rb, int ty, int cvb)
{
    RowRun rr;
    if(cvb < 0) {
        rr.r0 = (int64_t)blockIdx.x * rb + ty;
        rr.rend = rows;
        rr.stride = (int64_t)gridDim.x * rb;
        return rr;
    }
    const int64_t groups = (rows + rb - 1) / rb;
    const int64_t per = (groups + gridDim.x - 1) / gridDim.x;
    const int64_t g0 = (int64_t)blockIdx.x * per;
    int64_t g1 = g0 + per;
    if(g1 > groups)
        g1 = groups;
    rr.r0 = g0 * rb + ty;
    rr.rend = g1 * rb < rows ? g1 * rb : rows;
    rr.stride = rb;
    return rr;
}

// y = x*scale[c] + shift[c] (+ z) (relu).  MODE 0: scale/shift from s,b,m,v (inference);
// MODE 1: scale/shift precomputed in ss[0..C), ss[C..2C) (training, second pass).
template <typename T, int VN, int MODE>
__global__ void __launch_bounds__(256)
    bn_apply_cl(const T *__restrict__ x, int64_t px, const T *__restrict__ z, int64_t pz, T *__restrict__ y, int64_t py,
                const float *__restrict__ s, const float *__restrict__ b, const float *__restrict__ m,
                const float *__restrict__ v, const float *__restrict__ ss, float eps, int64_t rows, int C, int cvb_,
                int flags, uint8_t *__restrict__ mask = nullptr)
{
    // mask (VN == 8 only): one byte per row and 8-channel vector, bit j set where the stored y is > 0;
    // the backward pass of a fused add + relu layer reads it instead of y
    const int cvb = cvb_ < 0 ? -cvb_ : cvb_;
    const int tx = threadIdx.x % cvb, ty = threadIdx.x / cvb, rb = 256 / cvb;
    const int c0 = (blockIdx.y * cvb + tx) * VN;
    if(c0 >= C)
        return;
    float sc[VN], sh[VN];
#pragma unroll
    for(int j = 0; j < VN; j++) {
        if(MODE == 0) {
            sc[j] = s[c0 + j] * rsqrtf(v[c0 + j] + eps);
            sh[j] = b[c0 + j] - m[c0 + j] * sc[j];
        } else {
            sc[j] = ss[c0 + j];
            sh[j] = ss[C + c0 + j];
        }
    }
    const bool relu = flags & SAGA_BN_RELU, add = flags & SAGA_BN_ADD;
    typedef Ld<T, VN> L;
    typedef typename L::V V;
    // MODE 1 runs right after the statistics pass over the same rows: walking them in the
    // opposite direction meets the rows that pass touched last, which are the ones most
    // likely to be still cached
    const RowRun rr = row_run(rows, rb, ty, cvb_);
    const int64_t stride = rr.stride;
    auto row = [&](int64_t r) { return MODE == 1 ? rows - 1 - r : r; };
    auto finish = [&](const V &xr, const V &zr, int64_t r) {
        float o[VN];
#pragma unroll
        for(int j = 0; j < VN; j++) {
            float t = __builtin_fmaf(L::at(xr, j), sc[j], sh[j]);
            if(add)
                t += L::at(zr, j);
            if(relu)
                t = (t != t) ? t : fmaxf(t, 0.0f);
            o[j] = t;
        }
        L::store(y + r * py + c0, o);
        if constexpr(VN == 8) {
            if(mask) {
                unsigned bits = 0;
#pragma unroll
                for(int j = 0; j < VN; j++)
                    bits |= ((float)(T)o[j] > 0.0f ? 1u : 0u) << j;
                __builtin_nontemporal_store((uint8_t)bits, mask + r * (C / VN) + c0 / VN); // (read again in the backward pass only)
            }
        }
    };
    int64_t r = rr.r0;
    const int64_t rend = rr.rend;
    for(; r + 3 * stride < rend; r += 4 * stride) {
        V xr[4], zr[4];
#pragma unroll
        for(int u = 0; u < 4; u++) {
            xr[u] = L::raw(x + row(r + u * stride) * px + c0);
            zr[u] = add ? L::raw(z + row(r + u * stride) * pz + c0) : xr[u];
        }
#pragma unroll
        for(int u = 0; u < 4; u++)
            finish(xr[u], zr[u], row(r + u * stride));
    }
    for(; r < rend; r += stride) {
        const V xr = L::raw(x + row(r) * px + c0);
        const V zr = add ? L::raw(z + row(r) * pz + c0) : xr;
        finish(xr, zr, row(r));
    }
}

// Pass 1 of training forward: per-block partial sums of (x-K) and (x-K)^2, K = x[row 0].
template <typename T, int VN>
__global__ void __launch_bounds__(256)
    bn_stats_cl(const T *__restrict__ x, int64_t px, float *__restrict__ partial, int64_t rows, int C, int cvb_)
{
    __shared__ float red[256 * VN * 2];
    const int cvb = cvb_ < 0 ? -cvb_ : cvb_;
    const int tx = threadIdx.x % cvb, ty = threadIdx.x / cvb, rb = 256 / cvb;
    const int c0 = (blockIdx.y * cvb + tx) * VN;
    float a0[VN], a1[VN], k[VN];
#pragma unroll
    for(int j = 0; j < VN; j++)
        a0[j] = a1[j] = 0.0f;
    if(c0 < C) {
        typedef Ld<T, VN, false> L;
        typedef typename L::V V;
        L::load(x + c0, k);
        const RowRun rr = row_run(rows, rb, ty, cvb_);
        const int64_t stride = rr.stride;
        const int64_t rend = rr.rend;
        auto add = [&](const V &xr) {
#pragma unroll
            for(int j = 0; j < VN; j++) {
                const float d = L::at(xr, j) - k[j];
                a0[j] += d;
                a1[j] += d * d;
            }
        };
        int64_t r = rr.r0;
        for(; r + 7 * stride < rend; r += 8 * stride) {
            V xr[8];
#pragma unroll
            for(int u = 0; u < 8; u++)
                xr[u] = L::raw(x + (r + u * stride) * px + c0);
#pragma unroll
            for(int u = 0; u < 8; u++)
                add(xr[u]);
        }
        for(; r < rend; r += stride)
            add(L::raw(x + r * px + c0));
    }
#pragma unroll
    for(int j = 0; j < VN; j++) {
        red[(ty * cvb + tx) * VN * 2 + j] = a0[j];
        red[(ty * cvb + tx) * VN * 2 + VN + j] = a1[j];
    }
    __syncthreads();
    if(ty == 0 && c0 < C) {
        for(int t = 1; t < rb; t++) {
#pragma unroll
            for(int j = 0; j < VN; j++) {
                a0[j] += red[(t * cvb + tx) * VN * 2 + j];
                a1[j] += red[(t * cvb + tx) * VN * 2 + VN + j];
            }
        }
        float *o = partial + ((int64_t)blockIdx.x * C + c0) * 2;
#pragma unroll
        for(int j = 0; j < VN; j++) {
            o[j * 2] = a0[j];
            o[j * 2 + 1] = a1[j];
        }
    }
}

__device__ __forceinline__ double wave_sum_f64(double v)
{
#pragma unroll
    for(int o = 32; o > 0; o >>= 1)
        v += __shfl_xor(v, o, 64);
    return v;
}

// Adds the gx per-block partial pairs of channel c over the four wavefronts of a block, in a
// fixed order.  The loads of a thread are independent: eight are issued before any is consumed,
// and with 256 threads on one channel even 2048 partials are one such batch per thread, so the
// block pays the memory latency about once (these kernels are nothing but latency).
// The totals are valid in thread 0 only.
__device__ __forceinline__ void sum_partials(const float *__restrict__ partial, int gx, int C, int c, double &s0,
                                             double &s1)
{
    typedef float float2_t __attribute__((ext_vector_type(2)));
    __shared__ double red[4][2];
    const float2_t *p = (const float2_t *)partial + c;
    const int tid = threadIdx.x;
    double a0 = 0, a1 = 0;
    int g = tid;
    for(; g + 7 * 256 < gx; g += 8 * 256) {
        float2_t v[8];
#pragma unroll
        for(int u = 0; u < 8; u++)
            v[u] = p[(int64_t)(g + u * 256) * C];
#pragma unroll
        for(int u = 0; u < 8; u++) {
            a0 += v[u][0];
            a1 += v[u][1];
        }
    }
    {
        // the remainder, again as one batch: out-of-range slots read row 0 and are not added
        float2_t v[8];
#pragma unroll
        for(int u = 0; u < 8; u++) {
            const int r = g + u * 256;
            v[u] = p[(int64_t)(r < gx ? r : 0) * C];
        }
#pragma unroll
        for(int u = 0; u < 8; u++)
            if(g + u * 256 < gx) {
                a0 += v[u][0];
                a1 += v[u][1];
            }
    }
    a0 = wave_sum_f64(a0);
    a1 = wave_sum_f64(a1);
    if((tid & 63) == 0) {
        red[tid >> 6][0] = a0;
        red[tid >> 6][1] = a1;
    }
    __syncthreads();
    s0 = red[0][0] + red[1][0] + red[2][0] + red[3][0];
    s1 = red[0][1] + red[1][1] + red[2][1] + red[3][1];
}

// Finalize: mean, biased variance, invstd, running statistics, fused scale/shift.
// One block per channel adds the per-block partials (threads stride over the blocks).
template <typename T>
__global__ void __launch_bounds__(256)
    bn_stats_finalize(const float *__restrict__ partial, int gx, const T *__restrict__ xrow0, int64_t kstride,
                      const float *__restrict__ s, const float *__restrict__ b, float *run_m, float *run_v,
                      float *save_mean, float *save_invstd, float *ss, double M, int C, float eps, float expavg)
{
    const int c = blockIdx.x;
    // parameter loads first: they overlap the partial-sum loads instead of following them
    const double k = xrow0 ? (double)(float)xrow0[c * kstride] : 0.0;
    const float sv = s[c], bv = b[c];
    const float rm_old = run_m ? run_m[c] : 0.0f, rv_old = run_v ? run_v[c] : 0.0f;
    double s0, s1;
    sum_partials(partial, gx, C, c, s0, s1);
    if(threadIdx.x != 0)
        return;
    const double dm = s0 / M;
    double var = s1 / M - dm * dm;
    if(var < 0)
        var = 0;
    const double mean = k + dm;
    const float inv = (float)(1.0 / sqrt(var + (double)eps));
    if(save_mean)
        save_mean[c] = (float)mean;
    if(save_invstd)
        save_invstd[c] = inv;
    if(run_m)
        run_m[c] = (float)((1.0 - expavg) * rm_old + expavg * mean);
    if(run_v) {
        const double unb = M > 1 ? var * M / (M - 1.0) : var;
        run_v[c] = (float)((1.0 - expavg) * rv_old + expavg * unb);
    }
    const float sc = sv * inv;
    ss[c] = sc;
    ss[C + c] = __builtin_fmaf(-(float)mean, sc, bv); // same expression as the backward mask recompute
}

// Pass 1 of backward: partial sums of dy' and dy'*(x-mean); dy' = dy masked by y>0 when fused relu.
template <typename T, int VN, bool RC>
__global__ void __launch_bounds__(256)
    bn_bwd_stats_cl(const T *__restrict__ x, int64_t px, const T *__restrict__ y, int64_t py, const T *__restrict__ dy,
                    int64_t pdy, const float *__restrict__ save_mean, float *__restrict__ partial, int64_t rows, int C,
                    int cvb_, int flags, const float *__restrict__ rs, const float *__restrict__ rb_, const float *__restrict__ rinv,
                    T *__restrict__ dz, int64_t pdz, const uint8_t *__restrict__ mask = nullptr)
{
    // mask set (VN == 8): the relu mask comes from the byte per row and channel vector that the
    // forward pass left, and y is not read
    // dz set: the masked gradient dy' is stored there on the way (it is the residual branch's
    // gradient anyway), and the second pass reads it instead of y and dy
    // rs/rb_/rinv (scale, bias, saved 1/std) set: the relu mask is recomputed from x as
    // half(fma(x, sc, sh)) > 0, exactly what the forward stored, and y is not read
    __shared__ float red[256 * VN * 2];
    const int cvb = cvb_ < 0 ? -cvb_ : cvb_;
    const int tx = threadIdx.x % cvb, ty = threadIdx.x / cvb, rb = 256 / cvb;
    const int c0 = (blockIdx.y * cvb + tx) * VN;
    const bool relu = flags & SAGA_BN_RELU;
    constexpr bool recompute = RC;
    float a0[VN], a1[VN], mean[VN], sc[VN], sh[VN];
#pragma unroll
    for(int j = 0; j < VN; j++)
        a0[j] = a1[j] = 0.0f;
    if(c0 < C) {
#pragma unroll
        for(int j = 0; j < VN; j++) {
            mean[j] = save_mean[c0 + j];
            sc[j] = recompute ? rs[c0 + j] * rinv[c0 + j] : 0.0f;
            sh[j] = recompute ? __builtin_fmaf(-mean[j], sc[j], rb_[c0 + j]) : 0.0f;
        }
        typedef Ld<T, VN, false> L;
        typedef typename L::V V;
        const RowRun rr = row_run(rows, rb, ty, cvb_);
        const int64_t stride = rr.stride;
        const int64_t rend = rr.rend;
        auto add = [&](const V &xr, const V &gr, const V &yr, unsigned mb, int64_t r) {
            float gm[VN];
#pragma unroll
            for(int j = 0; j < VN; j++) {
                float g = L::at(gr, j);
                const float yv = recompute ? (float)(T)__builtin_fmaf(L::at(xr, j), sc[j], sh[j])
                                 : mask    ? (float)((mb >> j) & 1u)
                                           : L::at(yr, j);
                if(relu && !(yv > 0.0f))
                    g = 0.0f;
                a0[j] += g;
                a1[j] += g * (L::at(xr, j) - mean[j]);
                gm[j] = g;
            }
            if(dz)
                L::store(dz + r * pdz + c0, gm);
        };
        int64_t r = rr.r0;
        const int mp = C / VN, mc = c0 / VN; // mask row pitch and this thread's byte
        for(; r + 3 * stride < rend; r += 4 * stride) {
            V xr[4], gr[4], yr[4];
            unsigned mb[4];
#pragma unroll
            for(int u = 0; u < 4; u++) {
                xr[u] = L::raw(x + (r + u * stride) * px + c0);
                gr[u] = L::raw(dy + (r + u * stride) * pdy + c0);
                yr[u] = relu && !recompute && !mask ? L::raw(y + (r + u * stride) * py + c0) : gr[u];
                mb[u] = mask ? mask[(r + u * stride) * mp + mc] : 0u;
            }
#pragma unroll
            for(int u = 0; u < 4; u++)
                add(xr[u], gr[u], yr[u], mb[u], r + u * stride);
        }
        for(; r < rend; r += stride) {
            const V xr = L::raw(x + r * px + c0), gr = L::raw(dy + r * pdy + c0);
            add(xr, gr, relu && !recompute && !mask ? L::raw(y + r * py + c0) : gr, mask ? mask[r * mp + mc] : 0u, r);
        }
    }
#pragma unroll
    for(int j = 0; j < VN; j++) {
        red[(ty * cvb + tx) * VN * 2 + j] = a0[j];
        red[(ty * cvb + tx) * VN * 2 + VN + j] = a1[j];
    }
    __syncthreads();
    if(ty == 0 && c0 < C) {
        for(int t = 1; t < rb; t++) {
#pragma unroll
            for(int j = 0; j < VN; j++) {
                a0[j] += red[(t * cvb + tx) * VN * 2 + j];
                a1[j] += red[(t * cvb + tx) * VN * 2 + VN + j];
            }
        }
        float *o = partial + ((int64_t)blockIdx.x * C + c0) * 2;
#pragma unroll
        for(int j = 0; j < VN; j++) {
            o[j * 2] = a0[j];
            o[j * 2 + 1] = a1[j];
        }
    }
}

// coef[0..C) = s*invstd ; coef[C..2C) = db/M ; coef[2C..3C) = ds*invstd/M ; writes ds, db.
// One block per channel, as above.
__global__ void __launch_bounds__(256)
    bn_bwd_finalize(const float *__restrict__ partial, int gx, const float *__restrict__ s,
                    const float *__restrict__ save_invstd, float *ds, float *db, float *coef, double M, int C,
                    float beta_p)
{
    const int c = blockIdx.x;
    const double inv = save_invstd[c];
    const float sv = s[c];
    const float ds_old = beta_p != 0.0f ? ds[c] : 0.0f, db_old = beta_p != 0.0f ? db[c] : 0.0f;
    double s0, s1;
    sum_partials(partial, gx, C, c, s0, s1);
    if(threadIdx.x != 0)
        return;
    const double dsv = s1 * inv;
    ds[c] = (float)(beta_p != 0.0f ? dsv + (double)beta_p * ds_old : dsv);
    db[c] = (float)(beta_p != 0.0f ? s0 + (double)beta_p * db_old : s0);
    coef[c] = (float)(sv * inv);
    coef[C + c] = (float)(s0 / M);
    coef[2 * C + c] = (float)(dsv * inv / M);
}

// Pass 2 of backward: dx = s*invstd*(dy' - db/M - (x-mean)*invstd*ds/M) ; dz = dy'.
template <typename T, int VN, bool RC>
__global__ void __launch_bounds__(256)
    bn_bwd_apply_cl(const T *__restrict__ x, int64_t px, const T *__restrict__ y, int64_t py, const T *__restrict__ dy,
                    int64_t pdy, T *__restrict__ dx, int64_t pdx, T *__restrict__ dz, int64_t pdz,
                    const float *__restrict__ save_mean, const float *__restrict__ coef, int64_t rows, int C, int cvb_,
                    int flags, float beta_dx, float beta_dz, const float *__restrict__ rb_)
{
    const int cvb = cvb_ < 0 ? -cvb_ : cvb_;
    const int tx = threadIdx.x % cvb, ty = threadIdx.x / cvb, rb = 256 / cvb;
    const int c0 = (blockIdx.y * cvb + tx) * VN;
    if(c0 >= C)
        return;
    const bool relu = flags & SAGA_BN_RELU;
    constexpr bool recompute = RC;
    float mean[VN], a[VN], k0[VN], k1[VN], sh[VN];
#pragma unroll
    for(int j = 0; j < VN; j++) {
        mean[j] = save_mean[c0 + j];
        a[j] = coef[c0 + j]; // s * invstd: also the forward's scale
        k0[j] = coef[C + c0 + j];
        k1[j] = coef[2 * C + c0 + j];
        sh[j] = recompute ? __builtin_fmaf(-mean[j], a[j], rb_[c0 + j]) : 0.0f;
    }
    typedef Ld<T, VN> L;
    typedef typename L::V V;
    // rows are walked backwards: the statistics pass that ran just before ended at the top
    const RowRun rr = row_run(rows, rb, ty, cvb_);
    const int64_t stride = rr.stride;
    const int64_t rend = rr.rend;
    auto row = [&](int64_t r) { return rows - 1 - r; };
    auto finish = [&](const V &xr, const V &gr, const V &yr, int64_t r) {
        float gv[VN], ov[VN], res[VN];
#pragma unroll
        for(int j = 0; j < VN; j++) {
            gv[j] = L::at(gr, j);
            const float yv = recompute ? (float)(T)__builtin_fmaf(L::at(xr, j), a[j], sh[j]) : L::at(yr, j);
            if(relu && !(yv > 0.0f))
                gv[j] = 0.0f;
        }
        if(beta_dx != 0.0f)
            L::load(dx + r * pdx + c0, ov);
#pragma unroll
        for(int j = 0; j < VN; j++) {
            const float v = a[j] * (gv[j] - k0[j] - (L::at(xr, j) - mean[j]) * k1[j]);
            res[j] = beta_dx != 0.0f ? v + beta_dx * ov[j] : v;
        }
        L::store(dx + r * pdx + c0, res);
        if(dz) {
            if(beta_dz != 0.0f) {
                L::load(dz + r * pdz + c0, ov);
#pragma unroll
                for(int j = 0; j < VN; j++)
                    gv[j] += beta_dz * ov[j];
            }
            L::store(dz + r * pdz + c0, gv);
        }
    };
    int64_t r = rr.r0;
    for(; r + 3 * stride < rend; r += 4 * stride) {
        V xr[4], gr[4], yr[4];
#pragma unroll
        for(int u = 0; u < 4; u++) {
            const int64_t q = row(r + u * stride);
            xr[u] = L::raw(x + q * px + c0);
            gr[u] = L::raw(dy + q * pdy + c0);
            yr[u] = relu && !recompute ? L::raw(y + q * py + c0) : gr[u];
        }
#pragma unroll
        for(int u = 0; u < 4; u++)
            finish(xr[u], gr[u], yr[u], row(r + u * stride));
    }
    for(; r < rend; r += stride) {
        const int64_t q = row(r);
        const V xr = L::raw(x + q * px + c0), gr = L::raw(dy + q * pdy + c0);
        finish(xr, gr, relu && !recompute ? L::raw(y + q * py + c0) : gr, q);
    }
}

// ---------------------------------------------------------------- channels-first kernels
// One block per channel; HW runs are contiguous, lanes stride along them.

template <typename T> __device__ __forceinline__ void block_sum2(float &a, float &b)
{
    __shared__ float red[2][4];
    a = wave_sum(a);
    b = wave_sum(b);
    __syncthreads();
    if((threadIdx.x & 63) == 0) {
        red[0][threadIdx.x >> 6] = a;
        red[1][threadIdx.x >> 6] = b;
    }
    __syncthreads();
    a = red[0][0] + red[0][1] + red[0][2] + red[0][3];
    b = red[1][0] + red[1][1] + red[1][2] + red[1][3];
}

template <typename T>
__global__ void __launch_bounds__(256)
    bn_stats_cf(const T *__restrict__ x, int64_t npitch, int N, int C, int64_t HW, const float *__restrict__ s,
                const float *__restrict__ b, float *run_m, float *run_v, float *save_mean, float *save_invstd,
                float *ss, float eps, float expavg)
{
    const int c = blockIdx.x;
    const float k = (float)x[(int64_t)c * HW];
    float a0 = 0, a1 = 0;
    for(int n = 0; n < N; n++) {
        const T *p = x + n * npitch + (int64_t)c * HW;
        for(int64_t i = threadIdx.x; i < HW; i += 256) {
            const float d = (float)p[i] - k;
            a0 += d;
            a1 += d * d;
        }
    }
    block_sum2<T>(a0, a1);
    if(threadIdx.x == 0) {
        const double M = (double)N * HW;
        const double dm = a0 / M;
        double var = a1 / M - dm * dm;
        if(var < 0)
            var = 0;
        const double mean = k + dm;
        const float inv = (float)(1.0 / sqrt(var + (double)eps));
        if(save_mean)
            save_mean[c] = (float)mean;
        if(save_invstd)
            save_invstd[c] = inv;
        if(run_m)
            run_m[c] = (float)((1.0 - expavg) * run_m[c] + expavg * mean);
        if(run_v) {
            const double unb = M > 1 ? var * M / (M - 1.0) : var;
            run_v[c] = (float)((1.0 - expavg) * run_v[c] + expavg * unb);
        }
        const float sc = s[c] * inv;
        ss[c] = sc;
        ss[C + c] = b[c] - (float)mean * sc;
    }
}

template <typename T, int MODE>
__global__ void __launch_bounds__(256)
    bn_apply_cf(const T *__restrict__ x, int64_t npx, const T *__restrict__ z, int64_t npz, T *__restrict__ y,
                int64_t npy, const float *__restrict__ s, const float *__restrict__ b, const float *__restrict__ m,
                const float *__restrict__ v, const float *__restrict__ ss, float eps, int N, int C, int64_t HW,
                int flags)
{
    const int64_t total = (int64_t)N * C * HW;
    const bool relu = flags & SAGA_BN_RELU, add = flags & SAGA_BN_ADD;
    for(int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < total; i += (int64_t)gridDim.x * blockDim.x) {
        const int64_t nc = i / HW, hw = i - nc * HW;
        const int c = (int)(nc % C);
        const int64_t n = nc / C;
        float sc, sh;
        if(MODE == 0) {
            sc = s[c] * rsqrtf(v[c] + eps);
            sh = b[c] - m[c] * sc;
        } else {
            sc = ss[c];
            sh = ss[C + c];
        }
        float o = (float)x[n * npx + (int64_t)c * HW + hw] * sc + sh;
        if(add)
            o += (float)z[n * npz + (int64_t)c * HW + hw];
        if(relu)
            o = (o != o) ? o : fmaxf(o, 0.0f);
        y[n * npy + (int64_t)c * HW + hw] = (T)o;
    }
}

template <typename T>
__global__ void __launch_bounds__(256)
    bn_bwd_cf(const T *__restrict__ x, int64_t npx, const T *__restrict__ y, int64_t npy, const T *__restrict__ dy,
              int64_t npdy, T *__restrict__ dx, int64_t npdx, T *__restrict__ dz, int64_t npdz,
              const float *__restrict__ s, const float *__restrict__ save_mean, const float *__restrict__ save_invstd,
              float *ds, float *db, int N, int C, int64_t HW, int flags, float beta_dx, float beta_dz, float beta_p)
{
    const int c = blockIdx.x;
    const bool relu = flags & SAGA_BN_RELU;
    const float mean = save_mean[c], inv = save_invstd[c];
    float a0 = 0, a1 = 0;
    for(int n = 0; n < N; n++) {
        const int64_t o = (int64_t)c * HW;
        for(int64_t i = threadIdx.x; i < HW; i += 256) {
            float g = (float)dy[n * npdy + o + i];
            if(relu && !((float)y[n * npy + o + i] > 0.0f))
                g = 0.0f;
            a0 += g;
            a1 += g * ((float)x[n * npx + o + i] - mean);
        }
    }
    block_sum2<T>(a0, a1);
    const double M = (double)N * HW;
    const float dsv = a1 * inv;
    const float a = s[c] * inv, k0 = (float)(a0 / M), k1 = (float)(dsv * inv / M);
    for(int n = 0; n < N; n++) {
        const int64_t o = (int64_t)c * HW;
        for(int64_t i = threadIdx.x; i < HW; i += 256) {
            float g = (float)dy[n * npdy + o + i];
            if(relu && !((float)y[n * npy + o + i] > 0.0f))
                g = 0.0f;
            const float v = a * (g - k0 - ((float)x[n * npx + o + i] - mean) * k1);
            T *pd = dx + n * npdx + o + i;
            *pd = (T)(beta_dx != 0.0f ? v + beta_dx * (float)*pd : v);
            if(dz) {
                T *pz = dz + n * npdz + o + i;
                *pz = (T)(beta_dz != 0.0f ? g + beta_dz * (float)*pz : g);
            }
        }
    }
    if(threadIdx.x == 0) {
        ds[c] = beta_p != 0.0f ? dsv + beta_p * ds[c] : dsv;
        db[c] = beta_p != 0.0f ? a0 + beta_p * db[c] : a0;
    }
}

// ---------------------------------------------------------------- host side

struct Views {
    bool cl;
    CLInfo lx, ly, lz, ldy, ldx, ldz;
    CFInfo fx, fy, fz, fdy, fdx, fdz;
};

static int vec_width(int dtype, int C, std::initializer_list<const SagaTensorView *> vs,
                     std::initializer_list<int64_t> pitches)
{
    const int vn = dtype == SAGA_HALF ? 8 : 4;
    if(C % vn)
        return 1;
    for(auto v : vs)
        if(v && !aligned16(v->ptr))
            return 1;
    for(auto p : pitches)
        if(p % vn)
            return 1;
    return vn;
}

// SAGA_HIP_BN_GRIDSTRIDE: bits select the kernels that walk their rows grid-strided (row_run)
// (1 forward apply, 2 forward statistics, 4 backward statistics, 8 backward apply); default: the two apply passes
static int gridstride_mask()
{
    static const int v = env_int("SAGA_HIP_BN_GRIDSTRIDE", 9);
    return v;
}
#define WALK_CVB(bit) ((gridstride_mask() & (bit)) ? -sh.cvb : sh.cvb)
#define WALK_GRID(bit) ((gridstride_mask() & (bit)) ? dim3(sh.gx, sh.gy) : dim3(sh.gxa, sh.gy))

static bool force_y_mask()
{
    static int v = -1;
    if(v < 0) {
        const char *e = getenv("SAGA_HIP_BN_MASK_FROM_Y");
        v = (e && *e && *e != '0') ? 1 : 0;
    }
    return v == 1;
}

static size_t ws_floats(int64_t rows, int C, int dtype)
{
    // partials for the widest plan (vector width 1 gives the most blocks along y) + 3*C coefficients
    size_t best = 0;
    for(int vn : {1, dtype == SAGA_HALF ? 8 : 4}) {
        if(C % vn)
            continue;
        Shape sh = plan(rows, C / vn);
        size_t need = (size_t)sh.gx * C * 2;
        if(need > best)
            best = need;
    }
    return best + 3 * (size_t)C + 64;
}

} // namespace

int bn_launch_bwd_finalize(const float *partial, int rows, const float *s, const float *save_invstd, float *ds, float *db,
                           float *coef, double M, int C, float beta_p, hipStream_t st)
{
    bn_bwd_finalize<<<C, 256, 0, st>>>(partial, rows, s, save_invstd, ds, db, coef, M, C, beta_p);
    SAGA_CHECK_LAUNCH();
    return 0;
}

extern "C" {

size_t saga_hip_bn_workspace_size(const SagaTensorView *x)
{
    if(!x)
        return 0;
    const int64_t rows = (int64_t)x->dims[0] * x->dims[2] * x->dims[3];
    return ws_floats(rows, x->dims[1], x->dtype) * sizeof(float);
}

int saga_hip_bn_infer(const SagaTensorView *x, const SagaTensorView *z, const SagaTensorView *y, const float *s,
                      const float *b, const float *m, const float *v, float eps, int flags, saga_stream_t stream)
{
    if(!valid_view(x) || !valid_view(y) || !s || !b || !m || !v)
        return SAGA_HIP_EINVAL;
    const bool add = flags & SAGA_BN_ADD;
    if(add && !valid_view(z))
        return SAGA_HIP_EINVAL;
    if(!same_dims(x, y) || (add && !same_dims(x, z)))
        return SAGA_HIP_ESHAPE;
    if(x->dtype != y->dtype || (add && z->dtype != x->dtype) || (x->dtype != SAGA_HALF && x->dtype != SAGA_FLOAT))
        return SAGA_HIP_EUNSUPPORTED;
    hipStream_t st = as_stream(stream);
    CLInfo lx, ly, lz = {};
    CFInfo fx, fy, fz = {};
    if(as_channels_last(x, &lx) && as_channels_last(y, &ly) && (!add || as_channels_last(z, &lz))) {
        const int vn = vec_width(x->dtype, lx.C, {x, y, add ? z : nullptr}, {lx.pitch, ly.pitch, add ? lz.pitch : 0});
        Shape sh = plan(lx.rows, lx.C / vn);
        dim3 grid(sh.gx, sh.gy);
#define GO(T, VN)                                                                                                 \
    bn_apply_cl<T, VN, 0><<<WALK_GRID(1), 256, 0, st>>>((const T *)x->ptr, lx.pitch, add ? (const T *)z->ptr : nullptr,      \
                                                lz.pitch, (T *)y->ptr, ly.pitch, s, b, m, v, nullptr, eps, lx.rows, \
                                                lx.C, WALK_CVB(1), flags)
        if(x->dtype == SAGA_HALF) {
            if(vn == 8) GO(half_t, 8); else GO(half_t, 1);
        } else {
            if(vn == 4) GO(float, 4); else GO(float, 1);
        }
#undef GO
    } else if(as_channels_first(x, &fx) && as_channels_first(y, &fy) && (!add || as_channels_first(z, &fz))) {
        const int64_t total = (int64_t)fx.N * fx.C * fx.HW;
        const int g = grid_for(total, 256, 256 * 32);
        if(x->dtype == SAGA_HALF)
            bn_apply_cf<half_t, 0><<<g, 256, 0, st>>>((const half_t *)x->ptr, fx.npitch,
                                                      add ? (const half_t *)z->ptr : nullptr, fz.npitch,
                                                      (half_t *)y->ptr, fy.npitch, s, b, m, v, nullptr, eps, fx.N,
                                                      fx.C, fx.HW, flags);
        else
            bn_apply_cf<float, 0><<<g, 256, 0, st>>>((const float *)x->ptr, fx.npitch,
                                                     add ? (const float *)z->ptr : nullptr, fz.npitch,
                                                     (float *)y->ptr, fy.npitch, s, b, m, v, nullptr, eps, fx.N, fx.C,
                                                     fx.HW, flags);
    } else {
        return SAGA_HIP_EUNSUPPORTED;
    }
    SAGA_CHECK_LAUNCH();
    return 0;
}

int saga_hip_bn_train_fwd(const SagaTensorView *x, const SagaTensorView *z, const SagaTensorView *y,
                          const float *s, const float *b, float *run_m, float *run_v, float *save_mean,
                          float *save_invstd, float eps, float expavg, int flags, void *workspace,
                          size_t ws_bytes, saga_stream_t stream)
{
    if(!valid_view(x) || !valid_view(y) || !s || !b)
        return SAGA_HIP_EINVAL;
    const bool add = flags & SAGA_BN_ADD;
    if(add && !valid_view(z))
        return SAGA_HIP_EINVAL;
    if(!same_dims(x, y) || (add && !same_dims(x, z)))
        return SAGA_HIP_ESHAPE;
    if(x->dtype != y->dtype || (add && z->dtype != x->dtype) || (x->dtype != SAGA_HALF && x->dtype != SAGA_FLOAT))
        return SAGA_HIP_EUNSUPPORTED;
    if(!workspace || ws_bytes < saga_hip_bn_workspace_size(x))
        return SAGA_HIP_EWORKSPACE;
    hipStream_t st = as_stream(stream);
    float *ws = (float *)workspace;
    CLInfo lx, ly, lz = {};
    CFInfo fx, fy, fz = {};
    if(as_channels_last(x, &lx) && as_channels_last(y, &ly) && (!add || as_channels_last(z, &lz))) {
        const int C = lx.C;
        const int vn = vec_width(x->dtype, C, {x, y, add ? z : nullptr}, {lx.pitch, ly.pitch, add ? lz.pitch : 0});
        Shape sh = plan(lx.rows, C / vn);
        dim3 grid(sh.gx, sh.gy);
        float *partial = ws, *ss = ws + (size_t)sh.gx * C * 2;
#define GO(T, VN)                                                                                                   \
    do {                                                                                                            \
        bn_stats_cl<T, VN><<<grid, 256, 0, st>>>((const T *)x->ptr, lx.pitch, partial, lx.rows, C, WALK_CVB(2));           \
        bn_stats_finalize<T><<<C, 256, 0, st>>>(partial, sh.gx, (const T *)x->ptr, 1, s, b, run_m,      \
                                                              run_v, save_mean, save_invstd, ss, (double)lx.rows, C, \
                                                              eps, expavg);                                         \
        bn_apply_cl<T, VN, 1><<<WALK_GRID(1), 256, 0, st>>>((const T *)x->ptr, lx.pitch, add ? (const T *)z->ptr : nullptr,   \
                                                    lz.pitch, (T *)y->ptr, ly.pitch, nullptr, nullptr, nullptr,     \
                                                    nullptr, ss, eps, lx.rows, C, WALK_CVB(1), flags);                   \
    } while(0)
        if(x->dtype == SAGA_HALF) {
            if(vn == 8) GO(half_t, 8); else GO(half_t, 1);
        } else {
            if(vn == 4) GO(float, 4); else GO(float, 1);
        }
#undef GO
    } else if(as_channels_first(x, &fx) && as_channels_first(y, &fy) && (!add || as_channels_first(z, &fz))) {
        const int C = fx.C;
        float *ss = ws;
        const int64_t total = (int64_t)fx.N * C * fx.HW;
        const int g = grid_for(total, 256, 256 * 32);
#define GO(T)                                                                                                      \
    do {                                                                                                           \
        bn_stats_cf<T><<<C, 256, 0, st>>>((const T *)x->ptr, fx.npitch, fx.N, C, fx.HW, s, b, run_m, run_v,          \
                                          save_mean, save_invstd, ss, eps, expavg);                                \
        bn_apply_cf<T, 1><<<g, 256, 0, st>>>((const T *)x->ptr, fx.npitch, add ? (const T *)z->ptr : nullptr,        \
                                             fz.npitch, (T *)y->ptr, fy.npitch, nullptr, nullptr, nullptr, nullptr, \
                                             ss, eps, fx.N, C, fx.HW, flags);                                      \
    } while(0)
        if(x->dtype == SAGA_HALF) GO(half_t); else GO(float);
#undef GO
    } else {
        return SAGA_HIP_EUNSUPPORTED;
    }
    SAGA_CHECK_LAUNCH();
    return 0;
}

int saga_hip_bn_train_fwd_partials(const SagaTensorView *x, const SagaTensorView *z, const SagaTensorView *y,
                                   const float *s, const float *b, float *run_m, float *run_v, float *save_mean,
                                   float *save_invstd, float eps, float expavg, int flags, const float *partial,
                                   int partial_rows, uint8_t *relu_mask, void *workspace, size_t ws_bytes,
                                   saga_stream_t stream)
{
    if(!valid_view(x) || (y && !valid_view(y)) || !s || !b || !partial || partial_rows < 1)
        return SAGA_HIP_EINVAL;
    if(!y) {
        // statistics only: mean, 1/std and the running statistics as usual, and scale[c], shift[c] (2*C floats)
        // into the workspace, for a consumer that applies them itself (saga_hip_maxpool_fwd_codes_bn)
        if(z || relu_mask || (x->dtype != SAGA_HALF && x->dtype != SAGA_FLOAT))
            return SAGA_HIP_EINVAL;
        const int C = x->dims[1];
        if(!workspace || ws_bytes < 2 * (size_t)C * sizeof(float))
            return SAGA_HIP_EWORKSPACE;
        const double rows = (double)x->dims[0] * x->dims[2] * x->dims[3];
        if(x->dtype == SAGA_HALF)
            bn_stats_finalize<half_t><<<C, 256, 0, as_stream(stream)>>>(partial, partial_rows, (const half_t *)nullptr, 1, s, b,
                                                                        run_m, run_v, save_mean, save_invstd,
                                                                        (float *)workspace, rows, C, eps, expavg);
        else
            bn_stats_finalize<float><<<C, 256, 0, as_stream(stream)>>>(partial, partial_rows, (const float *)nullptr, 1, s, b,
                                                                       run_m, run_v, save_mean, save_invstd,
                                                                       (float *)workspace, rows, C, eps, expavg);
        SAGA_CHECK_LAUNCH();
        return 0;
    }
    const bool add = flags & SAGA_BN_ADD;
    if(add && !valid_view(z))
        return SAGA_HIP_EINVAL;
    if(!same_dims(x, y) || (add && !same_dims(x, z)))
        return SAGA_HIP_ESHAPE;
    if(x->dtype != y->dtype || (add && z->dtype != x->dtype) || (x->dtype != SAGA_HALF && x->dtype != SAGA_FLOAT))
        return SAGA_HIP_EUNSUPPORTED;
    CLInfo lx, ly, lz = {};
    if(!as_channels_last(x, &lx) || !as_channels_last(y, &ly) || (add && !as_channels_last(z, &lz)))
        return SAGA_HIP_EUNSUPPORTED;
    const int C = lx.C;
    if(!workspace || ws_bytes < 2 * (size_t)C * sizeof(float))
        return SAGA_HIP_EWORKSPACE;
    hipStream_t st = as_stream(stream);
    float *ss = (float *)workspace;
    const int vn = vec_width(x->dtype, C, {x, y, add ? z : nullptr}, {lx.pitch, ly.pitch, add ? lz.pitch : 0});
    // the mask has one byte per 8 fp16 channels: only the 8-wide fp16 kernel with relu writes it
    if(relu_mask && !(x->dtype == SAGA_HALF && vn == 8 && (flags & SAGA_BN_RELU)))
        return SAGA_HIP_EUNSUPPORTED;
    Shape sh = plan(lx.rows, C / vn);
    dim3 grid(sh.gx, sh.gy);
#define GO(T, VN)                                                                                                   \
    do {                                                                                                            \
        bn_stats_finalize<T><<<C, 256, 0, st>>>(partial, partial_rows, (const T *)nullptr, 1, s, b, run_m, \
                                                          run_v, save_mean, save_invstd, ss, (double)lx.rows, C,    \
                                                          eps, expavg);                                             \
        bn_apply_cl<T, VN, 1><<<WALK_GRID(1), 256, 0, st>>>((const T *)x->ptr, lx.pitch, add ? (const T *)z->ptr : nullptr,   \
                                                    lz.pitch, (T *)y->ptr, ly.pitch, nullptr, nullptr, nullptr,     \
                                                    nullptr, ss, eps, lx.rows, C, WALK_CVB(1), flags, relu_mask);        \
    } while(0)
    if(x->dtype == SAGA_HALF) {
        if(vn == 8) GO(half_t, 8); else GO(half_t, 1);
    } else {
        if(vn == 4) GO(float, 4); else GO(float, 1);
    }
#undef GO
    SAGA_CHECK_LAUNCH();
    return 0;
}

int saga_hip_bn_bwd(const SagaTensorView *x, const SagaTensorView *y, const SagaTensorView *dy,
                    const SagaTensorView *dx, const SagaTensorView *dz, const float *s, const float *save_mean,
                    const float *save_invstd, float *ds, float *db, float beta_dx, float beta_dz, float beta_p,
                    int flags, void *workspace, size_t ws_bytes, saga_stream_t stream)
{
    return saga_hip_bn_bwd_ex(x, y, dy, dx, dz, s, nullptr, save_mean, save_invstd, ds, db, beta_dx, beta_dz, beta_p,
                              flags, nullptr, workspace, ws_bytes, stream);
}

int saga_hip_bn_bwd_ex(const SagaTensorView *x, const SagaTensorView *y, const SagaTensorView *dy,
                       const SagaTensorView *dx, const SagaTensorView *dz, const float *s, const float *b,
                       const float *save_mean, const float *save_invstd, float *ds, float *db, float beta_dx,
                       float beta_dz, float beta_p, int flags, const uint8_t *relu_mask, void *workspace,
                       size_t ws_bytes, saga_stream_t stream)
{
    if(!valid_view(x) || !valid_view(dy) || !valid_view(dx) || !s || !save_mean || !save_invstd || !ds || !db)
        return SAGA_HIP_EINVAL;
    bool relu = flags & SAGA_BN_RELU;
    // with the bias at hand and no residual, the relu mask is a function of x: y is not needed
    CLInfo cl_probe;
    const bool recompute = relu && b && !(flags & SAGA_BN_ADD) && !force_y_mask() && as_channels_last(x, &cl_probe) &&
                           as_channels_last(dy, &cl_probe) && as_channels_last(dx, &cl_probe);
    if(relu && !recompute && !valid_view(y))
        return SAGA_HIP_EINVAL;
    if(recompute)
        y = nullptr;
    const bool need_y = relu && !recompute;
    relu = need_y; // below, "relu" guards every use of y
    if(dz && !valid_view(dz))
        return SAGA_HIP_EINVAL;
    if(!same_dims(x, dy) || !same_dims(x, dx) || (relu && !same_dims(x, y)) || (dz && !same_dims(x, dz)))
        return SAGA_HIP_ESHAPE;
    const int dt = x->dtype;
    if((dt != SAGA_HALF && dt != SAGA_FLOAT) || dy->dtype != dt || dx->dtype != dt || (relu && y->dtype != dt) ||
       (dz && dz->dtype != dt))
        return SAGA_HIP_EUNSUPPORTED;
    if(!workspace || ws_bytes < saga_hip_bn_workspace_size(x))
        return SAGA_HIP_EWORKSPACE;
    hipStream_t st = as_stream(stream);
    float *ws = (float *)workspace;
    CLInfo lx, ly = {}, ldy, ldx, ldz = {};
    CFInfo fx, fy = {}, fdy, fdx, fdz = {};
    if(as_channels_last(x, &lx) && as_channels_last(dy, &ldy) && as_channels_last(dx, &ldx) &&
       (!relu || as_channels_last(y, &ly)) && (!dz || as_channels_last(dz, &ldz))) {
        const int C = lx.C;
        const int vn = vec_width(dt, C, {x, dy, dx, relu ? y : nullptr, dz},
                                 {lx.pitch, ldy.pitch, ldx.pitch, relu ? ly.pitch : 0, dz ? ldz.pitch : 0});
        Shape sh = plan(lx.rows, C / vn, true);
        dim3 grid(sh.gx, sh.gy);
        float *partial = ws, *coef = ws + (size_t)sh.gx * C * 2;
        // residual layers: the first pass leaves dy' in dz, the second reads it in place of y and dy
        const bool early_dz = dz && beta_dz == 0.0f && relu && !recompute && dz->ptr != dy->ptr && dz->ptr != x->ptr &&
                              dz->ptr != y->ptr;
        // the forward pass's relu mask replaces y where only the first pass needs it
        const uint8_t *mk = relu_mask && early_dz && dt == SAGA_HALF && vn == 8 ? relu_mask : nullptr;
#define GO(T, VN)                                                                                                    \
    do {                                                                                                             \
        if(recompute)                                                                                                \
            GO2(T, VN, true);                                                                                        \
        else                                                                                                         \
            GO2(T, VN, false);                                                                                       \
    } while(0)
#define GO2(T, VN, RC)                                                                                               \
    do {                                                                                                             \
        bn_bwd_stats_cl<T, VN, RC><<<grid, 256, 0, st>>>((const T *)x->ptr, lx.pitch, relu ? (const T *)y->ptr : nullptr,  \
                                                     ly.pitch, (const T *)dy->ptr, ldy.pitch, save_mean, partial,    \
                                                     lx.rows, C, WALK_CVB(4), flags, recompute ? s : nullptr,             \
                                                     recompute ? b : nullptr, recompute ? save_invstd : nullptr,     \
                                                     early_dz ? (T *)dz->ptr : nullptr, ldz.pitch, mk);              \
        bn_bwd_finalize<<<C, 256, 0, st>>>(partial, sh.gx, s, save_invstd, ds, db, coef,                \
                                                         (double)lx.rows, C, beta_p);                                \
        if(early_dz)                                                                                                 \
            bn_bwd_apply_cl<T, VN, false><<<WALK_GRID(8), 256, 0, st>>>((const T *)x->ptr, lx.pitch, nullptr, 0,              \
                                                                (const T *)dz->ptr, ldz.pitch, (T *)dx->ptr,          \
                                                                ldx.pitch, nullptr, 0, save_mean, coef, lx.rows, C,   \
                                                                WALK_CVB(8), flags & ~SAGA_BN_RELU, beta_dx, 0.0f,         \
                                                                nullptr);                                             \
        else                                                                                                         \
            bn_bwd_apply_cl<T, VN, RC><<<WALK_GRID(8), 256, 0, st>>>(                                                        \
                (const T *)x->ptr, lx.pitch, relu ? (const T *)y->ptr : nullptr, ly.pitch, (const T *)dy->ptr,       \
                ldy.pitch, (T *)dx->ptr, ldx.pitch, dz ? (T *)dz->ptr : nullptr, ldz.pitch, save_mean, coef,         \
                lx.rows, C, WALK_CVB(8), flags, beta_dx, beta_dz, recompute ? b : nullptr);                               \
    } while(0)
        if(dt == SAGA_HALF) {
            if(vn == 8) GO(half_t, 8); else GO(half_t, 1);
        } else {
            if(vn == 4) GO(float, 4); else GO(float, 1);
        }
#undef GO
#undef GO2
    } else if(!recompute && as_channels_first(x, &fx) && as_channels_first(dy, &fdy) && as_channels_first(dx, &fdx) &&
              (!relu || as_channels_first(y, &fy)) && (!dz || as_channels_first(dz, &fdz))) {
#define GO(T)                                                                                                         \
    bn_bwd_cf<T><<<fx.C, 256, 0, st>>>((const T *)x->ptr, fx.npitch, relu ? (const T *)y->ptr : nullptr, fy.npitch,     \
                                       (const T *)dy->ptr, fdy.npitch, (T *)dx->ptr, fdx.npitch,                      \
                                       dz ? (T *)dz->ptr : nullptr, fdz.npitch, s, save_mean, save_invstd, ds, db,    \
                                       fx.N, fx.C, fx.HW, flags, beta_dx, beta_dz, beta_p)
        if(dt == SAGA_HALF) GO(half_t); else GO(float);
#undef GO
    } else {
        return SAGA_HIP_EUNSUPPORTED;
    }
    SAGA_CHECK_LAUNCH();
    return 0;
}

int saga_hip_bn_bwd_linked(const SagaTensorView *x, const SagaTensorView *g, const SagaTensorView *dx, const float *s,
                           const float *save_mean, const float *save_invstd, float *ds, float *db, float beta_dx,
                           float beta_p, const float *partial, int partial_rows, void *workspace, size_t ws_bytes,
                           saga_stream_t stream)
{
    if(!valid_view(x) || !valid_view(g) || !valid_view(dx) || !s || !save_mean || !save_invstd || !ds || !db || !partial ||
       partial_rows < 1)
        return SAGA_HIP_EINVAL;
    if(!same_dims(x, g) || !same_dims(x, dx))
        return SAGA_HIP_ESHAPE;
    const int dt = x->dtype;
    if((dt != SAGA_HALF && dt != SAGA_FLOAT) || g->dtype != dt || dx->dtype != dt)
        return SAGA_HIP_EUNSUPPORTED;
    CLInfo lx, lg, ldx;
    if(!as_channels_last(x, &lx) || !as_channels_last(g, &lg) || !as_channels_last(dx, &ldx))
        return SAGA_HIP_EUNSUPPORTED;
    const int C = lx.C;
    if(!workspace || ws_bytes < 3 * (size_t)C * sizeof(float))
        return SAGA_HIP_EWORKSPACE;
    hipStream_t st = as_stream(stream);
    float *coef = (float *)workspace;
    const int vn = vec_width(dt, C, {x, g, dx}, {lx.pitch, lg.pitch, ldx.pitch});
    const Shape sh = plan(lx.rows, C / vn, true);
    const dim3 grid(sh.gx, sh.gy);
    bn_bwd_finalize<<<C, 256, 0, st>>>(partial, partial_rows, s, save_invstd, ds, db, coef, (double)lx.rows, C, beta_p);
#define GO(T, VN)                                                                                                     \
    bn_bwd_apply_cl<T, VN, false><<<WALK_GRID(8), 256, 0, st>>>((const T *)x->ptr, lx.pitch, nullptr, 0, (const T *)g->ptr,    \
                                                        lg.pitch, (T *)dx->ptr, ldx.pitch, nullptr, 0, save_mean, coef, \
                                                        lx.rows, C, WALK_CVB(8), 0, beta_dx, 0.0f, nullptr)
    if(dt == SAGA_HALF) {
        if(vn == 8) GO(half_t, 8); else GO(half_t, 1);
    } else {
        if(vn == 4) GO(float, 4); else GO(float, 1);
    }
#undef GO
    SAGA_CHECK_LAUNCH();
    return 0;
}

} // extern "C"
