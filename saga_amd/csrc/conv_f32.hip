// fp32 convolution on the matrix cores: implicit GEMM with v_mfma_f32_32x32x2_f32, for tensors of
// any 4-D strides (fp32 tensors are NCHW unless the program forces channels-last), groups == 1.
//
// Forward (reference: cudnnConvolutionForward, src/cuda/cuda_dnn.cpp:338-347) and backward data
// (:447-493) are one gather kernel: GEMM rows are the pixels of the tensor being written, GEMM
// columns its channels, the reduction runs over (channel, tap) of the tensor being read.  Backward
// filter (:399-445) reduces over pixels, split across blocks into fp32 partial tiles that a second
// kernel adds in a fixed order (no atomics).
//
// What depends on the tensors' strides is taken out of the inner loops: a table built once per call
// holds, for every reduction index (c,r,s) or (k,r,s), the element offset of that channel in the
// gathered tensor, the tap's row / column displacement, and the offset of the matching filter
// element.  fp32 matrix instructions run at 1/16 of the fp16 rate, so plain register-staged tiles
// (global -> registers -> LDS, one barrier per slice, the next slice's loads in flight during the
// MFMAs) keep them busy; none of the fp16 path's load-to-LDS pipelining is needed here.
#include "conv.hpp"

namespace {

struct KTabA {
    long long off; // generic: offset of the channel in the gathered tensor; linear: that plus the tap's displacement
    int dr, ds;    // generic: tap displacement r*dil, s*dil; linear: dr = tap number r*S + s
};

struct TabArgs {
    KTabA *ta;
    long long *tb;            // offset of the filter element, without the GEMM-column term
    int n, RS, S, dil;
    long long a_sc;           // channel stride of the gathered tensor
    long long w_s_red, w_s2, w_s3; // filter strides: reduction channel, r, s
    long long lin_sh, lin_sw; // linear form: +-dil*sH, +-dil*sW of the gathered tensor; 0,0 selects the generic form
    int linear;
};

__global__ void __launch_bounds__(256) f32_build_ktab(TabArgs a)
{
    const int k = blockIdx.x * 256 + threadIdx.x;
    if(k >= a.n)
        return;
    const int ch = k / a.RS, rs = k - ch * a.RS;
    const int r = rs / a.S, s = rs - r * a.S;
    KTabA t;
    if(a.linear) {
        t.off = ch * a.a_sc + r * a.lin_sh + s * a.lin_sw;
        t.dr = rs;
        t.ds = 0;
    } else {
        t.off = ch * a.a_sc;
        t.dr = r * a.dil;
        t.ds = s * a.dil;
    }
    a.ta[k] = t;
    a.tb[k] = ch * a.w_s_red + r * a.w_s2 + s * a.w_s3;
}

struct GatherF32 {
    const float *a; // fwd: x ; bwd-data: dy
    const float *b; // filter
    float *out;     // fwd: y ; bwd-data: dx
    const KTabA *ta;
    const long long *tb;
    int M, Ngemm, Kred;
    int OH, OW; // spatial dims of the tensor written
    int IH, IW; // spatial dims of the tensor gathered from
    long long a_sn, a_sh, a_sw;
    long long o_sn, o_sc, o_sh, o_sw;
    long long b_sn; // filter stride of the GEMM column (fwd: k, bwd-data: c)
    int stride, pad, dil, R, S;
    float alpha, beta;
};

typedef float float16_t __attribute__((ext_vector_type(16)));

constexpr int FBM = 128, FBK = 16, FPAD = 8;

// 256 threads = 4 wavefronts (2 x 2), each a 64 x (BN/2) part of the 128 x BN tile.  The filter is
// the MFMA's first operand, so a lane ends up with 16 channels of ONE pixel and consecutive lanes
// with consecutive pixels: contiguous stores for NCHW outputs.
// LIN (stride 1 backward, any forward, at most 64 taps): the address of a tap is linear in the
// tap's displacement, so the table holds the finished offset, and whether a tap of this thread's
// pixel lies inside the image is one bit of a mask computed once.
template <int BN, bool BWD, bool LIN>
__global__ void __launch_bounds__(256) conv_f32_gather(GatherF32 g)
{
    constexpr int TN = BN / 64;        // 32-wide column tiles per wavefront
    constexpr int BPT = BN * FBK / 256; // filter elements per thread and slice
    __shared__ float As[2][FBK][FBM + FPAD];
    __shared__ float Bs[2][FBK][BN + FPAD];

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int nblk_n = (g.Ngemm + BN - 1) / BN;
    const int bm = blockIdx.x / nblk_n, bn = blockIdx.x - bm * nblk_n;
    const int m0 = bm * FBM, n0 = bn * BN;
    const int wm = (wave >> 1) * 64, wn = (wave & 1) * (BN / 2);

    // this thread's pixel of the A tile (fixed for the whole kernel) and its two reduction rows
    const int am = tid & (FBM - 1), ak0 = tid >> 7;
    const int m = m0 + am;
    const bool m_ok = m < g.M;
    int th0, tw0;
    long long a_base;
    {
        const int mm = m_ok ? m : 0;
        const int ow = mm % g.OW, t = mm / g.OW;
        const int oh = t % g.OH, n = t / g.OH;
        a_base = n * g.a_sn;
        th0 = BWD ? oh + g.pad : oh * g.stride - g.pad;
        tw0 = BWD ? ow + g.pad : ow * g.stride - g.pad;
    }
    unsigned long long tapmask = 0;
    if(LIN) {
        a_base += th0 * g.a_sh + tw0 * g.a_sw; // may point outside the tensor: only valid taps are read
        if(m_ok)
            for(int r = 0; r < g.R; r++) {
                const int ih = BWD ? th0 - r * g.dil : th0 + r * g.dil;
                if(ih < 0 || ih >= g.IH)
                    continue;
                for(int q = 0; q < g.S; q++) {
                    const int iw = BWD ? tw0 - q * g.dil : tw0 + q * g.dil;
                    if(iw >= 0 && iw < g.IW)
                        tapmask |= 1ull << (r * g.S + q);
                }
            }
    }
    // the filter tile: this thread's reduction row is fixed, its columns step by 16
    const int bk = tid & (FBK - 1), bn0 = tid >> 4;

    // The table entries of a slice are fetched one iteration before the data they address, so that
    // the data loads never wait for a table load (two dependent trips to memory per slice otherwise).
    float ra[FBK / 2], rb[BPT];
    KTabA ea[FBK / 2];
    long long eb = 0;
    auto load_table = [&](int k0) {
#pragma unroll
        for(int j = 0; j < FBK / 2; j++) {
            const int kg = k0 + ak0 + 2 * j;
            ea[j] = g.ta[kg < g.Kred ? kg : 0];
        }
        const int kg = k0 + bk;
        eb = g.tb[kg < g.Kred ? kg : 0];
    };
    auto load_slice = [&](int k0) {
#pragma unroll
        for(int j = 0; j < FBK / 2; j++) {
            const int kg = k0 + ak0 + 2 * j;
            const KTabA e = ea[j];
            float v = 0.0f;
            if(LIN) {
                if(kg < g.Kred && ((tapmask >> e.dr) & 1))
                    v = g.a[a_base + e.off];
            } else if(m_ok && kg < g.Kred) {
                int ih, iw;
                bool ok;
                if(BWD) {
                    const int th = th0 - e.dr, tw = tw0 - e.ds;
                    ih = th / g.stride;
                    iw = tw / g.stride;
                    ok = th >= 0 && tw >= 0 && ih * g.stride == th && iw * g.stride == tw && ih < g.IH && iw < g.IW;
                } else {
                    ih = th0 + e.dr;
                    iw = tw0 + e.ds;
                    ok = ih >= 0 && ih < g.IH && iw >= 0 && iw < g.IW;
                }
                if(ok)
                    v = g.a[a_base + e.off + ih * g.a_sh + iw * g.a_sw];
            }
            ra[j] = v;
        }
        const int kg = k0 + bk;
#pragma unroll
        for(int j = 0; j < BPT; j++) {
            const int n = n0 + bn0 + 16 * j;
            rb[j] = (kg < g.Kred && n < g.Ngemm) ? g.b[n * g.b_sn + eb] : 0.0f;
        }
    };
    auto store_slice = [&](int buf) {
#pragma unroll
        for(int j = 0; j < FBK / 2; j++)
            As[buf][ak0 + 2 * j][am] = ra[j];
#pragma unroll
        for(int j = 0; j < BPT; j++)
            Bs[buf][bk][bn0 + 16 * j] = rb[j];
    };

    float16_t acc[2][TN];
#pragma unroll
    for(int i = 0; i < 2; i++)
#pragma unroll
        for(int j = 0; j < TN; j++)
#pragma unroll
            for(int v = 0; v < 16; v++)
                acc[i][j][v] = 0.0f;

    const int KT = (g.Kred + FBK - 1) / FBK;
    load_table(0);
    load_slice(0);
    load_table(FBK);
    store_slice(0);
    __syncthreads();
    const int fr = lane & 31, fk = lane >> 5;
    for(int kt = 0; kt < KT; kt++) {
        const int buf = kt & 1;
        if(kt + 1 < KT) {
            load_slice((kt + 1) * FBK); // in flight during the MFMAs below
            load_table((kt + 2) * FBK);
        }
#pragma unroll
        for(int kk = 0; kk < FBK / 2; kk++) {
            float fa[2], fb[TN];
#pragma unroll
            for(int i = 0; i < 2; i++)
                fa[i] = As[buf][2 * kk + fk][wm + i * 32 + fr];
#pragma unroll
            for(int j = 0; j < TN; j++)
                fb[j] = Bs[buf][2 * kk + fk][wn + j * 32 + fr];
#pragma unroll
            for(int i = 0; i < 2; i++)
#pragma unroll
                for(int j = 0; j < TN; j++)
                    acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(fb[j], fa[i], acc[i][j], 0, 0, 0);
        }
        if(kt + 1 < KT)
            store_slice(buf ^ 1); // the other buffer was last read before the previous barrier
        __syncthreads();
    }

    // acc[i][j][v]: pixel wm + 32*i + lane%32, channel wn + 32*j + 8*(v/4) + 4*(lane/32) + v%4
#pragma unroll
    for(int i = 0; i < 2; i++) {
        const int mo = m0 + wm + i * 32 + fr;
        if(mo >= g.M)
            continue;
        const int ow = mo % g.OW, t = mo / g.OW;
        const int oh = t % g.OH, n = t / g.OH;
        float *op = g.out + n * g.o_sn + oh * g.o_sh + ow * g.o_sw;
#pragma unroll
        for(int j = 0; j < TN; j++)
#pragma unroll
            for(int v = 0; v < 16; v++) {
                const int c = n0 + wn + j * 32 + 8 * (v >> 2) + 4 * fk + (v & 3);
                if(c >= g.Ngemm)
                    continue;
                float val = g.alpha * acc[i][j][v];
                if(g.beta != 0.0f)
                    val += g.beta * op[c * g.o_sc];
                op[c * g.o_sc] = val;
            }
    }
}

// ---------------------------------------------------------------- backward filter

struct FilterF32 {
    const float *x, *dy;
    float *partial; // [splits][K][CRS]
    const KTabA *tab; // per column (c,r,s), generic form: off = c*sC(x), dr, ds
    int M, K, CRS;
    int P, Q, H, W;
    long long x_sn, x_sh, x_sw;
    long long dy_sn, dy_sc, dy_sh, dy_sw;
    int stride, pad;
    int tiles_k, tiles_c, m_per_split;
};

constexpr int WBM = 64, WBN = 64, WBK = 32;

// 4 wavefronts, one 32x32 tile each; reduction (pixels) in slices of 32 through LDS
__global__ void __launch_bounds__(256) conv_f32_bwd_filter(FilterF32 g)
{
    __shared__ float As[WBK][WBM + FPAD]; // [pixel][output channel]
    __shared__ float Bs[WBK][WBN + FPAD]; // [pixel][column]
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    int b = blockIdx.x;
    const int ntiles = g.tiles_k * g.tiles_c;
    const int split = b / ntiles;
    b -= split * ntiles;
    const int tk = b / g.tiles_c, tc = b - tk * g.tiles_c;
    const int k0 = tk * WBM, c0 = tc * WBN;
    const int m_begin = split * g.m_per_split;
    const int m_end = m_begin + g.m_per_split < g.M ? m_begin + g.m_per_split : g.M;
    const int wr = (wave >> 1) * 32, wc = (wave & 1) * 32;

    // loads: lanes run along the pixels (contiguous in NCHW), 8 rows / columns per thread
    const int lm = tid & 31, l0 = tid >> 5;
    KTabA cols[8];
    bool col_ok[8];
#pragma unroll
    for(int j = 0; j < 8; j++) {
        const int col = c0 + l0 + 8 * j;
        col_ok[j] = col < g.CRS;
        cols[j] = g.tab[col_ok[j] ? col : 0];
    }

    float16_t acc;
#pragma unroll
    for(int v = 0; v < 16; v++)
        acc[v] = 0.0f;
    float ra[8], rb[8];
    auto load_slice = [&](int ms) {
        const int m = ms + lm;
        const bool ok = m < m_end;
        const int mm = ok ? m : 0;
        const int q = mm % g.Q, t = mm / g.Q;
        const int p = t % g.P, n = t / g.P;
        const long long dyb = n * g.dy_sn + p * g.dy_sh + q * g.dy_sw;
        const long long xb = n * g.x_sn;
        const int ih0 = p * g.stride - g.pad, iw0 = q * g.stride - g.pad;
#pragma unroll
        for(int j = 0; j < 8; j++) {
            const int k = k0 + l0 + 8 * j;
            ra[j] = (ok && k < g.K) ? g.dy[dyb + k * g.dy_sc] : 0.0f;
            const int ih = ih0 + cols[j].dr, iw = iw0 + cols[j].ds;
            rb[j] = (ok && col_ok[j] && ih >= 0 && ih < g.H && iw >= 0 && iw < g.W)
                        ? g.x[xb + cols[j].off + ih * g.x_sh + iw * g.x_sw]
                        : 0.0f;
        }
    };
    const int fr = lane & 31, fk = lane >> 5;
    if(m_begin < m_end)
        load_slice(m_begin);
    for(int ms = m_begin; ms < m_end; ms += WBK) {
#pragma unroll
        for(int j = 0; j < 8; j++) {
            As[lm][l0 + 8 * j] = ra[j];
            Bs[lm][l0 + 8 * j] = rb[j];
        }
        __syncthreads();
        if(ms + WBK < m_end)
            load_slice(ms + WBK);
#pragma unroll
        for(int kk = 0; kk < WBK / 2; kk++) {
            const float fa = As[2 * kk + fk][wr + fr], fb = Bs[2 * kk + fk][wc + fr];
            acc = __builtin_amdgcn_mfma_f32_32x32x2f32(fa, fb, acc, 0, 0, 0);
        }
        __syncthreads();
    }
    // acc[v]: output channel wr + 8*(v/4) + 4*(lane/32) + v%4, column wc + lane%32
    float *out = g.partial + (long long)split * g.K * g.CRS;
    const int col = c0 + wc + fr;
    if(col < g.CRS) {
#pragma unroll
        for(int v = 0; v < 16; v++) {
            const int k = k0 + wr + 8 * (v >> 2) + 4 * fk + (v & 3);
            if(k < g.K)
                out[(long long)k * g.CRS + col] = acc[v];
        }
    }
}

__global__ void __launch_bounds__(256)
    conv_f32_filter_reduce(const float *__restrict__ partial, float *__restrict__ dw, const long long *__restrict__ tb, int K,
                           int CRS, int splits, long long w_sk, float alpha, float beta)
{
    const long long total = (long long)K * CRS;
    for(long long i = (long long)blockIdx.x * 256 + threadIdx.x; i < total; i += (long long)gridDim.x * 256) {
        const int k = (int)(i / CRS), col = (int)(i - (long long)k * CRS);
        float s = 0.0f;
        for(int p = 0; p < splits; p++)
            s += partial[(long long)p * total + i];
        float *o = dw + k * w_sk + tb[col];
        *o = beta != 0.0f ? alpha * s + beta * *o : alpha * s;
    }
}

// ---------------------------------------------------------------- host side

struct FilterSplit {
    int tiles_k, tiles_c, splits, m_per_split;
};

static FilterSplit plan_filter_f32(const ConvGeom &g)
{
    FilterSplit p;
    const int CRS = g.C * g.R * g.S;
    const long long M = (long long)g.N * g.P * g.Q;
    p.tiles_k = (g.K + WBM - 1) / WBM;
    p.tiles_c = (CRS + WBN - 1) / WBN;
    const int tiles = p.tiles_k * p.tiles_c;
    long long want = (2048 + tiles - 1) / tiles; // a few blocks per CU
    const long long maxs = (M + 511) / 512;      // at least 512 pixels per split
    if(want > maxs)
        want = maxs;
    if(want < 1)
        want = 1;
    long long per = (M + want - 1) / want;
    per = (per + WBK - 1) / WBK * WBK;
    p.m_per_split = (int)per;
    p.splits = (int)((M + per - 1) / per);
    return p;
}

static bool f32_ok(const SagaTensorView *a, const SagaTensorView *b, const SagaTensorView *c, const ConvGeom &g)
{
    if(a->dtype != SAGA_FLOAT || b->dtype != SAGA_FLOAT || c->dtype != SAGA_FLOAT || g.group != 1)
        return false;
    // pixel and reduction indices are 32-bit in the kernels
    const long long big = (long long)1 << 31;
    return (long long)g.N * g.H * g.W < big && (long long)g.N * g.P * g.Q < big && (long long)g.K * g.R * g.S < big &&
           (long long)g.C * g.R * g.S < big;
}

static size_t tab_bytes(int n) { return (((size_t)n * (sizeof(KTabA) + sizeof(long long))) + 255) & ~(size_t)255; }

} // namespace

size_t conv_f32_workspace(int kind, const SagaTensorView *x, const SagaTensorView *w, const SagaTensorView *y,
                          const ConvGeom &g)
{
    if(!f32_ok(x, w, y, g))
        return 0;
    if(kind == SAGA_CONV_FWD)
        return tab_bytes(g.C * g.R * g.S) + 256;
    if(kind == SAGA_CONV_BWD_DATA)
        return tab_bytes(g.K * g.R * g.S) + 256;
    const FilterSplit p = plan_filter_f32(g);
    return tab_bytes(g.C * g.R * g.S) + (size_t)p.splits * g.K * g.C * g.R * g.S * sizeof(float) + 256;
}

static int gather_launch(bool bwd, const SagaTensorView *a, const SagaTensorView *w, const SagaTensorView *out,
                         const ConvGeom &g, float alpha, float beta, void *ws, size_t ws_bytes, hipStream_t st)
{
    // forward: a = x (N,C,H,W), out = y (N,K,P,Q); backward data: a = dy (N,K,P,Q), out = dx (N,C,H,W)
    const int red_ch = bwd ? g.K : g.C;
    const int Kred = red_ch * g.R * g.S;
    if(!ws || ws_bytes < tab_bytes(Kred) || !aligned16(ws))
        return SAGA_HIP_EWORKSPACE;
    KTabA *ta = (KTabA *)ws;
    long long *tb = (long long *)(ta + Kred);
    const bool lin = (!bwd || g.stride == 1) && g.R * g.S <= 64;
    TabArgs t;
    t.ta = ta;
    t.tb = tb;
    t.n = Kred;
    t.RS = g.R * g.S;
    t.S = g.S;
    t.dil = g.dil;
    t.a_sc = a->strides[1];
    t.w_s_red = bwd ? w->strides[0] : w->strides[1];
    t.w_s2 = w->strides[2];
    t.w_s3 = w->strides[3];
    t.linear = lin;
    t.lin_sh = (bwd ? -1 : 1) * g.dil * a->strides[2];
    t.lin_sw = (bwd ? -1 : 1) * g.dil * a->strides[3];
    f32_build_ktab<<<(Kred + 255) / 256, 256, 0, st>>>(t);
    GatherF32 k;
    k.a = (const float *)a->ptr;
    k.b = (const float *)w->ptr;
    k.out = (float *)out->ptr;
    k.ta = ta;
    k.tb = tb;
    k.M = out->dims[0] * out->dims[2] * out->dims[3];
    k.Ngemm = out->dims[1];
    k.Kred = Kred;
    k.OH = out->dims[2];
    k.OW = out->dims[3];
    k.IH = a->dims[2];
    k.IW = a->dims[3];
    k.a_sn = a->strides[0];
    k.a_sh = a->strides[2];
    k.a_sw = a->strides[3];
    k.o_sn = out->strides[0];
    k.o_sc = out->strides[1];
    k.o_sh = out->strides[2];
    k.o_sw = out->strides[3];
    k.b_sn = bwd ? w->strides[1] : w->strides[0];
    k.stride = g.stride;
    k.pad = g.pad;
    k.dil = g.dil;
    k.R = g.R;
    k.S = g.S;
    k.alpha = alpha;
    k.beta = beta;
    const int bm = (k.M + FBM - 1) / FBM;
#define GO(BN, BLOCKS)                                                                  \
    do {                                                                                \
        if(bwd && lin)                                                                  \
            conv_f32_gather<BN, true, true><<<BLOCKS, 256, 0, st>>>(k);                 \
        else if(bwd)                                                                    \
            conv_f32_gather<BN, true, false><<<BLOCKS, 256, 0, st>>>(k);                \
        else if(lin)                                                                    \
            conv_f32_gather<BN, false, true><<<BLOCKS, 256, 0, st>>>(k);                \
        else                                                                            \
            conv_f32_gather<BN, false, false><<<BLOCKS, 256, 0, st>>>(k);               \
    } while(0)
    if(k.Ngemm > 64)
        GO(128, bm * ((k.Ngemm + 127) / 128));
    else
        GO(64, bm);
#undef GO
    SAGA_CHECK_LAUNCH();
    return 0;
}

int conv_f32_fwd(const SagaTensorView *x, const SagaTensorView *w, const SagaTensorView *y, const ConvGeom &g, float alpha,
                 float beta, void *ws, size_t ws_bytes, hipStream_t st)
{
    if(!f32_ok(x, w, y, g))
        return SAGA_HIP_EUNSUPPORTED;
    return gather_launch(false, x, w, y, g, alpha, beta, ws, ws_bytes, st);
}

int conv_f32_bwd_data(const SagaTensorView *dy, const SagaTensorView *w, const SagaTensorView *dx, const ConvGeom &g,
                      float alpha, float beta, void *ws, size_t ws_bytes, hipStream_t st)
{
    if(!f32_ok(dy, w, dx, g))
        return SAGA_HIP_EUNSUPPORTED;
    return gather_launch(true, dy, w, dx, g, alpha, beta, ws, ws_bytes, st);
}

int conv_f32_bwd_filter(const SagaTensorView *x, const SagaTensorView *dy, const SagaTensorView *dw, const ConvGeom &g,
                        float alpha, float beta, void *ws, size_t ws_bytes, hipStream_t st)
{
    if(!f32_ok(x, dy, dw, g))
        return SAGA_HIP_EUNSUPPORTED;
    const int CRS = g.C * g.R * g.S;
    const FilterSplit p = plan_filter_f32(g);
    const size_t need = tab_bytes(CRS) + (size_t)p.splits * g.K * CRS * sizeof(float);
    if(!ws || ws_bytes < need || !aligned16(ws))
        return SAGA_HIP_EWORKSPACE;
    KTabA *tab = (KTabA *)ws;
    long long *tb = (long long *)(tab + CRS);
    TabArgs t;
    t.ta = tab;
    t.tb = tb;
    t.n = CRS;
    t.RS = g.R * g.S;
    t.S = g.S;
    t.dil = g.dil;
    t.a_sc = x->strides[1];
    t.w_s_red = dw->strides[1];
    t.w_s2 = dw->strides[2];
    t.w_s3 = dw->strides[3];
    t.linear = 0;
    t.lin_sh = t.lin_sw = 0;
    f32_build_ktab<<<(CRS + 255) / 256, 256, 0, st>>>(t);
    FilterF32 k;
    k.x = (const float *)x->ptr;
    k.dy = (const float *)dy->ptr;
    k.partial = (float *)((char *)ws + tab_bytes(CRS));
    k.tab = tab;
    k.M = g.N * g.P * g.Q;
    k.K = g.K;
    k.CRS = CRS;
    k.P = g.P;
    k.Q = g.Q;
    k.H = g.H;
    k.W = g.W;
    k.x_sn = x->strides[0];
    k.x_sh = x->strides[2];
    k.x_sw = x->strides[3];
    k.dy_sn = dy->strides[0];
    k.dy_sc = dy->strides[1];
    k.dy_sh = dy->strides[2];
    k.dy_sw = dy->strides[3];
    k.stride = g.stride;
    k.pad = g.pad;
    k.tiles_k = p.tiles_k;
    k.tiles_c = p.tiles_c;
    k.m_per_split = p.m_per_split;
    conv_f32_bwd_filter<<<p.tiles_k * p.tiles_c * p.splits, 256, 0, st>>>(k);
    SAGA_CHECK_LAUNCH();
    const long long total = (long long)g.K * CRS;
    conv_f32_filter_reduce<<<grid_for(total, 256, 4096), 256, 0, st>>>(k.partial, (float *)dw->ptr, tb, g.K, CRS, p.splits,
                                                                     dw->strides[0], alpha, beta);
    SAGA_CHECK_LAUNCH();
    return 0;
}
