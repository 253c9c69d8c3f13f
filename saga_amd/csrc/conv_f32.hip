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

// acc[i][j][v]: pixel wm + 32*i + lane%32, channel wn + 32*j + 8*(v/4) + 4*(lane/32) + v%4
template <int TN>
__device__ __forceinline__ void f32_store_tile(const GatherF32 &g, const float16_t (&acc)[2][TN], int m0, int n0, int wm,
                                               int wn, int fr, int fk)
{
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

    f32_store_tile<TN>(g, acc, m0, n0, wm, wn, fr, fk);
}

// ---------------------------------------------------------------- gather kernel, wave-uniform addressing
//
// The same tile and data flow as conv_f32_gather<.., LIN = true>, with the address arithmetic moved off
// the vector unit (measured: the per-element 64-bit address and table handling above costs about as
// many issue cycles as the MFMAs).  The tile's loads are arranged so that every load instruction of a
// wavefront reads ONE reduction index: the table entry of that index then sits in scalar registers and the
// address is buffer base + table offset (scalar) + a 32-bit per-thread offset that is fixed for the
// whole kernel (buffer loads take exactly that triple).  Needs: the linear form (see LIN), byte offsets into the gathered tensor below 4 GB, and the
// filter copied once per call to wt[reduction index][output channel] (zero-padded to whole tiles, so the
// filter loads need neither a table nor bounds checks).

struct KTabU {
    unsigned off;           // byte offset of (channel, tap) from the buffer base (the tensor's address + minoff)
    unsigned unused;
    unsigned long long bit; // the tap's bit in the per-thread validity mask; 0 for the padding entries
};

struct UniTabArgs {
    KTabU *tu;
    float *wt;
    const float *w;
    int Kred, kpad, Ngemm, npad, RS, S;
    int tap_major, red_ch; // reduction index = tap * red_ch + channel instead of channel * RS + tap
    long long a_sc, lin_sh, lin_sw, shift; // elements; shift = bias + minoff, makes every offset non-negative
    long long w_sn, w_s_red, w_s2, w_s3;
};

__global__ void __launch_bounds__(256) f32_build_uniform(UniTabArgs a)
{
    const long long total = (long long)a.kpad * a.npad;
    for(long long i = (long long)blockIdx.x * 256 + threadIdx.x; i < total; i += (long long)gridDim.x * 256) {
        const int k = (int)(i / a.npad), n = (int)(i - (long long)k * a.npad);
        const int ch = a.tap_major ? k % a.red_ch : k / a.RS;
        const int rs = a.tap_major ? k / a.red_ch : k - ch * a.RS;
        const int r = rs / a.S, q = rs - r * a.S;
        const bool real = k < a.Kred;
        if(n == 0) {
            KTabU t;
            t.off = real ? (unsigned)((ch * a.a_sc + r * a.lin_sh + q * a.lin_sw - a.shift) * 4) : 0u;
            t.unused = 0;
            t.bit = real ? 1ull << rs : 0ull;
            a.tu[k] = t;
        }
        a.wt[i] = (real && n < a.Ngemm) ? a.w[n * a.w_sn + ch * a.w_s_red + r * a.w_s2 + q * a.w_s3] : 0.0f;
    }
}

struct GatherU32 {
    GatherF32 g;
    const KTabU *tu;
    const float *wt;
    long long minoff; // bytes, <= 0: the buffer base is the gathered tensor's address plus this
    int npad, bias;   // bias: pad for the forward pass (keeps the per-thread offset non-negative), else 0
};

#ifndef F32_UBK
#define F32_UBK 16
#endif
constexpr int UBK = F32_UBK; // reduction indices per slice of the wave-uniform kernel

// TAPU: the reduction index runs tap-major over a channel count that is a multiple of the slice depth,
// so all of a slice's indices share one tap and its validity is tested once per slice.
// A load of an invalid tap (or of a row past the end) gets an offset beyond the buffer's size and
// returns zero without touching memory.
constexpr unsigned U_RANGE = 0x80000000u;

template <int BM, int BN, bool BWD, bool TAPU>
__global__ void __launch_bounds__(256) conv_f32_gather_uniform(GatherU32 u)
{
    const GatherF32 &g = u.g;
    constexpr int WGN = 4 / (BM / 64);    // wavefronts along the channels: 2 (128 pixels) or 1 (256 pixels)
    constexpr int TN = BN / WGN / 32;     // 32-wide column tiles per wavefront
    constexpr int APT = BM * UBK / 256;   // gathered elements per thread and slice
    constexpr int AKS = 256 / BM;         // reduction rows between them
    constexpr int BPT = BN * UBK / 256; // filter elements per thread and slice
    constexpr int BKS = UBK / BPT;      // reduction rows between a thread's filter elements
    __shared__ float As[2][UBK][BM + FPAD];
    __shared__ float Bs[2][UBK][BN + FPAD];

    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int nblk_n = u.npad / BN;
    const int bm = blockIdx.x / nblk_n, bn = blockIdx.x - bm * nblk_n;
    const int m0 = bm * BM, n0 = bn * BN;
    const int wm = (wave / WGN) * 64, wn = (wave % WGN) * (BN / WGN);
    // every valid offset (scalar + per-thread) is below U_RANGE; the padded filter copy has no holes
    const __amdgpu_buffer_rsrc_t rsa =
        __builtin_amdgcn_make_buffer_rsrc((void *)((const char *)g.a + u.minoff), 0, (int)U_RANGE, 0x00020000);
    const __amdgpu_buffer_rsrc_t rsb = __builtin_amdgcn_make_buffer_rsrc((void *)u.wt, 0, (int)U_RANGE, 0x00020000);

    // A tile: this thread's pixel, reduction rows ak0, ak0 + AKS, ... (ak0 is the same for a whole wavefront)
    const int am = tid & (BM - 1), ak0 = BM == 256 ? 0 : wave >> 1;
    const int m = m0 + am;
    unsigned toff = 0;
    unsigned long long tapmask = 0;
    if(m < g.M) {
        const int ow = m % g.OW, t = m / g.OW;
        const int oh = t % g.OH, n = t / g.OH;
        const int th0 = BWD ? oh + g.pad : oh * g.stride - g.pad;
        const int tw0 = BWD ? ow + g.pad : ow * g.stride - g.pad;
        toff = (unsigned)((n * g.a_sn + (th0 + u.bias) * g.a_sh + (tw0 + u.bias) * g.a_sw) * 4);
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
    // B tile: this thread's output channel, reduction rows bk0, bk0 + BKS, ... (uniform as well)
    const int bnn = tid & (BN - 1), bk0 = BN == 64 ? wave : wave >> 1;
    const unsigned boff = (unsigned)bnn * 4;

    float ra[APT], rb[BPT];
    KTabU eu[APT];
    auto load_table = [&](int k0) { // k0 + UBK <= kpad always: the table has one slice of padding entries
#pragma unroll
        for(int j = 0; j < APT; j++)
            eu[j] = u.tu[k0 + ak0 + AKS * j];
    };
    auto load_slice = [&](int k0) {
        const unsigned vo0 = (tapmask & eu[0].bit) ? toff : U_RANGE;
#pragma unroll
        for(int j = 0; j < APT; j++) {
            const unsigned vo = TAPU ? vo0 : ((tapmask & eu[j].bit) ? toff : U_RANGE);
            ra[j] = __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(rsa, vo, eu[j].off, 0));
        }
#pragma unroll
        for(int j = 0; j < BPT; j++) {
            const unsigned so = (unsigned)(((k0 + bk0 + BKS * j) * u.npad + n0) * 4);
            rb[j] = __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(rsb, boff, so, 0));
        }
    };
    auto store_slice = [&](int buf) {
#pragma unroll
        for(int j = 0; j < APT; j++)
            As[buf][ak0 + AKS * j][am] = ra[j];
#pragma unroll
        for(int j = 0; j < BPT; j++)
            Bs[buf][bk0 + BKS * j][bnn] = rb[j];
    };

    float16_t acc[2][TN];
#pragma unroll
    for(int i = 0; i < 2; i++)
#pragma unroll
        for(int j = 0; j < TN; j++)
#pragma unroll
            for(int v = 0; v < 16; v++)
                acc[i][j][v] = 0.0f;

    const int KT = (g.Kred + UBK - 1) / UBK;
    load_table(0);
    load_slice(0);
    load_table(UBK);
    store_slice(0);
    __syncthreads();
    const int fr = lane & 31, fk = lane >> 5;
    for(int kt = 0; kt < KT; kt++) {
        const int buf = kt & 1;
        if(kt + 1 < KT) {
            load_slice((kt + 1) * UBK);
            if(kt + 2 < KT)
                load_table((kt + 2) * UBK);
        }
#pragma unroll
        for(int kk = 0; kk < UBK / 2; kk++) {
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
            store_slice(buf ^ 1);
        __syncthreads();
    }

    f32_store_tile<TN>(g, acc, m0, n0, wm, wn, fr, fk);
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

// ---------------------------------------------------------------- backward filter, wave-uniform addressing
//
// dw tile of 64 output channels x 128 columns per block, columns ordered tap-major (column = tap * C + c)
// with C a multiple of 32: each wavefront loads 32 consecutive columns, which share one tap, so the tap's
// validity is one test per thread and slice and every load is buffer base + scalar (channel) + per-thread
// (pixel) offset.  Slices are 64 pixels; lanes run along the pixels.  In LDS both operands are stored
// [row][pixel] and lane (fr, fk) walks the pixels fk*32 + 0..31, so that one 16-byte LDS read feeds four
// MFMAs (the order of the reduction is free as long as both operands use the same one).

constexpr int UW_K = 64, UW_C = 128, UW_P = 64, UW_PITCH = UW_P + 4;

struct FilterU32 {
    const float *x, *dy;
    float *partial; // [splits][K][CRS], columns tap-major
    int M, K, C, CRS;
    int P, Q, H, W, S;
    long long x_sn, x_sc, x_sh, x_sw;
    long long dy_sn, dy_sc, dy_sh, dy_sw;
    int stride, pad, dil;
    int tiles_k, tiles_c, m_per_split;
};

__global__ void __launch_bounds__(256) conv_f32_bwd_filter_uniform(FilterU32 g)
{
    __shared__ __attribute__((aligned(16))) float As[UW_K][UW_PITCH]; // [output channel][pixel]
    __shared__ __attribute__((aligned(16))) float Bs[UW_C][UW_PITCH]; // [column][pixel]
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    int b = blockIdx.x;
    const int ntiles = g.tiles_k * g.tiles_c;
    const int split = b / ntiles;
    b -= split * ntiles;
    const int tk = b / g.tiles_c, tc = b - tk * g.tiles_c;
    const int k0 = tk * UW_K, c0 = tc * UW_C;
    const int m_begin = split * g.m_per_split;
    const int m_end = m_begin + g.m_per_split < g.M ? m_begin + g.m_per_split : g.M;

    const __amdgpu_buffer_rsrc_t rsx = __builtin_amdgcn_make_buffer_rsrc((void *)g.x, 0, (int)U_RANGE, 0x00020000);
    const __amdgpu_buffer_rsrc_t rsy = __builtin_amdgcn_make_buffer_rsrc((void *)g.dy, 0, (int)U_RANGE, 0x00020000);

    // this wavefront's loads: output channels k0 + 16*wave + 0..15 of dy, columns c0 + 32*wave + 0..31 of x
    const int ky0 = k0 + 16 * wave;
    const int col0 = c0 + 32 * wave;
    const bool cols_ok = col0 < g.CRS;
    const int tap = cols_ok ? col0 / g.C : 0;
    const int ch0 = cols_ok ? col0 - tap * g.C : 0;
    const int tr = (tap / g.S) * g.dil, ts = (tap % g.S) * g.dil;
    const unsigned so_x0 = (unsigned)(ch0 * g.x_sc * 4), so_xs = (unsigned)(g.x_sc * 4);
    const unsigned so_y0 = (unsigned)(ky0 * g.dy_sc * 4), so_ys = (unsigned)(g.dy_sc * 4);

    float ra[16], rb[32];
    auto load_slice = [&](int ms) {
        const int m = ms + lane;
        unsigned vy = U_RANGE, vx = U_RANGE;
        if(m < m_end) {
            const int q = m % g.Q, t = m / g.Q;
            const int p = t % g.P, n = t / g.P;
            vy = (unsigned)((n * g.dy_sn + p * g.dy_sh + q * g.dy_sw) * 4);
            const int ih = p * g.stride - g.pad + tr, iw = q * g.stride - g.pad + ts;
            if(cols_ok && ih >= 0 && ih < g.H && iw >= 0 && iw < g.W)
                vx = (unsigned)((n * g.x_sn + ih * g.x_sh + iw * g.x_sw) * 4);
        }
#pragma unroll
        for(int j = 0; j < 16; j++) {
            const bool row = ky0 + j < g.K; // uniform
            ra[j] = __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(rsy, row ? vy : U_RANGE,
                                                                                  row ? so_y0 + j * so_ys : 0u, 0));
        }
#pragma unroll
        for(int j = 0; j < 32; j++)
            rb[j] = __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(rsx, vx, so_x0 + j * so_xs, 0));
    };

    float16_t acc[2];
#pragma unroll
    for(int i = 0; i < 2; i++)
#pragma unroll
        for(int v = 0; v < 16; v++)
            acc[i][v] = 0.0f;
    const int fr = lane & 31, fk = lane >> 5;
    const int wr = (wave >> 1) * 32, wc = (wave & 1) * 64;
    if(m_begin < m_end)
        load_slice(m_begin);
    for(int ms = m_begin; ms < m_end; ms += UW_P) {
#pragma unroll
        for(int j = 0; j < 16; j++)
            As[16 * wave + j][lane] = ra[j];
#pragma unroll
        for(int j = 0; j < 32; j++)
            Bs[32 * wave + j][lane] = rb[j];
        __syncthreads();
        if(ms + UW_P < m_end)
            load_slice(ms + UW_P);
#pragma unroll
        for(int kk = 0; kk < 32; kk += 4) {
            const float4_t fa = *(const float4_t *)&As[wr + fr][fk * 32 + kk];
            const float4_t fb0 = *(const float4_t *)&Bs[wc + fr][fk * 32 + kk];
            const float4_t fb1 = *(const float4_t *)&Bs[wc + 32 + fr][fk * 32 + kk];
#pragma unroll
            for(int e = 0; e < 4; e++) {
                acc[0] = __builtin_amdgcn_mfma_f32_32x32x2f32(fa[e], fb0[e], acc[0], 0, 0, 0);
                acc[1] = __builtin_amdgcn_mfma_f32_32x32x2f32(fa[e], fb1[e], acc[1], 0, 0, 0);
            }
        }
        __syncthreads();
    }
    // acc[i][v]: output channel wr + 8*(v/4) + 4*(lane/32) + v%4, column wc + 32*i + lane%32
    float *out = g.partial + (long long)split * g.K * g.CRS;
#pragma unroll
    for(int i = 0; i < 2; i++) {
        const int col = c0 + wc + 32 * i + fr;
        if(col >= g.CRS)
            continue;
#pragma unroll
        for(int v = 0; v < 16; v++) {
            const int k = k0 + wr + 8 * (v >> 2) + 4 * fk + (v & 3);
            if(k < g.K)
                out[(long long)k * g.CRS + col] = acc[i][v];
        }
    }
}

// dw[k][c][r][s] = alpha * sum_p partial[p][k][tap * C + c] + beta * dw, any filter strides
__global__ void __launch_bounds__(256)
    conv_f32_filter_reduce_tapmajor(const float *__restrict__ partial, float *__restrict__ dw, int K, int C, int S, int CRS,
                                    int splits, long long w_sk, long long w_sc, long long w_sr, long long w_ss, float alpha,
                                    float beta)
{
    const long long total = (long long)K * CRS;
    for(long long i = (long long)blockIdx.x * 256 + threadIdx.x; i < total; i += (long long)gridDim.x * 256) {
        const int k = (int)(i / CRS), col = (int)(i - (long long)k * CRS);
        const int tap = col / C, c = col - tap * C;
        float s = 0.0f;
        for(int p = 0; p < splits; p++)
            s += partial[(long long)p * total + i];
        float *o = dw + k * w_sk + c * w_sc + (tap / S) * w_sr + (tap % S) * w_ss;
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

static FilterSplit plan_filter_uniform(const ConvGeom &g)
{
    FilterSplit p;
    const int CRS = g.C * g.R * g.S;
    const long long M = (long long)g.N * g.P * g.Q;
    p.tiles_k = (g.K + UW_K - 1) / UW_K;
    p.tiles_c = (CRS + UW_C - 1) / UW_C;
    const int tiles = p.tiles_k * p.tiles_c;
    long long want = (768 + tiles - 1) / tiles; // three blocks per CU
    const long long maxs = (M + 1023) / 1024;   // at least 1024 pixels per split
    if(want > maxs)
        want = maxs;
    if(want < 1)
        want = 1;
    long long per = (M + want - 1) / want;
    per = (per + UW_P - 1) / UW_P * UW_P;
    p.m_per_split = (int)per;
    p.splits = (int)((M + per - 1) / per);
    return p;
}

static long long extent_bytes(const SagaTensorView *v)
{
    long long ext = 1;
    for(int i = 0; i < 4; i++) {
        if(v->strides[i] < 0)
            return -1;
        ext += (long long)(v->dims[i] - 1) * v->strides[i];
    }
    return ext * 4;
}

// the wave-uniform backward-filter kernel: 32 consecutive columns must share a tap, offsets fit the buffer range
static bool filter_uniform_ok(const SagaTensorView *x, const SagaTensorView *dy, const ConvGeom &g)
{
    if(getenv("SAGA_HIP_F32_NO_UNIFORM") || g.C % 32)
        return false;
    const long long ex = extent_bytes(x), ey = extent_bytes(dy);
    return ex > 0 && ey > 0 && ex + 64 < (long long)U_RANGE && ey + 64 < (long long)U_RANGE;
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

// the wave-uniform gather kernel: padded table + transposed, padded filter
struct UniPlan {
    int kpad, npad, bn, bm;
    size_t tab, bytes;
};

static UniPlan plan_uniform(int Kred, int Ngemm)
{
    UniPlan p;
    p.bn = Ngemm > 64 ? 128 : 64;
    p.bm = 128; // 256-pixel tiles (64 x 64 per wavefront) measured equal
    p.kpad = ((Kred + UBK - 1) / UBK + 1) * UBK;
    p.npad = (Ngemm + p.bn - 1) / p.bn * p.bn;
    p.tab = ((size_t)p.kpad * sizeof(KTabU) + 255) & ~(size_t)255;
    p.bytes = p.tab + (((size_t)p.kpad * p.npad * sizeof(float) + 255) & ~(size_t)255);
    return p;
}

// usable when the taps are linear in the address (see LIN), fit the 64-bit mask, and every byte offset
// the kernel forms stays below 4 GB
static bool uniform_ok(bool bwd, const SagaTensorView *a, const ConvGeom &g)
{
    if(getenv("SAGA_HIP_F32_NO_UNIFORM"))
        return false;
    if((bwd && g.stride != 1) || g.R * g.S > 64)
        return false;
    long long ext = 1;
    for(int i = 0; i < 4; i++) {
        if(a->strides[i] < 0)
            return false;
        ext += (long long)(a->dims[i] - 1) * a->strides[i];
    }
    const long long reach = (long long)(g.pad + (g.R > g.S ? g.R : g.S) * g.dil + 1) * (a->strides[2] + a->strides[3]);
    const int red = (bwd ? g.K : g.C) * g.R * g.S, cols = bwd ? g.C : g.K;
    const UniPlan up = plan_uniform(red, cols);
    return (ext + 2 * reach + 64) * 4 < (long long)U_RANGE && (long long)up.kpad * up.npad * 4 < (long long)U_RANGE;
}

} // namespace

size_t conv_f32_workspace(int kind, const SagaTensorView *x, const SagaTensorView *w, const SagaTensorView *y,
                          const ConvGeom &g)
{
    if(!f32_ok(x, w, y, g))
        return 0;
    if(kind == SAGA_CONV_FWD) {
        const size_t a = tab_bytes(g.C * g.R * g.S), b = plan_uniform(g.C * g.R * g.S, g.K).bytes;
        return (a > b ? a : b) + 256;
    }
    if(kind == SAGA_CONV_BWD_DATA) {
        const size_t a = tab_bytes(g.K * g.R * g.S), b = plan_uniform(g.K * g.R * g.S, g.C).bytes;
        return (a > b ? a : b) + 256;
    }
    const FilterSplit p = plan_filter_f32(g), pu = plan_filter_uniform(g);
    const int splits = p.splits > pu.splits ? p.splits : pu.splits;
    return tab_bytes(g.C * g.R * g.S) + (size_t)splits * g.K * g.C * g.R * g.S * sizeof(float) + 256;
}

static int gather_launch(bool bwd, const SagaTensorView *a, const SagaTensorView *w, const SagaTensorView *out,
                         const ConvGeom &g, float alpha, float beta, void *ws, size_t ws_bytes, hipStream_t st)
{
    // forward: a = x (N,C,H,W), out = y (N,K,P,Q); backward data: a = dy (N,K,P,Q), out = dx (N,C,H,W)
    const int red_ch = bwd ? g.K : g.C;
    const int Kred = red_ch * g.R * g.S;
    if(!ws || ws_bytes < tab_bytes(Kred) || !aligned16(ws))
        return SAGA_HIP_EWORKSPACE;
    if(uniform_ok(bwd, a, g)) {
        const UniPlan up = plan_uniform(Kred, out->dims[1]);
        if(ws_bytes < up.bytes)
            return SAGA_HIP_EWORKSPACE;
        const int sign = bwd ? -1 : 1, bias = bwd ? 0 : g.pad;
        UniTabArgs t;
        t.tu = (KTabU *)ws;
        t.wt = (float *)((char *)ws + up.tab);
        t.w = (const float *)w->ptr;
        t.Kred = Kred;
        t.kpad = up.kpad;
        t.Ngemm = out->dims[1];
        t.npad = up.npad;
        t.RS = g.R * g.S;
        t.S = g.S;
        t.tap_major = red_ch % UBK == 0;
        t.red_ch = red_ch;
        t.a_sc = a->strides[1];
        t.lin_sh = sign * g.dil * a->strides[2];
        t.lin_sw = sign * g.dil * a->strides[3];
        // the smallest (channel 0) table offset: forward -bias, backward the far corner of the taps
        const long long minoff = bwd ? -(long long)g.dil * ((g.R - 1) * a->strides[2] + (g.S - 1) * a->strides[3])
                                     : -(long long)bias * (a->strides[2] + a->strides[3]);
        t.shift = (long long)bias * (a->strides[2] + a->strides[3]) + minoff;
        t.w_sn = bwd ? w->strides[1] : w->strides[0];
        t.w_s_red = bwd ? w->strides[0] : w->strides[1];
        t.w_s2 = w->strides[2];
        t.w_s3 = w->strides[3];
        f32_build_uniform<<<grid_for((long long)up.kpad * up.npad, 256, 4096), 256, 0, st>>>(t);
        GatherU32 k;
        k.g.a = (const float *)a->ptr;
        k.g.b = nullptr;
        k.g.out = (float *)out->ptr;
        k.g.ta = nullptr;
        k.g.tb = nullptr;
        k.g.M = out->dims[0] * out->dims[2] * out->dims[3];
        k.g.Ngemm = out->dims[1];
        k.g.Kred = Kred;
        k.g.OH = out->dims[2];
        k.g.OW = out->dims[3];
        k.g.IH = a->dims[2];
        k.g.IW = a->dims[3];
        k.g.a_sn = a->strides[0];
        k.g.a_sh = a->strides[2];
        k.g.a_sw = a->strides[3];
        k.g.o_sn = out->strides[0];
        k.g.o_sc = out->strides[1];
        k.g.o_sh = out->strides[2];
        k.g.o_sw = out->strides[3];
        k.g.b_sn = 0;
        k.g.stride = g.stride;
        k.g.pad = g.pad;
        k.g.dil = g.dil;
        k.g.R = g.R;
        k.g.S = g.S;
        k.g.alpha = alpha;
        k.g.beta = beta;
        k.tu = t.tu;
        k.wt = t.wt;
        k.npad = up.npad;
        k.bias = bias;
        k.minoff = minoff * 4;
        const int blocks = ((k.g.M + up.bm - 1) / up.bm) * (up.npad / up.bn);
#define GOU(BM, BN, TAPU)                                                              \
    do {                                                                           \
        if(bwd)                                                                    \
            conv_f32_gather_uniform<BM, BN, true, TAPU><<<blocks, 256, 0, st>>>(k);    \
        else                                                                       \
            conv_f32_gather_uniform<BM, BN, false, TAPU><<<blocks, 256, 0, st>>>(k);   \
    } while(0)
        if(up.bn == 128) {
            if(t.tap_major) GOU(128, 128, true); else GOU(128, 128, false);
        } else {
            if(t.tap_major) GOU(128, 64, true); else GOU(128, 64, false);
        }
#undef GOU
        SAGA_CHECK_LAUNCH();
        return 0;
    }
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
    if(filter_uniform_ok(x, dy, g)) {
        const FilterSplit p = plan_filter_uniform(g);
        if(!ws || ws_bytes < (size_t)p.splits * g.K * CRS * sizeof(float) || !aligned16(ws))
            return SAGA_HIP_EWORKSPACE;
        FilterU32 k;
        k.x = (const float *)x->ptr;
        k.dy = (const float *)dy->ptr;
        k.partial = (float *)ws;
        k.M = g.N * g.P * g.Q;
        k.K = g.K;
        k.C = g.C;
        k.CRS = CRS;
        k.P = g.P;
        k.Q = g.Q;
        k.H = g.H;
        k.W = g.W;
        k.S = g.S;
        k.x_sn = x->strides[0];
        k.x_sc = x->strides[1];
        k.x_sh = x->strides[2];
        k.x_sw = x->strides[3];
        k.dy_sn = dy->strides[0];
        k.dy_sc = dy->strides[1];
        k.dy_sh = dy->strides[2];
        k.dy_sw = dy->strides[3];
        k.stride = g.stride;
        k.pad = g.pad;
        k.dil = g.dil;
        k.tiles_k = p.tiles_k;
        k.tiles_c = p.tiles_c;
        k.m_per_split = p.m_per_split;
        conv_f32_bwd_filter_uniform<<<p.tiles_k * p.tiles_c * p.splits, 256, 0, st>>>(k);
        SAGA_CHECK_LAUNCH();
        const long long total = (long long)g.K * CRS;
        conv_f32_filter_reduce_tapmajor<<<grid_for(total, 256, 4096), 256, 0, st>>>(
            k.partial, (float *)dw->ptr, g.K, g.C, g.S, CRS, p.splits, dw->strides[0], dw->strides[1], dw->strides[2],
            dw->strides[3], alpha, beta);
        SAGA_CHECK_LAUNCH();
        return 0;
    }
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
