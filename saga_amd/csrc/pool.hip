// Max / average pooling, forward and backward, for any 4-D strides.
// Channels-last tensors are processed in vectors of channels (16-byte loads, lanes on
// consecutive channel groups); everything else runs one element per lane with w fastest.
// Backward is a gather over the windows that cover each input position, so no atomics are
// needed and fp16 gradients are summed in fp32 registers.
#include "common.hpp"

namespace {

template <typename T, int VN> struct PV {
    static __device__ __forceinline__ void load(const T *p, float (&o)[VN])
    {
        if constexpr(VN == 1) {
            o[0] = (float)*p;
        } else if constexpr(sizeof(T) == 2) {
            const half8_t v = *(const half8_t *)p;
#pragma unroll
            for(int j = 0; j < VN; j++)
                o[j] = (float)v[j];
        } else {
            const float4_t v = *(const float4_t *)p;
#pragma unroll
            for(int j = 0; j < VN; j++)
                o[j] = v[j];
        }
    }
    static __device__ __forceinline__ void store(T *p, const float (&o)[VN])
    {
        if constexpr(VN == 1) {
            *p = (T)o[0];
        } else if constexpr(sizeof(T) == 2) {
            half8_t v;
#pragma unroll
            for(int j = 0; j < VN; j++)
                v[j] = (T)o[j];
            *(half8_t *)p = v;
        } else {
            float4_t v;
#pragma unroll
            for(int j = 0; j < VN; j++)
                v[j] = o[j];
            *(float4_t *)p = v;
        }
    }    // the same for data that is touched once: non-temporal
    static __device__ __forceinline__ void load_nt(const T *p, float (&o)[VN])
    {
        if constexpr(VN == 8 && sizeof(T) == 2) {
            const half8_t v = __builtin_nontemporal_load((const half8_t *)p);
#pragma unroll
            for(int j = 0; j < VN; j++)
                o[j] = (float)v[j];
        } else {
            load(p, o);
        }
    }
    static __device__ __forceinline__ void store_nt(T *p, const float (&o)[VN])
    {
        if constexpr(VN == 8 && sizeof(T) == 2) {
            half8_t v;
#pragma unroll
            for(int j = 0; j < VN; j++)
                v[j] = (T)o[j];
            __builtin_nontemporal_store(v, (half8_t *)p);
        } else {
            store(p, o);
        }
    }
};

__device__ __forceinline__ int64_t off4(const DView &v, int n, int c, int h, int w)
{
    return n * v.s[0] + c * v.s[1] + h * v.s[2] + w * v.s[3];
}

// Decodes a linear work index into (n, c0, h, w) for a tensor of dims (N, C, H, W) walked in
// vectors of VN channels; channel vectors are fastest when VN > 1, w otherwise.
template <int VN>
__device__ __forceinline__ void decode(int64_t i, int C, int H, int W, int &n, int &c, int &h, int &w)
{
    if(VN > 1) {
        const int cv = C / VN;
        c = (int)(i % cv) * VN;
        i /= cv;
        w = (int)(i % W);
        i /= W;
        h = (int)(i % H);
        n = (int)(i / H);
    } else {
        w = (int)(i % W);
        i /= W;
        h = (int)(i % H);
        i /= H;
        c = (int)(i % C);
        n = (int)(i / C);
    }
}

// v replaces best when it is larger, or when it is the first NaN: "not (v <= best)" holds for both, and a NaN
// already held is never replaced (two compares; the spelled-out form costs three and more mask logic)
__device__ __forceinline__ bool better(float v, float best) { return !(v <= best) && best == best; }
__device__ __forceinline__ bool same(float a, float b) { return a == b || (a != a && b != b); }

template <typename T, int VN, int MODE>
__global__ void __launch_bounds__(256)
    pool_fwd_k(DView x, DView y, DView idx, int has_idx, int k, int pad, int stride, int64_t total)
{
    const int C = y.d[1], P = y.d[2], Q = y.d[3], H = x.d[2], W = x.d[3];
    const float inv = 1.0f / (float)(k * k);
    for(int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < total; i += (int64_t)gridDim.x * blockDim.x) {
        int n, c, p, q;
        decode<VN>(i, C, P, Q, n, c, p, q);
        float acc[VN];
        int best[VN];
        bool first = true; // the first in-bounds position seeds the maximum for every channel
#pragma unroll
        for(int j = 0; j < VN; j++) {
            acc[j] = MODE == SAGA_POOL_MAX ? -INFINITY : 0.0f;
            best[j] = -1;
        }
        for(int r = 0; r < k; r++) {
            const int h = p * stride - pad + r;
            if(h < 0 || h >= H)
                continue;
            for(int s = 0; s < k; s++) {
                const int w = q * stride - pad + s;
                if(w < 0 || w >= W)
                    continue;
                float v[VN];
                PV<T, VN>::load((const T *)x.ptr + off4(x, n, c, h, w), v);
                const int pos = h * W + w;
#pragma unroll
                for(int j = 0; j < VN; j++) {
                    if(MODE == SAGA_POOL_MAX) {
                        const bool take = first | better(v[j], acc[j]);
                        acc[j] = take ? v[j] : acc[j];
                        best[j] = take ? pos : best[j];
                    } else {
                        acc[j] += v[j];
                    }
                }
                first = false;
            }
        }
        if(MODE == SAGA_POOL_AVG) {
#pragma unroll
            for(int j = 0; j < VN; j++)
                acc[j] *= inv;
        }
        PV<T, VN>::store((T *)y.ptr + off4(y, n, c, p, q), acc);
        if(MODE == SAGA_POOL_MAX && has_idx) {
#pragma unroll
            for(int j = 0; j < VN; j++)
                ((int32_t *)idx.ptr)[off4(idx, n, c + j, p, q)] = best[j];
        }
    }
}

// Average pooling over windows of 1024 positions or more (global pooling of a large image): one
// block per output vector, the window positions striped over its 256 threads, then a tree sum in LDS.
template <typename T, int VN>
__global__ void __launch_bounds__(256) avgpool_fwd_wide_k(DView x, DView y, int k, int pad, int stride)
{
    __shared__ float part[256][VN];
    const int C = y.d[1], P = y.d[2], Q = y.d[3], H = x.d[2], W = x.d[3];
    int n, c, p, q;
    decode<VN>(blockIdx.x, C, P, Q, n, c, p, q);
    float acc[VN];
#pragma unroll
    for(int j = 0; j < VN; j++)
        acc[j] = 0.0f;
    for(int t = threadIdx.x; t < k * k; t += 256) {
        const int h = p * stride - pad + t / k, w = q * stride - pad + t % k;
        if(h < 0 || h >= H || w < 0 || w >= W)
            continue;
        float v[VN];
        PV<T, VN>::load((const T *)x.ptr + off4(x, n, c, h, w), v);
#pragma unroll
        for(int j = 0; j < VN; j++)
            acc[j] += v[j];
    }
#pragma unroll
    for(int j = 0; j < VN; j++)
        part[threadIdx.x][j] = acc[j];
    __syncthreads();
    for(int w = 128; w > 0; w >>= 1) {
        if((int)threadIdx.x < w) {
#pragma unroll
            for(int j = 0; j < VN; j++)
                part[threadIdx.x][j] += part[threadIdx.x + w][j];
        }
        __syncthreads();
    }
    if(threadIdx.x == 0) {
        const float inv = 1.0f / (float)(k * k);
#pragma unroll
        for(int j = 0; j < VN; j++)
            acc[j] = part[0][j] * inv;
        PV<T, VN>::store((T *)y.ptr + off4(y, n, c, p, q), acc);
    }
}

static __device__ __forceinline__ int cdiv_floor(int a, int b) { return a >= 0 ? a / b : -((-a + b - 1) / b); }

template <typename T, int VN, int MODE>
__global__ void __launch_bounds__(256)
    pool_bwd_k(DView x, DView y, DView dy, DView dx, int k, int pad, int stride, float beta, int64_t total)
{
    const int C = dx.d[1], H = dx.d[2], W = dx.d[3], P = dy.d[2], Q = dy.d[3];
    const float inv = 1.0f / (float)(k * k);
    for(int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < total; i += (int64_t)gridDim.x * blockDim.x) {
        int n, c, h, w;
        decode<VN>(i, C, H, W, n, c, h, w);
        float acc[VN], xv[VN];
#pragma unroll
        for(int j = 0; j < VN; j++)
            acc[j] = 0.0f;
        if(MODE == SAGA_POOL_MAX)
            PV<T, VN>::load((const T *)x.ptr + off4(x, n, c, h, w), xv);
        int p0 = cdiv_floor(h + pad - k + stride, stride), p1 = cdiv_floor(h + pad, stride);
        int q0 = cdiv_floor(w + pad - k + stride, stride), q1 = cdiv_floor(w + pad, stride);
        if(p0 < 0) p0 = 0;
        if(q0 < 0) q0 = 0;
        if(p1 > P - 1) p1 = P - 1;
        if(q1 > Q - 1) q1 = Q - 1;
        for(int p = p0; p <= p1; p++) {
            for(int q = q0; q <= q1; q++) {
                float g[VN];
                PV<T, VN>::load((const T *)dy.ptr + off4(dy, n, c, p, q), g);
                if(MODE == SAGA_POOL_AVG) {
#pragma unroll
                    for(int j = 0; j < VN; j++)
                        acc[j] += g[j] * inv;
                    continue;
                }
                float yv[VN];
                PV<T, VN>::load((const T *)y.ptr + off4(y, n, c, p, q), yv);
                bool hit[VN];
                bool any = false;
#pragma unroll
                for(int j = 0; j < VN; j++) {
                    hit[j] = same(xv[j], yv[j]);
                    any |= hit[j];
                }
                if(!any)
                    continue;
                // the gradient goes to the FIRST position of the window that holds the maximum
                const int hs = p * stride - pad, ws = q * stride - pad;
                for(int r = 0; r < k && any; r++) {
                    const int hh = hs + r;
                    if(hh < 0 || hh >= H)
                        continue;
                    if(hh > h)
                        break;
                    for(int s = 0; s < k; s++) {
                        const int ww = ws + s;
                        if(ww < 0 || ww >= W)
                            continue;
                        if(hh == h && ww >= w)
                            break;
                        float e[VN];
                        PV<T, VN>::load((const T *)x.ptr + off4(x, n, c, hh, ww), e);
                        any = false;
#pragma unroll
                        for(int j = 0; j < VN; j++) {
                            if(hit[j] && same(e[j], yv[j]))
                                hit[j] = false;
                            any |= hit[j];
                        }
                    }
                }
#pragma unroll
                for(int j = 0; j < VN; j++)
                    if(hit[j])
                        acc[j] += g[j];
            }
        }
        T *o = (T *)dx.ptr + off4(dx, n, c, h, w);
        if(beta != 0.0f) {
            float old[VN];
            PV<T, VN>::load(o, old);
#pragma unroll
            for(int j = 0; j < VN; j++)
                acc[j] += beta * old[j];
        }
        PV<T, VN>::store(o, acc);
    }
}

// Max-pool backward for channels-last vectors, in two phases per block so that the tie-break
// (the gradient goes to the FIRST position of a window equal to its maximum) is resolved once
// per window instead of once per (input position, window):
//  1. every window that overlaps the block's TH x TW patch of input positions scans its
//     k*k inputs in order and leaves the code r*k+s of the first one equal to y (255: none)
//     in LDS, one byte per channel;
//  2. every input position sums dy over the windows that cover it and whose code names it.
// Lanes run over CVB channel vectors first, then over positions.
constexpr int POOL_TH = 16, POOL_TW = 16, POOL_CVB = 8;

template <typename T, int VN>
__global__ void __launch_bounds__(256) maxpool_bwd_tiled(DView x, DView y, DView dy, DView dx, int k, int pad,
                                                         int stride, float beta, int tiles_w, int WPmax, int WQmax)
{
    extern __shared__ __attribute__((aligned(16))) unsigned char codes[]; // [WPmax*WQmax][CVB][VN]
    const int C = dx.d[1], H = dx.d[2], W = dx.d[3], P = dy.d[2], Q = dy.d[3];
    const int tile = blockIdx.x, n = blockIdx.z;
    const int h0 = (tile / tiles_w) * POOL_TH, w0 = (tile % tiles_w) * POOL_TW;
    const int cvl = threadIdx.x % POOL_CVB, lpos = threadIdx.x / POOL_CVB;
    const int c = (blockIdx.y * POOL_CVB + cvl) * VN;
    const bool cok = c < C;
    const int h1 = min(h0 + POOL_TH, H) - 1, w1 = min(w0 + POOL_TW, W) - 1;
    const int p_lo = max(0, cdiv_floor(h0 + pad - k + stride, stride)), p_hi = min(P - 1, cdiv_floor(h1 + pad, stride));
    const int q_lo = max(0, cdiv_floor(w0 + pad - k + stride, stride)), q_hi = min(Q - 1, cdiv_floor(w1 + pad, stride));
    const int np = p_hi - p_lo + 1, nq = q_hi - q_lo + 1;

    for(int wi = lpos; wi < np * nq; wi += 256 / POOL_CVB) {
        if(!cok)
            break;
        const int p = p_lo + wi / nq, q = q_lo + wi % nq;
        float yv[VN];
        PV<T, VN>::load((const T *)y.ptr + off4(y, n, c, p, q), yv);
        int code[VN];
#pragma unroll
        for(int j = 0; j < VN; j++)
            code[j] = 255;
        const int hs = p * stride - pad, ws = q * stride - pad;
        for(int r = 0; r < k; r++) {
            const int hh = hs + r;
            if(hh < 0 || hh >= H)
                continue;
            for(int s = 0; s < k; s++) {
                const int ww = ws + s;
                if(ww < 0 || ww >= W)
                    continue;
                float e[VN];
                PV<T, VN>::load((const T *)x.ptr + off4(x, n, c, hh, ww), e);
#pragma unroll
                for(int j = 0; j < VN; j++)
                    code[j] = (code[j] == 255 && same(e[j], yv[j])) ? r * k + s : code[j];
            }
        }
        unsigned char *o = codes + ((wi / nq) * WQmax + wi % nq) * (POOL_CVB * VN) + cvl * VN;
#pragma unroll
        for(int j = 0; j < VN; j++)
            o[j] = (unsigned char)code[j];
    }
    __syncthreads();
    if(!cok)
        return;
    for(int pi = lpos; pi < POOL_TH * POOL_TW; pi += 256 / POOL_CVB) {
        const int h = h0 + pi / POOL_TW, w = w0 + pi % POOL_TW;
        if(h >= H || w >= W)
            continue;
        float acc[VN];
#pragma unroll
        for(int j = 0; j < VN; j++)
            acc[j] = 0.0f;
        const int p0 = max(p_lo, cdiv_floor(h + pad - k + stride, stride)), p1 = min(p_hi, cdiv_floor(h + pad, stride));
        const int q0 = max(q_lo, cdiv_floor(w + pad - k + stride, stride)), q1 = min(q_hi, cdiv_floor(w + pad, stride));
        for(int p = p0; p <= p1; p++) {
            for(int q = q0; q <= q1; q++) {
                float g[VN];
                PV<T, VN>::load((const T *)dy.ptr + off4(dy, n, c, p, q), g);
                const int mine = (h - (p * stride - pad)) * k + (w - (q * stride - pad));
                const unsigned char *o = codes + ((p - p_lo) * WQmax + (q - q_lo)) * (POOL_CVB * VN) + cvl * VN;
#pragma unroll
                for(int j = 0; j < VN; j++)
                    acc[j] += o[j] == mine ? g[j] : 0.0f;
            }
        }
        T *o = (T *)dx.ptr + off4(dx, n, c, h, w);
        if(beta != 0.0f) {
            float old[VN];
            PV<T, VN>::load(o, old);
#pragma unroll
            for(int j = 0; j < VN; j++)
                acc[j] += beta * old[j];
        }
        PV<T, VN>::store(o, acc);
    }
}

// ---------------------------------------------------------------- max pooling with position codes
//
// Training variant for channels-last tensors: the forward pass also leaves, per output element,
// one byte naming the window position (r*K + s) of its first maximum; the backward pass then
// needs neither x nor y - an input position receives dy of every window whose code names it.
// All loads of a thread are issued before the first is consumed (addresses of positions outside
// the image are clamped and their values ignored).

template <int VN> struct CodeVec;
template <> struct CodeVec<8> {
    typedef unsigned type __attribute__((ext_vector_type(2)));
};
template <> struct CodeVec<4> {
    typedef unsigned type;
};

// Work mapping without integer division (a thread handles 16 bytes; eight divisions by run-time
// values cost more than its memory traffic): blockIdx.z = sample, blockIdx.y = output row,
// threadIdx.x = channel vector, threadIdx.y (+ blockIdx.x) = output column.  K and the stride
// are template parameters so that the window arithmetic folds to shifts and constants.
// ss (may be null): 2*C floats scale[c], shift[c] of a batch norm whose output the pooling reads - the windows then
// hold relu(x * scale + shift) (relu when `relu` is set), rounded to T as the norm would have stored it, computed
// here from the norm's INPUT x, and the normalised tensor never exists.
template <typename T, int VN, int K, int S>
__global__ void __launch_bounds__(256) maxpool_fwd_codes_k(DView x, DView y, uint8_t *__restrict__ codes, int pad,
                                                           const float *__restrict__ ss = nullptr, int relu = 0)
{
    const int C = y.d[1], P = y.d[2], Q = y.d[3], H = x.d[2], W = x.d[3];
    const int n = blockIdx.z, p = blockIdx.y;
    const int q = blockIdx.x * blockDim.y + threadIdx.y;
    const int c = threadIdx.x * VN;
    if(q >= Q || c >= C)
        return;
    const int h0 = p * S - pad, w0 = q * S - pad;
    float v[K * K][VN];
    bool ok[K * K];
#pragma unroll
    for(int r = 0; r < K; r++)
#pragma unroll
        for(int s = 0; s < K; s++) {
            const int h = h0 + r, w = w0 + s;
            ok[r * K + s] = h >= 0 && h < H && w >= 0 && w < W;
            const int hc = h < 0 ? 0 : (h >= H ? H - 1 : h), wc = w < 0 ? 0 : (w >= W ? W - 1 : w);
            PV<T, VN>::load((const T *)x.ptr + off4(x, n, c, hc, wc), v[r * K + s]);
        }
    if(ss) {
        float sc[VN], sh[VN];
#pragma unroll
        for(int j = 0; j < VN; j++) {
            sc[j] = ss[c + j];
            sh[j] = ss[C + c + j];
        }
#pragma unroll
        for(int k = 0; k < K * K; k++)
#pragma unroll
            for(int j = 0; j < VN; j++) {
                float t = __builtin_fmaf(v[k][j], sc[j], sh[j]); // bn_apply_cl's expression
                if(relu)
                    t = (t != t) ? t : fmaxf(t, 0.0f);
                v[k][j] = (float)(T)t;
            }
    }
    float acc[VN];
    unsigned code[VN];
#pragma unroll
    for(int j = 0; j < VN; j++) {
        acc[j] = -INFINITY;
        code[j] = 0;
    }
    bool first = true; // the first position inside the image seeds the maximum of every channel
#pragma unroll
    for(int k = 0; k < K * K; k++) {
#pragma unroll
        for(int j = 0; j < VN; j++) {
            const bool take = ok[k] && (first || better(v[k][j], acc[j]));
            acc[j] = take ? v[k][j] : acc[j];
            code[j] = take ? (unsigned)k : code[j];
        }
        first = first && !ok[k];
    }
    PV<T, VN>::store((T *)y.ptr + off4(y, n, c, p, q), acc);
    typename CodeVec<VN>::type packed;
    if constexpr(VN == 8) {
        packed[0] = code[0] | code[1] << 8 | code[2] << 16 | code[3] << 24;
        packed[1] = code[4] | code[5] << 8 | code[6] << 16 | code[7] << 24;
    } else {
        packed = code[0] | code[1] << 8 | code[2] << 16 | code[3] << 24;
    }
    if(codes)
        *(typename CodeVec<VN>::type *)(codes + ((((size_t)n * P + p) * Q + q) * C + c)) = packed;
}

// The same pooling for 3x3 windows of stride 2 and padding 1 on fp16 channels-last tensors, whole image rows in LDS.
// maxpool_fwd_codes_k loads every window for itself: an input element is fetched 2.25 times (the caches serve most
// of that, but neighbouring output rows run on different dies and the rows they share come from memory twice: 618 MB
// for the 411 MB stem output of ResNet-50) and, on a batch norm's input, normalised 2.25 times; and its comparisons,
// two float compares and two selects per element and window position, make it bound by the vector ALU, not by memory
// (236 us for that tensor, 2.4 TB/s).
// Here one persistent block per CU owns strips of TR output rows of an image.  The 2 * TR + 1 input rows go to LDS
// once (buffer_load ... lds; rows above / below the image fall outside a buffer resource that covers just the image),
// the next strip's while this one is worked on.  Every element is normalised once, in place, and left there as a
// 16-bit ORDER KEY, two to a register: 0x8000 + |v| for v >= 0 and 0x7fff - |v| for v < 0, minus 0x03ff, so that
// unsigned integer order is the order of the values (-inf = 0 ... +inf = 0xf801), -0, raised to +0 before, shares
// its key (a tie, as in a float compare) and every NaN, of either sign and any payload, is the one largest key
// 0xf802 (the first NaN of a window wins, as there).  relu is max(key, key of 0).  The window maximum is then 8
// packed integer maxima per register and the position code of the FIRST maximum is min over k of
// (key_k == maximum ? k : 0xffff), also packed: 4 instructions per two elements and window position instead of
// some 20.  A position outside the image reads the window's centre row / column instead and is numbered 16 + k.
// Pooled values and codes equal maxpool_fwd_codes_k's, except that a pooled -0 comes out as +0 and a pooled NaN as
// a quiet one of positive sign.  144 us for the tensor above.
typedef __attribute__((address_space(3))) void *pool_lds_ptr_t;
typedef unsigned short pool_u16x2 __attribute__((ext_vector_type(2)));
typedef short pool_i16x2 __attribute__((ext_vector_type(2)));
typedef _Float16 pool_h2 __attribute__((ext_vector_type(2)));
typedef unsigned pool_u32x4 __attribute__((ext_vector_type(4)));
constexpr int POOL_ROWS_NT = 1024; // threads per block
constexpr int POOL_ROWS_NLD = 5;   // 16-byte chunks per lane of a strip's rows (at most 80 KB; two buffers of them)
struct PoolRowsArgs {
    const half_t *x;
    half_t *y;
    uint8_t *codes;
    const float *ss;
    int C, H, W, P, Q, CV;   // CV = C / 8 channel vectors per pixel (a power of two)
    int xs0, xs2, xs3;       // pitches of x in elements: image, row, pixel
    int64_t ys0, ys2, ys3;   // of y
    int TR, spi, nstrips;    // output rows per strip, strips per image, strips
    int chunks;              // (2 * TR + 1) * W * CV
    int relu;
    unsigned ximg_bytes;     // H * xs2 * 2
};

// (packed 16-bit integer operations as inline assembly: written as vector expressions the compiler recognises
// min(x, 1) as a comparison and falls back to one compare and one select per half)
__device__ __forceinline__ unsigned pk_max_u16(unsigned a, unsigned b)
{
    unsigned r;
    asm("v_pk_max_u16 %0, %1, %2" : "=v"(r) : "v"(a), "v"(b));
    return r;
}
__device__ __forceinline__ unsigned pk_min_u16(unsigned a, unsigned b)
{
    unsigned r;
    asm("v_pk_min_u16 %0, %1, %2" : "=v"(r) : "v"(a), "v"(b));
    return r;
}
// a * b + c per half, saturating at 0xffff
__device__ __forceinline__ unsigned pk_mad_sat_u16(unsigned a, unsigned b, unsigned c)
{
    unsigned r;
    asm("v_pk_mad_u16 %0, %1, %2, %3 clamp" : "=v"(r) : "v"(a), "v"(b), "v"(c));
    return r;
}
// a - b and a + b per half, wrapping
__device__ __forceinline__ unsigned pk_sub_u16(unsigned a, unsigned b)
{
    unsigned r;
    asm("v_pk_sub_u16 %0, %1, %2" : "=v"(r) : "v"(a), "v"(b));
    return r;
}
__device__ __forceinline__ unsigned pk_add_u16(unsigned a, unsigned b)
{
    unsigned r;
    asm("v_pk_add_u16 %0, %1, %2" : "=v"(r) : "v"(a), "v"(b));
    return r;
}
// per half: 0xffff when bit 15 is set, else 0
__device__ __forceinline__ unsigned pk_sign_u16(unsigned a)
{
    return __builtin_bit_cast(unsigned, (pool_i16x2)(__builtin_bit_cast(pool_i16x2, a) >> (pool_i16x2){15, 15}));
}

// (LDS accesses of the kernel below as inline assembly: before an LDS access of its own the compiler waits for every
// buffer_load ... lds in flight, the next strip's included)
__device__ __forceinline__ pool_u32x4 lds_read16(unsigned addr)
{
    pool_u32x4 r;
    asm volatile("ds_read_b128 %0, %1" : "=v"(r) : "v"(addr) : "memory");
    return r;
}
__device__ __forceinline__ void lds_write16(unsigned addr, pool_u32x4 v)
{
    asm volatile("ds_write_b128 %0, %1" : : "v"(addr), "v"(v) : "memory");
}

template <bool RELU>
__global__ void __launch_bounds__(POOL_ROWS_NT, 1) maxpool_3x3s2_rows_k(PoolRowsArgs t)
{
    extern __shared__ __attribute__((aligned(16))) char smem[];
    constexpr unsigned OOB = 0xffffffffu; // (beyond every image: the load writes zeros)
    constexpr int NT = POOL_ROWS_NT, NW = NT / 64;
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const unsigned lds0 = (unsigned)(uintptr_t)(pool_lds_ptr_t)smem;
    // chunk L = (q * NW + wave) * 64 + lane of a strip: channel vector L % CV of pixel (L / CV) % W of row L / CV / W
    unsigned roff[POOL_ROWS_NLD];
#pragma unroll
    for(int q = 0; q < POOL_ROWS_NLD; q++) {
        const int L = (q * NW + wave) * 64 + lane;
        const int pix = L / t.CV, cv = L - pix * t.CV;
        const int r = pix / t.W, w = pix - r * t.W;
        roff[q] = L < t.chunks ? (unsigned)((r * t.xs2 + w * t.xs3 + cv * 8) * 2) : OOB;
    }
    // two buffers of whole 1 KB pieces (one load of a wave each)
    const int buf_bytes = ((t.chunks + 63) >> 6) << 10;
    // this thread's channel vector is the same for every chunk and output it handles (the block's size is a multiple of CV)
    const int cv = tid & (t.CV - 1);
    float sc[8], sh[8];
#pragma unroll
    for(int j = 0; j < 8; j++) {
        sc[j] = t.ss ? t.ss[cv * 8 + j] : 1.0f;
        sh[j] = t.ss ? t.ss[t.C + cv * 8 + j] : 0.0f;
    }
    const unsigned floor_key = 0x7c017c01u; // relu: no key below that of +0
    const int nout = t.TR * t.Q * t.CV;
    // a strip's rows into buffer b
    auto request = [&](int strip, int b) {
        const int n = strip / t.spi;
        const int p0 = (strip - n * t.spi) * t.TR;
        const __amdgpu_buffer_rsrc_t rx =
            __builtin_amdgcn_make_buffer_rsrc((void *)(t.x + (int64_t)n * t.xs0), 0, t.ximg_bytes, 0x00020000);
        const unsigned base = (unsigned)((2 * p0 - 1) * t.xs2 * 2); // (negative for the first strip: out of range)
#pragma unroll
        for(int q = 0; q < POOL_ROWS_NLD; q++) {
            const unsigned off = roff[q] == OOB ? OOB : roff[q] + base;
            if((q * NW + wave) * 64 < t.chunks)
                __builtin_amdgcn_raw_ptr_buffer_load_lds(rx, (pool_lds_ptr_t)(smem + b * buf_bytes + (q * NW + wave) * 1024), 16, off, 0, 0, 0);
        }
    };
    // the three window columns of output column q: LDS offset within a row (the centre column's for one outside the
    // image: a duplicate changes no maximum) and 16 per half for a column outside, to number its positions 16 + k
    auto columns = [&](int q, unsigned (&col)[3], unsigned (&kcc)[3]) {
#pragma unroll
        for(int c = 0; c < 3; c++) {
            const int w = 2 * q - 1 + c;
            const bool ok = w >= 0 && w < t.W;
            col[c] = (unsigned)(((ok ? w : 2 * q) * t.CV + cv) * 16);
            kcc[c] = ok ? 0u : 0x00100010u;
        }
    };
    // output (p, q) of image n, p the strip's row pl, for this thread's 8 channels
    auto pool_one = [&](unsigned buf, int n, int p, int pl, int q, const unsigned (&col)[3], const unsigned (&kcc)[3]) {
        const unsigned row_bytes = (unsigned)(t.W * t.CV * 16);
        pool_u32x4 v[9];
        unsigned kc[9];
#pragma unroll
        for(int r = 0; r < 3; r++) {
            const int h = 2 * p - 1 + r;
            const bool okr = h >= 0 && h < t.H;
            const unsigned row = buf + (unsigned)(2 * pl + (okr ? r : 1)) * row_bytes;
            const unsigned kcr = okr ? 0u : 0x00100010u;
#pragma unroll
            for(int c = 0; c < 3; c++) {
                v[r * 3 + c] = lds_read16(row + col[c]);
                kc[r * 3 + c] = kcr | kcc[c] | (unsigned)(r * 3 + c) * 0x00010001u;
            }
        }
        asm volatile("s_waitcnt lgkmcnt(0)"
                     : "+v"(v[0]), "+v"(v[1]), "+v"(v[2]), "+v"(v[3]), "+v"(v[4]), "+v"(v[5]), "+v"(v[6]), "+v"(v[7]), "+v"(v[8])
                     :
                     : "memory");
        pool_u32x4 out;
        unsigned code[4];
#pragma unroll
        for(int i = 0; i < 4; i++) {
            unsigned m = v[0][i];
#pragma unroll
            for(int k = 1; k < 9; k++)
                m = pk_max_u16(m, v[k][i]);
            // the first position that holds the maximum: min over k of (k, or 0xffff where v[k] differs from it)
            unsigned first = 0xffffffffu;
#pragma unroll
            for(int k = 0; k < 9; k++)
                first = pk_min_u16(first, pk_mad_sat_u16(v[k][i] ^ m, 0xffffffffu, kc[k]));
            code[i] = (first & 0xffu) | (first >> 8 & 0xff00u);
            // key -> fp16 bits (0xfc01 and above: NaN, made quiet)
            unsigned ord = pk_add_u16(m, 0x03ff03ffu);
            ord |= pk_sub_u16(pk_max_u16(ord, 0xfc00fc00u), 0xfc00fc00u) << 9; // (0xfc01 at most: 0 or 1 per half)
            out[i] = ord ^ (~pk_sign_u16(ord) | 0x80008000u);
        }
        *(pool_u32x4 *)(t.y + n * t.ys0 + p * t.ys2 + q * t.ys3 + cv * 8) = out;
        if(t.codes) {
            typedef unsigned u2 __attribute__((ext_vector_type(2)));
            u2 packed;
            packed[0] = code[0] | code[1] << 16;
            packed[1] = code[2] | code[3] << 16;
            // (non-temporal: nobody reads the codes before the backward pass)
            __builtin_nontemporal_store(packed, (u2 *)(t.codes + ((((size_t)n * t.P + p) * t.Q + q) * t.C + cv * 8)));
        }
    };
    // one output per thread and strip at most (the usual case): its row, column and column offsets, once
    const bool one_pass = nout <= NT;
    const int pl1 = (tid / t.CV) / t.Q, q1 = (tid / t.CV) - pl1 * t.Q;
    unsigned col1[3], kcc1[3];
    columns(q1, col1, kcc1);
    int b = 0;
    if((int)blockIdx.x < t.nstrips)
        request(blockIdx.x, 0);
    for(int strip = blockIdx.x; strip < t.nstrips; strip += gridDim.x, b ^= 1) {
        const int n = strip / t.spi;
        const int p0 = (strip - n * t.spi) * t.TR;
        const unsigned buf = lds0 + b * buf_bytes;
        // this strip's rows have landed; every wave is done with the other buffer (and the stores of its last strip)
        asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)\n\ts_barrier" ::: "memory");
        if(strip + (int)gridDim.x < t.nstrips)
            request(strip + gridDim.x, b ^ 1);
        // values -> order keys, in place
        for(int L = tid; L < t.chunks; L += NT) {
            pool_u32x4 win = lds_read16(buf + L * 16);
            asm volatile("s_waitcnt lgkmcnt(0)" : "+v"(win) : : "memory"); // (the operand keeps the uses behind the wait)
            // bn_apply_cl's expression, fma(float(x), scale, shift) rounded to fp16 (scale 1 and shift 0 without a norm: the
            // value itself).  Not v_fma_mixlo_f16 / mixhi: they round the exact sum once, bn_apply_cl's fp32 fma and
            // conversion round twice, and the results differ in one element of some ten thousand.
            unsigned pair[4];
#pragma unroll
            for(int i = 0; i < 4; i++) {
                const unsigned wi = win[i]; // (bit_cast of the element expression itself reads element 0 for every i)
                const pool_h2 h = __builtin_bit_cast(pool_h2, wi);
                const float f0 = __builtin_fmaf((float)h[0], sc[2 * i], sh[2 * i]);
                const float f1 = __builtin_fmaf((float)h[1], sc[2 * i + 1], sh[2 * i + 1]);
                asm("v_cvt_pk_f16_f32 %0, %1, %2" : "=v"(pair[i]) : "v"(f0), "v"(f1));
            }
            unsigned key[4];
#pragma unroll
            for(int i = 0; i < 4; i++) {
                unsigned bits = pair[i];
                if constexpr(!RELU) // -0 -> +0 (with relu the floor below does it)
                    asm("v_pk_add_f16 %0, %1, 0" : "=v"(bits) : "v"(bits));
                // order of the values: 0x8000 + |v| for v >= 0, 0x7fff - |v| for v < 0; shifted down by 0x03ff (wrapping)
                // -inf becomes 0, +inf 0xf801 and every NaN, of either sign, lies above: all NaN -> 0xf802
                const unsigned ord = bits ^ (pk_sign_u16(bits) | 0x80008000u);
                key[i] = pk_min_u16(pk_sub_u16(ord, 0x03ff03ffu), 0xf802f802u);
                if constexpr(RELU)
                    key[i] = pk_max_u16(key[i], floor_key);
            }
            lds_write16(buf + L * 16, (pool_u32x4){key[0], key[1], key[2], key[3]});
        }
        asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
        if(one_pass) {
            if(tid < nout && p0 + pl1 < t.P)
                pool_one(buf, n, p0 + pl1, pl1, q1, col1, kcc1);
        } else {
            for(int o = tid; o < nout; o += NT) {
                const int pq = o / t.CV;
                const int pl = pq / t.Q, q = pq - pl * t.Q;
                if(p0 + pl >= t.P)
                    continue;
                unsigned col[3], kcc[3];
                columns(q, col, kcc);
                pool_one(buf, n, p0 + pl, pl, q, col, kcc);
            }
        }
    }
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
}

// floor(a / S) for a that may be negative, S a compile-time constant
template <int S> __device__ __forceinline__ int floor_div(int a) { return a >= 0 ? a / S : -((-a + S - 1) / S); }

// blockIdx.z = sample, blockIdx.y = input row, threadIdx.x = channel vector, threadIdx.y = input column
template <typename T, int VN, int K, int S>
__global__ void __launch_bounds__(256)
    maxpool_bwd_codes_k(const uint8_t *__restrict__ codes, DView dy, DView dx, int pad, float beta)
{
    constexpr int MAXW = (K + S - 1) / S; // the most windows that cover one input position along one axis
    const int C = dx.d[1], W = dx.d[3], P = dy.d[2], Q = dy.d[3];
    const int n = blockIdx.z, h = blockIdx.y;
    const int w = blockIdx.x * blockDim.y + threadIdx.y;
    const int c = threadIdx.x * VN;
    if(w >= W || c >= C)
        return;
    // windows p with p*S - pad <= h <= p*S - pad + K - 1
    int p0 = floor_div<S>(h + pad - K + S), p1 = floor_div<S>(h + pad);
    int q0 = floor_div<S>(w + pad - K + S), q1 = floor_div<S>(w + pad);
    p0 = p0 < 0 ? 0 : p0;
    q0 = q0 < 0 ? 0 : q0;
    p1 = p1 > P - 1 ? P - 1 : p1;
    q1 = q1 > Q - 1 ? Q - 1 : q1;
    float g[MAXW * MAXW][VN];
    typename CodeVec<VN>::type cd[MAXW * MAXW];
    bool ok[MAXW * MAXW];
    unsigned expect[MAXW * MAXW];
#pragma unroll
    for(int a = 0; a < MAXW; a++)
#pragma unroll
        for(int b = 0; b < MAXW; b++) {
            const int p = p0 + a, q = q0 + b;
            const int e = a * MAXW + b;
            ok[e] = p <= p1 && q <= q1;
            const int pc = p <= p1 ? p : p0 > p1 ? 0 : p1, qc = q <= q1 ? q : q0 > q1 ? 0 : q1;
            expect[e] = (unsigned)((h + pad - pc * S) * K + (w + pad - qc * S));
            PV<T, VN>::load((const T *)dy.ptr + off4(dy, n, c, pc, qc), g[e]);
            cd[e] = *(const typename CodeVec<VN>::type *)(codes + ((((size_t)n * P + pc) * Q + qc) * C + c));
        }
    float acc[VN];
#pragma unroll
    for(int j = 0; j < VN; j++)
        acc[j] = 0.0f;
#pragma unroll
    for(int e = 0; e < MAXW * MAXW; e++)
#pragma unroll
        for(int j = 0; j < VN; j++) {
            unsigned cj;
            if constexpr(VN == 8)
                cj = (cd[e][j >> 2] >> (8 * (j & 3))) & 255u;
            else
                cj = (cd[e] >> (8 * j)) & 255u;
            acc[j] += (ok[e] && cj == expect[e]) ? g[e][j] : 0.0f;
        }
    T *out = (T *)dx.ptr + off4(dx, n, c, h, w);
    if(beta != 0.0f) {
        float old[VN];
        PV<T, VN>::load(out, old);
#pragma unroll
        for(int j = 0; j < VN; j++)
            acc[j] += beta * old[j];
    }
    PV<T, VN>::store(out, acc);
}

// The same for 3x3 windows at stride 2, four input positions per thread.  In padded coordinates (hh = h + pad)
// window p covers rows 2p .. 2p+2, so the input rows 2a-1 and 2a are reached by the windows a-1 and a only, and
// the 2x2 patch (2a-1 .. 2a) x (2b-1 .. 2b) by the four windows (a-1 .. a) x (b-1 .. b): four gradient vectors
// and four code vectors are loaded for four results (the kernel above loads four of each per result).  Which
// window position a patch element is for each window is fixed:
//   (2a-1, 2b-1): position 4 of window (a-1, b-1)
//   (2a-1, 2b)  : 5 of (a-1, b-1), 3 of (a-1, b)
//   (2a,   2b-1): 7 of (a-1, b-1), 1 of (a, b-1)
//   (2a,   2b)  : 8 of (a-1, b-1), 6 of (a-1, b), 2 of (a, b-1), 0 of (a, b)
// blockIdx.z = sample, blockIdx.y = a, threadIdx.x = channel vector, threadIdx.y (+ blockIdx.x) = b
template <typename T, int VN>
__global__ void __launch_bounds__(256)
    maxpool_bwd_codes_3x3s2_k(const uint8_t *__restrict__ codes, DView dy, DView dx, int pad, float beta)
{
    const int C = dx.d[1], H = dx.d[2], W = dx.d[3], P = dy.d[2], Q = dy.d[3];
    const int n = blockIdx.z, a = blockIdx.y;
    const int b = blockIdx.x * blockDim.y + threadIdx.y;
    const int c = threadIdx.x * VN;
    if(c >= C || 2 * b - 1 - pad >= W)
        return;
    float g[4][VN];
    typename CodeVec<VN>::type cd[4];
    bool okw[4];
#pragma unroll
    for(int e = 0; e < 4; e++) {
        const int p = a - 1 + (e >> 1), q = b - 1 + (e & 1);
        okw[e] = p >= 0 && p < P && q >= 0 && q < Q;
        const int pc = p < 0 ? 0 : p >= P ? P - 1 : p, qc = q < 0 ? 0 : q >= Q ? Q - 1 : q;
        PV<T, VN>::load((const T *)dy.ptr + off4(dy, n, c, pc, qc), g[e]);
        cd[e] = *(const typename CodeVec<VN>::type *)(codes + ((((size_t)n * P + pc) * Q + qc) * C + c));
    }
    auto code = [&](int e, int j) -> unsigned {
        if constexpr(VN == 8)
            return (cd[e][j >> 2] >> (8 * (j & 3))) & 255u;
        else
            return (cd[e] >> (8 * j)) & 255u;
    };
    // term(e, k, j): what window e gives the position it calls k
    auto term = [&](int e, unsigned k, int j) { return (okw[e] && code(e, j) == k) ? g[e][j] : 0.0f; };
    float out[4][VN];
#pragma unroll
    for(int j = 0; j < VN; j++) {
        out[0][j] = term(0, 4, j);
        out[1][j] = term(0, 5, j) + term(1, 3, j);
        out[2][j] = term(0, 7, j) + term(2, 1, j);
        out[3][j] = term(0, 8, j) + term(1, 6, j) + term(2, 2, j) + term(3, 0, j);
    }
#pragma unroll
    for(int e = 0; e < 4; e++) {
        const int h = 2 * a - 1 + (e >> 1) - pad, w = 2 * b - 1 + (e & 1) - pad;
        if(h < 0 || h >= H || w < 0 || w >= W)
            continue;
        T *o = (T *)dx.ptr + off4(dx, n, c, h, w);
        if(beta != 0.0f) {
            float old[VN];
            PV<T, VN>::load(o, old);
#pragma unroll
            for(int j = 0; j < VN; j++)
                out[e][j] += beta * old[j];
        }
        PV<T, VN>::store(o, out[e]);
    }
}

// Backward of max pooling (3x3, stride 2, position codes) and of the batch norm (+ relu) in front of it in one:
// the pooled gradient is gathered as in maxpool_bwd_codes_3x3s2_k - a thread owns a 2x2 input patch and the four
// windows that reach it - rounded to T as the unfused pooling would have stored it, masked by the norm's relu
// (recomputed from the norm's input x as half(fma(x, sc, sh)) > 0, the forward's own expression), and goes
// straight into the norm's backward: MODE 0 leaves per block and channel the sums of g and g * (x - mean),
// MODE 1 writes dx = a * (g - k0 - (x - mean) * k1) (+ beta * dx).  The norm's output gradient never exists.
// A block walks AG consecutive patch rows, so that there are few partial rows.
// blockIdx.z = sample, blockIdx.y = group of patch rows, threadIdx.x = channel vector, threadIdx.y (+ blockIdx.x) = b
constexpr int BNPOOL_AG = 16; // patch rows per block (measured on the 112x112 stem: 1 row 579 us, 8 rows 450 us, 16 or 64 rows 430 us)
template <typename T, int VN, int MODE, int AG>
__global__ void __launch_bounds__(256)
    bn_pool_bwd_3x3s2_k(const uint8_t *__restrict__ codes, DView dp, DView x, DView dx, int pad, int na,
                        const float *__restrict__ mean_, const float *__restrict__ s_, const float *__restrict__ invstd_,
                        const float *__restrict__ b_, int relu, const float *__restrict__ coef, float *__restrict__ partial,
                        float beta)
{
    __shared__ float red[MODE == 0 ? 256 * VN * 2 : 1];
    const int C = x.d[1], H = x.d[2], W = x.d[3], P = dp.d[2], Q = dp.d[3];
    const int n = blockIdx.z;
    const int b = blockIdx.x * blockDim.y + threadIdx.y;
    const int c = threadIdx.x * VN;
    const bool live = c < C && 2 * b - 1 - pad < W;
    float mean[VN], sc[VN], sh[VN], k0[VN], k1[VN], a0[VN], a1[VN];
#pragma unroll
    for(int j = 0; j < VN; j++) {
        a0[j] = a1[j] = 0.0f;
        mean[j] = sc[j] = sh[j] = k0[j] = k1[j] = 0.0f;
        if(live) {
            mean[j] = mean_[c + j];
            sc[j] = MODE == 1 ? coef[c + j] : s_[c + j] * invstd_[c + j]; // s * invstd, also the forward's scale
            sh[j] = relu ? __builtin_fmaf(-mean[j], sc[j], b_[c + j]) : 0.0f;
            if(MODE == 1) {
                k0[j] = coef[C + c + j];
                k1[j] = coef[2 * C + c + j];
            }
        }
    }
    const int a_end = (blockIdx.y + 1) * AG < na ? (blockIdx.y + 1) * AG : na;
    if(live)
        for(int a = blockIdx.y * AG; a < a_end; a++) {
            float g[4][VN];
            typename CodeVec<VN>::type cd[4];
            bool okw[4];
#pragma unroll
            for(int e = 0; e < 4; e++) {
                const int p = a - 1 + (e >> 1), q = b - 1 + (e & 1);
                okw[e] = p >= 0 && p < P && q >= 0 && q < Q;
                const int pc = p < 0 ? 0 : p >= P ? P - 1 : p, qc = q < 0 ? 0 : q >= Q ? Q - 1 : q;
                PV<T, VN>::load((const T *)dp.ptr + off4(dp, n, c, pc, qc), g[e]);
                cd[e] = *(const typename CodeVec<VN>::type *)(codes + ((((size_t)n * P + pc) * Q + qc) * C + c));
            }
            float xv[4][VN];
            bool in[4];
#pragma unroll
            for(int e = 0; e < 4; e++) {
                const int h = 2 * a - 1 + (e >> 1) - pad, w = 2 * b - 1 + (e & 1) - pad;
                in[e] = h >= 0 && h < H && w >= 0 && w < W;
                const int hc = h < 0 ? 0 : h >= H ? H - 1 : h, wc = w < 0 ? 0 : w >= W ? W - 1 : w;
                if constexpr(MODE == 1) // (the second and last pass over x)
                    PV<T, VN>::load_nt((const T *)x.ptr + off4(x, n, c, hc, wc), xv[e]);
                else
                    PV<T, VN>::load((const T *)x.ptr + off4(x, n, c, hc, wc), xv[e]);
            }
            auto code = [&](int e, int j) -> unsigned {
                if constexpr(VN == 8)
                    return (cd[e][j >> 2] >> (8 * (j & 3))) & 255u;
                else
                    return (cd[e] >> (8 * j)) & 255u;
            };
            auto term = [&](int e, unsigned k, int j) { return (okw[e] && code(e, j) == k) ? g[e][j] : 0.0f; };
            float out[4][VN];
#pragma unroll
            for(int j = 0; j < VN; j++) {
                out[0][j] = term(0, 4, j);
                out[1][j] = term(0, 5, j) + term(1, 3, j);
                out[2][j] = term(0, 7, j) + term(2, 1, j);
                out[3][j] = term(0, 8, j) + term(1, 6, j) + term(2, 2, j) + term(3, 0, j);
            }
#pragma unroll
            for(int e = 0; e < 4; e++) {
                if(!in[e])
                    continue;
                float res[VN];
#pragma unroll
                for(int j = 0; j < VN; j++) {
                    float gv = (float)(T)out[e][j]; // as the pooling's backward would have stored it
                    if(relu && !((float)(T)__builtin_fmaf(xv[e][j], sc[j], sh[j]) > 0.0f))
                        gv = 0.0f;
                    const float xm = xv[e][j] - mean[j];
                    if(MODE == 0) {
                        a0[j] += gv;
                        a1[j] += gv * xm;
                    } else {
                        res[j] = sc[j] * (gv - k0[j] - xm * k1[j]);
                    }
                }
                if(MODE == 1) {
                    const int h = 2 * a - 1 + (e >> 1) - pad, w = 2 * b - 1 + (e & 1) - pad;
                    T *o = (T *)dx.ptr + off4(dx, n, c, h, w);
                    if(beta != 0.0f) {
                        float old[VN];
                        PV<T, VN>::load(o, old);
#pragma unroll
                        for(int j = 0; j < VN; j++)
                            res[j] += beta * old[j];
                    }
                    PV<T, VN>::store_nt(o, res);
                }
            }
        }
    if constexpr(MODE == 0) {
        // threads along y hold different columns of the same channels: add them up in a fixed order
        const int t = threadIdx.y * blockDim.x + threadIdx.x;
#pragma unroll
        for(int j = 0; j < VN; j++) {
            red[t * VN * 2 + j] = a0[j];
            red[t * VN * 2 + VN + j] = a1[j];
        }
        __syncthreads();
        if(threadIdx.y == 0 && c < C) {
            for(int ty = 1; ty < (int)blockDim.y; ty++) {
                const int u = ty * blockDim.x + threadIdx.x;
#pragma unroll
                for(int j = 0; j < VN; j++) {
                    a0[j] += red[u * VN * 2 + j];
                    a1[j] += red[u * VN * 2 + VN + j];
                }
            }
            const int64_t row = ((int64_t)blockIdx.z * gridDim.y + blockIdx.y) * gridDim.x + blockIdx.x;
            float *o = partial + (row * C + c) * 2;
#pragma unroll
            for(int j = 0; j < VN; j++) {
                o[j * 2] = a0[j];
                o[j * 2 + 1] = a1[j];
            }
        }
    }
}

static int vec_for(int dtype, std::initializer_list<const SagaTensorView *> vs)
{
    const int vn = dtype == SAGA_HALF ? 8 : 4;
    for(auto v : vs) {
        if(!v)
            continue;
        if(v->dims[1] % vn || (v->dims[1] > 1 && v->strides[1] != 1) || !aligned16(v->ptr))
            return 1;
        for(int i : {0, 2, 3})
            if(v->dims[i] > 1 && v->strides[i] % vn)
                return 1;
    }
    return vn;
}

static int pool_dim(int in, int k, int pad, int stride) { return 1 + (in + 2 * pad - k) / stride; }

} // namespace

static bool codes_ok(const SagaTensorView *a, const SagaTensorView *b, int size, int pad, int stride);
static void launch_maxpool_codes(const SagaTensorView *x, const SagaTensorView *y, uint8_t *codes, int size, int pad,
                                 int stride, hipStream_t st, const float *ss = nullptr, int relu = 0);

extern "C" {

int saga_hip_pool_fwd(int mode, const SagaTensorView *x, const SagaTensorView *y, const SagaTensorView *idx,
                      int size, int pad, int stride, saga_stream_t stream)
{
    if(!valid_view(x) || !valid_view(y) || size < 1 || stride < 1 || pad < 0 || (idx && !valid_view(idx)))
        return SAGA_HIP_EINVAL;
    if(mode != SAGA_POOL_MAX && mode != SAGA_POOL_AVG)
        return SAGA_HIP_EINVAL;
    if(y->dims[0] != x->dims[0] || y->dims[1] != x->dims[1] || y->dims[2] != pool_dim(x->dims[2], size, pad, stride) ||
       y->dims[3] != pool_dim(x->dims[3], size, pad, stride) || (idx && !same_dims(idx, y)))
        return SAGA_HIP_ESHAPE;
    if(x->dtype != y->dtype || (x->dtype != SAGA_HALF && x->dtype != SAGA_FLOAT) || (idx && idx->dtype != SAGA_I32))
        return SAGA_HIP_EUNSUPPORTED;
    const int vn = vec_for(x->dtype, {x, y});
    const int64_t total = view_elements(y) / vn;
    const int g = grid_for(total, 256, 256 * 32);
    hipStream_t st = as_stream(stream);
    // max pooling without indices over 2x2 / 3x3 windows of a channels-last tensor: the kernel of the training
    // variant, which has all loads of a window in flight at once (no division in the work mapping), without its
    // position codes (the 112x112 stem output of ResNet-50 b256: 150 -> 110 us)
    if(mode == SAGA_POOL_MAX && !idx && codes_ok(x, y, size, pad, stride)) {
        launch_maxpool_codes(x, y, nullptr, size, pad, stride, st);
        SAGA_CHECK_LAUNCH();
        return 0;
    }
    DView dvx = dview(x), dvy = dview(y), dvi = idx ? dview(idx) : dview(y);
#define GO(T, VN)                                                                                        \
    do {                                                                                                 \
        if(mode == SAGA_POOL_MAX)                                                                        \
            pool_fwd_k<T, VN, SAGA_POOL_MAX><<<g, 256, 0, st>>>(dvx, dvy, dvi, idx != nullptr, size, pad, \
                                                                stride, total);                          \
        else if(size >= 32 && total < ((int64_t)1 << 30))                                                \
            avgpool_fwd_wide_k<T, VN><<<(int)total, 256, 0, st>>>(dvx, dvy, size, pad, stride);           \
        else                                                                                             \
            pool_fwd_k<T, VN, SAGA_POOL_AVG><<<g, 256, 0, st>>>(dvx, dvy, dvi, 0, size, pad, stride, total); \
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

int saga_hip_pool_bwd(int mode, const SagaTensorView *x, const SagaTensorView *y, const SagaTensorView *dy,
                      const SagaTensorView *dx, int size, int pad, int stride, float beta, saga_stream_t stream)
{
    if(!valid_view(dy) || !valid_view(dx) || size < 1 || stride < 1 || pad < 0)
        return SAGA_HIP_EINVAL;
    if(mode != SAGA_POOL_MAX && mode != SAGA_POOL_AVG)
        return SAGA_HIP_EINVAL;
    const bool mx = mode == SAGA_POOL_MAX;
    if(mx && (!valid_view(x) || !valid_view(y)))
        return SAGA_HIP_EINVAL;
    if(dy->dims[0] != dx->dims[0] || dy->dims[1] != dx->dims[1] ||
       dy->dims[2] != pool_dim(dx->dims[2], size, pad, stride) || dy->dims[3] != pool_dim(dx->dims[3], size, pad, stride) ||
       (mx && (!same_dims(x, dx) || !same_dims(y, dy))))
        return SAGA_HIP_ESHAPE;
    const int dt = dx->dtype;
    if((dt != SAGA_HALF && dt != SAGA_FLOAT) || dy->dtype != dt || (mx && (x->dtype != dt || y->dtype != dt)))
        return SAGA_HIP_EUNSUPPORTED;
    const int vn = vec_for(dt, {dx, dy, mx ? x : nullptr, mx ? y : nullptr});
    const int64_t total = view_elements(dx) / vn;
    const int g = grid_for(total, 256, 256 * 32);
    hipStream_t st = as_stream(stream);
    DView dvx = mx ? dview(x) : dview(dx), dvy = mx ? dview(y) : dview(dy), dvdy = dview(dy), dvdx = dview(dx);
    if(mx && vn > 1 && size * size < 255) {
        const int H = dx->dims[2], W = dx->dims[3];
        const int WP = (POOL_TH + size - 2) / stride + 2, WQ = (POOL_TW + size - 2) / stride + 2;
        const size_t lds = (size_t)WP * WQ * POOL_CVB * vn;
        if(lds <= 64 * 1024 && dx->dims[0] <= 65535) {
            const int tw = (W + POOL_TW - 1) / POOL_TW, th = (H + POOL_TH - 1) / POOL_TH;
            const dim3 grid(tw * th, (dx->dims[1] / vn + POOL_CVB - 1) / POOL_CVB, dx->dims[0]);
            if(dt == SAGA_HALF)
                maxpool_bwd_tiled<half_t, 8><<<grid, 256, lds, st>>>(dvx, dvy, dvdy, dvdx, size, pad, stride, beta, tw, WP, WQ);
            else
                maxpool_bwd_tiled<float, 4><<<grid, 256, lds, st>>>(dvx, dvy, dvdy, dvdx, size, pad, stride, beta, tw, WP, WQ);
            SAGA_CHECK_LAUNCH();
            return 0;
        }
    }
#define GO(T, VN)                                                                                              \
    do {                                                                                                       \
        if(mx)                                                                                                 \
            pool_bwd_k<T, VN, SAGA_POOL_MAX><<<g, 256, 0, st>>>(dvx, dvy, dvdy, dvdx, size, pad, stride, beta, total); \
        else                                                                                                   \
            pool_bwd_k<T, VN, SAGA_POOL_AVG><<<g, 256, 0, st>>>(dvx, dvy, dvdy, dvdx, size, pad, stride, beta, total); \
    } while(0)
    if(dt == SAGA_HALF) {
        if(vn == 8) GO(half_t, 8); else GO(half_t, 1);
    } else {
        if(vn == 4) GO(float, 4); else GO(float, 1);
    }
#undef GO
    SAGA_CHECK_LAUNCH();
    return 0;
}

// Max pooling that records where each maximum came from (one byte per output element, dense
// N,P,Q,C order); only channels-last tensors whose channels fill whole 16-byte vectors, 2x2 or
// 3x3 windows.  SAGA_HIP_EUNSUPPORTED otherwise: the caller then uses saga_hip_pool_fwd/bwd.
static bool codes_ok(const SagaTensorView *a, const SagaTensorView *b, int size, int pad, int stride)
{
    if(size < 2 || size > 3 || stride < 1 || stride > size || pad < 0 || pad >= size)
        return false;
    if(a->dtype != b->dtype || (a->dtype != SAGA_HALF && a->dtype != SAGA_FLOAT))
        return false;
    if(vec_for(a->dtype, {a, b}) == 1)
        return false;
    const int vn = a->dtype == SAGA_HALF ? 8 : 4;
    // one block spans all channel vectors of a pixel; rows and samples are grid dimensions
    return a->dims[1] / vn <= 256 && a->dims[0] <= 65535 && a->dims[2] <= 65535 && b->dims[2] <= 65535;
}

// block = (channel vectors rounded up to a power of two) x (columns to fill 256 threads)
static void codes_launch_shape(int cv, int cols, int rows, int n, dim3 &grid, dim3 &block)
{
    int bx = 1;
    while(bx < cv)
        bx <<= 1;
    const int by = 256 / bx;
    block = dim3(bx, by, 1);
    grid = dim3((cols + by - 1) / by, rows, n);
}

int saga_hip_maxpool_fwd_codes(const SagaTensorView *x, const SagaTensorView *y, uint8_t *codes, int size, int pad,
                               int stride, saga_stream_t stream)
{
    if(!valid_view(x) || !valid_view(y) || !codes)
        return SAGA_HIP_EINVAL;
    if(x->dims[0] != y->dims[0] || x->dims[1] != y->dims[1] || y->dims[2] != pool_dim(x->dims[2], size, pad, stride) ||
       y->dims[3] != pool_dim(x->dims[3], size, pad, stride))
        return SAGA_HIP_ESHAPE;
    if(!codes_ok(x, y, size, pad, stride) || ((uintptr_t)codes & 7))
        return SAGA_HIP_EUNSUPPORTED;
    launch_maxpool_codes(x, y, codes, size, pad, stride, as_stream(stream));
    SAGA_CHECK_LAUNCH();
    return 0;
}

int saga_hip_maxpool_fwd_codes_bn(const SagaTensorView *x, const SagaTensorView *y, uint8_t *codes, int size, int pad,
                                  int stride, const float *scale_shift, int flags, saga_stream_t stream)
{
    if(!valid_view(x) || !valid_view(y) || !codes || !scale_shift)
        return SAGA_HIP_EINVAL;
    if(flags & ~SAGA_BN_RELU)
        return SAGA_HIP_EUNSUPPORTED; // a residual would be a third tensor per window position
    if(x->dims[0] != y->dims[0] || x->dims[1] != y->dims[1] || y->dims[2] != pool_dim(x->dims[2], size, pad, stride) ||
       y->dims[3] != pool_dim(x->dims[3], size, pad, stride))
        return SAGA_HIP_ESHAPE;
    if(!codes_ok(x, y, size, pad, stride) || ((uintptr_t)codes & 7))
        return SAGA_HIP_EUNSUPPORTED;
    launch_maxpool_codes(x, y, codes, size, pad, stride, as_stream(stream), scale_shift, flags & SAGA_BN_RELU ? 1 : 0);
    SAGA_CHECK_LAUNCH();
    return 0;
}

} // extern "C"

// The row-resident kernel for 3x3 / stride 2 / padding 1 on fp16 channels-last tensors whose rows do not overlap;
// false when the shapes do not fit it (SAGA_HIP_POOL_ROWS=0 switches it off).
static bool launch_maxpool_rows(const SagaTensorView *x, const SagaTensorView *y, uint8_t *codes, int size, int pad,
                                int stride, hipStream_t st, const float *ss, int relu)
{
    static const bool off = getenv("SAGA_HIP_POOL_ROWS") && atoi(getenv("SAGA_HIP_POOL_ROWS")) == 0;
    if(off || x->dtype != SAGA_HALF || size != 3 || stride != 2 || pad != 1)
        return false;
    const int N = x->dims[0], C = x->dims[1], H = x->dims[2], W = x->dims[3], P = y->dims[2], Q = y->dims[3];
    const int cv = C / 8;
    if(C % 8 || (cv & (cv - 1)) || cv > 256)
        return false;
    const int64_t xs0 = x->strides[0], xs2 = x->strides[2], xs3 = x->strides[3];
    if(H < 2 || W < 2 || P < 2 || Q < 2) // (a dimension of one element may carry any pitch)
        return false;
    if((C > 1 && (x->strides[1] != 1 || y->strides[1] != 1)) || xs3 < C || xs3 % 8 || xs2 % 8 ||
       (int64_t)(W - 1) * xs3 + C > xs2 || (int64_t)H * xs2 * 2 >= 0x7fff0000)
        return false;
    if(N > 1 && (xs0 % 8 || (int64_t)H * xs2 > xs0 || xs0 >= 0x7fffffff || y->strides[0] % 8 || y->strides[0] < 0))
        return false;
    for(int i : {2, 3})
        if(y->strides[i] % 8 || y->strides[i] < 0)
            return false;
    if(!aligned16(x->ptr) || !aligned16(y->ptr))
        return false;
    // the most output rows whose 2 * TR + 1 input rows fit the kernel's chunks per lane
    const int64_t row_chunks = (int64_t)W * cv;
    int tr = (int)((POOL_ROWS_NLD * POOL_ROWS_NT / row_chunks - 1) / 2);
    tr = std::min(tr, P);
    if(tr < 1)
        return false;
    static int cus = 0;
    if(!cus) {
        int dev = 0;
        hipDeviceProp_t prop;
        if(hipGetDevice(&dev) != hipSuccess || hipGetDeviceProperties(&prop, dev) != hipSuccess)
            return false;
        cus = prop.multiProcessorCount;
        if(hipFuncSetAttribute((const void *)maxpool_3x3s2_rows_k<false>, hipFuncAttributeMaxDynamicSharedMemorySize,
                               2 * POOL_ROWS_NLD * POOL_ROWS_NT * 16) != hipSuccess ||
           hipFuncSetAttribute((const void *)maxpool_3x3s2_rows_k<true>, hipFuncAttributeMaxDynamicSharedMemorySize,
                               2 * POOL_ROWS_NLD * POOL_ROWS_NT * 16) != hipSuccess) {
            cus = 0;
            return false;
        }
    }
    PoolRowsArgs t;
    t.x = (const half_t *)x->ptr;
    t.y = (half_t *)y->ptr;
    t.codes = codes;
    t.ss = ss;
    t.C = C, t.H = H, t.W = W, t.P = P, t.Q = Q, t.CV = cv;
    t.xs0 = N > 1 ? (int)xs0 : 0, t.xs2 = (int)xs2, t.xs3 = (int)xs3;
    t.ys0 = N > 1 ? y->strides[0] : 0, t.ys2 = y->strides[2], t.ys3 = y->strides[3];
    t.TR = tr;
    t.spi = (P + tr - 1) / tr;
    if((int64_t)t.spi * N > 0x7fffffff)
        return false;
    t.nstrips = t.spi * N;
    t.chunks = (int)((2 * tr + 1) * row_chunks);
    t.relu = relu;
    t.ximg_bytes = (unsigned)(H * xs2 * 2);
    const int lds = 2 * (((t.chunks + 63) >> 6) << 10);
    if(lds > 2 * POOL_ROWS_NLD * POOL_ROWS_NT * 16)
        return false;
    const int blocks = std::min(t.nstrips, cus);
    if(relu)
        maxpool_3x3s2_rows_k<true><<<blocks, POOL_ROWS_NT, lds, st>>>(t);
    else
        maxpool_3x3s2_rows_k<false><<<blocks, POOL_ROWS_NT, lds, st>>>(t);
    return true;
}

static void launch_maxpool_codes(const SagaTensorView *x, const SagaTensorView *y, uint8_t *codes, int size, int pad,
                                 int stride, hipStream_t st, const float *ss, int relu)
{
    const int vn = x->dtype == SAGA_HALF ? 8 : 4;
    if(launch_maxpool_rows(x, y, codes, size, pad, stride, st, ss, relu))
        return;
    dim3 grid, block;
    codes_launch_shape(y->dims[1] / vn, y->dims[3], y->dims[2], y->dims[0], grid, block);
    const DView dvx = dview(x), dvy = dview(y);
#define GO2(T, VN, K, S) maxpool_fwd_codes_k<T, VN, K, S><<<grid, block, 0, st>>>(dvx, dvy, codes, pad, ss, relu)
#define GO(T, VN)                                                                                              \
    do {                                                                                                       \
        switch(size * 4 + stride) {                                                                            \
        case 13: GO2(T, VN, 3, 1); break;                                                                      \
        case 14: GO2(T, VN, 3, 2); break;                                                                      \
        case 15: GO2(T, VN, 3, 3); break;                                                                      \
        case 9: GO2(T, VN, 2, 1); break;                                                                       \
        default: GO2(T, VN, 2, 2); break;                                                                      \
        }                                                                                                      \
    } while(0)
    if(x->dtype == SAGA_HALF)
        GO(half_t, 8);
    else
        GO(float, 4);
#undef GO
#undef GO2
}

extern "C" {

int saga_hip_maxpool_bwd_codes(const uint8_t *codes, const SagaTensorView *dy, const SagaTensorView *dx, int size, int pad,
                               int stride, float beta, saga_stream_t stream)
{
    if(!valid_view(dy) || !valid_view(dx) || !codes)
        return SAGA_HIP_EINVAL;
    if(dy->dims[0] != dx->dims[0] || dy->dims[1] != dx->dims[1] ||
       dy->dims[2] != pool_dim(dx->dims[2], size, pad, stride) || dy->dims[3] != pool_dim(dx->dims[3], size, pad, stride))
        return SAGA_HIP_ESHAPE;
    if(!codes_ok(dx, dy, size, pad, stride) || ((uintptr_t)codes & 7))
        return SAGA_HIP_EUNSUPPORTED;
    const int vn = dx->dtype == SAGA_HALF ? 8 : 4;
    dim3 grid, block;
    hipStream_t st = as_stream(stream);
    const DView dvdy = dview(dy), dvdx = dview(dx);
    if(size == 3 && stride == 2) {
        // patches (2a-1 .. 2a) x (2b-1 .. 2b) in padded coordinates: a = 0 .. (H - 1 + pad + 1) / 2
        const int na = (dx->dims[2] + pad) / 2 + 1, nb = (dx->dims[3] + pad) / 2 + 1;
        codes_launch_shape(dx->dims[1] / vn, nb, na, dx->dims[0], grid, block);
        if(dx->dtype == SAGA_HALF)
            maxpool_bwd_codes_3x3s2_k<half_t, 8><<<grid, block, 0, st>>>(codes, dvdy, dvdx, pad, beta);
        else
            maxpool_bwd_codes_3x3s2_k<float, 4><<<grid, block, 0, st>>>(codes, dvdy, dvdx, pad, beta);
        SAGA_CHECK_LAUNCH();
        return 0;
    }
    codes_launch_shape(dx->dims[1] / vn, dx->dims[3], dx->dims[2], dx->dims[0], grid, block);
#define GO2(T, VN, K, S) maxpool_bwd_codes_k<T, VN, K, S><<<grid, block, 0, st>>>(codes, dvdy, dvdx, pad, beta)
#define GO(T, VN)                                                                                              \
    do {                                                                                                       \
        switch(size * 4 + stride) {                                                                            \
        case 13: GO2(T, VN, 3, 1); break;                                                                      \
        case 14: GO2(T, VN, 3, 2); break;                                                                      \
        case 15: GO2(T, VN, 3, 3); break;                                                                      \
        case 9: GO2(T, VN, 2, 1); break;                                                                       \
        default: GO2(T, VN, 2, 2); break;                                                                      \
        }                                                                                                      \
    } while(0)
    if(dx->dtype == SAGA_HALF)
        GO(half_t, 8);
    else
        GO(float, 4);
#undef GO
#undef GO2
    SAGA_CHECK_LAUNCH();
    return 0;
}

} // extern "C"

// Shape of the fused launch: patches along rows in groups of BNPOOL_AG; returns the number of partial rows.
static int64_t bn_pool_launch_shape(const SagaTensorView *x, int pad, dim3 &grid, dim3 &block, int *na_out, int ag = BNPOOL_AG)
{
    const int vn = x->dtype == SAGA_HALF ? 8 : 4;
    const int na = (x->dims[2] + pad) / 2 + 1, nb = (x->dims[3] + pad) / 2 + 1;
    codes_launch_shape(x->dims[1] / vn, nb, (na + ag - 1) / ag, x->dims[0], grid, block);
    if(na_out)
        *na_out = na;
    return (int64_t)grid.x * grid.y * grid.z;
}

static bool bn_pool_ok(const SagaTensorView *x, const SagaTensorView *dp, const SagaTensorView *dx, int size, int pad, int stride)
{
    if(!valid_view(x) || !valid_view(dp) || size != 3 || stride != 2 || pad < 0 || pad > 2)
        return false;
    if(dx && (!valid_view(dx) || !same_dims(x, dx) || dx->dtype != x->dtype))
        return false;
    if(dp->dims[0] != x->dims[0] || dp->dims[1] != x->dims[1] || dp->dims[2] != pool_dim(x->dims[2], size, pad, stride) ||
       dp->dims[3] != pool_dim(x->dims[3], size, pad, stride) || dp->dtype != x->dtype)
        return false;
    return codes_ok(x, dp, size, pad, stride) && (!dx || codes_ok(dx, dp, size, pad, stride));
}

extern "C" {

size_t saga_hip_bn_bwd_pooled_workspace_size(const SagaTensorView *x, const SagaTensorView *dp, int size, int pad, int stride)
{
    if(!x || !dp || !bn_pool_ok(x, dp, nullptr, size, pad, stride))
        return 0;
    dim3 grid, block;
    const int64_t rows = bn_pool_launch_shape(x, pad, grid, block, nullptr);
    return ((size_t)rows * x->dims[1] * 2 + 3 * (size_t)x->dims[1] + 64) * sizeof(float);
}

int saga_hip_bn_bwd_pooled(const SagaTensorView *x, const SagaTensorView *dp, const uint8_t *codes, const SagaTensorView *dx,
                           const float *s, const float *b, const float *save_mean, const float *save_invstd, float *ds,
                           float *db, float beta_dx, float beta_p, int flags, int size, int pad, int stride, void *workspace,
                           size_t ws_bytes, saga_stream_t stream)
{
    if(!x || !dp || !dx || !codes || !s || !save_mean || !save_invstd || !ds || !db)
        return SAGA_HIP_EINVAL;
    if(flags & ~SAGA_BN_RELU)
        return SAGA_HIP_EUNSUPPORTED;
    const int relu = flags & SAGA_BN_RELU ? 1 : 0;
    if(relu && !b)
        return SAGA_HIP_EINVAL; // the mask is rebuilt from x, which takes the bias
    if(!bn_pool_ok(x, dp, dx, size, pad, stride) || ((uintptr_t)codes & 7))
        return SAGA_HIP_EUNSUPPORTED;
    const size_t need = saga_hip_bn_bwd_pooled_workspace_size(x, dp, size, pad, stride);
    if(!workspace || ws_bytes < need)
        return SAGA_HIP_EWORKSPACE;
    dim3 grid, block;
    int na = 0;
    const int64_t rows = bn_pool_launch_shape(x, pad, grid, block, &na);
    if(rows >= (1ll << 31))
        return SAGA_HIP_EUNSUPPORTED;

    const int C = x->dims[1];
    float *partial = (float *)workspace, *coef = partial + (size_t)rows * C * 2;
    hipStream_t st = as_stream(stream);
    const DView dvp = dview(dp), dvx = dview(x), dvdx = dview(dx);
    const double M = (double)x->dims[0] * x->dims[2] * x->dims[3];
#define GO(T, VN)                                                                                                       \
    do {                                                                                                                \
        bn_pool_bwd_3x3s2_k<T, VN, 0, BNPOOL_AG><<<grid, block, 0, st>>>(codes, dvp, dvx, dvdx, pad, na, save_mean, s,     \
                                                                        save_invstd, b, relu, nullptr, partial, 0.0f); \
        const int rc = bn_launch_bwd_finalize(partial, (int)rows, s, save_invstd, ds, db, coef, M, C, beta_p, st);       \
        if(rc)                                                                                                          \
            return rc;                                                                                                  \
        bn_pool_bwd_3x3s2_k<T, VN, 1, BNPOOL_AG><<<grid, block, 0, st>>>(codes, dvp, dvx, dvdx, pad, na, save_mean, s,           \
                                                                  save_invstd, b, relu, coef, nullptr, beta_dx);        \
    } while(0)
    if(x->dtype == SAGA_HALF)
        GO(half_t, 8);
    else
        GO(float, 4);
#undef GO
    SAGA_CHECK_LAUNCH();
    return 0;
}

} // extern "C"
