// Element-wise kernels: activations, add, axpby (transform), convert, bias add, fill.
// All are HBM-bound: the fast paths move 16 bytes per lane per access and keep every
// wavefront on consecutive addresses; odd layouts fall back to a strided gather.
#include "common.hpp"
#include <atomic>

namespace {

// ---------------------------------------------------------------- functors (fp32 math)

struct ActFwd {
    int mode;
    float alpha, beta;
    __device__ float operator()(float x, float, float old) const
    {
        float r;
        switch(mode) {
        case SAGA_ACT_RELU: r = (x != x) ? x : fmaxf(x, 0.0f); break;
        case SAGA_ACT_SIGMOID: r = 1.0f / (1.0f + __expf(-x)); break;
        case SAGA_ACT_TANH: r = tanhf(x); break;
        case SAGA_ACT_SWISH: r = x / (1.0f + __expf(-x)); break;
        default: r = x > 0 ? x : x * alpha; break;
        }
        return beta != 0.0f ? r + beta * old : r;
    }
};

// a = x (relu, swish, leaky) or y (sigmoid, tanh); b = dy
struct ActBwd {
    int mode;
    float alpha, beta;
    __device__ float operator()(float a, float dy, float old) const
    {
        float d;
        switch(mode) {
        case SAGA_ACT_RELU: d = a > 0 ? 1.0f : 0.0f; break;
        case SAGA_ACT_SIGMOID: d = a * (1.0f - a); break;
        case SAGA_ACT_TANH: d = 1.0f - a * a; break;
        case SAGA_ACT_SWISH: {
            const float sg = 1.0f / (1.0f + __expf(-a));
            d = sg + a * sg * (1.0f - sg);
            break;
        }
        default: d = a > 0 ? 1.0f : alpha; break;
        }
        const float r = d * dy;
        return beta != 0.0f ? r + beta * old : r;
    }
};

struct AddFn {
    __device__ float operator()(float a, float b, float) const { return a + b; }
};

struct AxpbyFn {
    float alpha, beta;
    __device__ float operator()(float a, float, float old) const
    {
        const float r = alpha * a;
        return beta != 0.0f ? r + beta * old : r;
    }
};

// ---------------------------------------------------------------- kernels

template <typename T> struct Vec;
template <> struct Vec<half_t> {
    typedef half8_t type;
    static constexpr int n = 8;
};
template <> struct Vec<float> {
    typedef float4_t type;
    static constexpr int n = 4;
};

// Flat, dense, same layout for every operand: 16-byte vectors.  A block owns a contiguous run of tiles of
// 4 x 256 vectors (16 KB per operand) and requests the four vectors of a lane before it stores the first
// result; the grid has up to 65535 blocks, dispatched in order, so that at any time the chip works on one
// compact window of the tensors.  Measured on MI355X with a 1 GiB copy: 5.4 - 6.0 TB/s this way, 4.1 - 4.5 TB/s
// with a grid-stride loop whose four vectors lie a whole grid apart, 5.2 TB/s for the runtime's own copy.
template <typename T, int NIN, bool READ_OLD, typename F>
__global__ void __launch_bounds__(256) ew_flat(T *__restrict__ out, const T *__restrict__ a, const T *__restrict__ b,
                                               int64_t nvec, int64_t total, F f)
{
    typedef typename Vec<T>::type V;
    constexpr int VN = Vec<T>::n;
    constexpr int U = 4;
    auto apply = [&](const V &va, const V &vb, const V &vo) {
        V r;
#pragma unroll
        for(int j = 0; j < VN; j++)
            r[j] = (T)f((float)va[j], (float)vb[j], (float)vo[j]);
        return r;
    };
    const int64_t tiles = (nvec + 256 * U - 1) / (256 * U);
    const int64_t per = (tiles + gridDim.x - 1) / gridDim.x;
    const int64_t t0 = (int64_t)blockIdx.x * per;
    const int64_t t1 = t0 + per < tiles ? t0 + per : tiles;
    for(int64_t t = t0; t < t1; t++) {
        const int64_t i = t * (256 * U) + threadIdx.x;
        if(i + (U - 1) * 256 < nvec) {
            V va[U], vb[U], vo[U];
#pragma unroll
            for(int u = 0; u < U; u++) {
                va[u] = ((const V *)a)[i + u * 256];
                vb[u] = NIN > 1 ? ((const V *)b)[i + u * 256] : va[u];
                vo[u] = READ_OLD ? ((const V *)out)[i + u * 256] : va[u];
            }
#pragma unroll
            for(int u = 0; u < U; u++)
                ((V *)out)[i + u * 256] = apply(va[u], vb[u], vo[u]);
        } else {
            for(int64_t k = i; k < nvec; k += 256) {
                const V va = ((const V *)a)[k];
                const V vb = NIN > 1 ? ((const V *)b)[k] : va;
                const V vo = READ_OLD ? ((const V *)out)[k] : va;
                ((V *)out)[k] = apply(va, vb, vo);
            }
        }
    }
    const int64_t stride = (int64_t)gridDim.x * blockDim.x;
    // tail
    const int64_t base = nvec * VN;
    for(int64_t i = base + (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < total; i += stride) {
        const float va = (float)a[i];
        const float vb = NIN > 1 ? (float)b[i] : va;
        const float vo = READ_OLD ? (float)out[i] : 0.0f;
        out[i] = (T)f(va, vb, vo);
    }
}

// Channels-last rows with individual pitches (channel slices): vectors along C.
template <typename T, int NIN, bool READ_OLD, typename F>
__global__ void __launch_bounds__(256)
    ew_rows(T *__restrict__ out, int64_t po, const T *__restrict__ a, int64_t pa, const T *__restrict__ b, int64_t pb,
            int64_t rows, int cvec, F f)
{
    typedef typename Vec<T>::type V;
    constexpr int VN = Vec<T>::n;
    const int64_t total = rows * cvec;
    const int64_t stride = (int64_t)gridDim.x * blockDim.x;
    for(int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < total; i += stride) {
        const int64_t r = i / cvec;
        const int c = (int)(i - r * cvec) * VN;
        V va = *(const V *)(a + r * pa + c);
        V vb = NIN > 1 ? *(const V *)(b + r * pb + c) : va;
        V vo = READ_OLD ? *(const V *)(out + r * po + c) : va;
        V res;
#pragma unroll
        for(int j = 0; j < VN; j++)
            res[j] = (T)f((float)va[j], (float)vb[j], (float)vo[j]);
        *(V *)(out + r * po + c) = res;
    }
}

// Anything else: one element per lane, addresses from the 4-D strides.  `cl` selects the
// decode order so that neighbouring lanes are neighbours in the output's memory.
template <typename TO, typename TA, typename TB, int NIN, bool READ_OLD, typename F>
__global__ void __launch_bounds__(256) ew_strided(DView out, DView a, DView b, int64_t total, int cl, F f)
{
    const int64_t stride = (int64_t)gridDim.x * blockDim.x;
    const int N = out.d[0], C = out.d[1], H = out.d[2], W = out.d[3];
    (void)N;
    for(int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < total; i += stride) {
        int n, c, h, w;
        int64_t t = i;
        if(cl) {
            c = (int)(t % C);
            t /= C;
            w = (int)(t % W);
            t /= W;
            h = (int)(t % H);
            n = (int)(t / H);
        } else {
            w = (int)(t % W);
            t /= W;
            h = (int)(t % H);
            t /= H;
            c = (int)(t % C);
            n = (int)(t / C);
        }
        const int64_t oa = n * a.s[0] + c * a.s[1] + h * a.s[2] + w * a.s[3];
        const int64_t oo = n * out.s[0] + c * out.s[1] + h * out.s[2] + w * out.s[3];
        const float va = (float)((const TA *)a.ptr)[oa];
        float vb = va;
        if(NIN > 1) {
            const int64_t ob = n * b.s[0] + c * b.s[1] + h * b.s[2] + w * b.s[3];
            vb = (float)((const TB *)b.ptr)[ob];
        }
        TO *po = (TO *)out.ptr + oo;
        const float vo = READ_OLD ? (float)*po : 0.0f;
        *po = (TO)f(va, vb, vo);
    }
}

static bool same_strides(const SagaTensorView *a, const SagaTensorView *b)
{
    for(int i = 0; i < 4; i++)
        if(a->dims[i] > 1 && a->strides[i] != b->strides[i])
            return false;
    return true;
}

static bool dense(const SagaTensorView *v)
{
    CLInfo cl;
    CFInfo cf;
    if(as_channels_last(v, &cl) && cl.pitch == cl.C)
        return true;
    if(as_channels_first(v, &cf) && cf.npitch == (int64_t)cf.C * cf.HW)
        return true;
    return false;
}

// Dispatch for same-dtype unary / binary element-wise ops.
template <typename T, int NIN, bool READ_OLD, typename F>
int launch_ew_t(const SagaTensorView *out, const SagaTensorView *a, const SagaTensorView *b, F f, hipStream_t st)
{
    const int64_t total = view_elements(out);
    constexpr int VN = Vec<T>::n;
    const bool al = aligned16(out->ptr) && aligned16(a->ptr) && (NIN < 2 || aligned16(b->ptr));
    if(dense(out) && same_strides(out, a) && (NIN < 2 || same_strides(out, b)) && al) {
        const int64_t nvec = total / VN;
        ew_flat<T, NIN, READ_OLD, F><<<grid_for(nvec ? (nvec + 3) / 4 : 1, 256, 65535), 256, 0, st>>>(
            (T *)out->ptr, (const T *)a->ptr, (const T *)(NIN > 1 ? b->ptr : a->ptr), nvec, total, f);
        SAGA_CHECK_LAUNCH();
        return 0;
    }
    CLInfo co, ca, cb;
    if(al && as_channels_last(out, &co) && as_channels_last(a, &ca) && (NIN < 2 || as_channels_last(b, &cb)) &&
       co.C % VN == 0 && co.pitch % VN == 0 && ca.pitch % VN == 0 && (NIN < 2 || cb.pitch % VN == 0)) {
        const int cvec = co.C / VN;
        ew_rows<T, NIN, READ_OLD, F><<<grid_for(co.rows * cvec, 256, 256 * 16), 256, 0, st>>>(
            (T *)out->ptr, co.pitch, (const T *)a->ptr, ca.pitch, (const T *)(NIN > 1 ? b->ptr : a->ptr),
            NIN > 1 ? cb.pitch : ca.pitch, co.rows, cvec, f);
        SAGA_CHECK_LAUNCH();
        return 0;
    }
    const int cl = (out->dims[1] == 1 || out->strides[1] == 1) ? 1 : 0;
    ew_strided<T, T, T, NIN, READ_OLD, F><<<grid_for(total, 256, 256 * 32), 256, 0, st>>>(
        dview(out), dview(a), dview(NIN > 1 ? b : a), total, cl, f);
    SAGA_CHECK_LAUNCH();
    return 0;
}

template <int NIN, typename F>
int launch_ew(const SagaTensorView *out, const SagaTensorView *a, const SagaTensorView *b, bool read_old, F f,
              hipStream_t st)
{
    if(!valid_view(out) || !valid_view(a) || (NIN > 1 && !valid_view(b)))
        return SAGA_HIP_EINVAL;
    if(!same_dims(out, a) || (NIN > 1 && !same_dims(out, b)))
        return SAGA_HIP_ESHAPE;
    if(out->dtype != a->dtype || (NIN > 1 && out->dtype != b->dtype))
        return SAGA_HIP_EUNSUPPORTED;
    if(out->dtype == SAGA_HALF)
        return read_old ? launch_ew_t<half_t, NIN, true, F>(out, a, b, f, st)
                        : launch_ew_t<half_t, NIN, false, F>(out, a, b, f, st);
    if(out->dtype == SAGA_FLOAT)
        return read_old ? launch_ew_t<float, NIN, true, F>(out, a, b, f, st)
                        : launch_ew_t<float, NIN, false, F>(out, a, b, f, st);
    return SAGA_HIP_EUNSUPPORTED;
}

struct ScaleFn {
    float scale;
    __device__ float operator()(float a, float, float) const { return a * scale; }
};

template <typename TS, typename TD>
int launch_convert(const SagaTensorView *src, const SagaTensorView *dst, float scale, hipStream_t st)
{
    const int64_t total = view_elements(dst);
    const int cl = (dst->dims[1] == 1 || dst->strides[1] == 1) ? 1 : 0;
    ew_strided<TD, TS, TS, 1, false, ScaleFn><<<grid_for(total, 256, 256 * 32), 256, 0, st>>>(
        dview(dst), dview(src), dview(src), total, cl, ScaleFn{scale});
    SAGA_CHECK_LAUNCH();
    return 0;
}

// y[row, c] += b[c] on channels-last rows.
template <typename T, typename TB>
__global__ void __launch_bounds__(256) bias_add_cl(T *y, int64_t pitch, const TB *b, int64_t rows, int C)
{
    const int64_t total = rows * C;
    const int64_t stride = (int64_t)gridDim.x * blockDim.x;
    for(int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < total; i += stride) {
        const int64_t r = i / C;
        const int c = (int)(i - r * C);
        T *p = y + r * pitch + c;
        *p = (T)((float)*p + (float)b[c]);
    }
}

template <typename T, typename TB>
__global__ void __launch_bounds__(256) bias_add_cf(T *y, int64_t npitch, const TB *b, int N, int C, int64_t HW)
{
    const int64_t total = (int64_t)N * C * HW;
    const int64_t stride = (int64_t)gridDim.x * blockDim.x;
    for(int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < total; i += stride) {
        const int64_t nc = i / HW;
        const int c = (int)(nc % C);
        const int64_t n = nc / C;
        T *p = y + n * npitch + (int64_t)c * HW + (i - nc * HW);
        *p = (T)((float)*p + (float)b[c]);
    }
}

// db[c] = beta*db[c] + sum over rows, channels-last: one block handles 64 channels x all rows
// striped over 4 waves; lanes read consecutive channels.
template <typename T, typename TB>
__global__ void __launch_bounds__(256) bias_bwd_cl(const T *dy, int64_t pitch, TB *db, int64_t rows, int C, float beta)
{
    __shared__ float part[4][64];
    const int lane = threadIdx.x & 63, wv = threadIdx.x >> 6;
    const int c = blockIdx.x * 64 + lane;
    float acc = 0;
    if(c < C)
        for(int64_t r = wv; r < rows; r += 4)
            acc += (float)dy[r * pitch + c];
    part[wv][lane] = acc;
    __syncthreads();
    if(wv == 0 && c < C) {
        const float s = part[0][lane] + part[1][lane] + part[2][lane] + part[3][lane];
        db[c] = (TB)(beta != 0.0f ? s + beta * (float)db[c] : s);
    }
}

// Large channels-last tensors: the rows are split over gridDim.x blocks, each leaving one fp32
// partial per channel; bias_bwd_final adds them in block order (deterministic, no atomics).
// Block = 64 channels x 4 row lanes, as above.
template <typename T>
__global__ void __launch_bounds__(256)
    bias_bwd_partial_cl(const T *__restrict__ dy, int64_t pitch, float *__restrict__ partial, int64_t rows, int C)
{
    __shared__ float part[4][64];
    const int lane = threadIdx.x & 63, wv = threadIdx.x >> 6;
    const int c = blockIdx.y * 64 + lane;
    float acc = 0;
    if(c < C) {
        const int64_t stride = (int64_t)gridDim.x * 4;
        int64_t r = (int64_t)blockIdx.x * 4 + wv;
        for(; r + 7 * stride < rows; r += 8 * stride) {
            float v[8];
#pragma unroll
            for(int u = 0; u < 8; u++)
                v[u] = (float)dy[(r + u * stride) * pitch + c];
#pragma unroll
            for(int u = 0; u < 8; u++)
                acc += v[u];
        }
        for(; r < rows; r += stride)
            acc += (float)dy[r * pitch + c];
    }
    part[wv][lane] = acc;
    __syncthreads();
    if(wv == 0 && c < C)
        partial[(int64_t)blockIdx.x * C + c] = part[0][lane] + part[1][lane] + part[2][lane] + part[3][lane];
}

// The same with 16-byte loads along C (C, the pitch and the base address multiples of the vector):
// cvp (a power of two, at most 256) threads cover the channel vectors of one row, 256 / cvp rows at a time.
template <typename T>
__global__ void __launch_bounds__(256) bias_bwd_partial_vec(const T *__restrict__ dy, int64_t pitch,
                                                            float *__restrict__ partial, int64_t rows, int C, int cvp)
{
    typedef typename Vec<T>::type V;
    constexpr int VN = Vec<T>::n;
    __shared__ float part[256][VN + 1];
    const int cv = C / VN;
    const int ci = blockIdx.y * cvp + (threadIdx.x & (cvp - 1));
    const int rl = threadIdx.x / cvp, nrl = 256 / cvp;
    float acc[VN];
#pragma unroll
    for(int j = 0; j < VN; j++)
        acc[j] = 0.0f;
    if(ci < cv) {
        const int64_t stride = (int64_t)gridDim.x * nrl;
        int64_t r = (int64_t)blockIdx.x * nrl + rl;
        const T *base = dy + (int64_t)ci * VN;
        for(; r + 3 * stride < rows; r += 4 * stride) {
            V v[4];
#pragma unroll
            for(int u = 0; u < 4; u++)
                v[u] = *(const V *)(base + (r + u * stride) * pitch);
#pragma unroll
            for(int u = 0; u < 4; u++)
#pragma unroll
                for(int j = 0; j < VN; j++)
                    acc[j] += (float)v[u][j];
        }
        for(; r < rows; r += stride) {
            const V v = *(const V *)(base + r * pitch);
#pragma unroll
            for(int j = 0; j < VN; j++)
                acc[j] += (float)v[j];
        }
    }
#pragma unroll
    for(int j = 0; j < VN; j++)
        part[threadIdx.x][j] = acc[j];
    __syncthreads();
    if(rl == 0 && ci < cv) {
        for(int k = 1; k < nrl; k++)
#pragma unroll
            for(int j = 0; j < VN; j++)
                acc[j] += part[threadIdx.x + k * cvp][j];
#pragma unroll
        for(int j = 0; j < VN; j++)
            partial[(int64_t)blockIdx.x * C + ci * VN + j] = acc[j];
    }
}

// One block per 32 channels: 8 lanes per channel each add every 8th partial (four loads in flight),
// then lane 0 adds the 8 lane sums in order.
template <typename TB>
__global__ void __launch_bounds__(256) bias_bwd_final(const float *__restrict__ partial, int gx, TB *db, int C, float beta)
{
    __shared__ float part[8][32];
    const int cl = threadIdx.x & 31, gl = threadIdx.x >> 5;
    const int c = blockIdx.x * 32 + cl;
    float s = 0;
    if(c < C) {
        int g = gl;
        for(; g + 24 < gx; g += 32) {
            const float v0 = partial[(int64_t)g * C + c], v1 = partial[(int64_t)(g + 8) * C + c];
            const float v2 = partial[(int64_t)(g + 16) * C + c], v3 = partial[(int64_t)(g + 24) * C + c];
            s += (v0 + v1) + (v2 + v3);
        }
        for(; g < gx; g += 8)
            s += partial[(int64_t)g * C + c];
    }
    part[gl][cl] = s;
    __syncthreads();
    if(gl == 0 && c < C) {
        for(int k = 1; k < 8; k++)
            s += part[k][cl];
        db[c] = (TB)(beta != 0.0f ? s + beta * (float)db[c] : s);
    }
}

// blocks along the rows for the two-pass form; 1 = the single-pass kernel is enough
static int bias_bwd_splits(int64_t rows, int C)
{
    if(rows * C < (int64_t)1 << 20)
        return 1;
    int64_t gx = C >= 512 ? 512 : 1024; // at least four blocks of the vector kernel per CU
    if(gx > rows / 64)
        gx = rows / 64;
    return gx < 2 ? 1 : (int)gx;
}

template <typename T, typename TB>
__global__ void __launch_bounds__(256) bias_bwd_cf(const T *dy, int64_t npitch, TB *db, int N, int C, int64_t HW, float beta)
{
    __shared__ float part[4];
    const int c = blockIdx.x;
    float acc = 0;
    for(int n = 0; n < N; n++) {
        const T *p = dy + n * npitch + (int64_t)c * HW;
        for(int64_t i = threadIdx.x; i < HW; i += 256)
            acc += (float)p[i];
    }
    acc = wave_sum(acc);
    if((threadIdx.x & 63) == 0)
        part[threadIdx.x >> 6] = acc;
    __syncthreads();
    if(threadIdx.x == 0) {
        const float s = part[0] + part[1] + part[2] + part[3];
        db[c] = (TB)(beta != 0.0f ? s + beta * (float)db[c] : s);
    }
}

__global__ void __launch_bounds__(256) fill_bytes(uint8_t *p, uint8_t v, size_t n)
{
    const size_t stride = (size_t)gridDim.x * blockDim.x;
    const size_t i0 = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    const uint32_t v4 = v * 0x01010101u;
    const size_t head = (size_t)((16 - ((uintptr_t)p & 15)) & 15);
    const size_t h = head < n ? head : n;
    for(size_t i = i0; i < h; i += stride)
        p[i] = v;
    uint4 *q = (uint4 *)(p + h);
    const size_t nv = (n - h) / 16;
    for(size_t i = i0; i < nv; i += stride)
        q[i] = make_uint4(v4, v4, v4, v4);
    for(size_t i = h + nv * 16 + i0; i < n; i += stride)
        p[i] = v;
}

} // namespace

// ---------------------------------------------------------------- dropout
// keep(i) for the logical element index i (N,C,H,W order) comes from a counter-based generator: a 64-bit
// mix of (seed, offset, i) whose top 32 bits are compared with prob * 2^32.  The backward pass calls the
// same function with the same key, so no mask is stored.
__device__ __forceinline__ bool dropout_keep(uint64_t key, uint64_t i, unsigned threshold)
{
    uint64_t z = key + i * 0x9e3779b97f4a7c15ull; // splitmix64 finaliser over a Weyl sequence
    z = (z ^ (z >> 30)) * 0xbf58476d1ce4e5b9ull;
    z = (z ^ (z >> 27)) * 0x94d049bb133111ebull;
    z ^= z >> 31;
    return (unsigned)(z >> 32) >= threshold;
}

template <typename T, bool READ_OLD>
__global__ void __launch_bounds__(256)
    dropout_k(DView out, DView a, int64_t total, int cl, uint64_t key, unsigned threshold, float scale, float beta)
{
    const int64_t stride = (int64_t)gridDim.x * blockDim.x;
    const int C = out.d[1], H = out.d[2], W = out.d[3];
    for(int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < total; i += stride) {
        int n, c, h, w;
        int64_t t = i;
        if(cl) { // walk in the order of a channels-last tensor's memory
            c = (int)(t % C);
            t /= C;
            w = (int)(t % W);
            t /= W;
            h = (int)(t % H);
            n = (int)(t / H);
        } else {
            w = (int)(t % W);
            t /= W;
            h = (int)(t % H);
            t /= H;
            c = (int)(t % C);
            n = (int)(t / C);
        }
        const int64_t logical = (((int64_t)n * C + c) * H + h) * W + w;
        const int64_t oa = n * a.s[0] + c * a.s[1] + h * a.s[2] + w * a.s[3];
        const int64_t oo = n * out.s[0] + c * out.s[1] + h * out.s[2] + w * out.s[3];
        float v = dropout_keep(key, (uint64_t)logical, threshold) ? (float)((const T *)a.ptr)[oa] * scale : 0.0f;
        if(READ_OLD)
            v += beta * (float)((T *)out.ptr)[oo];
        ((T *)out.ptr)[oo] = (T)v;
    }
}

static int dropout_launch(const SagaTensorView *a, const SagaTensorView *out, float prob, uint64_t seed, uint64_t offset,
                          float beta, saga_stream_t stream)
{
    if(!valid_view(a) || !valid_view(out) || !(prob >= 0.0f) || !(prob < 1.0f))
        return SAGA_HIP_EINVAL;
    if(!same_dims(a, out))
        return SAGA_HIP_ESHAPE;
    if(a->dtype != out->dtype || (a->dtype != SAGA_HALF && a->dtype != SAGA_FLOAT))
        return SAGA_HIP_EUNSUPPORTED;
    const int64_t total = view_elements(out);
    const int cl = out->dims[1] > 1 && out->strides[1] == 1;
    const unsigned threshold = (unsigned)((double)prob * 4294967296.0);
    const float scale = 1.0f / (1.0f - prob);
    // one key per (seed, call): the Weyl step inside dropout_keep spreads the element index
    uint64_t key = seed * 0xd1342543de82ef95ull + offset * 0x2545f4914f6cdd1dull + 0x632be59bd9b4e019ull;
    hipStream_t st = as_stream(stream);
    const int g = grid_for(total, 256, 256 * 32);
#define GO(T)                                                                                                   \
    do {                                                                                                        \
        if(beta != 0.0f)                                                                                        \
            dropout_k<T, true><<<g, 256, 0, st>>>(dview(out), dview(a), total, cl, key, threshold, scale, beta);  \
        else                                                                                                    \
            dropout_k<T, false><<<g, 256, 0, st>>>(dview(out), dview(a), total, cl, key, threshold, scale, 0.0f); \
    } while(0)
    if(a->dtype == SAGA_HALF)
        GO(half_t);
    else
        GO(float);
#undef GO
    SAGA_CHECK_LAUNCH();
    return 0;
}

extern "C" {

int saga_hip_act_fwd(int mode, float alpha, const SagaTensorView *x, const SagaTensorView *y, float beta,
                     saga_stream_t stream)
{
    if(mode < SAGA_ACT_RELU || mode > SAGA_ACT_LEAKYRELU)
        return SAGA_HIP_EINVAL;
    return launch_ew<1>(y, x, nullptr, beta != 0.0f, ActFwd{mode, alpha, beta}, as_stream(stream));
}

int saga_hip_act_bwd(int mode, float alpha, const SagaTensorView *x, const SagaTensorView *y,
                     const SagaTensorView *dy, const SagaTensorView *dx, float beta, saga_stream_t stream)
{
    if(mode < SAGA_ACT_RELU || mode > SAGA_ACT_LEAKYRELU)
        return SAGA_HIP_EINVAL;
    const bool uses_y = mode == SAGA_ACT_SIGMOID || mode == SAGA_ACT_TANH;
    const SagaTensorView *a = uses_y ? y : x;
    return launch_ew<2>(dx, a, dy, beta != 0.0f, ActBwd{mode, alpha, beta}, as_stream(stream));
}

int saga_hip_add(const SagaTensorView *a, const SagaTensorView *b, const SagaTensorView *y, saga_stream_t stream)
{
    return launch_ew<2>(y, a, b, false, AddFn{}, as_stream(stream));
}

int saga_hip_axpby(const SagaTensorView *src, const SagaTensorView *dst, float alpha, float beta,
                   saga_stream_t stream)
{
    return launch_ew<1>(dst, src, nullptr, beta != 0.0f, AxpbyFn{alpha, beta}, as_stream(stream));
}

int saga_hip_convert(const SagaTensorView *src, const SagaTensorView *dst, float scale, saga_stream_t stream)
{
    if(!valid_view(src) || !valid_view(dst))
        return SAGA_HIP_EINVAL;
    if(!same_dims(src, dst))
        return SAGA_HIP_ESHAPE;
    hipStream_t st = as_stream(stream);
    const int s = src->dtype, d = dst->dtype;
    if(s == d && (s == SAGA_HALF || s == SAGA_FLOAT))
        return saga_hip_axpby(src, dst, scale, 0.0f, stream);
    if(s == SAGA_U8 && d == SAGA_FLOAT) return launch_convert<uint8_t, float>(src, dst, scale, st);
    if(s == SAGA_U8 && d == SAGA_HALF) return launch_convert<uint8_t, half_t>(src, dst, scale, st);
    if(s == SAGA_I16 && d == SAGA_HALF) return launch_convert<int16_t, half_t>(src, dst, scale, st);
    if(s == SAGA_I16 && d == SAGA_FLOAT) return launch_convert<int16_t, float>(src, dst, scale, st);
    if(s == SAGA_FLOAT && d == SAGA_HALF) return launch_convert<float, half_t>(src, dst, scale, st);
    if(s == SAGA_HALF && d == SAGA_FLOAT) return launch_convert<half_t, float>(src, dst, scale, st);
    return SAGA_HIP_EUNSUPPORTED;
}

int saga_hip_bias_add(const SagaTensorView *y, const SagaTensorView *b, saga_stream_t stream)
{
    if(!valid_view(y) || !valid_view(b))
        return SAGA_HIP_EINVAL;
    if(view_elements(b) != y->dims[1])
        return SAGA_HIP_ESHAPE;
    hipStream_t st = as_stream(stream);
    const int64_t total = view_elements(y);
    CLInfo cl;
    CFInfo cf;
#define BIAS_ADD(T, TB)                                                                                       \
    if(as_channels_last(y, &cl))                                                                              \
        bias_add_cl<T, TB><<<grid_for(total, 256, 256 * 32), 256, 0, st>>>((T *)y->ptr, cl.pitch,               \
                                                                           (const TB *)b->ptr, cl.rows, cl.C); \
    else if(as_channels_first(y, &cf))                                                                        \
        bias_add_cf<T, TB><<<grid_for(total, 256, 256 * 32), 256, 0, st>>>((T *)y->ptr, cf.npitch,              \
                                                                           (const TB *)b->ptr, cf.N, cf.C, cf.HW); \
    else                                                                                                      \
        return SAGA_HIP_EUNSUPPORTED;
    if(y->dtype == SAGA_HALF && b->dtype == SAGA_HALF) {
        BIAS_ADD(half_t, half_t)
    } else if(y->dtype == SAGA_HALF && b->dtype == SAGA_FLOAT) {
        BIAS_ADD(half_t, float)
    } else if(y->dtype == SAGA_FLOAT && b->dtype == SAGA_FLOAT) {
        BIAS_ADD(float, float)
    } else
        return SAGA_HIP_EUNSUPPORTED;
#undef BIAS_ADD
    SAGA_CHECK_LAUNCH();
    return 0;
}

size_t saga_hip_bias_bwd_workspace_size(const SagaTensorView *dy)
{
    CLInfo cl;
    if(!valid_view(dy) || !as_channels_last(dy, &cl))
        return 0;
    const int gx = bias_bwd_splits(cl.rows, cl.C);
    return gx > 1 ? (size_t)gx * cl.C * sizeof(float) : 0;
}

// Shared by saga_hip_bias_bwd (the caller's workspace) and saga_hip_bias_bwd_noalloc (the library's scratch array).
static int bias_bwd_run(const SagaTensorView *dy, const SagaTensorView *db, float beta, void *workspace, size_t ws_bytes,
                        saga_stream_t stream)
{
    if(!valid_view(dy) || !valid_view(db))
        return SAGA_HIP_EINVAL;
    if(view_elements(db) != dy->dims[1])
        return SAGA_HIP_ESHAPE;
    hipStream_t st = as_stream(stream);
    CLInfo cl;
    CFInfo cf;
    const size_t need = saga_hip_bias_bwd_workspace_size(dy);
    if(need && (!workspace || ws_bytes < need))
        return SAGA_HIP_EWORKSPACE;
#define BIAS_BWD(T, TB)                                                                                     \
    if(as_channels_last(dy, &cl) && need) {                                                                 \
        const int gx = bias_bwd_splits(cl.rows, cl.C);                                                      \
        constexpr int VN = Vec<T>::n;                                                                       \
        if(cl.C % VN == 0 && cl.pitch % VN == 0 && (uintptr_t)dy->ptr % 16 == 0) {                          \
            int cvp = 1;                                                                                    \
            while(cvp < cl.C / VN && cvp < 256)                                                             \
                cvp *= 2;                                                                                   \
            bias_bwd_partial_vec<T><<<dim3(gx, (cl.C / VN + cvp - 1) / cvp), 256, 0, st>>>(                  \
                (const T *)dy->ptr, cl.pitch, (float *)workspace, cl.rows, cl.C, cvp);                      \
        } else                                                                                              \
            bias_bwd_partial_cl<T><<<dim3(gx, (cl.C + 63) / 64), 256, 0, st>>>(                             \
                (const T *)dy->ptr, cl.pitch, (float *)workspace, cl.rows, cl.C);                           \
        bias_bwd_final<TB><<<(cl.C + 31) / 32, 256, 0, st>>>((const float *)workspace, gx, (TB *)db->ptr,  \
                                                               cl.C, beta);                                 \
    } else if(as_channels_last(dy, &cl))                                                                    \
        bias_bwd_cl<T, TB><<<(cl.C + 63) / 64, 256, 0, st>>>((const T *)dy->ptr, cl.pitch, (TB *)db->ptr,     \
                                                             cl.rows, cl.C, beta);                          \
    else if(as_channels_first(dy, &cf))                                                                     \
        bias_bwd_cf<T, TB><<<cf.C, 256, 0, st>>>((const T *)dy->ptr, cf.npitch, (TB *)db->ptr, cf.N, cf.C,   \
                                                 cf.HW, beta);                                              \
    else                                                                                                    \
        return SAGA_HIP_EUNSUPPORTED;
    if(dy->dtype == SAGA_HALF && db->dtype == SAGA_HALF) {
        BIAS_BWD(half_t, half_t)
    } else if(dy->dtype == SAGA_HALF && db->dtype == SAGA_FLOAT) {
        BIAS_BWD(half_t, float)
    } else if(dy->dtype == SAGA_FLOAT && db->dtype == SAGA_FLOAT) {
        BIAS_BWD(float, float)
    } else
        return SAGA_HIP_EUNSUPPORTED;
#undef BIAS_BWD
    SAGA_CHECK_LAUNCH();
    return 0;
}

int saga_hip_bias_bwd(const SagaTensorView *dy, const SagaTensorView *db, float beta, void *workspace, size_t ws_bytes,
                      saga_stream_t stream)
{
    return bias_bwd_run(dy, db, beta, workspace, ws_bytes, stream);
}

// ---- the entry point that allocates nothing.  The per-block partial sums of the two-pass reduction go to a
// fixed array in device memory instead of a workspace.  Every GPU holds its own copy of the array at its own
// address, resolved once per device (saga_hip_init, or the first call on that device) and kept in
// bias_scratch_ptr; host code passes that pointer, never the array's name, to the kernels.  The partial kernels
// overwrite every [block][channel] entry the final kernel reads, so nothing has to be cleared between calls.
static __device__ __align__(256) float scratch[SAGA_HIP_BIAS_BWD_NOALLOC_MAX_BYTES / sizeof(float)];
static constexpr int MAX_SCRATCH_DEVICES = 64;
static std::atomic<float *> bias_scratch_ptr[MAX_SCRATCH_DEVICES];

// `device` must be the current device.
static int resolve_bias_scratch(int device, float **out)
{
    if(device < 0 || device >= MAX_SCRATCH_DEVICES)
        return SAGA_HIP_EINVAL;
    float *p = bias_scratch_ptr[device].load(std::memory_order_acquire);
    if(!p) {
        const hipError_t e = hipGetSymbolAddress((void **)&p, HIP_SYMBOL(scratch));
        if(e != hipSuccess)
            return (int)e;
        if(!p)
            return SAGA_HIP_EINVAL;
        bias_scratch_ptr[device].store(p, std::memory_order_release);
    }
    if(out)
        *out = p;
    return 0;
}

int saga_hip_bias_bwd_noalloc(const SagaTensorView *dy, const SagaTensorView *db, float beta, saga_stream_t stream)
{
    if(!valid_view(dy) || !valid_view(db))
        return SAGA_HIP_EINVAL;
    const size_t need = saga_hip_bias_bwd_workspace_size(dy);
    if(need > SAGA_HIP_BIAS_BWD_NOALLOC_MAX_BYTES)
        return SAGA_HIP_ETOOLARGE;
    float *ws = nullptr;
    if(need) {
        int device = -1;
        const hipError_t e = hipGetDevice(&device);
        if(e != hipSuccess)
            return (int)e;
        if(device < 0 || device >= MAX_SCRATCH_DEVICES)
            return SAGA_HIP_EINVAL;
        // the scratch array belongs to the current device: a stream of another device would hand its kernels
        // an address of the wrong GPU
        hipDevice_t stream_device = device;
        if(stream && hipStreamGetDevice(as_stream(stream), &stream_device) == hipSuccess && (int)stream_device != device)
            return SAGA_HIP_EINVAL;
        if(!bias_scratch_ptr[device].load(std::memory_order_acquire)) {
            // resolving the symbol loads the code object and materialises the array: not under stream capture,
            // where saga_hip_init(device) has to have done it beforehand
            hipStreamCaptureStatus capturing = hipStreamCaptureStatusNone;
            if(hipStreamIsCapturing(as_stream(stream), &capturing) == hipSuccess &&
               capturing != hipStreamCaptureStatusNone)
                return SAGA_HIP_EINVAL;
        }
        const int rc = resolve_bias_scratch(device, &ws);
        if(rc)
            return rc;
    }
    return bias_bwd_run(dy, db, beta, ws, need, stream);
}

int saga_hip_fill(void *ptr, int value, size_t bytes, saga_stream_t stream)
{
    if(!ptr && bytes)
        return SAGA_HIP_EINVAL;
    if(bytes == 0)
        return 0;
    fill_bytes<<<grid_for((int64_t)(bytes / 16 + 1), 256, 256 * 16), 256, 0, as_stream(stream)>>>(
        (uint8_t *)ptr, (uint8_t)value, bytes);
    SAGA_CHECK_LAUNCH();
    return 0;
}

const char *saga_hip_error_string(int code)
{
    switch(code) {
    case SAGA_HIP_OK: return "ok";
    case SAGA_HIP_EINVAL: return "invalid argument";
    case SAGA_HIP_ESHAPE: return "operand shapes do not agree";
    case SAGA_HIP_EUNSUPPORTED: return "unsupported dtype or layout";
    case SAGA_HIP_EWORKSPACE: return "workspace missing or too small";
    case SAGA_HIP_ETOOLARGE: return "operand needs more scratch than the entry point that allocates nothing holds";
    }
    if(code > 0)
        return hipGetErrorString((hipError_t)code);
    return "unknown error";
}

int saga_hip_init(int device, int *cus)
{
    hipError_t e = hipSetDevice(device);
    if(e != hipSuccess)
        return (int)e;
    hipDeviceProp_t prop;
    e = hipGetDeviceProperties(&prop, device);
    if(e != hipSuccess)
        return (int)e;
    if(cus)
        *cus = prop.multiProcessorCount;
    return resolve_bias_scratch(device, nullptr);
}

int saga_hip_dropout_fwd(const SagaTensorView *x, const SagaTensorView *y, float prob, uint64_t seed, uint64_t offset,
                         saga_stream_t stream)
{
    return dropout_launch(x, y, prob, seed, offset, 0.0f, stream);
}

int saga_hip_dropout_bwd(const SagaTensorView *dy, const SagaTensorView *dx, float prob, uint64_t seed, uint64_t offset,
                         float beta, saga_stream_t stream)
{
    return dropout_launch(dy, dx, prob, seed, offset, beta, stream);
}

} // extern "C"
