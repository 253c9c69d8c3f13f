// Row-major GEMM used by the fully-connected node: C = alpha*op(A)*op(B) + beta*C, either
// operand may be stored transposed.
//  * fp16: gemm_mfma_f16, 64x64x32 block tiles on v_mfma_f32_32x32x16_f16 (one 32x32 tile per
//    wave), operands staged through LDS with the reduction index contiguous; an operand
//    stored with the other index contiguous is transposed on its way into LDS.
//  * fp32: gemm_mfma_f32, the same 64x64x16 LDS tiles on v_mfma_f32_32x32x2_f32 (gemm_tiled, a 4x4
//    register block per lane, is kept as the non-matrix-core reference of the same tiling).
#include "common.hpp"

namespace {

template <typename T>
__global__ void __launch_bounds__(256)
    gemm_tiled(int tA, int tB, int M, int N, int K, float alpha, const T *__restrict__ A, int lda,
               const T *__restrict__ B, int ldb, float beta, T *__restrict__ C, int ldc)
{
    constexpr int BM = 64, BN = 64, BK = 16;
    __shared__ float As[BK][BM + 4];
    __shared__ float Bs[BK][BN + 4];
    const int tid = threadIdx.x;
    const int tx = tid % 16, ty = tid / 16;
    const int m0 = blockIdx.y * BM, n0 = blockIdx.x * BN;
    float acc[4][4] = {};
    for(int k0 = 0; k0 < K; k0 += BK) {
        // A tile: BM x BK
        for(int e = tid; e < BM * BK; e += 256) {
            int mm, kk;
            if(tA) { mm = e % BM; kk = e / BM; } else { kk = e % BK; mm = e / BK; }
            const int gm = m0 + mm, gk = k0 + kk;
            float v = 0;
            if(gm < M && gk < K)
                v = (float)(tA ? A[(int64_t)gk * lda + gm] : A[(int64_t)gm * lda + gk]);
            As[kk][mm] = v;
        }
        for(int e = tid; e < BN * BK; e += 256) {
            int nn, kk;
            if(tB) { kk = e % BK; nn = e / BK; } else { nn = e % BN; kk = e / BN; }
            const int gn = n0 + nn, gk = k0 + kk;
            float v = 0;
            if(gn < N && gk < K)
                v = (float)(tB ? B[(int64_t)gn * ldb + gk] : B[(int64_t)gk * ldb + gn]);
            Bs[kk][nn] = v;
        }
        __syncthreads();
#pragma unroll
        for(int kk = 0; kk < BK; kk++) {
            float a[4], b[4];
#pragma unroll
            for(int i = 0; i < 4; i++) {
                a[i] = As[kk][ty * 4 + i];
                b[i] = Bs[kk][tx * 4 + i];
            }
#pragma unroll
            for(int i = 0; i < 4; i++)
#pragma unroll
                for(int j = 0; j < 4; j++)
                    acc[i][j] += a[i] * b[j];
        }
        __syncthreads();
    }
#pragma unroll
    for(int i = 0; i < 4; i++) {
        const int gm = m0 + ty * 4 + i;
        if(gm >= M)
            continue;
#pragma unroll
        for(int j = 0; j < 4; j++) {
            const int gn = n0 + tx * 4 + j;
            if(gn >= N)
                continue;
            T *o = C + (int64_t)gm * ldc + gn;
            const float v = alpha * acc[i][j];
            *o = (T)(beta != 0.0f ? v + beta * (float)*o : v);
        }
    }
}

// fp32 on the matrix cores: the tiles of gemm_tiled, multiplied with v_mfma_f32_32x32x2_f32 (one
// 32x32 tile per wavefront, 8 instructions per 16-deep slice) instead of a 4x4 register block per
// lane.  A lane feeds A[m = lane%32][k = lane/32] and B[k][n = lane%32] and ends up with column
// n = lane%32, rows 8*(v/4) + 4*(lane/32) + v%4 of the tile.
__global__ void __launch_bounds__(256)
    gemm_mfma_f32(int tA, int tB, int M, int N, int K, float alpha, const float *__restrict__ A, int lda,
                  const float *__restrict__ B, int ldb, float beta, float *__restrict__ C, int ldc)
{
    typedef float float16_t __attribute__((ext_vector_type(16)));
    constexpr int BM = 64, BN = 64, BK = 16;
    __shared__ float As[BK][BM + 4];
    __shared__ float Bs[BK][BN + 4];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int m0 = blockIdx.y * BM, n0 = blockIdx.x * BN;
    const int wr = (wave >> 1) * 32, wc = (wave & 1) * 32;
    const int fr = lane & 31, fk = lane >> 5;
    float16_t acc;
#pragma unroll
    for(int v = 0; v < 16; v++)
        acc[v] = 0.0f;
    for(int k0 = 0; k0 < K; k0 += BK) {
        for(int e = tid; e < BM * BK; e += 256) {
            int mm, kk;
            if(tA) { mm = e % BM; kk = e / BM; } else { kk = e % BK; mm = e / BK; }
            const int gm = m0 + mm, gk = k0 + kk;
            float v = 0;
            if(gm < M && gk < K)
                v = tA ? A[(int64_t)gk * lda + gm] : A[(int64_t)gm * lda + gk];
            As[kk][mm] = v;
        }
        for(int e = tid; e < BN * BK; e += 256) {
            int nn, kk;
            if(tB) { kk = e % BK; nn = e / BK; } else { nn = e % BN; kk = e / BN; }
            const int gn = n0 + nn, gk = k0 + kk;
            float v = 0;
            if(gn < N && gk < K)
                v = tB ? B[(int64_t)gn * ldb + gk] : B[(int64_t)gk * ldb + gn];
            Bs[kk][nn] = v;
        }
        __syncthreads();
#pragma unroll
        for(int kk = 0; kk < BK / 2; kk++)
            acc = __builtin_amdgcn_mfma_f32_32x32x2f32(As[2 * kk + fk][wr + fr], Bs[2 * kk + fk][wc + fr], acc, 0, 0, 0);
        __syncthreads();
    }
    const int gn = n0 + wc + fr;
    if(gn >= N)
        return;
#pragma unroll
    for(int v = 0; v < 16; v++) {
        const int gm = m0 + wr + 8 * (v >> 2) + 4 * fk + (v & 3);
        if(gm >= M)
            continue;
        float *o = C + (int64_t)gm * ldc + gn;
        const float r = alpha * acc[v];
        *o = beta != 0.0f ? r + beta * *o : r;
    }
}

// One operand tile (64 rows x 32 reduction steps) from global memory into LDS rows of LDK
// halves.  kcontig: element (row, k) is at base[row*ld + k], else at base[k*ld + row].
// Every lane moves 8 elements that are contiguous in memory, with one 16-byte load when the
// run is in range and aligned.
// An iteration of the main loop takes GBK = 128 reduction steps (four 32-wide pieces per operand, eight 16-byte
// loads per lane in flight): with 32 the loop of a tall reduction (fc 2048 -> 1000 at batch 256: 64 blocks of 64
// iterations) paid one trip to memory per iteration and took 69 us; LDS rows are GLDK halves.
constexpr int GBK = 128;
constexpr int GLDK = GBK + 8;

__device__ __forceinline__ void gemm_stage(half_t (*dst)[GLDK], const half_t *__restrict__ base, int ld, bool kcontig,
                                           int row0, int rows, int k0, int K, bool vec_ok, int tid)
{
    half8_t v;
    if(kcontig) {
        const int r = tid >> 2, kk = (tid & 3) * 8;
        const int gr = row0 + r, gk = k0 + kk;
        const half_t *src = base + (int64_t)gr * ld + gk;
        if(vec_ok && gr < rows && gk + 8 <= K) {
            v = *(const half8_t *)src;
        } else {
#pragma unroll
            for(int j = 0; j < 8; j++)
                v[j] = (gr < rows && gk + j < K) ? src[j] : (half_t)0;
        }
        *(half8_t *)&dst[r][kk] = v;
    } else {
        const int kk = tid >> 3, r = (tid & 7) * 8;
        const int gr = row0 + r, gk = k0 + kk;
        const half_t *src = base + (int64_t)gk * ld + gr;
        if(vec_ok && gk < K && gr + 8 <= rows) {
            v = *(const half8_t *)src;
        } else {
#pragma unroll
            for(int j = 0; j < 8; j++)
                v[j] = (gk < K && gr + j < rows) ? src[j] : (half_t)0;
        }
#pragma unroll
        for(int j = 0; j < 8; j++)
            dst[r + j][kk] = v[j];
    }
}

__global__ void __launch_bounds__(256)
    gemm_mfma_f16(int tA, int tB, int M, int N, int K, float alpha, const half_t *__restrict__ A, int lda,
                  const half_t *__restrict__ B, int ldb, float beta, half_t *__restrict__ C, int ldc, int a_vec,
                  int b_vec)
{
    __shared__ __attribute__((aligned(16))) half_t As[2][64][GLDK];
    __shared__ __attribute__((aligned(16))) half_t Bs[2][64][GLDK];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int m0 = blockIdx.y * 64, n0 = blockIdx.x * 64;
    const int wm = (wave >> 1) * 32, wn = (wave & 1) * 32;
    float16_t acc;
#pragma unroll
    for(int v = 0; v < 16; v++)
        acc[v] = 0.0f;
    const int frow = lane & 31, fk = (lane >> 5) * 8;
    const int KT = (K + GBK - 1) / GBK;
    // Vector path (both operands 16-byte loadable): all eight loads of an iteration are issued before the first
    // LDS write waits for one - branch-free, out-of-range runs read the operand's first bytes and are zeroed -
    // so an iteration pays one trip to memory, not eight.
    const bool fast = a_vec && b_vec;
    auto fetch = [&](const half_t *__restrict__ base, int ld, bool kcontig, int row0, int rows, int k0, bool &ok) {
        int gr, gk;
        if(kcontig) {
            gr = row0 + (tid >> 2); gk = k0 + (tid & 3) * 8;
            ok = gr < rows && gk + 8 <= K;
            return *(const half8_t *)(base + (ok ? (int64_t)gr * ld + gk : 0));
        }
        gk = k0 + (tid >> 3); gr = row0 + (tid & 7) * 8;
        ok = gk < K && gr + 8 <= rows;
        return *(const half8_t *)(base + (ok ? (int64_t)gk * ld + gr : 0));
    };
    auto put = [&](half_t(*dst)[GLDK], bool kcontig, half8_t v, bool ok) {
        if(!ok)
            v = half8_t{0, 0, 0, 0, 0, 0, 0, 0};
        if(kcontig) {
            *(half8_t *)&dst[tid >> 2][(tid & 3) * 8] = v;
        } else {
#pragma unroll
            for(int j = 0; j < 8; j++)
                dst[(tid & 7) * 8 + j][tid >> 3] = v[j];
        }
    };
    // a run that is only partly in range (K or the row count no multiple of 8) is rare: those tiles take the
    // element-wise path of gemm_stage
    auto partial = [&](int row0, int rows, int k0, bool kcontig) {
        return kcontig ? (K % 8 != 0 && k0 + GBK > K) : (rows % 8 != 0 && row0 + 64 > rows);
    };
    auto stage = [&](int buf, int k0) {
        if(fast && !partial(m0, M, k0, !tA) && !partial(n0, N, k0, tB)) {
            half8_t va[GBK / 32], vb[GBK / 32];
            bool oa[GBK / 32], ob[GBK / 32];
#pragma unroll
            for(int j = 0; j < GBK / 32; j++) {
                va[j] = fetch(A, lda, !tA, m0, M, k0 + 32 * j, oa[j]);
                vb[j] = fetch(B, ldb, tB, n0, N, k0 + 32 * j, ob[j]);
            }
#pragma unroll
            for(int j = 0; j < GBK / 32; j++) {
                put((half_t(*)[GLDK]) & As[buf][0][32 * j], !tA, va[j], oa[j]);
                put((half_t(*)[GLDK]) & Bs[buf][0][32 * j], tB, vb[j], ob[j]);
            }
            return;
        }
#pragma unroll
        for(int j = 0; j < GBK / 32; j++) {
            gemm_stage((half_t(*)[GLDK]) & As[buf][0][32 * j], A, lda, !tA, m0, M, k0 + 32 * j, K, a_vec, tid);
            gemm_stage((half_t(*)[GLDK]) & Bs[buf][0][32 * j], B, ldb, tB, n0, N, k0 + 32 * j, K, b_vec, tid);
        }
    };
    stage(0, 0);
    for(int kt = 0; kt < KT; kt++) {
        __syncthreads();
        const int cur = kt & 1;
        if(kt + 1 < KT)
            stage(cur ^ 1, (kt + 1) * GBK);
#pragma unroll
        for(int kk = 0; kk < GBK / 16; kk++) {
            const half8_t fa = *(const half8_t *)&As[cur][wm + frow][kk * 16 + fk];
            const half8_t fb = *(const half8_t *)&Bs[cur][wn + frow][kk * 16 + fk];
            acc = __builtin_amdgcn_mfma_f32_32x32x16_f16(fa, fb, acc, 0, 0, 0);
        }
    }
    const int n = n0 + wn + (lane & 31);
    if(n >= N)
        return;
#pragma unroll
    for(int v = 0; v < 16; v++) {
        const int m = m0 + wm + (v >> 2) * 8 + (lane >> 5) * 4 + (v & 3);
        if(m >= M)
            continue;
        half_t *o = C + (int64_t)m * ldc + n;
        const float r = alpha * acc[v];
        *o = (half_t)(beta != 0.0f ? r + beta * (float)*o : r);
    }
}

} // namespace

extern "C" int saga_hip_gemm(int transA, int transB, int M, int N, int K, float alpha, const void *A, int lda,
                             const void *B, int ldb, float beta, void *C, int ldc, int dtype, saga_stream_t stream)
{
    if(!A || !B || !C || M < 1 || N < 1 || K < 1)
        return SAGA_HIP_EINVAL;
    if(lda < (transA ? M : K) || ldb < (transB ? K : N) || ldc < N)
        return SAGA_HIP_ESHAPE;
    dim3 grid((N + 63) / 64, (M + 63) / 64);
    hipStream_t st = as_stream(stream);
    if(dtype == SAGA_HALF) {
        const int a_vec = lda % 8 == 0 && ((uintptr_t)A & 15) == 0, b_vec = ldb % 8 == 0 && ((uintptr_t)B & 15) == 0;
        gemm_mfma_f16<<<grid, 256, 0, st>>>(transA, transB, M, N, K, alpha, (const half_t *)A, lda, (const half_t *)B,
                                            ldb, beta, (half_t *)C, ldc, a_vec, b_vec);
    } else if(dtype == SAGA_FLOAT)
        gemm_mfma_f32<<<grid, 256, 0, st>>>(transA, transB, M, N, K, alpha, (const float *)A, lda, (const float *)B, ldb,
                                            beta, (float *)C, ldc);
    else
        return SAGA_HIP_EUNSUPPORTED;
    SAGA_CHECK_LAUNCH();
    return 0;
}
