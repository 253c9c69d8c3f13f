// Row-major GEMM used by the fully-connected node: C = alpha*op(A)*op(B) + beta*C.
// LDS-tiled 64x64x16 with a 4x4 register block per lane and fp32 accumulation; either
// operand may be stored transposed.  (The fc layers of the target networks are a small
// fraction of the step; convolutions take the MFMA path in conv_mfma.hip.)
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
    if(dtype == SAGA_HALF)
        gemm_tiled<half_t><<<grid, 256, 0, st>>>(transA, transB, M, N, K, alpha, (const half_t *)A, lda,
                                                 (const half_t *)B, ldb, beta, (half_t *)C, ldc);
    else if(dtype == SAGA_FLOAT)
        gemm_tiled<float><<<grid, 256, 0, st>>>(transA, transB, M, N, K, alpha, (const float *)A, lda,
                                                (const float *)B, ldb, beta, (float *)C, ldc);
    else
        return SAGA_HIP_EUNSUPPORTED;
    SAGA_CHECK_LAUNCH();
    return 0;
}
