// True 32-bit matrix product: C[M,N] (+)= A[M,K] * W[N,K]^T with float FMA only (no
// matrix-core reduced-precision mode).  Every output element is accumulated over k in
// ascending order by one thread, so its value does not depend on M, on the tile it
// falls in, or on the other rows of the batch.
//
// reference: op_linear_proj, kernels/megakernel_ops.hip:166-276 (one block per output
// row, f32 accumulate); the LDS-tiled 64x64x16 form here is the CDNA layout of the
// same sum.
#include "common.h"

#define BM 64
#define BN 64
#define BK 16

// mode 0: C = AW^T ; mode 1: C += AW^T (C holds the residual stream)
template <int MODE>
__global__ __launch_bounds__(256) void gemm_f32_kernel(const float* __restrict__ A, const float* __restrict__ W,
                                                       float* __restrict__ C, int M, int N, int K,
                                                       size_t lda, size_t ldc) {
    __shared__ float As[BK][BM + 4];
    __shared__ float Ws[BK][BN + 4];
    const int tid = threadIdx.x;
    const int tx = tid & 15, ty = tid >> 4;
    const int m0 = blockIdx.y * BM, n0 = blockIdx.x * BN;
    const int lr = tid >> 2, lk = (tid & 3) * 4;  // loader: row lr, k offset lk..lk+3
    float acc[4][4];
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[i][j] = 0.f;

    for (int k0 = 0; k0 < K; k0 += BK) {
        {
            const int m = m0 + lr, n = n0 + lr;
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                const int k = k0 + lk + e;
                As[lk + e][lr] = (m < M && k < K) ? A[(size_t)m * lda + k] : 0.f;
                Ws[lk + e][lr] = (n < N && k < K) ? W[(size_t)n * K + k] : 0.f;
            }
        }
        __syncthreads();
#pragma unroll
        for (int k = 0; k < BK; ++k) {
            float a[4], w[4];
#pragma unroll
            for (int i = 0; i < 4; ++i) a[i] = As[k][ty * 4 + i];
#pragma unroll
            for (int j = 0; j < 4; ++j) w[j] = Ws[k][tx * 4 + j];
#pragma unroll
            for (int i = 0; i < 4; ++i)
#pragma unroll
                for (int j = 0; j < 4; ++j) acc[i][j] = fmaf(a[i], w[j], acc[i][j]);
        }
        __syncthreads();
    }
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const int m = m0 + ty * 4 + i;
        if (m >= M) continue;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int n = n0 + tx * 4 + j;
            if (n >= N) continue;
            float* c = C + (size_t)m * ldc + n;
            if (MODE == 1) *c = *c + acc[i][j]; else *c = acc[i][j];
        }
    }
}

extern "C" int br_gemm_f32(const float* A, const float* W, float* C, int M, int N, int K,
                           size_t lda, size_t ldc, int accumulate, hipStream_t s) {
    if (M <= 0 || N <= 0) return BR_OK;
    if (K <= 0 || lda < (size_t)K || ldc < (size_t)N) return BR_BAD_ARG;
    dim3 grid((N + BN - 1) / BN, (M + BM - 1) / BM);
    if (grid.y > 65535) return BR_BAD_ARG;
    if (accumulate) gemm_f32_kernel<1><<<grid, 256, 0, s>>>(A, W, C, M, N, K, lda, ldc);
    else gemm_f32_kernel<0><<<grid, 256, 0, s>>>(A, W, C, M, N, K, lda, ldc);
    return br_check_launch();
}
