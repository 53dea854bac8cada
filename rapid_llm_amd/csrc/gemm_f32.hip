// True float32 matrix product C[M,N] = A[M,K] * W[N,K]^T with float32 FMA only: no matrix
// cores, no reduced-precision mode.  The sum over k runs in ascending order in every
// thread, so an output element does not depend on M, on the tile it falls in, or on what
// else is in the batch.
#include "common.h"

#define TM 64
#define TN 64
#define TK 16
#define PAD 1

__global__ __launch_bounds__(256) void gemm_f32_kernel(const float* __restrict__ A,
                                                       const float* __restrict__ W,
                                                       float* __restrict__ C, int M, int N, int K,
                                                       int lda, int ldw, int ldc) {
    __shared__ float As[TK][TM + PAD];
    __shared__ float Ws[TK][TN + PAD];
    const int tid = threadIdx.x;
    const int m0 = blockIdx.y * TM;
    const int n0 = blockIdx.x * TN;
    const int lr = tid / 4;        // 0..63: row of the tile this thread loads
    const int lk = (tid % 4) * 4;  // 0,4,8,12: first of its four k
    const int ty = tid / 16, tx = tid % 16;
    float acc[4][4];
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[i][j] = 0.f;

    for (int k0 = 0; k0 < K; k0 += TK) {
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const int k = k0 + lk + i;
            const int am = m0 + lr, wn = n0 + lr;
            As[lk + i][lr] = (am < M && k < K) ? A[(size_t)am * lda + k] : 0.f;
            Ws[lk + i][lr] = (wn < N && k < K) ? W[(size_t)wn * ldw + k] : 0.f;
        }
        __syncthreads();
#pragma unroll
        for (int k = 0; k < TK; ++k) {
            float a[4], b[4];
#pragma unroll
            for (int i = 0; i < 4; ++i) a[i] = As[k][ty * 4 + i];
#pragma unroll
            for (int j = 0; j < 4; ++j) b[j] = Ws[k][tx * 4 + j];
#pragma unroll
            for (int i = 0; i < 4; ++i)
#pragma unroll
                for (int j = 0; j < 4; ++j) acc[i][j] = fmaf(a[i], b[j], acc[i][j]);
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
            if (n < N) C[(size_t)m * ldc + n] = acc[i][j];
        }
    }
}

extern "C" int rl_gemm_f32(const float* A, const float* W, float* C, int M, int N, int K, int lda,
                           int ldw, int ldc, hipStream_t stream) {
    if (M <= 0 || N <= 0) return RL_OK;
    if (K <= 0 || lda < K || ldw < K || ldc < N) return RL_ERR_ARG;
    dim3 grid((N + TN - 1) / TN, (M + TM - 1) / TM), block(256);
    if (grid.y > 65535) return RL_ERR_ARG;
    hipLaunchKernelGGL(gemm_f32_kernel, grid, block, 0, stream, A, W, C, M, N, K, lda, ldw, ldc);
    return rl_launch_status();
}
