// True float32 matrix product C[M,N] = A[M,K] * W[N,K]^T on the matrix cores' float32
// instruction (v_mfma_f32_16x16x4_f32: float32 operands, float32 accumulation; no
// reduced-precision mode).
//
// One order of summation for every output element, whatever M, the tile it falls in or what
// else is in the batch, so that results are equal bit for bit however the rows are cut:
//   * K is cut in chunks of 16; the chunks are dealt to the 8 waves of a workgroup as 8
//     contiguous runs of ceil(chunks / 8);
//   * a wave walks its chunks in ascending order; a chunk is four matrix instructions on one
//     accumulator, instruction j taking the k  {j, 4 + j, 8 + j, 12 + j}  of the chunk (lane
//     group g supplies k = 4 g + j, from one 16-byte load of k = 4g .. 4g + 3);
//   * the 8 partial results are added in the order of the waves.
// k beyond K contribute zeros.
//
// The transposed product is computed (W supplies the A operand, the rows of A the B operand),
// so a lane's four results are four consecutive n of one row of C.  A workgroup owns NT x MT
// tiles of 16 x 16; NT and MT only decide how often an operand is reused.
#include "common.h"

typedef float f32x4 __attribute__((ext_vector_type(4)));

#define FW 8    // waves per workgroup = runs of K
#define FCH 16  // k per chunk
#define RED_TILES 4  // tiles reduced through LDS at a time

// four consecutive floats of a row, zeros beyond `limit` (elements left in the row)
template <bool VEC>
__device__ inline f32x4 load_k4(const float* p, int limit) {
    if (VEC) {
        if (limit >= 4) return *reinterpret_cast<const f32x4*>(p);
        return (f32x4){0.f, 0.f, 0.f, 0.f};  // VEC: K is a multiple of 4, a piece is whole or absent
    }
    f32x4 v;
#pragma unroll
    for (int i = 0; i < 4; ++i) v[i] = i < limit ? p[i] : 0.f;
    return v;
}

template <int NT, int MT, bool VEC>
__global__ __launch_bounds__(FW* RL_WAVE) void gemm_f32_kernel(
    const float* __restrict__ A, const float* __restrict__ W, float* __restrict__ C, int M, int N,
    int K, int lda, int ldw, int ldc) {
    __shared__ float red[FW][RED_TILES * 256];

    const int lane = threadIdx.x & (RL_WAVE - 1);
    const int wave = threadIdx.x / RL_WAVE;
    const int r16 = lane & 15;
    const int g = lane >> 4;
    const int n0 = blockIdx.x * NT * 16;
    const int m0 = blockIdx.y * MT * 16;

    // rows beyond the matrices read the last row; their results are dropped at the end
    const float* wrow[NT];
    const float* arow[MT];
    bool aok[MT];
#pragma unroll
    for (int nt = 0; nt < NT; ++nt)
        wrow[nt] = W + (size_t)min(n0 + nt * 16 + r16, N - 1) * ldw + 4 * g;
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) {
        aok[mt] = m0 + mt * 16 + r16 < M;
        arow[mt] = A + (size_t)min(m0 + mt * 16 + r16, M - 1) * lda + 4 * g;
    }

    f32x4 acc[NT][MT];
#pragma unroll
    for (int nt = 0; nt < NT; ++nt)
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) acc[nt][mt] = (f32x4){0.f, 0.f, 0.f, 0.f};

    const int chunks = (K + FCH - 1) / FCH;
    const int per = (chunks + FW - 1) / FW;
    const int c_lo = min(chunks, wave * per), c_hi = min(chunks, c_lo + per);

    // With one tile (few rows: the weights are streamed once) four chunks are asked for
    // together, so that the four lane groups read 256 contiguous bytes of every row and more
    // loads are in flight; the products still run chunk by chunk in ascending order
    constexpr int U = (NT * MT == 1) ? 4 : 1;
    f32x4 wv[U][NT], av[U][MT], wn[U][NT], an[U][MT];
    auto load = [&](int c, f32x4* wd, f32x4* ad) {
        const int k = c * FCH + 4 * g;  // this lane's first k of the chunk
#pragma unroll
        for (int nt = 0; nt < NT; ++nt) wd[nt] = load_k4<VEC>(wrow[nt] + c * FCH, K - k);
#pragma unroll
        for (int mt = 0; mt < MT; ++mt)
            ad[mt] = aok[mt] ? load_k4<VEC>(arow[mt] + c * FCH, K - k) : (f32x4){0.f, 0.f, 0.f, 0.f};
    };
    auto load_group = [&](int c, f32x4 (*wd)[NT], f32x4 (*ad)[MT]) {
#pragma unroll
        for (int u = 0; u < U; ++u)
            if (c + u < c_hi) load(c + u, wd[u], ad[u]);
    };
    if (c_lo < c_hi) load_group(c_lo, wv, av);
    for (int c = c_lo; c < c_hi; c += U) {
        if (c + U < c_hi) load_group(c + U, wn, an);  // the next group's loads fly during this one's products
#pragma unroll
        for (int u = 0; u < U; ++u) {
            if (c + u >= c_hi) break;
#pragma unroll
            for (int j = 0; j < 4; ++j)
#pragma unroll
                for (int nt = 0; nt < NT; ++nt)
#pragma unroll
                    for (int mt = 0; mt < MT; ++mt)
                        acc[nt][mt] = __builtin_amdgcn_mfma_f32_16x16x4f32(wv[u][nt][j], av[u][mt][j],
                                                                          acc[nt][mt], 0, 0, 0);
        }
#pragma unroll
        for (int u = 0; u < U; ++u) {
#pragma unroll
            for (int nt = 0; nt < NT; ++nt) wv[u][nt] = wn[u][nt];
#pragma unroll
            for (int mt = 0; mt < MT; ++mt) av[u][mt] = an[u][mt];
        }
    }

    // the waves' partial tiles are added in the order of the waves, RED_TILES tiles at a time
    constexpr int TILES = NT * MT;
#pragma unroll
    for (int t0 = 0; t0 < TILES; t0 += RED_TILES) {
        if (t0 > 0) __syncthreads();
#pragma unroll
        for (int t = t0; t < t0 + RED_TILES && t < TILES; ++t)
#pragma unroll
            for (int i = 0; i < 4; ++i)
                red[wave][((t - t0) * 4 + i) * 64 + lane] = acc[t / MT][t % MT][i];
        __syncthreads();
        const int count = min(RED_TILES, TILES - t0) * 256;
        for (int e = threadIdx.x; e < count; e += FW * RL_WAVE) {
            const int ln = e & 63;
            const int i = (e >> 6) & 3;
            const int t = t0 + (e >> 8);
            const int n = n0 + (t / MT) * 16 + 4 * (ln >> 4) + i;
            const int m = m0 + (t % MT) * 16 + (ln & 15);
            if (n >= N || m >= M) continue;
            float v = red[0][e];
#pragma unroll
            for (int w = 1; w < FW; ++w) v += red[w][e];
            C[(size_t)m * ldc + n] = v;
        }
    }
}

template <int NT, int MT>
static int launch(const float* A, const float* W, float* C, int M, int N, int K, int lda, int ldw,
                  int ldc, hipStream_t stream) {
    dim3 grid((N + NT * 16 - 1) / (NT * 16), (M + MT * 16 - 1) / (MT * 16)), block(FW * RL_WAVE);
    if (grid.y > 65535) return RL_ERR_ARG;
    const bool vec = K % 4 == 0 && lda % 4 == 0 && ldw % 4 == 0 &&
                     (reinterpret_cast<uintptr_t>(A) & 15) == 0 &&
                     (reinterpret_cast<uintptr_t>(W) & 15) == 0;
    if (vec)
        hipLaunchKernelGGL((gemm_f32_kernel<NT, MT, true>), grid, block, 0, stream, A, W, C, M, N, K,
                           lda, ldw, ldc);
    else
        hipLaunchKernelGGL((gemm_f32_kernel<NT, MT, false>), grid, block, 0, stream, A, W, C, M, N,
                           K, lda, ldw, ldc);
    return rl_launch_status();
}

// Rows of A and W may be strided; the inner dimension is contiguous.  The tiling follows M:
// few rows stream the weights once with as many workgroups as there are 16-row tiles of W;
// many rows reuse each operand four times.
extern "C" int rl_gemm_f32(const float* A, const float* W, float* C, int M, int N, int K, int lda,
                           int ldw, int ldc, hipStream_t stream) {
    if (M <= 0 || N <= 0) return RL_OK;
    if (K <= 0 || lda < K || ldw < K || ldc < N) return RL_ERR_ARG;
    if (M <= 16) return launch<1, 1>(A, W, C, M, N, K, lda, ldw, ldc, stream);
    if (M <= 32) return launch<2, 2>(A, W, C, M, N, K, lda, ldw, ldc, stream);
    return launch<4, 4>(A, W, C, M, N, K, lda, ldw, ldc, stream);
}
