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
#pragma unroll
    for (int nt = 0; nt < NT; ++nt)
        wrow[nt] = W + (size_t)min(n0 + nt * 16 + r16, N - 1) * ldw + 4 * g;
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) arow[mt] = A + (size_t)min(m0 + mt * 16 + r16, M - 1) * lda + 4 * g;

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
    // loads are in flight; the products still run chunk by chunk in ascending order.
    constexpr int U = (NT * MT == 1) ? 4 : 1;
    // a chunk's operands: rows beyond A read A's last row (their results are dropped), so
    // that no load depends on the lane
    auto load = [&](int c, f32x4 (&wd)[NT], f32x4 (&ad)[MT]) {  // a whole chunk: no predicate
#pragma unroll
        for (int nt = 0; nt < NT; ++nt) wd[nt] = *reinterpret_cast<const f32x4*>(wrow[nt] + c * FCH);
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) ad[mt] = *reinterpret_cast<const f32x4*>(arow[mt] + c * FCH);
    };
    auto load_checked = [&](int c, f32x4 (&wd)[NT], f32x4 (&ad)[MT]) {
        const int k = c * FCH + 4 * g;  // this lane's first k of the chunk
#pragma unroll
        for (int nt = 0; nt < NT; ++nt) wd[nt] = load_k4<VEC>(wrow[nt] + c * FCH, K - k);
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) ad[mt] = load_k4<VEC>(arow[mt] + c * FCH, K - k);
    };
    auto products = [&](f32x4 (&wd)[NT], f32x4 (&ad)[MT]) {
#pragma unroll
        for (int j = 0; j < 4; ++j)
#pragma unroll
            for (int nt = 0; nt < NT; ++nt)
#pragma unroll
                for (int mt = 0; mt < MT; ++mt)
                    acc[nt][mt] =
                        __builtin_amdgcn_mfma_f32_16x16x4f32(wd[nt][j], ad[mt][j], acc[nt][mt], 0, 0, 0);
    };
    auto load_group = [&](int c, f32x4 (&wd)[U][NT], f32x4 (&ad)[U][MT]) {
#pragma unroll
        for (int u = 0; u < U; ++u) load(c + u, wd[u], ad[u]);
        // the loads stay here, in front of the other group's products (left to itself the
        // scheduler moves them down to their use and nothing is in flight during the products)
        __builtin_amdgcn_sched_barrier(0);
    };
    auto group_products = [&](f32x4 (&wd)[U][NT], f32x4 (&ad)[U][MT]) {
#pragma unroll
        for (int u = 0; u < U; ++u) products(wd[u], ad[u]);
    };
    // Groups of whole chunks go through two sets of registers in turn: the group after next
    // is asked for before this one is multiplied.  Inside the loop no load stands behind a
    // condition (behind one the compiler counts it as absent and makes the oldest operand wait
    // for the newest load); what the loop leaves, and the chunks that are not whole or do not
    // fill a group, follow one by one.  The order of the sum is that of the chunks either way.
    int c = c_lo;
    {
        const int whole = VEC ? min(c_hi, K / FCH) : c_lo;  // unaligned rows: every chunk is checked
        int left = whole > c_lo ? (whole - c_lo) / U : 0;
        if (left > 0) {
            f32x4 wa[U][NT], aa[U][MT], wb[U][NT], ab[U][MT];
            load_group(c, wa, aa);
            while (left > 2) {
                load_group(c + U, wb, ab);
                group_products(wa, aa);
                load_group(c + 2 * U, wa, aa);
                group_products(wb, ab);
                c += 2 * U;
                left -= 2;
            }
            if (left == 2) {
                load_group(c + U, wb, ab);
                group_products(wa, aa);
                group_products(wb, ab);
                c += 2 * U;
            } else {
                group_products(wa, aa);
                c += U;
            }
        }
    }
    for (; c < c_hi; ++c) {
        f32x4 w1[NT], a1[MT];
        load_checked(c, w1, a1);
        products(w1, a1);
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
