// Bandwidth-bound bfloat16 product for few rows (decode): out[M,N] = X[M,K] * W[N,K]^T with
// M <= 64, float32 accumulation on the matrix cores, optionally fused with SwiGLU.
//
// Every weight byte is read once, in long contiguous runs: a workgroup owns NT tiles of 16
// weight rows and its 8 waves interleave over K in steps of 128 elements, so that at any
// moment the waves of a group stream 2 KB of each row.  The transposed product is computed,
//   C^T[n, m] = W[n, k] * X^T[k, m]        (A = W tile, B = X^T),
// so W is the A operand exactly as it lies in memory: lane (n = lane % 16, g = lane / 16)
// loads the 64 contiguous bytes W[n][k0 + 32 g .. + 31] and feeds its four 8-element pieces
// to four v_mfma_f32_16x16x32_bf16; X supplies the same k pieces as the B operand.  The
// waves' partial tiles are added through LDS in a fixed order (no atomics).
//
// With SWIGLU the workgroup's tiles alternate between gate rows n and up rows I + n of the
// packed [gate | up] matrix and the epilogue writes silu(gate) * up
// (rapid_llm/kernels/ops/activation/swiglu.py:91-121), so the [M, 2I] intermediate never
// exists.
#include "common.h"

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float f32x4 __attribute__((ext_vector_type(4)));

#define GW 8            // waves per workgroup
#define KSTEP 128       // k elements one wave consumes per iteration

__device__ inline bf16x8 ld16(const bf16_t* p) {
    return __builtin_bit_cast(bf16x8, *reinterpret_cast<const uint4*>(p));
}
__device__ inline bf16x8 z8() {
    bf16x8 z;
#pragma unroll
    for (int i = 0; i < 8; ++i) z[i] = (__bf16)0.f;
    return z;
}

template <typename T>
__device__ inline void store_out(T* p, float v);
template <>
__device__ inline void store_out<float>(float* p, float v) {
    *p = v;
}
template <>
__device__ inline void store_out<bf16_t>(bf16_t* p, float v) {
    *p = float_to_bf16(v);
}

// MB: blocks of 16 rows of X (M <= 16 MB); NT: tiles of 16 weight rows per workgroup.
// SWIGLU: tiles 2j / 2j+1 are gate rows / up rows; N is then the width I of the result.
template <int MB, int NT, typename OutT, bool SWIGLU>
__global__ __launch_bounds__(GW* RL_WAVE) void gemm_skinny_kernel(
    const bf16_t* __restrict__ X, const bf16_t* __restrict__ W, OutT* __restrict__ out, int M,
    int N, int K, int ldx, int ldw, int ldo) {
    __shared__ float red[GW][NT * MB * 256];

    const int lane = threadIdx.x & (RL_WAVE - 1);
    const int wave = threadIdx.x / RL_WAVE;
    const int r16 = lane & 15;
    const int g = lane >> 4;

    // weight rows of this lane, one per tile (row >= limit: zeros)
    const bf16_t* wrow[NT];
    bool wok[NT];
#pragma unroll
    for (int nt = 0; nt < NT; ++nt) {
        int row;
        if (SWIGLU) {
            const int n = (blockIdx.x * (NT / 2) + nt / 2) * 16 + r16;
            wok[nt] = n < N;
            row = (nt & 1) ? N + n : n;
        } else {
            row = (blockIdx.x * NT + nt) * 16 + r16;
            wok[nt] = row < N;
        }
        wrow[nt] = W + (size_t)(wok[nt] ? row : 0) * ldw;
    }
    const bf16_t* xrow[MB];
    bool xok[MB];
#pragma unroll
    for (int mb = 0; mb < MB; ++mb) {
        const int m = mb * 16 + r16;
        xok[mb] = m < M;
        xrow[mb] = X + (size_t)(xok[mb] ? m : 0) * ldx;
    }

    f32x4 acc[NT][MB];
#pragma unroll
    for (int nt = 0; nt < NT; ++nt)
#pragma unroll
        for (int mb = 0; mb < MB; ++mb) acc[nt][mb] = (f32x4){0.f, 0.f, 0.f, 0.f};

    // the loop bound is the same for every lane of a wave: matrix instructions need them all
    for (int kw = wave * KSTEP; kw < K; kw += GW * KSTEP) {
        const int k0 = kw + 32 * g;
        bf16x8 a[NT][4], x[MB][4];
        // K is a multiple of 8: a piece is either whole or absent
#pragma unroll
        for (int nt = 0; nt < NT; ++nt)
#pragma unroll
            for (int j = 0; j < 4; ++j)
                a[nt][j] = (wok[nt] && k0 + 8 * j < K) ? ld16(wrow[nt] + k0 + 8 * j) : z8();
#pragma unroll
        for (int mb = 0; mb < MB; ++mb)
#pragma unroll
            for (int j = 0; j < 4; ++j)
                x[mb][j] = (xok[mb] && k0 + 8 * j < K) ? ld16(xrow[mb] + k0 + 8 * j) : z8();
#pragma unroll
        for (int j = 0; j < 4; ++j)
#pragma unroll
            for (int nt = 0; nt < NT; ++nt)
#pragma unroll
                for (int mb = 0; mb < MB; ++mb)
                    acc[nt][mb] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a[nt][j], x[mb][j],
                                                                          acc[nt][mb], 0, 0, 0);
    }

    // partial tiles of the waves -> LDS; lane-major so that reads below are conflict-free
#pragma unroll
    for (int nt = 0; nt < NT; ++nt)
#pragma unroll
        for (int mb = 0; mb < MB; ++mb)
#pragma unroll
            for (int i = 0; i < 4; ++i)
                red[wave][((nt * MB + mb) * 4 + i) * 64 + lane] = acc[nt][mb][i];
    __syncthreads();

    // thread -> (tile pair / tile, block of X rows, lane of the tile); sums the waves in order
    constexpr int OUT_TILES = SWIGLU ? NT / 2 : NT;
    for (int e = threadIdx.x; e < OUT_TILES * MB * 64; e += GW * RL_WAVE) {
        const int ln = e & 63;
        const int mb = (e >> 6) % MB;
        const int ot = (e >> 6) / MB;
        const int m = mb * 16 + (ln & 15);
        const int nbase = (blockIdx.x * OUT_TILES + ot) * 16 + 4 * (ln >> 4);
        if (m >= M) continue;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const int n = nbase + i;
            if (n >= N) continue;
            float v;
            if (SWIGLU) {
                float gate = 0.f, up = 0.f;
#pragma unroll
                for (int w = 0; w < GW; ++w) {
                    gate += red[w][(((2 * ot) * MB + mb) * 4 + i) * 64 + ln];
                    up += red[w][(((2 * ot + 1) * MB + mb) * 4 + i) * 64 + ln];
                }
                // the activation reads its operands rounded to bfloat16, as the unfused
                // path does where the product's result is stored before the activation
                gate = bf16_to_float(float_to_bf16(gate));
                up = bf16_to_float(float_to_bf16(up));
                v = gate / (1.f + expf(-gate)) * up;
            } else {
                v = 0.f;
#pragma unroll
                for (int w = 0; w < GW; ++w) v += red[w][((ot * MB + mb) * 4 + i) * 64 + ln];
            }
            store_out<OutT>(out + (size_t)m * ldo + n, v);
        }
    }
}

template <int MB, int NT, typename OutT, bool SWIGLU>
static int launch(const bf16_t* X, const bf16_t* W, OutT* out, int M, int N, int K, int ldx,
                  int ldw, int ldo, hipStream_t stream) {
    constexpr int rows_per_block = (SWIGLU ? NT / 2 : NT) * 16;
    dim3 grid((N + rows_per_block - 1) / rows_per_block), block(GW * RL_WAVE);
    hipLaunchKernelGGL((gemm_skinny_kernel<MB, NT, OutT, SWIGLU>), grid, block, 0, stream, X, W,
                       out, M, N, K, ldx, ldw, ldo);
    return rl_launch_status();
}

template <typename OutT, bool SWIGLU>
static int dispatch(const bf16_t* X, const bf16_t* W, OutT* out, int M, int N, int K, int ldx,
                    int ldw, int ldo, int nt, hipStream_t stream) {
    const int mb = (M + 15) / 16;
#define RL_CASE(MBV, NTV)                                                                      \
    if (mb <= MBV && nt == NTV)                                                                \
        return launch<MBV, NTV, OutT, SWIGLU>(X, W, out, M, N, K, ldx, ldw, ldo, stream);
    if (SWIGLU) {
        RL_CASE(1, 2) RL_CASE(1, 4) RL_CASE(2, 2)
    } else {
        RL_CASE(1, 1) RL_CASE(1, 2) RL_CASE(1, 4) RL_CASE(2, 1) RL_CASE(2, 2) RL_CASE(4, 1)
    }
#undef RL_CASE
    return RL_ERR_ARG;
}

// out_type: RL_F32 or RL_BF16.  nt: weight-row tiles per workgroup (see the host wrapper).
extern "C" int rl_gemm_skinny(const void* X, const void* W, void* out, int M, int N, int K,
                              int ldx, int ldw, int ldo, int out_type, int nt,
                              hipStream_t stream) {
    if (M <= 0 || N <= 0) return RL_OK;
    if (M > 64 || K < 8 || K % 8 || ldx % 8 || ldw % 8 || ldx < K || ldw < K || ldo < N)
        return RL_ERR_ARG;
    if (out_type == RL_F32)
        return dispatch<float, false>((const bf16_t*)X, (const bf16_t*)W, (float*)out, M, N, K,
                                      ldx, ldw, ldo, nt, stream);
    if (out_type == RL_BF16)
        return dispatch<bf16_t, false>((const bf16_t*)X, (const bf16_t*)W, (bf16_t*)out, M, N, K,
                                       ldx, ldw, ldo, nt, stream);
    return RL_ERR_ARG;
}

// out[M, I] = silu(X Wg^T) * (X Wu^T) with W = [Wg | Wu] stacked by rows, [2I, K].
extern "C" int rl_gemm_skinny_swiglu(const void* X, const void* W, void* out, int M, int I, int K,
                                     int ldx, int ldw, int ldo, int nt, hipStream_t stream) {
    if (M <= 0 || I <= 0) return RL_OK;
    if (M > 32 || K < 8 || K % 8 || ldx % 8 || ldw % 8 || ldx < K || ldw < K || ldo < I)
        return RL_ERR_ARG;
    return dispatch<bf16_t, true>((const bf16_t*)X, (const bf16_t*)W, (bf16_t*)out, M, I, K, ldx,
                                  ldw, ldo, nt, stream);
}
