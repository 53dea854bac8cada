// Bandwidth-bound bfloat16 product for few rows (decode): out[M,N] = X[M,K] * W[N,K]^T with
// M <= 16, float32 accumulation on the matrix cores, optionally fused with SwiGLU.
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

// NT: tiles of 16 weight rows per workgroup.  M <= 16: the rows of X are the 16 columns of
// one matrix instruction.  SWIGLU: tiles 2j / 2j+1 are gate rows / up rows; N is then the
// width I of the result.
//
// The A operand wants lane (n, g) to hold W[n][k0 + 32g ..]: read straight from memory that
// is sixteen rows per quarter wave, 16 bytes each.  Instead a quarter wave reads 256
// contiguous bytes of one row (instruction j covers rows 4j .. 4j+3 of the tile) and the tile
// is turned into the operand layout through a wave-private piece of LDS; no barrier is
// needed, the wave reads what it wrote itself.
//
// Measured on MI355X (graph replays, weights rotated through 800 MB so that nothing stays in
// cache), 8 rows, microseconds for the four products of a Qwen3-8B layer (50 / 34 / 101 / 201
// MB): strided reads 16.2 / 10.5 / 22.8 / 46.9; this kernel 14.7 / 9.4 / 20.5 / 41.0; weights
// stored pre-tiled so that every instruction reads 1 KB contiguous 14.3 / 9.2 / 19.9 / 41.2
// (no better, and the library product of the prefill could not read them); a plain read of
// the same bytes 10 / 6.5 / 16 / 34.  Deeper unrolling, non-temporal loads, more waves, K
// split over workgroups and staggered K offsets did not help.
#define WT_PITCH 272  // bytes between the 16 rows of the LDS tile: 256 + 16, conflict-free reads

template <int NT, typename OutT, bool SWIGLU>
__global__ __launch_bounds__(GW* RL_WAVE) void gemm_skinny_kernel(
    const bf16_t* __restrict__ X, const bf16_t* __restrict__ W, OutT* __restrict__ out, int M,
    int N, int K, int ldx, int ldw, int ldo) {
    __shared__ float red[GW][NT * 256];
    __shared__ __attribute__((aligned(16))) unsigned char wtile[GW][16 * WT_PITCH];

    const int lane = threadIdx.x & (RL_WAVE - 1);
    const int wave = threadIdx.x / RL_WAVE;
    const int r16 = lane & 15;
    const int g = lane >> 4;

    // first weight row of each tile; rows beyond the matrix read the last row and their
    // results are dropped in the epilogue
    int tile_row[NT];
#pragma unroll
    for (int nt = 0; nt < NT; ++nt) {
        if (SWIGLU)
            tile_row[nt] = (blockIdx.x * (NT / 2) + nt / 2) * 16 + ((nt & 1) ? N : 0);
        else
            tile_row[nt] = (blockIdx.x * NT + nt) * 16;
    }
    const int row_limit = SWIGLU ? 2 * N - 1 : N - 1;
    const int seg_limit = N - 1;  // within the gate (or up) half
    // coalesced reads: instruction j of tile nt reads row 4j + g of the tile at bytes 16 r16
    const bf16_t* wld[NT][4];
#pragma unroll
    for (int nt = 0; nt < NT; ++nt)
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            int row = tile_row[nt] + 4 * j + g;
            if (SWIGLU) {
                const int base = (nt & 1) ? N : 0;
                row = base + min(row - base, seg_limit);
            }
            row = min(row, row_limit);
            wld[nt][j] = W + (size_t)row * ldw + 8 * r16;
        }
    // strided reads (the last, partial chunk only): row r16 of the tile at elements 32 g
    const bf16_t* wrow[NT];
#pragma unroll
    for (int nt = 0; nt < NT; ++nt) {
        int row = tile_row[nt] + r16;
        if (SWIGLU) {
            const int base = (nt & 1) ? N : 0;
            row = base + min(row - base, seg_limit);
        }
        row = min(row, row_limit);
        wrow[nt] = W + (size_t)row * ldw + 32 * g;
    }
    const bool xok = r16 < M;
    const bf16_t* xrow = X + (size_t)(xok ? r16 : 0) * ldx + 32 * g;
    unsigned char* mytile = wtile[wave];

    f32x4 acc[NT];
#pragma unroll
    for (int nt = 0; nt < NT; ++nt) acc[nt] = (f32x4){0.f, 0.f, 0.f, 0.f};

    // whole chunks of 128: no predicates.  The bound is the same for every lane of a wave.
    const int kfull = K & ~(KSTEP - 1);
    for (int kw = wave * KSTEP; kw < kfull; kw += GW * KSTEP) {
        uint4 raw[NT][4];
        bf16x8 x[4];
#pragma unroll
        for (int nt = 0; nt < NT; ++nt)
#pragma unroll
            for (int j = 0; j < 4; ++j) raw[nt][j] = *reinterpret_cast<const uint4*>(wld[nt][j] + kw);
#pragma unroll
        for (int j = 0; j < 4; ++j) x[j] = xok ? ld16(xrow + kw + 8 * j) : z8();
#pragma unroll
        for (int nt = 0; nt < NT; ++nt) {
            // the tiles of a wave go through the same piece of LDS one after the other
#pragma unroll
            for (int j = 0; j < 4; ++j)
                *reinterpret_cast<uint4*>(mytile + (4 * j + g) * WT_PITCH + 16 * r16) = raw[nt][j];
            bf16x8 a[4];
#pragma unroll
            for (int j = 0; j < 4; ++j)
                a[j] = __builtin_bit_cast(
                    bf16x8, *reinterpret_cast<const uint4*>(mytile + r16 * WT_PITCH + 64 * g + 16 * j));
#pragma unroll
            for (int j = 0; j < 4; ++j)
                acc[nt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a[j], x[j], acc[nt], 0, 0, 0);
        }
    }
    // the last, partial chunk (K is a multiple of 8: a piece is whole or absent)
    if (kfull < K && wave == (kfull / KSTEP) % GW) {
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const bool ok = kfull + 32 * g + 8 * j < K;
            const bf16x8 xv = (ok && xok) ? ld16(xrow + kfull + 8 * j) : z8();
#pragma unroll
            for (int nt = 0; nt < NT; ++nt) {
                const bf16x8 av = ok ? ld16(wrow[nt] + kfull + 8 * j) : z8();
                acc[nt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(av, xv, acc[nt], 0, 0, 0);
            }
        }
    }

    // partial tiles of the waves -> LDS; lane-major so that reads below are conflict-free
#pragma unroll
    for (int nt = 0; nt < NT; ++nt)
#pragma unroll
        for (int i = 0; i < 4; ++i) red[wave][(nt * 4 + i) * 64 + lane] = acc[nt][i];
    __syncthreads();

    // thread -> (tile pair / tile, lane of the tile); sums the waves in order
    constexpr int OUT_TILES = SWIGLU ? NT / 2 : NT;
    for (int e = threadIdx.x; e < OUT_TILES * 64; e += GW * RL_WAVE) {
        const int ln = e & 63;
        const int ot = e >> 6;
        const int m = ln & 15;
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
                    gate += red[w][((2 * ot) * 4 + i) * 64 + ln];
                    up += red[w][((2 * ot + 1) * 4 + i) * 64 + ln];
                }
                // the activation reads its operands rounded to bfloat16, as the unfused
                // path does where the product's result is stored before the activation
                gate = bf16_to_float(float_to_bf16(gate));
                up = bf16_to_float(float_to_bf16(up));
                v = gate / (1.f + expf(-gate)) * up;
            } else {
                v = 0.f;
#pragma unroll
                for (int w = 0; w < GW; ++w) v += red[w][(ot * 4 + i) * 64 + ln];
            }
            store_out<OutT>(out + (size_t)m * ldo + n, v);
        }
    }
}

template <int NT, typename OutT, bool SWIGLU>
static int launch(const bf16_t* X, const bf16_t* W, OutT* out, int M, int N, int K, int ldx,
                  int ldw, int ldo, hipStream_t stream) {
    constexpr int rows_per_block = (SWIGLU ? NT / 2 : NT) * 16;
    dim3 grid((N + rows_per_block - 1) / rows_per_block), block(GW * RL_WAVE);
    hipLaunchKernelGGL((gemm_skinny_kernel<NT, OutT, SWIGLU>), grid, block, 0, stream, X, W, out,
                       M, N, K, ldx, ldw, ldo);
    return rl_launch_status();
}

template <typename OutT, bool SWIGLU>
static int dispatch(const bf16_t* X, const bf16_t* W, OutT* out, int M, int N, int K, int ldx,
                    int ldw, int ldo, int nt, hipStream_t stream) {
#define RL_CASE(NTV)                                                                           \
    if (nt == NTV) return launch<NTV, OutT, SWIGLU>(X, W, out, M, N, K, ldx, ldw, ldo, stream);
    if (SWIGLU) {
        RL_CASE(2) RL_CASE(4)
    } else {
        RL_CASE(1) RL_CASE(2)
    }
#undef RL_CASE
    return RL_ERR_ARG;
}

// out_type: RL_F32 or RL_BF16.  nt: weight-row tiles per workgroup (see the host wrapper).
extern "C" int rl_gemm_skinny(const void* X, const void* W, void* out, int M, int N, int K,
                              int ldx, int ldw, int ldo, int out_type, int nt,
                              hipStream_t stream) {
    if (M <= 0 || N <= 0) return RL_OK;
    if (M > 16 || K < 8 || K % 8 || ldx % 8 || ldw % 8 || ldx < K || ldw < K || ldo < N)
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
    if (M > 16 || K < 8 || K % 8 || ldx % 8 || ldw % 8 || ldx < K || ldw < K || ldo < I)
        return RL_ERR_ARG;
    return dispatch<bf16_t, true>((const bf16_t*)X, (const bf16_t*)W, (bf16_t*)out, M, I, K, ldx,
                                  ldw, ldo, nt, stream);
}
