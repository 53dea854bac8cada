// Bandwidth-bound bfloat16 product for few rows (decode): out[M,N] = X[M,K] * W[N,K]^T with
// M <= 16, float32 accumulation on the matrix cores, optionally fused with SwiGLU.  (The last
// section of the file holds the products for 17 rows and more of narrow and of small matrices.)
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
//
// Two optional epilogues fold the residual norm between two products into the products
// themselves, so that a decode step needs no norm kernel (rapid_llm/kernels/ops/layernorm/
// skip_rmsnorm.py:51-85 is what they compute together):
//   * "residual": the producer adds its result (rounded to bfloat16, as a stored result
//     would be) to the float32 residual rows in place, writes the rows times the norm's
//     weight as bfloat16, and leaves the sum of squares of its 16 columns of every row in
//     `partial[workgroup][row]`;
//   * "scaled input": the consumer reads those rows as its X and multiplies its own result
//     by  rsqrt(sum of the partials / width + eps)  of the row: the norm's factor is a
//     scalar per row and commutes with the product.
// Sums run in a fixed order (the workgroups' partials in index order).
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
// the same bytes 10 / 6.5 / 16 / 34.  Non-temporal loads, more waves, K split over workgroups
// and staggered K offsets did not help.  Two chunks in flight per wave, in two sets of
// registers (see the main loop), then gave 14.0 / 9.4 / 21.9 / 38.4 where one chunk at a time
// gave 14.9 / 9.7 / 22.2 / 42.6 in the same run; four chunks in flight (where a compute unit holds
// one workgroup anyway) were no faster than two (9.8 against 9.3, 22.1 against 21.9).
// sum over the four lanes l, l + 16, l + 32, l + 48 (two lane swaps of gfx950), left in all four
__device__ inline float sum_rows_of_16(float v) {
    const unsigned u = __float_as_uint(v);
    const auto a = __builtin_amdgcn_permlane32_swap(u, u, false, false);
    const unsigned w = __float_as_uint(__uint_as_float(a[0]) + __uint_as_float(a[1]));
    const auto b = __builtin_amdgcn_permlane16_swap(w, w, false, false);
    return __uint_as_float(b[0]) + __uint_as_float(b[1]);
}

#define WT_PITCH 272  // bytes between the 16 rows of the LDS tile: 256 + 16, conflict-free reads

struct SkinnyExtra {
    // scaled input (null: X is used as it is)
    const float* x_partial;  // [x_parts][16] sums of squares
    int x_parts;
    float x_inv_size, x_eps;
    // residual epilogue (null: the result is stored)
    float* residual;      // [M, N] float32, updated in place
    const float* norm_w;  // [N]
    bf16_t* xt;           // [M, N] residual * norm_w
    float* partial;       // [workgroups][16]
};

// LASTQ: groups of four rows of the last tile that belong to the workgroup: 4, or 2 for
// workgroups of 24 rows (NT == 2), which put a matrix of 384 tiles on 256 compute units
// evenly; the other rows of that tile are neither read nor stored.
template <int NT, typename OutT, bool SWIGLU, bool SCALED, int LASTQ = 4>
__global__ __launch_bounds__(GW* RL_WAVE) void gemm_skinny_kernel(
    const bf16_t* __restrict__ X, const bf16_t* __restrict__ W, OutT* __restrict__ out, int M,
    int N, int K, int ldx, int ldw, int ldo, SkinnyExtra ex) {
    __shared__ float red[GW][NT * 256];

    __shared__ __attribute__((aligned(16))) unsigned char wtile[GW][16 * WT_PITCH];
    __shared__ float wave_part[SCALED ? GW : 1][16];  // a scaled input's sums of squares by wave
    static_assert(LASTQ == 4 || (LASTQ == 2 && NT == 2 && !SWIGLU), "half a last tile: two plain tiles only");
    constexpr int ROWS = (NT - 1) * 16 + 4 * LASTQ;  // weight rows of a workgroup (not SWIGLU)

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
            tile_row[nt] = blockIdx.x * ROWS + nt * 16;
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

    // What the residual epilogue needs from memory is asked for now and arrives while the
    // weights stream: the residual and norm weights of the results this thread will write.
    // (Asking for a scaled input's partial sums this early was measured and lost 1.5 us a
    // product: loads return in order, and the weights then wait behind them.)
    static_assert(NT * 64 <= GW * RL_WAVE, "every result of the workgroup has a thread of its own");
    float res_in[4] = {0.f, 0.f, 0.f, 0.f}, nw_in[4] = {0.f, 0.f, 0.f, 0.f};
    if (!SWIGLU && ex.residual && threadIdx.x < NT * 64) {
        const int ln = threadIdx.x & 63, ot = threadIdx.x >> 6, m = ln & 15;
        const int nbase = blockIdx.x * ROWS + ot * 16 + 4 * (ln >> 4);
        const bool mine = ot * 16 + 4 * (ln >> 4) < ROWS;
#pragma unroll
        for (int i = 0; i < 4; ++i)
            if (m < M && mine && nbase + i < N) {
                res_in[i] = ex.residual[(size_t)m * N + nbase + i];
                nw_in[i] = ex.norm_w[nbase + i];
            }
    }

    // whole chunks of 128: no predicates.  The bound is the same for every lane of a wave.
    const int kfull = K & ~(KSTEP - 1);
    // Two chunks in flight per wave, in two sets of registers used in turn: the loads of the
    // chunk after next are issued before this chunk's products.  Inside the loop no load
    // stands behind a condition (behind one the compiler counts it as absent and makes the
    // oldest operand wait for the newest load); what is left, one chunk or two, follows it.
    // Rows beyond M read row 0 (their results are never stored), so no load is predicated.
    constexpr int XP_AHEAD = 8;  // partial sums a thread asks for ahead: 256 parts in all
    float x_part[XP_AHEAD];
    {
        bf16x8 wa[NT][4], wb[NT][4], xa[4], xb[4];
        auto load = [&](bf16x8 (&r)[NT][4], bf16x8 (&xx)[4], int kw) {
#pragma unroll
            for (int nt = 0; nt < NT; ++nt)
#pragma unroll
                for (int j = 0; j < (nt == NT - 1 ? LASTQ : 4); ++j) r[nt][j] = ld16(wld[nt][j] + kw);
#pragma unroll
            for (int j = 0; j < 4; ++j) xx[j] = ld16(xrow + kw + 8 * j);
        };
        auto products = [&](bf16x8 (&r)[NT][4], bf16x8 (&xx)[4]) {
#pragma unroll
            for (int nt = 0; nt < NT; ++nt) {
#pragma unroll
                for (int j = 0; j < (nt == NT - 1 ? LASTQ : 4); ++j)  // rows beyond stay what they were
                    *reinterpret_cast<bf16x8*>(mytile + (4 * j + g) * WT_PITCH + 16 * r16) = r[nt][j];
                bf16x8 a[4];
#pragma unroll
                for (int j = 0; j < 4; ++j)
                    a[j] = *reinterpret_cast<const bf16x8*>(mytile + r16 * WT_PITCH + 64 * g + 16 * j);
#pragma unroll
                for (int j = 0; j < 4; ++j)
                    acc[nt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a[j], xx[j], acc[nt], 0, 0, 0);
            }
        };
        // A scaled input's partial sums of squares (thread (run j, row m) owns the partials
        // j, j + 32, ..) are asked for behind the wave's last weights, without a condition,
        // and arrive with them; they are added after the last products.  Asked for after the
        // loop, their whole latency stood in the open in front of the epilogue (5 us a product
        // where a compute unit holds one workgroup).
        auto partial_loads = [&]() {
            if constexpr (SCALED) {
                const int m = threadIdx.x & 15, j = threadIdx.x >> 4;  // 512 threads: 32 runs
#pragma unroll
                for (int i = 0; i < XP_AHEAD; ++i)
                    x_part[i] = ex.x_partial[min(j + 32 * i, ex.x_parts - 1) * 16 + m];
            }
        };
        constexpr int S = GW * KSTEP;
        int kw = wave * KSTEP;
        if (kw >= kfull) partial_loads();
        if (kw < kfull) {
            int left = (kfull - kw + S - 1) / S;  // chunks of this wave, the loaded one included
            load(wa, xa, kw);
            while (left > 2) {
                load(wb, xb, kw + S);
                products(wa, xa);
                load(wa, xa, kw + 2 * S);
                products(wb, xb);
                kw += 2 * S;
                left -= 2;
            }
            if (left == 2) {
                load(wb, xb, kw + S);
                partial_loads();
                products(wa, xa);
                products(wb, xb);
            } else {
                partial_loads();
                products(wa, xa);
            }
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

    // The norm's factor of every row of a scaled input: thread (run j, row m) adds its partials
    // j, j + 32, .. in order; the four runs of a wave are added by lane swaps, the eight waves'
    // sums by every thread that needs the row's factor, in the order of the waves.  No barrier
    // beyond the one that the waves' partial tiles need anyway.
    // (the residual epilogue's small array lives where the weight tiles were)
    float* sq = reinterpret_cast<float*>(&wtile[0][0]);  // [NT * 64]
    static_assert(sizeof(wtile) >= NT * 64 * sizeof(float), "epilogue array fits");
    if constexpr (SCALED) {
        const int m = threadIdx.x & 15, j = threadIdx.x >> 4;
        float run = 0.f;
#pragma unroll
        for (int i = 0; i < XP_AHEAD; ++i) run += (j + 32 * i < ex.x_parts) ? x_part[i] : 0.f;
        for (int p = j + 32 * XP_AHEAD; p < ex.x_parts; p += 32) run += ex.x_partial[p * 16 + m];
        run = sum_rows_of_16(run);
        if (g == 0) wave_part[wave][m] = run;
    }
    // partial tiles of the waves -> LDS; lane-major so that reads below are conflict-free
#pragma unroll
    for (int nt = 0; nt < NT; ++nt)
#pragma unroll
        for (int i = 0; i < 4; ++i) red[wave][(nt * 4 + i) * 64 + lane] = acc[nt][i];
    __syncthreads();  // also: every wave has left the main loop, the weight tiles are free

    // thread -> (tile pair / tile, lane of the tile); sums the waves in order
    constexpr int OUT_TILES = SWIGLU ? NT / 2 : NT;
    for (int e = threadIdx.x; e < OUT_TILES * 64; e += GW * RL_WAVE) {  // at most one round
        const int ln = e & 63;
        const int ot = e >> 6;
        const int m = ln & 15;
        const int nbase = SWIGLU ? (blockIdx.x * OUT_TILES + ot) * 16 + 4 * (ln >> 4)
                                 : blockIdx.x * ROWS + ot * 16 + 4 * (ln >> 4);
        const bool mine = SWIGLU || ot * 16 + 4 * (ln >> 4) < ROWS;  // not in the unused part of the last tile
        float scale = 1.f;
        if constexpr (SCALED) {
            float ss = 0.f;
#pragma unroll
            for (int w = 0; w < GW; ++w) ss += wave_part[w][m];
            scale = rsqrtf(ss * ex.x_inv_size + ex.x_eps);
        }
        float sumsq = 0.f;
        if (m < M && mine) {
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
                    gate = bf16_to_float(float_to_bf16(gate * scale));
                    up = bf16_to_float(float_to_bf16(up * scale));
                    v = gate / (1.f + expf(-gate)) * up;
                } else {
                    v = 0.f;
#pragma unroll
                    for (int w = 0; w < GW; ++w) v += red[w][(ot * 4 + i) * 64 + ln];
                    v *= scale;
                }
                if (!SWIGLU && ex.residual) {
                    const size_t at = (size_t)m * N + n;
                    const float r = res_in[i] + bf16_to_float(float_to_bf16(v));
                    ex.residual[at] = r;
                    ex.xt[at] = float_to_bf16(r * nw_in[i]);
                    sumsq += r * r;
                } else {
                    store_out<OutT>(out + (size_t)m * ldo + n, v);
                }
            }
        }
        if (!SWIGLU && ex.residual) sq[e] = sumsq;
    }
    if (!SWIGLU && ex.residual) {
        __syncthreads();
        // row m of this workgroup's columns: the epilogue threads with lane % 16 == m, in order
        if (threadIdx.x < 16) {
            float ss = 0.f;
            for (int e = threadIdx.x; e < OUT_TILES * 64; e += 16) ss += sq[e];
            ex.partial[(size_t)blockIdx.x * 16 + threadIdx.x] = ss;
        }
    }
}

template <int NT, typename OutT, bool SWIGLU, bool SCALED, int LASTQ = 4>
static int launch(const bf16_t* X, const bf16_t* W, OutT* out, int M, int N, int K, int ldx,
                  int ldw, int ldo, const SkinnyExtra& ex, hipStream_t stream) {
    constexpr int rows_per_block = SWIGLU ? (NT / 2) * 16 : (NT - 1) * 16 + 4 * LASTQ;
    dim3 grid((N + rows_per_block - 1) / rows_per_block), block(GW * RL_WAVE);
    hipLaunchKernelGGL((gemm_skinny_kernel<NT, OutT, SWIGLU, SCALED, LASTQ>), grid, block, 0, stream, X, W,
                       out, M, N, K, ldx, ldw, ldo, ex);
    return rl_launch_status();
}

// --------------------------------------------------------------------------- //
// The gate/up product where the matrix has more (gate, up) pairs of tiles than the chip has
// compute units.  The kernel above needs the registers of a whole compute unit for one
// workgroup (two chunks of two tiles in flight per wave), so its workgroups follow each other
// on a unit, and between two of them the unit streams nothing: the last waves drain, the
// epilogue runs, the next workgroup asks for its first weights (cycle stamps: three workgroups
// of 12.3 us a unit for the 24,576 rows of Qwen3-8B, 1.5 us of each the epilogue and as much
// again before its loads come back).  Here a unit gets one workgroup that walks its pairs
// b, b + G, b + 2G, .. as one stream of chunks: a wave that has its last chunk of a pair in
// flight asks for its first of the next, puts the pair's sums into LDS when they are complete,
// and the one epilogue at the end folds the waves' sums of every pair, in the order of the
// waves: bit for bit what the kernel above computes.
// --------------------------------------------------------------------------- //
#define SW_MAX_TILES 7  // pairs a workgroup may walk (their partial sums wait in LDS: 16 KB a pair)

template <bool SCALED>
__global__ __launch_bounds__(GW* RL_WAVE) void gemm_swiglu_stream_kernel(
    const bf16_t* __restrict__ X, const bf16_t* __restrict__ W, bf16_t* __restrict__ out, int M,
    int I, int K, int ldx, int ldw, int ldo, int pairs, SkinnyExtra ex) {
    __shared__ float red[SW_MAX_TILES][GW][2 * 256];
    __shared__ __attribute__((aligned(16))) unsigned char wtile[GW][16 * WT_PITCH];
    __shared__ float wave_part[SCALED ? GW : 1][16];

    const int lane = threadIdx.x & (RL_WAVE - 1);
    const int wave = threadIdx.x / RL_WAVE;
    const int r16 = lane & 15;
    const int g = lane >> 4;
    // pairs of this workgroup: blockIdx.x, + gridDim.x, ..  (host: at most SW_MAX_TILES)
    const int T = (pairs - (int)blockIdx.x + (int)gridDim.x - 1) / (int)gridDim.x;
    const size_t pair_stride = (size_t)gridDim.x * 16 * ldw;  // elements between two of its pairs
    // instruction j of tile nt (0: gate, 1: up) reads row 4j + g of the tile at bytes 16 r16
    const bf16_t* wld[2][4];
#pragma unroll
    for (int nt = 0; nt < 2; ++nt)
#pragma unroll
        for (int j = 0; j < 4; ++j)
            wld[nt][j] = W + (size_t)(nt * I + blockIdx.x * 16 + 4 * j + g) * ldw + 8 * r16;
    const bf16_t* xrow = X + (size_t)(r16 < M ? r16 : 0) * ldx + 32 * g;
    unsigned char* mytile = wtile[wave];

    f32x4 acc[2];
    acc[0] = acc[1] = (f32x4){0.f, 0.f, 0.f, 0.f};
    constexpr int XP_AHEAD = 8;
    float x_part[XP_AHEAD];
    constexpr int S = GW * KSTEP;
    const int k0 = wave * KSTEP;
    const int nchunk = (K - k0 + S - 1) / S;  // chunks of this wave in a pair: at least one (host)
    {
        bf16x8 wa[2][4], wb[2][4], xa[4], xb[4];
        auto load = [&](bf16x8 (&r)[2][4], bf16x8 (&xx)[4], int t, int kw) {
            const size_t off = (size_t)t * pair_stride + kw;
#pragma unroll
            for (int nt = 0; nt < 2; ++nt)
#pragma unroll
                for (int j = 0; j < 4; ++j) r[nt][j] = ld16(wld[nt][j] + off);
#pragma unroll
            for (int j = 0; j < 4; ++j) xx[j] = ld16(xrow + kw + 8 * j);
        };
        // the chunk's products; `last`: the wave's last chunk of pair t, whose sums go to LDS
        auto products = [&](bf16x8 (&r)[2][4], bf16x8 (&xx)[4], int t, bool last) {
#pragma unroll
            for (int nt = 0; nt < 2; ++nt) {
#pragma unroll
                for (int j = 0; j < 4; ++j)
                    *reinterpret_cast<bf16x8*>(mytile + (4 * j + g) * WT_PITCH + 16 * r16) = r[nt][j];
                bf16x8 a[4];
#pragma unroll
                for (int j = 0; j < 4; ++j)
                    a[j] = *reinterpret_cast<const bf16x8*>(mytile + r16 * WT_PITCH + 64 * g + 16 * j);
#pragma unroll
                for (int j = 0; j < 4; ++j)
                    acc[nt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a[j], xx[j], acc[nt], 0, 0, 0);
            }
            if (last) {  // the same for every lane of the wave
#pragma unroll
                for (int nt = 0; nt < 2; ++nt)
#pragma unroll
                    for (int i = 0; i < 4; ++i) {
                        red[t][wave][(nt * 4 + i) * 64 + lane] = acc[nt][i];
                        acc[nt][i] = 0.f;
                    }
            }
        };
        auto partial_loads = [&]() {
            if constexpr (SCALED) {
                const int m = threadIdx.x & 15, j = threadIdx.x >> 4;  // 512 threads: 32 runs
#pragma unroll
                for (int i = 0; i < XP_AHEAD; ++i)
                    x_part[i] = ex.x_partial[min(j + 32 * i, ex.x_parts - 1) * 16 + m];
            }
        };
        // the wave's chunks of all its pairs as one sequence: (pair t, chunk i), two in flight
        int ta = 0, ia = 0, tb = 0, ib = 0;
        auto next = [&](int& t, int& i, int t0, int i0) {
            i = i0 + 1;
            t = t0;
            if (i == nchunk) {
                i = 0;
                t = t0 + 1;
            }
        };
        int left = T * nchunk;
        load(wa, xa, 0, k0);
        while (left > 2) {
            next(tb, ib, ta, ia);
            load(wb, xb, tb, k0 + ib * S);
            products(wa, xa, ta, ia == nchunk - 1);
            next(ta, ia, tb, ib);
            load(wa, xa, ta, k0 + ia * S);
            products(wb, xb, tb, ib == nchunk - 1);
            left -= 2;
        }
        if (left == 2) {
            next(tb, ib, ta, ia);
            load(wb, xb, tb, k0 + ib * S);
            partial_loads();
            products(wa, xa, ta, ia == nchunk - 1);
            products(wb, xb, tb, true);
        } else {
            partial_loads();
            products(wa, xa, ta, true);
        }
    }
    if constexpr (SCALED) {
        const int m = threadIdx.x & 15, j = threadIdx.x >> 4;
        float run = 0.f;
#pragma unroll
        for (int i = 0; i < XP_AHEAD; ++i) run += (j + 32 * i < ex.x_parts) ? x_part[i] : 0.f;
        for (int p = j + 32 * XP_AHEAD; p < ex.x_parts; p += 32) run += ex.x_partial[p * 16 + m];
        run = sum_rows_of_16(run);
        if (g == 0) wave_part[wave][m] = run;
    }
    __syncthreads();  // every wave's sums of every pair are in LDS

    // thread -> (pair t, lane of its tile); sums the waves in order
    for (int e = threadIdx.x; e < T * 64; e += GW * RL_WAVE) {
        const int ln = e & 63;
        const int t = e >> 6;
        const int m = ln & 15;
        if (m >= M) continue;
        const int nbase = ((int)blockIdx.x + t * (int)gridDim.x) * 16 + 4 * (ln >> 4);
        float scale = 1.f;
        if constexpr (SCALED) {
            float ss = 0.f;
#pragma unroll
            for (int w = 0; w < GW; ++w) ss += wave_part[w][m];
            scale = rsqrtf(ss * ex.x_inv_size + ex.x_eps);
        }
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            float gate = 0.f, up = 0.f;
#pragma unroll
            for (int w = 0; w < GW; ++w) {
                gate += red[t][w][i * 64 + ln];
                up += red[t][w][(4 + i) * 64 + ln];
            }
            // operands rounded to bfloat16, as where the product's result is stored first
            gate = bf16_to_float(float_to_bf16(gate * scale));
            up = bf16_to_float(float_to_bf16(up * scale));
            out[(size_t)m * ldo + nbase + i] = float_to_bf16(gate / (1.f + expf(-gate)) * up);
        }
    }
}

// true (and *rc set) if the stream kernel took the product; `units`: the chip's compute units
// as the host read them (one workgroup of the stream kernel each)
static bool swiglu_stream(const bf16_t* X, const bf16_t* W, bf16_t* out, int M, int I, int K, int ldx,
                          int ldw, int ldo, int units, const SkinnyExtra& ex, hipStream_t stream, int* rc) {
    const int pairs = I / 16;
    if (units <= 0 || I % 16 || K % KSTEP || K < GW * KSTEP || pairs <= units) return false;
    const int per = (pairs + units - 1) / units;  // pairs a workgroup
    if (per > SW_MAX_TILES) return false;
    dim3 grid((pairs + per - 1) / per), block(GW * RL_WAVE);
    if (ex.x_partial)
        hipLaunchKernelGGL((gemm_swiglu_stream_kernel<true>), grid, block, 0, stream, X, W, out, M, I, K,
                           ldx, ldw, ldo, pairs, ex);
    else
        hipLaunchKernelGGL((gemm_swiglu_stream_kernel<false>), grid, block, 0, stream, X, W, out, M, I, K,
                           ldx, ldw, ldo, pairs, ex);
    *rc = rl_launch_status();
    return true;
}

template <typename OutT, bool SWIGLU>
static int dispatch(const bf16_t* X, const bf16_t* W, OutT* out, int M, int N, int K, int ldx,
                    int ldw, int ldo, int nt, const SkinnyExtra& ex, hipStream_t stream) {
#define RL_CASE(NTV)                                                                           \
    if (nt == NTV)                                                                             \
        return ex.x_partial                                                                    \
                   ? launch<NTV, OutT, SWIGLU, true>(X, W, out, M, N, K, ldx, ldw, ldo, ex, stream) \
                   : launch<NTV, OutT, SWIGLU, false>(X, W, out, M, N, K, ldx, ldw, ldo, ex, stream);
    // the gate/up variant holds a (gate, up) pair of tiles; two pairs would not fit the registers
    // of two chunks in flight
    if constexpr (SWIGLU) {
        RL_CASE(2)
    } else {
        RL_CASE(1) RL_CASE(2)
        // nt == 3: workgroups of 24 rows, one tile and a half; plain results only
        if (nt == 3 && !ex.residual)
            return ex.x_partial
                       ? launch<2, OutT, false, true, 2>(X, W, out, M, N, K, ldx, ldw, ldo, ex, stream)
                       : launch<2, OutT, false, false, 2>(X, W, out, M, N, K, ldx, ldw, ldo, ex, stream);
    }
#undef RL_CASE
    return RL_ERR_ARG;
}

static bool skinny_args_ok(int M, int K, int ldx, int ldw) {
    return M <= 16 && K >= 8 && K % 8 == 0 && ldx % 8 == 0 && ldw % 8 == 0 && ldx >= K && ldw >= K;
}

// x_partial (optional): X holds rows whose norm factor is still to be applied,
// rsqrt(sum over x_parts of x_partial[part][row] / x_size + x_eps); the result is multiplied
// by it.
static SkinnyExtra scaled_input(const float* x_partial, int x_parts, int x_size, float x_eps) {
    SkinnyExtra ex = {};
    if (x_partial) {
        ex.x_partial = x_partial;
        ex.x_parts = x_parts;
        ex.x_inv_size = 1.f / (float)x_size;
        ex.x_eps = x_eps;
    }
    return ex;
}

// out_type: RL_F32 or RL_BF16.  nt: weight-row tiles per workgroup, 1 or 2, or 3 for one and a
// half (24 rows), see the host wrapper.
extern "C" int rl_gemm_skinny(const void* X, const void* W, void* out, int M, int N, int K,
                              int ldx, int ldw, int ldo, int out_type, int nt,
                              const float* x_partial, int x_parts, int x_size, float x_eps,
                              hipStream_t stream) {
    if (M <= 0 || N <= 0) return RL_OK;
    if (!skinny_args_ok(M, K, ldx, ldw) || ldo < N || (x_partial && (x_parts < 1 || x_size < 1)))
        return RL_ERR_ARG;
    const SkinnyExtra ex = scaled_input(x_partial, x_parts, x_size, x_eps);
    if (out_type == RL_F32)
        return dispatch<float, false>((const bf16_t*)X, (const bf16_t*)W, (float*)out, M, N, K,
                                      ldx, ldw, ldo, nt, ex, stream);
    if (out_type == RL_BF16)
        return dispatch<bf16_t, false>((const bf16_t*)X, (const bf16_t*)W, (bf16_t*)out, M, N, K,
                                       ldx, ldw, ldo, nt, ex, stream);
    return RL_ERR_ARG;
}

// out[M, I] = silu(X Wg^T) * (X Wu^T) with W = [Wg | Wu] stacked by rows, [2I, K].  A matrix
// with more pairs of tiles than the chip has compute units (`units`, as the host's launch rules
// read them) goes to the stream kernel (nt < 0: never, the kernel of one pair a workgroup with
// -nt tiles: for comparing the two).
extern "C" int rl_gemm_skinny_swiglu(const void* X, const void* W, void* out, int M, int I, int K,
                                     int ldx, int ldw, int ldo, int nt, int units, const float* x_partial,
                                     int x_parts, int x_size, float x_eps, hipStream_t stream) {
    if (M <= 0 || I <= 0) return RL_OK;
    if (!skinny_args_ok(M, K, ldx, ldw) || ldo < I || (x_partial && (x_parts < 1 || x_size < 1)))
        return RL_ERR_ARG;
    const SkinnyExtra ex = scaled_input(x_partial, x_parts, x_size, x_eps);
    int rc = RL_OK;
    if (nt >= 0 && swiglu_stream((const bf16_t*)X, (const bf16_t*)W, (bf16_t*)out, M, I, K, ldx, ldw, ldo, units,
                                 ex, stream, &rc))
        return rc;
    return dispatch<bf16_t, true>((const bf16_t*)X, (const bf16_t*)W, (bf16_t*)out, M, I, K, ldx,
                                  ldw, ldo, nt < 0 ? -nt : nt, ex, stream);
}

// The product with the residual epilogue: residual[M, N] += X W^T (rounded to bfloat16),
// xt[M, N] = residual * norm_w as bfloat16, partial[workgroup][16] = sums of squares of the
// workgroup's columns per row.  Returns the number of workgroups through *parts (the caller
// sizes `partial` with rl_gemm_skinny_parts).
extern "C" int rl_gemm_skinny_parts(int N, int nt) { return (N + nt * 16 - 1) / (nt * 16); }

extern "C" int rl_gemm_skinny_residual(const void* X, const void* W, int M, int N, int K, int ldx,
                                       int ldw, int nt, float* residual, const float* norm_w,
                                       void* xt, float* partial, hipStream_t stream) {
    if (M <= 0 || N <= 0) return RL_OK;
    if (!skinny_args_ok(M, K, ldx, ldw) || !residual || !norm_w || !xt || !partial) return RL_ERR_ARG;
    SkinnyExtra ex = {};
    ex.residual = residual;
    ex.norm_w = norm_w;
    ex.xt = (bf16_t*)xt;
    ex.partial = partial;
    return dispatch<bf16_t, false>((const bf16_t*)X, (const bf16_t*)W, (bf16_t*)nullptr, M, N, K,
                                   ldx, ldw, N, nt, ex, stream);
}

// =========================================================================== //
// 17 .. 192 rows: the runs of K of a product whose result feeds the residual
// =========================================================================== //
// The library's product reads X once for every 16 or 32 weight rows at these sizes and
// stays near 3 TB/s.  Here a workgroup is four waves with 16 weight rows each; the chunk of X
// they all need ([64 rows x 128 k], double-buffered) goes through LDS once per workgroup, the
// weights stream as in the skinny product (two chunks in flight per wave, no load behind a
// condition).  A matrix of 4,096 rows gives only 64 such workgroups, so K is cut into `ks`
// runs (grid.y) whose float32 results [ks][M][N] are added by the norm kernel that consumes
// them (rl_add_rmsnorm_parts).  Measured against the library at 64 rows (Qwen3-8B shapes,
// microseconds): 4,096 x 4,096 11.8 / 14.9, 4,096 x 12,288 26.6 / 38.1; at 32 rows 9.9 / 13.9
// and 23.0 / 28.6.  The wide products (6,144 and 24,576 rows) gain nothing (18.3 / 18.1 and
// 55 / 46) and stay with the library.  More than 64 rows run as blocks of 64 rows (grid.z), each
// reading the weights again: up to about 192 rows that is still faster than the library's kernels
// for such shapes (the host's rule holds the measurements).
#define MW 4  // waves per workgroup

template <int MB>
__global__ __launch_bounds__(MW* RL_WAVE) void gemm_mid_kernel(
    const bf16_t* __restrict__ X, const bf16_t* __restrict__ W, float* __restrict__ part, int M,
    int N, int K, int ldx, int ldw, int chunks_per_run) {
    __shared__ __attribute__((aligned(16))) unsigned char xs[2][MB * 16 * WT_PITCH];
    __shared__ __attribute__((aligned(16))) unsigned char wtile[MW][16 * WT_PITCH];
    const int tid = threadIdx.x, lane = tid & (RL_WAVE - 1), wave = tid / RL_WAVE;
    const int r16 = lane & 15, g = lane >> 4;
    const int n0 = (blockIdx.x * MW + wave) * 16;
    const int run = blockIdx.y;
    const int m0 = blockIdx.z * 64;  // more than 64 rows: blocks of 64 (grid.z)
    const int c_lo = run * chunks_per_run, c_hi = min(K / KSTEP, c_lo + chunks_per_run);
    // weights: instruction j reads row 4j + g of the wave's tile at bytes 16 r16 (as the skinny
    // product does); rows beyond the matrix read its last row, their results are dropped
    const bf16_t* wld[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) wld[j] = W + (size_t)min(n0 + 4 * j + g, N - 1) * ldw + 8 * r16;
    // X: thread reads bytes 16 (tid % 16) of rows tid / 16 + 16 i; rows beyond M read the last
    const bf16_t* xld[MB];
#pragma unroll
    for (int i = 0; i < MB; ++i) xld[i] = X + (size_t)min(m0 + tid / 16 + 16 * i, M - 1) * ldx + 8 * (tid % 16);
    unsigned char* mytile = wtile[wave];
    f32x4 acc[MB];
#pragma unroll
    for (int mb = 0; mb < MB; ++mb) acc[mb] = (f32x4){0.f, 0.f, 0.f, 0.f};

    bf16x8 wa[4], wb[4], xa[MB], xb[MB];
    auto load = [&](bf16x8 (&w)[4], bf16x8 (&x)[MB], int c) {
#pragma unroll
        for (int j = 0; j < 4; ++j) w[j] = ld16(wld[j] + c * KSTEP);
#pragma unroll
        for (int i = 0; i < MB; ++i) x[i] = ld16(xld[i] + c * KSTEP);
        __builtin_amdgcn_sched_barrier(0);  // the loads stay in front of the other chunk's products
    };
    auto stage = [&](bf16x8 (&x)[MB], int buf) {
#pragma unroll
        for (int i = 0; i < MB; ++i)
            *reinterpret_cast<bf16x8*>(xs[buf] + (tid / 16 + 16 * i) * WT_PITCH + 16 * (tid % 16)) = x[i];
    };
    auto products = [&](bf16x8 (&w)[4], int buf) {
#pragma unroll
        for (int j = 0; j < 4; ++j)
            *reinterpret_cast<bf16x8*>(mytile + (4 * j + g) * WT_PITCH + 16 * r16) = w[j];
        bf16x8 a[4];
#pragma unroll
        for (int j = 0; j < 4; ++j)
            a[j] = *reinterpret_cast<const bf16x8*>(mytile + r16 * WT_PITCH + 64 * g + 16 * j);
#pragma unroll
        for (int mb = 0; mb < MB; ++mb) {
            bf16x8 xf[4];
#pragma unroll
            for (int j = 0; j < 4; ++j)
                xf[j] = *reinterpret_cast<const bf16x8*>(xs[buf] + (mb * 16 + r16) * WT_PITCH + 64 * g + 16 * j);
#pragma unroll
            for (int j = 0; j < 4; ++j)
                acc[mb] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a[j], xf[j], acc[mb], 0, 0, 0);
        }
    };
    // Chunk c's X lives in buffer (c - c_lo) & 1.  One barrier per chunk: the X of chunk c + 1 is
    // written to the other buffer after the barrier that all readers of chunk c - 1 have passed.
    // The bounds are the same for every thread of the workgroup.
    int left = c_hi - c_lo;
    if (left > 0) {
        int c = c_lo;
        load(wa, xa, c);
        stage(xa, 0);
        while (left > 2) {
            load(wb, xb, c + 1);
            __syncthreads();
            products(wa, 0);
            stage(xb, 1);
            load(wa, xa, c + 2);
            __syncthreads();
            products(wb, 1);
            stage(xa, 0);
            c += 2;
            left -= 2;
        }
        if (left == 2) {
            load(wb, xb, c + 1);
            __syncthreads();
            products(wa, 0);
            stage(xb, 1);
            __syncthreads();
            products(wb, 1);
        } else {
            __syncthreads();
            products(wa, 0);
        }
    }
    // acc[mb][i]: row 16 mb + r16 of X, weight row n0 + 4 g + i
#pragma unroll
    for (int mb = 0; mb < MB; ++mb) {
        const int m = m0 + mb * 16 + r16;
        if (m >= M) continue;
        float* dst = part + ((size_t)run * M + m) * N + n0 + 4 * g;
        if (n0 + 4 * g + 3 < N) {
            *reinterpret_cast<float4*>(dst) = make_float4(acc[mb][0], acc[mb][1], acc[mb][2], acc[mb][3]);
        } else {
#pragma unroll
            for (int i = 0; i < 4; ++i)
                if (n0 + 4 * g + i < N) dst[i] = acc[mb][i];
        }
    }
}

// part [ks, M, N] float32: run r holds X[:, r-th run of K] W[:, the same]^T.  K a multiple of
// 128, N a multiple of 4; more than 64 rows run as blocks of 64.
extern "C" int rl_gemm_mid_parts(const void* X, const void* W, float* part, int M, int N, int K,
                                 int ldx, int ldw, int ks, hipStream_t stream) {
    if (M <= 0 || N <= 0) return RL_OK;
    if (M > 64 * 65535 || K < KSTEP || K % KSTEP || N % 4 || ldx % 8 || ldw % 8 || ldx < K || ldw < K || ks < 1 ||
        ks > K / KSTEP || !part)
        return RL_ERR_ARG;
    const int chunks = K / KSTEP, per = (chunks + ks - 1) / ks;
    if ((per * (ks - 1)) >= chunks) return RL_ERR_ARG;  // every run holds a chunk
    dim3 grid((N + MW * 16 - 1) / (MW * 16), ks, (M + 63) / 64), block(MW * RL_WAVE);
    const bf16_t* x = (const bf16_t*)X;
    const bf16_t* w = (const bf16_t*)W;
    if (M <= 16)
        hipLaunchKernelGGL((gemm_mid_kernel<1>), grid, block, 0, stream, x, w, part, M, N, K, ldx, ldw, per);
    else if (M <= 32)
        hipLaunchKernelGGL((gemm_mid_kernel<2>), grid, block, 0, stream, x, w, part, M, N, K, ldx, ldw, per);
    else if (M <= 48)
        hipLaunchKernelGGL((gemm_mid_kernel<3>), grid, block, 0, stream, x, w, part, M, N, K, ldx, ldw, per);
    else
        hipLaunchKernelGGL((gemm_mid_kernel<4>), grid, block, 0, stream, x, w, part, M, N, K, ldx, ldw, per);
    return rl_launch_status();
}

// =========================================================================== //
// 17 .. 512 rows over matrices of a few megabytes: the whole product in one launch
// =========================================================================== //
// Where a model's matrices are a few megabytes (Qwen3-0.6B: 4 to 13 MB) a decode step of tens
// or hundreds of rows is bound by how long each kernel takes to get going, not by its bytes,
// and the library's kernels for such shapes take 10 to 15 us each (few, large tiles that
// walk K in sixteen dependent steps).  This is the mid-size kernel's tile (four waves of 16
// weight rows, a chunk of X through LDS, two chunks of weights in flight) over a grid of
// weight-row blocks x row blocks of X, writing bfloat16 directly; MB blocks of 16 rows of X a
// workgroup.  SWIGLU: waves 0, 1 hold gate rows n .. n + 31, waves 2, 3 the up rows of the same
// columns; the up halves cross LDS and the gate waves write silu(gate) * up, both rounded to
// bfloat16 first as a stored product would be.
template <int MB, bool SWIGLU>
__global__ __launch_bounds__(MW* RL_WAVE) void gemm_tile_kernel(
    const bf16_t* __restrict__ X, const bf16_t* __restrict__ W, bf16_t* __restrict__ out, int M,
    int N, int K, int ldx, int ldw, int ldo) {
    __shared__ __attribute__((aligned(16))) unsigned char xs[2][MB * 16 * WT_PITCH];
    __shared__ __attribute__((aligned(16))) unsigned char wtile[MW][16 * WT_PITCH];
    const int tid = threadIdx.x, lane = tid & (RL_WAVE - 1), wave = tid / RL_WAVE;
    const int r16 = lane & 15, g = lane >> 4;
    const int m0 = blockIdx.y * (16 * MB);
    // first output column of the wave's tile, and the weight row that holds it
    const int n0 = SWIGLU ? blockIdx.x * 32 + 16 * (wave & 1) : (blockIdx.x * MW + wave) * 16;
    const int w0 = (SWIGLU && wave >= 2) ? N : 0;  // the up rows follow the N gate rows
    const bf16_t* wld[4];
#pragma unroll
    for (int j = 0; j < 4; ++j)
        wld[j] = W + (size_t)(w0 + min(n0 + 4 * j + g, N - 1)) * ldw + 8 * r16;
    const bf16_t* xld[MB];
#pragma unroll
    for (int i = 0; i < MB; ++i)
        xld[i] = X + (size_t)min(m0 + tid / 16 + 16 * i, M - 1) * ldx + 8 * (tid % 16);
    unsigned char* mytile = wtile[wave];
    f32x4 acc[MB];
#pragma unroll
    for (int mb = 0; mb < MB; ++mb) acc[mb] = (f32x4){0.f, 0.f, 0.f, 0.f};

    bf16x8 wa[4], wb[4], xa[MB], xb[MB];
    auto load = [&](bf16x8 (&w)[4], bf16x8 (&x)[MB], int c) {
#pragma unroll
        for (int j = 0; j < 4; ++j) w[j] = ld16(wld[j] + c * KSTEP);
#pragma unroll
        for (int i = 0; i < MB; ++i) x[i] = ld16(xld[i] + c * KSTEP);
        __builtin_amdgcn_sched_barrier(0);  // the loads stay in front of the other chunk's products
    };
    auto stage = [&](bf16x8 (&x)[MB], int buf) {
#pragma unroll
        for (int i = 0; i < MB; ++i)
            *reinterpret_cast<bf16x8*>(xs[buf] + (tid / 16 + 16 * i) * WT_PITCH + 16 * (tid % 16)) = x[i];
    };
    auto products = [&](bf16x8 (&w)[4], int buf) {
#pragma unroll
        for (int j = 0; j < 4; ++j)
            *reinterpret_cast<bf16x8*>(mytile + (4 * j + g) * WT_PITCH + 16 * r16) = w[j];
        bf16x8 a[4];
#pragma unroll
        for (int j = 0; j < 4; ++j)
            a[j] = *reinterpret_cast<const bf16x8*>(mytile + r16 * WT_PITCH + 64 * g + 16 * j);
#pragma unroll
        for (int mb = 0; mb < MB; ++mb) {
            bf16x8 xf[4];
#pragma unroll
            for (int j = 0; j < 4; ++j)
                xf[j] = *reinterpret_cast<const bf16x8*>(xs[buf] + (mb * 16 + r16) * WT_PITCH + 64 * g + 16 * j);
#pragma unroll
            for (int j = 0; j < 4; ++j)
                acc[mb] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a[j], xf[j], acc[mb], 0, 0, 0);
        }
    };
    // as in the mid-size kernel: chunk c's X lives in buffer c & 1, one barrier per chunk
    int left = K / KSTEP;  // at least one (host-checked)
    int c = 0;
    load(wa, xa, c);
    stage(xa, 0);
    while (left > 2) {
        load(wb, xb, c + 1);
        __syncthreads();
        products(wa, 0);
        stage(xb, 1);
        load(wa, xa, c + 2);
        __syncthreads();
        products(wb, 1);
        stage(xa, 0);
        c += 2;
        left -= 2;
    }
    if (left == 2) {
        load(wb, xb, c + 1);
        __syncthreads();
        products(wa, 0);
        stage(xb, 1);
        __syncthreads();
        products(wb, 1);
    } else {
        __syncthreads();
        products(wa, 0);
    }
    // acc[mb][i]: row m0 + 16 mb + r16 of X, column n0 + 4 g + i
    if (SWIGLU) {
        float* up = reinterpret_cast<float*>(xs);  // [2 waves][MB][4][64 lanes], where X was
        static_assert(sizeof(float) * 2 * MB * 4 * RL_WAVE <= sizeof(xs), "the up halves fit where X was");
        __syncthreads();  // every wave has read its last chunk of X
        if (wave >= 2) {
#pragma unroll
            for (int mb = 0; mb < MB; ++mb)
#pragma unroll
                for (int i = 0; i < 4; ++i) up[(((wave - 2) * MB + mb) * 4 + i) * RL_WAVE + lane] = acc[mb][i];
        }
        __syncthreads();
        if (wave >= 2) return;
#pragma unroll
        for (int mb = 0; mb < MB; ++mb)
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const float gate = bf16_to_float(float_to_bf16(acc[mb][i]));
                const float u = bf16_to_float(float_to_bf16(up[((wave * MB + mb) * 4 + i) * RL_WAVE + lane]));
                acc[mb][i] = gate / (1.f + expf(-gate)) * u;
            }
    }
#pragma unroll
    for (int mb = 0; mb < MB; ++mb) {
        const int m = m0 + mb * 16 + r16;
        if (m >= M) continue;
        bf16_t* dst = out + (size_t)m * ldo + n0 + 4 * g;
        if (n0 + 4 * g + 3 < N) {
            struct {
                bf16_t v[4];
            } o;
#pragma unroll
            for (int i = 0; i < 4; ++i) o.v[i] = float_to_bf16(acc[mb][i]);
            *reinterpret_cast<uint2*>(dst) = __builtin_bit_cast(uint2, o);
        } else {
#pragma unroll
            for (int i = 0; i < 4; ++i)
                if (n0 + 4 * g + i < N) dst[i] = float_to_bf16(acc[mb][i]);
        }
    }
}

// out[M, N] = X W^T as bfloat16 (swiglu == 0), or out[M, N] = silu(X Wg^T) * (X Wu^T) with
// W = [Wg | Wu] stacked by rows, [2N, K].  K a multiple of 128, ldo a multiple of 4.
extern "C" int rl_gemm_tile(const void* X, const void* W, void* out, int M, int N, int K, int ldx,
                            int ldw, int ldo, int swiglu, hipStream_t stream) {
    if (M <= 0 || N <= 0) return RL_OK;
    if (K < KSTEP || K % KSTEP || ldx % 8 || ldw % 8 || ldx < K || ldw < K || ldo % 4 || ldo < N || !out)
        return RL_ERR_ARG;
    const int row_blocks = (M + 63) / 64;
    const int mb = ((M + row_blocks - 1) / row_blocks + 15) / 16;  // 16-row blocks a workgroup
    if (row_blocks > 65535) return RL_ERR_ARG;
    const int cols = swiglu ? 32 : MW * 16;
    dim3 grid((N + cols - 1) / cols, (M + 16 * mb - 1) / (16 * mb)), block(MW * RL_WAVE);
    const bf16_t* x = (const bf16_t*)X;
    const bf16_t* w = (const bf16_t*)W;
    bf16_t* o = (bf16_t*)out;
#define RL_TILE(MBV)                                                                              \
    do {                                                                                          \
        if (swiglu)                                                                               \
            hipLaunchKernelGGL((gemm_tile_kernel<MBV, true>), grid, block, 0, stream, x, w, o, M, \
                               N, K, ldx, ldw, ldo);                                              \
        else                                                                                      \
            hipLaunchKernelGGL((gemm_tile_kernel<MBV, false>), grid, block, 0, stream, x, w, o,   \
                               M, N, K, ldx, ldw, ldo);                                           \
    } while (0)
    if (mb == 1)
        RL_TILE(1);
    else if (mb == 2)
        RL_TILE(2);
    else if (mb == 3)
        RL_TILE(3);
    else
        RL_TILE(4);
#undef RL_TILE
    return rl_launch_status();
}
