// 17 .. 64 rows over wide bfloat16 matrices (the packed query/key/value and gate/up matrices,
// the output projection over the vocabulary): out[M, N] = X[M, K] W[N, K]^T, float32
// accumulation on the matrix cores, optionally with SwiGLU in the epilogue.
//
// A decode step of a few dozen requests is still bound by the weights' bytes, but X no longer
// fits the few-row kernel's scheme, where every wave reads the rows of X itself for every 16 or
// 32 weight rows: at 64 rows that is more traffic through the first-level cache than the
// weights are.  Here a compute unit gets one workgroup that owns a contiguous share of the
// matrix's tiles of 16 weight rows (its share of `units` tiles, or (gate, up) pairs of them),
// up to TB tiles, and walks K once for all of them:
//   * the waves interleave over K in chunks of 128 elements, as in the few-row kernel;
//   * for a chunk a wave turns its [16 MB x 128] piece of X into matrix-core operands once and
//     keeps them in registers for all TB tiles (X crosses the cache once per workgroup, not
//     once per tile); the next chunk's piece is asked for while this chunk is multiplied;
//   * weights and X are both read in runs of 256 contiguous bytes a quarter wave and brought
//     into the operand layout through a wave-private piece of LDS (no barrier: a wave reads
//     what it wrote itself); DEPTH tiles of weights are in flight per wave, no load stands
//     behind a condition;
//   * the waves' partial sums meet in LDS at the end and are added in wave order (no atomics:
//     the same bits every run).
// Workgroups of four waves have a SIMD's whole register file each (up to 10 tiles of
// accumulators beside two sets of X); eight waves where registers allow stream a little faster.
// Tiles beyond a workgroup's share read its last tile again and store nothing.
//
// Measured on MI355X against the library's product (plus the activation kernel where it
// applies), graph replays over weights rotated through 900 MB, microseconds at 17 / 32 / 64
// rows, the library first: Qwen3-8B gate/up with SwiGLU (201 MB) 48.7 / 40 .. 42, 50.9 / 41,
// 49.7 / 46; its vocabulary product with float32 results (1,245 MB) 269 / 240, 279 / 249,
// 282 / 285; its packed QKV matrix (50 MB), where a unit owns a tile and a half and X is two
// thirds of all traffic, 14.8 / 15.3, 16.4 / 16.4, 18.1 / 20.5.
#include "common.h"

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float f32x4 __attribute__((ext_vector_type(4)));

#define RK 128        // k elements a wave consumes per chunk
#define RT_PITCH 272  // bytes between the 16 rows of the LDS tile: 256 + 16, conflict-free reads

__device__ inline bf16x8 rows_ld16(const bf16_t* p) {
    return __builtin_bit_cast(bf16x8, *reinterpret_cast<const uint4*>(p));
}

template <typename T>
__device__ inline void rows_store4(T* p, const float (&v)[4]);
template <>
__device__ inline void rows_store4<float>(float* p, const float (&v)[4]) {
    *reinterpret_cast<float4*>(p) = make_float4(v[0], v[1], v[2], v[3]);
}
template <>
__device__ inline void rows_store4<bf16_t>(bf16_t* p, const float (&v)[4]) {
    struct {
        bf16_t b[4];
    } o;
#pragma unroll
    for (int i = 0; i < 4; ++i) o.b[i] = float_to_bf16(v[i]);
    *reinterpret_cast<uint2*>(p) = __builtin_bit_cast(uint2, o);
}

// TB: tiles of 16 weight rows a workgroup holds (SWIGLU: TB / 2 (gate, up) pairs; a "unit" is a
// tile, or a pair).  MB: blocks of 16 rows of X.  DEPTH: tiles of weights in flight per wave
// (TB % DEPTH == 0, so that the ring of register sets closes within a chunk).  NW: waves.
// N: result columns (SWIGLU: the width I of the result, W then has 2 N rows, gate rows first).
// Workgroup b owns units [b * units / gridDim.x, (b + 1) * units / gridDim.x): at most TB (host).
template <int TB, int MB, bool SWIGLU, typename OutT, int DEPTH, int NW>
__global__ __launch_bounds__(NW* RL_WAVE) void gemm_rows_kernel(
    const bf16_t* __restrict__ X, const bf16_t* __restrict__ W, OutT* __restrict__ out, int M,
    int N, int K, int ldx, int ldw, int ldo) {
    static_assert(TB % DEPTH == 0, "the ring of tiles in flight closes within a chunk");
    static_assert(!SWIGLU || TB % 2 == 0, "gate and up tiles come in pairs");
    constexpr int TPU = SWIGLU ? 2 : 1;  // tiles per unit
    constexpr int UNITS = TB / TPU;      // units a workgroup holds at most
    // units whose partial sums cross LDS together: what fits 96 KB (every barrier of the epilogue
    // stands in the open, nothing streams behind it)
    constexpr int UPR_FIT = 96 / (NW * TPU * MB);
    constexpr int UPR = UPR_FIT < 1 ? 1 : (UPR_FIT > UNITS ? UNITS : UPR_FIT);
    __shared__ __attribute__((aligned(16))) unsigned char wtile[NW][16 * RT_PITCH];
    __shared__ float red[NW][UPR * TPU * MB * 256];

    const int lane = threadIdx.x & (RL_WAVE - 1);
    const int wave = threadIdx.x / RL_WAVE;
    const int r16 = lane & 15;
    const int g = lane >> 4;
    const int units = N / 16;
    const int lo = (int)((long)blockIdx.x * units / (int)gridDim.x);
    const int hi = (int)((long)(blockIdx.x + 1) * units / (int)gridDim.x);
    if (hi <= lo) return;  // the same for every thread of the workgroup

    // first weight row of tile t (the same for all lanes); tiles beyond the workgroup's share
    // read its last unit again
    auto tile_row = [&](int t) -> int {
        const int u = min(lo + t / TPU, hi - 1);
        return u * 16 + ((SWIGLU && (t & 1)) ? N : 0);
    };
    // instruction j of a tile reads row 4 j + g of the tile at bytes 16 r16
    const bf16_t* wl = W + (size_t)g * ldw + 8 * r16;
    const bf16_t* xl[MB][4];
#pragma unroll
    for (int mb = 0; mb < MB; ++mb)
#pragma unroll
        for (int j = 0; j < 4; ++j) xl[mb][j] = X + (size_t)min(mb * 16 + 4 * j + g, M - 1) * ldx + 8 * r16;
    unsigned char* mytile = wtile[wave];

    f32x4 acc[TB][MB];
#pragma unroll
    for (int t = 0; t < TB; ++t)
#pragma unroll
        for (int mb = 0; mb < MB; ++mb) acc[t][mb] = (f32x4){0.f, 0.f, 0.f, 0.f};

    constexpr int S = NW * RK;
    const int nchunk = (K / RK - wave + NW - 1) / NW;  // chunks of this wave (K a multiple of 128)
    if (nchunk > 0) {
        bf16x8 wr[DEPTH][4];
        bf16x8 xr[MB][4], xf[MB][4];
        auto wload = [&](bf16x8 (&r)[4], int t, int kw) {
            const bf16_t* base = wl + (size_t)tile_row(t) * ldw + kw;
#pragma unroll
            for (int j = 0; j < 4; ++j) r[j] = rows_ld16(base + (size_t)(4 * j) * ldw);
        };
        auto xload = [&](int kw) {
#pragma unroll
            for (int mb = 0; mb < MB; ++mb)
#pragma unroll
                for (int j = 0; j < 4; ++j) xr[mb][j] = rows_ld16(xl[mb][j] + kw);
        };
        // a tile as it was read (instruction j: rows 4 j + g, bytes 16 r16) into the operand
        // layout (lane (r16, g): row r16, elements 32 g + 8 j ..)
        auto turn = [&](const bf16x8 (&raw)[4], bf16x8 (&frag)[4]) {
#pragma unroll
            for (int j = 0; j < 4; ++j)
                *reinterpret_cast<bf16x8*>(mytile + (4 * j + g) * RT_PITCH + 16 * r16) = raw[j];
#pragma unroll
            for (int j = 0; j < 4; ++j)
                frag[j] = *reinterpret_cast<const bf16x8*>(mytile + r16 * RT_PITCH + 64 * g + 16 * j);
        };
        const int k_first = wave * RK;
        const int k_last = k_first + (nchunk - 1) * S;
        xload(k_first);
#pragma unroll
        for (int d = 0; d < DEPTH; ++d) wload(wr[d], d, k_first);
        for (int c = 0; c < nchunk; ++c) {
            const int kw = k_first + c * S;
            const int kn = min(kw + S, k_last);  // the chunk after (the last one again at the end)
#pragma unroll
            for (int mb = 0; mb < MB; ++mb) turn(xr[mb], xf[mb]);
            xload(kn);
#pragma unroll
            for (int t = 0; t < TB; ++t) {
                bf16x8(&r)[4] = wr[t % DEPTH];
                bf16x8 a[4];
                turn(r, a);
                // the tile DEPTH further on, into the registers just stored
                if (t + DEPTH < TB)
                    wload(r, t + DEPTH, kw);
                else
                    wload(r, t + DEPTH - TB, kn);
#pragma unroll
                for (int j = 0; j < 4; ++j)
#pragma unroll
                    for (int mb = 0; mb < MB; ++mb)
                        acc[t][mb] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a[j], xf[mb][j], acc[t][mb], 0, 0, 0);
            }
        }
    }

    // the waves' partial sums of UPR units at a time through LDS, added in wave order
    constexpr int ROUNDS = (UNITS + UPR - 1) / UPR;
#pragma unroll
    for (int rd = 0; rd < ROUNDS; ++rd) {
        if (rd) __syncthreads();
#pragma unroll
        for (int uu = 0; uu < UPR; ++uu)
#pragma unroll
            for (int tt = 0; tt < TPU; ++tt) {
                const int t = (rd * UPR + uu) * TPU + tt;
                if (t < TB) {
#pragma unroll
                    for (int mb = 0; mb < MB; ++mb)
#pragma unroll
                        for (int i = 0; i < 4; ++i)
                            red[wave][(((uu * TPU + tt) * MB + mb) * 4 + i) * 64 + lane] = acc[t < TB ? t : 0][mb][i];
                }
            }
        __syncthreads();
        for (int e = threadIdx.x; e < UPR * MB * 64; e += NW * RL_WAVE) {
            const int ln = e & 63, mb = (e >> 6) % MB, uu = e / (MB * 64);
            const int m = mb * 16 + (ln & 15);
            const int unit = lo + rd * UPR + uu;
            if (m >= M || unit >= hi || rd * UPR + uu >= UNITS) continue;
            float v[4];
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                if (SWIGLU) {
                    float gate = 0.f, up = 0.f;
#pragma unroll
                    for (int w = 0; w < NW; ++w) {
                        gate += red[w][(((uu * 2 + 0) * MB + mb) * 4 + i) * 64 + ln];
                        up += red[w][(((uu * 2 + 1) * MB + mb) * 4 + i) * 64 + ln];
                    }
                    // the activation reads its operands rounded to bfloat16, as the unfused path
                    // does where the product's result is stored before the activation
                    // (rapid_llm/kernels/ops/activation/swiglu.py:91-121)
                    gate = bf16_to_float(float_to_bf16(gate));
                    up = bf16_to_float(float_to_bf16(up));
                    v[i] = gate / (1.f + expf(-gate)) * up;
                } else {
                    float s = 0.f;
#pragma unroll
                    for (int w = 0; w < NW; ++w) s += red[w][((uu * MB + mb) * 4 + i) * 64 + ln];
                    v[i] = s;
                }
            }
            rows_store4<OutT>(out + (size_t)m * ldo + unit * 16 + 4 * (ln >> 4), v);
        }
    }
}

template <int TB, int MB, bool SWIGLU, typename OutT, int DEPTH, int NW>
static int rows_launch(const void* X, const void* W, void* out, int M, int N, int K, int ldx, int ldw,
                       int ldo, int groups, hipStream_t stream) {
    hipLaunchKernelGGL((gemm_rows_kernel<TB, MB, SWIGLU, OutT, DEPTH, NW>), dim3(groups), dim3(NW * RL_WAVE), 0,
                       stream, (const bf16_t*)X, (const bf16_t*)W, (OutT*)out, M, N, K, ldx, ldw, ldo);
    return rl_launch_status();
}

// Eight waves where their registers hold the accumulators and both sets of X, four waves with a
// SIMD's whole register file each otherwise.
constexpr int rows_waves(int tb, int mb) { return (tb <= 3 || (tb <= 6 && mb <= 3)) ? 8 : 4; }

template <int TB, bool SWIGLU, typename OutT, int DEPTH>
static int rows_by_blocks(const void* X, const void* W, void* out, int M, int N, int K, int ldx, int ldw,
                          int ldo, int groups, hipStream_t stream) {
    switch ((M + 15) / 16) {
        case 1:
        case 2:
            return rows_launch<TB, 2, SWIGLU, OutT, DEPTH, rows_waves(TB, 2)>(X, W, out, M, N, K, ldx, ldw, ldo, groups, stream);
        case 3:
            return rows_launch<TB, 3, SWIGLU, OutT, DEPTH, rows_waves(TB, 3)>(X, W, out, M, N, K, ldx, ldw, ldo, groups, stream);
        default:
            return rows_launch<TB, 4, SWIGLU, OutT, DEPTH, rows_waves(TB, 4)>(X, W, out, M, N, K, ldx, ldw, ldo, groups, stream);
    }
}

// Whether a kernel is built that holds `per_group` units (tiles of 16 result columns; with SwiGLU
// a gate and an up tile each) a workgroup at M rows: the host picks among these and sets the
// number of workgroups.  Five pairs beside 64 rows of X overflow a SIMD's registers into its
// accumulation registers and back (measured: 179 us where three pairs take 136); seven pairs
// were slower than the library at every row count and are not built.
extern "C" int rl_gemm_rows_holds(int swiglu, int per_group, int M) {
    if (M < 1 || M > 64) return 0;
    if (swiglu) return per_group == 2 || per_group == 3 || (per_group == 5 && M <= 48);
    return per_group == 1 || per_group == 2 || per_group == 3 || per_group == 6;
}

// out[M, N] = X W^T (swiglu == 0; out_type RL_F32 or RL_BF16), or out[M, N] = silu(X Wg^T) *
// (X Wu^T) as bfloat16 with W = [Wg | Wu] stacked by rows, [2 N, K].  1 <= M <= 64, N a multiple
// of 16, K a multiple of 128.  `groups` workgroups share the N / 16 units evenly, each at most
// `per_group` of them (one of rl_gemm_rows_holds).
extern "C" int rl_gemm_rows(const void* X, const void* W, void* out, int M, int N, int K, int ldx, int ldw,
                            int ldo, int swiglu, int out_type, int per_group, int groups, hipStream_t stream) {
    if (M <= 0 || N <= 0) return RL_OK;
    if (M > 64 || N % 16 || K < RK || K % RK || ldx % 8 || ldw % 8 || ldx < K || ldw < K || ldo % 4 || ldo < N ||
        !X || !W || !out || groups < 1)
        return RL_ERR_ARG;
    const int units = N / 16;
    if (groups > units || (units + groups - 1) / groups > per_group || !rl_gemm_rows_holds(swiglu, per_group, M))
        return RL_ERR_ARG;
#define RL_ROWS(PER, TBV, SW, OT, DV) \
    if (per_group == PER) return rows_by_blocks<TBV, SW, OT, DV>(X, W, out, M, N, K, ldx, ldw, ldo, groups, stream);
    if (swiglu) {
        if (out_type != RL_BF16) return RL_ERR_ARG;
        RL_ROWS(2, 4, true, bf16_t, 2)
        RL_ROWS(3, 6, true, bf16_t, 2)
        RL_ROWS(5, 10, true, bf16_t, 2)
        return RL_ERR_ARG;
    }
    if (out_type == RL_BF16) {
        RL_ROWS(1, 1, false, bf16_t, 1)
        RL_ROWS(2, 2, false, bf16_t, 2)
        RL_ROWS(3, 3, false, bf16_t, 3)
        RL_ROWS(6, 6, false, bf16_t, 3)
        return RL_ERR_ARG;
    }
    if (out_type == RL_F32) {
        RL_ROWS(1, 1, false, float, 1)
        RL_ROWS(2, 2, false, float, 2)
        RL_ROWS(3, 3, false, float, 3)
        RL_ROWS(6, 6, false, float, 3)
        return RL_ERR_ARG;
    }
#undef RL_ROWS
    return RL_ERR_ARG;
}
