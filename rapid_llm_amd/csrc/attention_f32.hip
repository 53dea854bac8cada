// Paged causal attention in true float32 on the matrix cores' float32 instruction
// (v_mfma_f32_16x16x4_f32), compiled for one head size RL_HEAD_DIM (a multiple of 16).
//
// One workgroup of four waves per (tile of 16 rows, kv head).  Rows are (token, query head of
// the kv group) pairs of ONE request, so grouped heads and neighbouring tokens share every key
// that is read.  The key tiles are dealt to the waves by their absolute index (tile i goes to
// wave i % 4), each wave keeps a softmax state of its own, and the four states are folded in
// the order of the waves: a single token's long context is then read by four waves at once.  As in the bfloat16 kernels the transposed products are computed,
//   S^T[keys, rows] = K[keys, d] Q^T[d, rows],   O^T[d, rows] += V^T[d, keys] P^T[keys, rows],
// which leaves a lane with the scores of keys 4g .. 4g + 3 of its own row: exactly its
// operand of the second product, whose other operand is one 16-byte read of the transposed
// value cache.  Softmax state is one scalar per lane.
//
// A row's result does not depend on the tile it falls in, on the other rows there, or on how
// a prompt was cut into steps: keys are taken in tiles of 16 at absolute positions 0, 16, ..,
// each wave takes its tiles in ascending order; within a tile the order of every sum is fixed
// by the key's position; a tile that holds no visible key of a row leaves that row's state as
// it is, exactly (factor 1, terms 0), and so does a wave without visible keys in the fold.  Masked keys contribute exactly zero
// (rapid_llm/kernels/ops/attention/flashdecoding.py:223-237); scores are (q . k) / sqrt(d)
// (rapid_llm/modules/attention.py:62), softmax over keys in float32
// (rapid_llm/kernels/ops/attention/flashattention2_nopad.py:138-168).
#include "common.h"

#ifndef RL_HEAD_DIM
#error "compile with -DRL_HEAD_DIM=<head size>"
#endif

namespace f32attn {

constexpr int D = RL_HEAD_DIM;
constexpr int DB = D / 16;  // 16-channel chunks of the first product = blocks of the output
constexpr int AW = 4;       // waves per workgroup: key tile i belongs to wave i % AW
typedef float f32x4 __attribute__((ext_vector_type(4)));

__device__ inline f32x4 ld4(const float* p) { return *reinterpret_cast<const f32x4*>(p); }

// the four lanes (r, g = 0..3) that share a row: the same bits in each of them
__device__ inline float row_max(float v) {
    v = fmaxf(v, __shfl_xor(v, 16, RL_WAVE));
    return fmaxf(v, __shfl_xor(v, 32, RL_WAVE));
}
__device__ inline float row_sum(float v) {
    v += __shfl_xor(v, 16, RL_WAVE);
    return v + __shfl_xor(v, 32, RL_WAVE);
}

// tile_info: [tiles][3] = index of the request's first token in the step, its tokens in the
// step, first row of the tile.  The request's first position is read from `positions`.
__global__ __launch_bounds__(AW* RL_WAVE) void attn_f32_kernel(
    const float* __restrict__ q, const float* __restrict__ k_cache,
    const float* __restrict__ v_cache, float* __restrict__ out,
    const int* __restrict__ tile_info, const int* __restrict__ positions,
    const int* __restrict__ token_slot, const int* __restrict__ block_table, int table_stride,
    int page_size, int nq, int nkv, int window, float scale) {
    const int tile = blockIdx.x;
    const int hk = blockIdx.y;
    const int G = nq / nkv;
    const int at = tile_info[3 * tile], n = tile_info[3 * tile + 1], row0 = tile_info[3 * tile + 2];
    __shared__ float fold_ml[AW - 1][2][RL_WAVE];
    __shared__ float fold_acc[AW - 1][DB * 4][RL_WAVE];
    const int lane = threadIdx.x & (RL_WAVE - 1);
    const int wave = threadIdx.x / RL_WAVE;
    const int r16 = lane & 15;
    const int g = lane >> 4;
    const int start = positions[at];
    const int* table = block_table + (size_t)token_slot[at] * table_stride;

    const int rows = n * G;
    const int row = row0 + r16;
    const bool row_ok = row < rows;
    const int tok = (row_ok ? row : rows - 1) / G;
    const int head = hk * G + (row_ok ? row : rows - 1) % G;
    const int pos = start + tok;
    const int kend = pos + 1;
    const int kstart = (window > 0 && pos - window + 1 > 0) ? pos - window + 1 : 0;

    // the keys any row of the tile sees: from the first row's first key (rows ascend with
    // the tokens), in whole tiles of 16, up to the last row's own position
    const int first_pos = start + row0 / G;
    const int last_pos = start + (min(rows, row0 + 16) - 1) / G;
    const int first_key = (window > 0 && first_pos - window + 1 > 0) ? first_pos - window + 1 : 0;
    const int lo = first_key & ~15;
    const int hi = last_pos + 1;  // keys below hi are in the cache

    // Q^T: lane (row r16, g) holds channels 16c + 4g .. + 3 of its row
    f32x4 qf[DB];
    {
        const float* qrow = q + ((size_t)(at + tok) * nq + head) * D + 4 * g;
#pragma unroll
        for (int c = 0; c < DB; ++c) qf[c] = row_ok ? ld4(qrow + 16 * c) : (f32x4){0.f, 0.f, 0.f, 0.f};
    }

    float m = -INFINITY, l = 0.f;
    f32x4 acc[DB];
#pragma unroll
    for (int b = 0; b < DB; ++b) acc[b] = (f32x4){0.f, 0.f, 0.f, 0.f};

    // operands of one tile of 16 keys: lane (key r16, g) reads channels 16c + 4g .. + 3 of its
    // key; lane (channel r16, g) reads keys kb + 4g .. + 3 of its channel in every block
    struct Frags {
        f32x4 k[DB], v[DB];
    };
    auto load = [&](int kb, Frags& f) {
        const int key = min(kb + r16, hi - 1);  // beyond the cache: any real key, masked below
        const float* krow =
            k_cache + (((size_t)table[key / page_size] * nkv + hk) * page_size + key % page_size) * D + 4 * g;
#pragma unroll
        for (int c = 0; c < DB; ++c) f.k[c] = ld4(krow + 16 * c);
        const int key4 = min(kb + 4 * g, (hi - 1) & ~3);
        const float* vrow = v_cache +
                            (((size_t)table[key4 / page_size] * nkv + hk) * D + r16) * page_size +
                            key4 % page_size;
#pragma unroll
        for (int b = 0; b < DB; ++b) f.v[b] = ld4(vrow + (size_t)16 * b * page_size);
    };

    // S^T = K Q^T of one tile, the chunks dealt to four accumulators that are added at the
    // end (one chain of dependent instructions would leave the matrix core idle)
    auto scores = [&](const Frags& f) -> f32x4 {
        f32x4 part[4];
#pragma unroll
        for (int a4 = 0; a4 < 4; ++a4) part[a4] = (f32x4){0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int c = 0; c < DB; ++c)
#pragma unroll
            for (int j = 0; j < 4; ++j)
                part[c & 3] =
                    __builtin_amdgcn_mfma_f32_16x16x4f32(f.k[c][j], qf[c][j], part[c & 3], 0, 0, 0);
        return (part[0] + part[1]) + (part[2] + part[3]);
    };

    // softmax and second product of the tile at kb, given its scores and its values
    auto finish_tile = [&](int kb, f32x4 s, const f32x4 (&vcur)[DB]) {
        // ---- this lane's keys kb + 4g + i of its own row ------------------------------------
        float tmax = -INFINITY;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const int key = kb + 4 * g + i;
            const bool seen = row_ok && key >= kstart && key < kend;
            s[i] = seen ? s[i] * scale : -INFINITY;
            tmax = fmaxf(tmax, s[i]);
        }
        tmax = row_max(tmax);
        const float m_new = fmaxf(m, tmax);
        float alpha = 1.f;  // no visible key so far and none here: nothing changes
        f32x4 p = (f32x4){0.f, 0.f, 0.f, 0.f};
        if (m_new != -INFINITY) {
            alpha = expf(m - m_new);  // m = -inf before the row's first key: 0
#pragma unroll
            for (int i = 0; i < 4; ++i) p[i] = expf(s[i] - m_new);  // masked: exactly 0
        }
        l = l * alpha + row_sum((p[0] + p[1]) + (p[2] + p[3]));
        m = m_new;
        // ---- O^T = O^T alpha + V^T P^T --------------------------------------------------------
#pragma unroll
        for (int b = 0; b < DB; ++b) {
            f32x4 vf = vcur[b];
            // keys no row of the tile sees (beyond the cache, or before the window, whose
            // pages may have been given back) may hold anything: 0 * it must be 0
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const int key = kb + 4 * g + i;
                if (key >= hi || key < first_key) vf[i] = 0.f;
            }
#pragma unroll
            for (int i = 0; i < 4; ++i) acc[b][i] *= alpha;
#pragma unroll
            for (int j = 0; j < 4; ++j)
                acc[b] = __builtin_amdgcn_mfma_f32_16x16x4f32(vf[j], p[j], acc[b], 0, 0, 0);
        }
    };

    // Software pipeline over the wave's tiles: while a tile goes through softmax and the second
    // product, the scores of the next have been multiplied and the operands of the one after
    // are in flight.  The last two tiles stand outside the loop, so that inside it the loads
    // are issued without a condition and stay where they are written (behind a condition the
    // compiler counts a load as absent and makes every older operand wait for it; left to
    // itself the scheduler moves loads down to their use).
    constexpr int STEP = 16 * AW;
    const int mine = lo + 16 * ((wave - lo / 16) & (AW - 1));  // first tile >= lo with index % AW == wave
    if (mine < hi) {
        int left = (hi - mine + STEP - 1) / STEP;  // tiles of this wave, the current one included
        int kb = mine;
        Frags nxt;
        f32x4 vcur[DB], vnext[DB];
        load(kb, nxt);
        f32x4 sc = scores(nxt);
#pragma unroll
        for (int b = 0; b < DB; ++b) vcur[b] = nxt.v[b];
        if (left > 1) load(kb + STEP, nxt);
        while (left > 2) {
            const f32x4 s_next = scores(nxt);
#pragma unroll
            for (int b = 0; b < DB; ++b) vnext[b] = nxt.v[b];
            load(kb + 2 * STEP, nxt);
            __builtin_amdgcn_sched_barrier(0);
            finish_tile(kb, sc, vcur);
            sc = s_next;
#pragma unroll
            for (int b = 0; b < DB; ++b) vcur[b] = vnext[b];
            kb += STEP;
            --left;
        }
        if (left == 2) {
            const f32x4 s_next = scores(nxt);
            finish_tile(kb, sc, vcur);
            finish_tile(kb + STEP, s_next, nxt.v);
        } else {
            finish_tile(kb, sc, vcur);
        }
    }
    // ---- fold the waves' states in their order (a wave without visible keys has m = -inf,
    // l = 0 and zero sums: it changes nothing, exactly) ----------------------------------------
    if (wave > 0) {
        fold_ml[wave - 1][0][lane] = m;
        fold_ml[wave - 1][1][lane] = l;
#pragma unroll
        for (int b = 0; b < DB; ++b)
#pragma unroll
            for (int i = 0; i < 4; ++i) fold_acc[wave - 1][4 * b + i][lane] = acc[b][i];
    }
    __syncthreads();
    if (wave > 0) return;
#pragma unroll
    for (int w = 0; w < AW - 1; ++w) {
        const float m_w = fold_ml[w][0][lane], l_w = fold_ml[w][1][lane];
        const float m_new = fmaxf(m, m_w);
        if (m_new == -INFINITY) continue;
        const float fa = expf(m - m_new), fb = expf(m_w - m_new);
        l = l * fa + l_w * fb;
#pragma unroll
        for (int b = 0; b < DB; ++b)
#pragma unroll
            for (int i = 0; i < 4; ++i) acc[b][i] = acc[b][i] * fa + fold_acc[w][4 * b + i][lane] * fb;
        m = m_new;
    }
    if (!row_ok) return;
    // acc[b][i] is channel 16b + 4g + i of the lane's row
    float* orow = out + ((size_t)(at + tok) * nq + head) * D + 4 * g;
    const float inv = 1.f / l;
#pragma unroll
    for (int b = 0; b < DB; ++b)
        *reinterpret_cast<f32x4*>(orow + 16 * b) =
            (f32x4){acc[b][0] * inv, acc[b][1] * inv, acc[b][2] * inv, acc[b][3] * inv};
}

}  // namespace f32attn

// Every token of the step, single tokens and portions alike.  page_size must be a multiple
// of 4 (the four keys of a lane lie in one page).
extern "C" int rl_attn_f32(const float* q, const float* k_cache, const float* v_cache, float* out,
                           const int* tile_info, int num_tiles, const int* positions,
                           const int* token_slot, const int* block_table, int table_stride,
                           int page_size, int nq, int nkv, int window, float scale,
                           hipStream_t stream) {
    if (num_tiles <= 0) return RL_OK;
    if (nkv < 1 || nq % nkv || page_size < 4 || page_size % 4 || nkv > 65535) return RL_ERR_ARG;
    hipLaunchKernelGGL(f32attn::attn_f32_kernel, dim3(num_tiles, nkv), dim3(f32attn::AW * RL_WAVE), 0, stream, q,
                       k_cache, v_cache, out, tile_info, positions, token_slot, block_table,
                       table_stride, page_size, nq, nkv, window, scale);
    return rl_launch_status();
}
