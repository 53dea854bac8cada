// Matrix-core (MFMA) paged attention for bfloat16 on gfx950, compiled for one head size
// RL_HEAD_DIM (a multiple of 16 up to 256).
//
// Both kernels compute the *transposed* products, so that nothing ever has to change
// layout between the two matrix products:
//
//   S^T[keys, rows]  = K[keys, d]   * Q^T[d, rows]      (A = K,   B = Q^T)
//   O^T[d, rows]    += V^T[d, keys] * P^T[keys, rows]   (A = V^T, B = P^T)
//
// with v_mfma_f32_16x16x32_bf16: a wave owns 16 "rows" (queries) as the N dimension.  The
// result of the first product leaves lane (row r, group g = lane / 16) with the scores of
// four tile rows 4g..4g+3 of each 16-key block.  Which key a tile row holds is free, and it is
// chosen so that the two blocks of a 32-key step leave the lane with the eight *consecutive*
// keys 8g..8g+7: tile row i of block kb holds key 8 (i / 4) + 4 kb + i % 4.  Those eight
// scores are then exactly the lane's contraction slots of the second product, whose A
// operand needs, for channel d, the values of the same eight keys: one 16-byte read, which is
// why the cache stores values transposed (V[page][head][d][slot]).  Softmax state (running
// maximum and sum) is one scalar per lane, since a lane only ever sees one row.
//
// Rows are (token, query head of the kv group) pairs, so grouped-query attention reads each
// key once for all heads of its group.  Softmax runs in the exp2 domain in float32
// (rapid_llm/kernels/ops/attention/flashattention2_nopad.py:138-168); P is rounded to
// bfloat16 for the second product (:162), sums use the unrounded values.
//
//   rl_attn_prefill: portions of prompts.  Workgroup = 4 waves x 32 rows; K and V^T tiles of
//                    64 keys go through LDS, the next tile travelling from memory while this
//                    one is multiplied (straight into a second set of tiles for heads of 128
//                    channels, through registers otherwise); one softmax step per 64 keys.
//   rl_attn_decode:  single tokens.  Workgroup = (request, kv head, split of the keys); its
//                    4 waves stride over 32-key steps reading K and V^T straight from
//                    global memory (nothing is reused), combine through LDS,
//                    and a merge kernel folds the splits (rapid_llm/kernels/ops/attention/
//                    flashdecoding.py:115-263 stage 1, :334-407 stage 2).  In its fused form
//                    it also norms and rotates q and k and writes the token's k and v.
#include "common.h"

#ifndef RL_HEAD_DIM
#error "compile with -DRL_HEAD_DIM=<head size>"
#endif

#define D RL_HEAD_DIM
static_assert(D % 16 == 0 && D >= 16 && D <= 256, "head size must be a multiple of 16 up to 256");

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef unsigned u32x2 __attribute__((ext_vector_type(2)));

constexpr int DC = (D + 31) / 32;     // 32-channel chunks of the first product
constexpr int DB = D / 16;            // 16-channel blocks of the output
constexpr bool D_TAIL = (D % 32) != 0;  // the last chunk holds 16 channels, the rest is zero

__device__ inline bf16x8 zero8() {
    bf16x8 z;
#pragma unroll
    for (int i = 0; i < 8; ++i) z[i] = (__bf16)0.f;
    return z;
}

__device__ inline bf16x8 load16(const bf16_t* p) {
    return __builtin_bit_cast(bf16x8, *reinterpret_cast<const uint4*>(p));
}

// two groups of four consecutive bfloat16 -> one operand
__device__ inline bf16x8 load8x2(const bf16_t* p0, const bf16_t* p1) {
    struct {
        uint2 a, b;
    } v;
    v.a = *reinterpret_cast<const uint2*>(p0);
    v.b = *reinterpret_cast<const uint2*>(p1);
    return __builtin_bit_cast(bf16x8, v);
}

__device__ inline f32x4 mfma(bf16x8 a, bf16x8 b, f32x4 c) {
    return __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b, c, 0, 0, 0);
}

// Maximum and sum over the four lanes (one in each row of 16) that hold the same query row:
// two lane swaps of gfx950 (the halves of the wave, then neighbouring rows of 16) instead of
// two trips through the LDS crossbar.
__device__ inline float row_max4(float v) {
    const unsigned u = __float_as_uint(v);
    const auto a = __builtin_amdgcn_permlane32_swap(u, u, false, false);
    const unsigned w = __float_as_uint(fmaxf(__uint_as_float(a[0]), __uint_as_float(a[1])));
    const auto b = __builtin_amdgcn_permlane16_swap(w, w, false, false);
    return fmaxf(__uint_as_float(b[0]), __uint_as_float(b[1]));
}
__device__ inline float row_sum4(float v) {
    const unsigned u = __float_as_uint(v);
    const auto a = __builtin_amdgcn_permlane32_swap(u, u, false, false);
    const unsigned w = __float_as_uint(__uint_as_float(a[0]) + __uint_as_float(a[1]));
    const auto b = __builtin_amdgcn_permlane16_swap(w, w, false, false);
    return __uint_as_float(b[0]) + __uint_as_float(b[1]);
}

// --------------------------------------------------------------------------- //
// One 32-key step of the online softmax for one block of 16 rows.
//   s0, s1: raw scores (q . k) of the two 16-key blocks: this lane's keys 8g..8g+3, 8g+4..8g+7
//   ok0, ok1: bit i set when key i of those four is visible to this lane's row
// Updates (m, l), scales the accumulators, returns P^T as the B operand.
// --------------------------------------------------------------------------- //
__device__ inline bf16x8 softmax_step(f32x4 s0, f32x4 s1, unsigned ok0, unsigned ok1,
                                      float scale_log2, float& m, float& l, f32x4* acc) {
    float x[8];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        x[i] = ((ok0 >> i) & 1u) ? s0[i] * scale_log2 : -INFINITY;
        x[4 + i] = ((ok1 >> i) & 1u) ? s1[i] * scale_log2 : -INFINITY;
    }
    float mx = x[0];
#pragma unroll
    for (int i = 1; i < 8; ++i) mx = fmaxf(mx, x[i]);
    mx = row_max4(mx);
    const float m_new = fmaxf(m, mx);
    // a row that has seen no visible key yet keeps m = -inf; exp2 of (-inf) - 0 is 0
    const float m_safe = (m_new == -INFINITY) ? 0.f : m_new;
    const float alpha = exp2f(m - m_safe);
    float psum = 0.f;
    bf16x8 p;
#pragma unroll
    for (int i = 0; i < 8; ++i) {
        const float e = exp2f(x[i] - m_safe);
        psum += e;
        p[i] = (__bf16)e;
    }
    l = l * alpha + psum;  // per-lane partial sum; the four groups are added at the end
    m = m_new;
#pragma unroll
    for (int b = 0; b < DB; ++b) {
        acc[b][0] *= alpha;
        acc[b][1] *= alpha;
        acc[b][2] *= alpha;
        acc[b][3] *= alpha;
    }
    return p;
}

// =========================================================================== //
// decode
// =========================================================================== //
#ifndef RL_DEC_WAVES
#define RL_DEC_WAVES 4
#endif
#define DEC_WAVES RL_DEC_WAVES
#define DEC_MAX_PAGES 1024  // pages one split may span (their ids are staged in LDS)

// Keys of one 32-key step as the two matrix products see them.  Tile row i of key block kb
// is the physical key  base + 8 (i / 4) + 4 kb + (i % 4),  so that lane (row, g) leaves the
// first product with the scores of the eight *consecutive* keys base + 8g .. base + 8g + 7:
// exactly its contraction slots of the second product, whose A operand (values, stored
// transposed) is then one 16-byte read of those eight positions of a channel.
struct DecodeFrags {
    bf16x8 k[2][DC];
    bf16x8 v[DB];
};

template <bool V16>
__device__ inline void decode_load(DecodeFrags& f, const bf16_t* k_cache, const bf16_t* v_cache,
                                   const int* pages,
                                   int page0, int page_size, int nkv, int hk, int base,
                                   int last_key, int col, int g) {
#pragma unroll
    for (int kb = 0; kb < 2; ++kb) {
        const int key = min(base + 8 * (col >> 2) + 4 * kb + (col & 3), last_key);  // masked later
        const int page = pages[key / page_size - page0];
        const bf16_t* krow =
            k_cache + (((size_t)page * nkv + hk) * page_size + key % page_size) * D;
#pragma unroll
        for (int c = 0; c < DC; ++c) {
            const bool chan_ok = !(D_TAIL && c == DC - 1 && g >= 2);
            f.k[kb][c] = chan_ok ? load16(krow + 32 * c + 8 * g) : zero8();
        }
    }
    if (V16) {
        // eight positions of one page row; clamped as a group so that the read stays inside
        // the request's last page (what is read there is zeroed before use)
        const int key = min(base + 8 * g, last_key & ~7);
        const int page = pages[key / page_size - page0];
        const bf16_t* vrow = v_cache + (((size_t)page * nkv + hk) * D) * page_size + key % page_size;
#pragma unroll
        for (int b = 0; b < DB; ++b) f.v[b] = load16(vrow + (size_t)(16 * b + col) * page_size);
    } else {
        const bf16_t* vrow[2];
#pragma unroll
        for (int h = 0; h < 2; ++h) {
            const int key = min(base + 8 * g + 4 * h, last_key & ~3);
            const int page = pages[key / page_size - page0];
            vrow[h] = v_cache + (((size_t)page * nkv + hk) * D) * page_size + key % page_size;
        }
#pragma unroll
        for (int b = 0; b < DB; ++b) {
            const size_t doff = (size_t)(16 * b + col) * page_size;
            f.v[b] = load8x2(vrow[0] + doff, vrow[1] + doff);
        }
    }
}

// What the kernels need to finish a head themselves: the per-head norm weights (null: no
// norm), the rotation tables (null: no rotation), where the token's own key and value go (the
// decode kernel; null: this layer writes no cache).
struct DecodeExtra {
    const float* q_norm_w;
    const float* k_norm_w;
    const float* cos_tab;
    const float* sin_tab;
    bf16_t* k_write;
    bf16_t* v_write;
    float eps;
    int qkv_stride;  // elements between the rows of `q` (fused: the packed q|k|v row)
};

// Q^T as the B operand of one row (lane (col, g) holds channels 32 c + 8 g .. + 7 of its row) from
// the raw head in the packed row: norm over the head, then the rotation of channel i with
// i + D / 2 by the position's angle (rapid_llm/models/base.py:134-140), in float32, rounded to
// bfloat16 once.  Needs D % 64 == 0: a lane then holds both channels of every pair.
__device__ inline void prepared_query(bf16x8 (&qf)[DC], const bf16_t* qrow, bool row_ok, int pos, int g,
                                      const DecodeExtra& ex) {
    float x[DC][8];
    float ss = 0.f;
#pragma unroll
    for (int c = 0; c < DC; ++c) {
        const bf16x8 raw = row_ok ? load16(qrow + 32 * c + 8 * g) : zero8();
#pragma unroll
        for (int j = 0; j < 8; ++j) {
            x[c][j] = (float)raw[j];
            ss += x[c][j] * x[c][j];
        }
    }
    if (ex.q_norm_w) {
        const float rrms = rsqrtf(row_sum4(ss) / (float)D + ex.eps);
#pragma unroll
        for (int c = 0; c < DC; ++c)
#pragma unroll
            for (int j = 0; j < 8; ++j) x[c][j] *= rrms * ex.q_norm_w[32 * c + 8 * g + j];
    }
    if (ex.cos_tab) {
        constexpr int HC = DC / 2;  // chunk c pairs with chunk c + HC, same lane and slot
#pragma unroll
        for (int c = 0; c < HC; ++c)
#pragma unroll
            for (int j = 0; j < 8; ++j) {
                const int i = 32 * c + 8 * g + j;
                const float cs = ex.cos_tab[(size_t)pos * (D / 2) + i];
                const float sn = ex.sin_tab[(size_t)pos * (D / 2) + i];
                const float a = x[c][j], bb = x[c + HC][j];
                x[c][j] = a * cs - bb * sn;
                x[c + HC][j] = bb * cs + a * sn;
            }
    }
#pragma unroll
    for (int c = 0; c < DC; ++c)
#pragma unroll
        for (int j = 0; j < 8; ++j) qf[c][j] = (__bf16)x[c][j];
}

// k_cache and v_cache carry no promise of being the only way to their memory: in the fused
// form the token's own key and value are stored through ex.k_write / ex.v_write, which point
// into the same tensors, and read back through them after a fence and a barrier.
// FUSED: `q` holds raw packed [q | k | v] rows.  The workgroup norms and rotates the query
// heads of its kv head itself (rapid_llm/models/base.py:134-140), and the workgroup whose
// split holds the token's own position norms, rotates and writes the new key and value
// before anyone reads them (rapid_llm/modules/attention.py:126-138), so that a decode step
// needs no separate kernel for that.  Needs D % 64 == 0: a lane then holds both channels of
// every rotation pair.
template <bool V16, bool FUSED>
__global__ __launch_bounds__(DEC_WAVES* RL_WAVE) void attn_decode_kernel(
    const bf16_t* __restrict__ q, const bf16_t* k_cache, const bf16_t* v_cache,
    bf16_t* __restrict__ out, float* __restrict__ part_o,
    float* __restrict__ part_ml, const int* __restrict__ seq_token,
    const int* __restrict__ seq_order, const int* __restrict__ positions,
    const int* __restrict__ token_slot, const int* __restrict__ block_table, int table_stride,
    int page_size, int nq, int nkv, int window, float scale_log2, int split_chunk, int nsplit,
    DecodeExtra ex) {
    __shared__ float lds_o[DEC_WAVES / 2][D * 16];
    __shared__ float lds_m[DEC_WAVES / 2][16];
    __shared__ float lds_l[DEC_WAVES / 2][16];
    __shared__ int lds_pages[DEC_MAX_PAGES + 2];

    const int G = nq / nkv;
    const int head_chunks = (G + 15) / 16;
    // Workgroups are handed out in the order of their linear index, x fastest, and go to the
    // chip's eight dies in turn.  The kv heads are x, so that each die gets its share of every
    // request whatever the requests' lengths are (with the requests as x, 256 requests of 64 to
    // 1,152 keys took 174 us; so 125); a die takes another head of every next request, so that
    // its reads spread over the pages' bytes as before (without that, 64 requests of 2,100 keys
    // went from 102 to 106 us).  The requests are y, and seq_order (optional) names them longest
    // first, so that the short ones fill the gaps at the end.
    const int seq = seq_order ? seq_order[blockIdx.y] : blockIdx.y;
    const int hx = (blockIdx.x + blockIdx.y) % gridDim.x;
    const int hk = hx / head_chunks;
    const int hc = hx % head_chunks;
    const int split = blockIdx.z;
    const int lane = threadIdx.x & (RL_WAVE - 1);
    const int wave = threadIdx.x / RL_WAVE;
    const int col = lane & 15;  // row of the attention problem = query head of the group
    const int g = lane >> 4;

    const int t = seq_token ? seq_token[seq] : seq;  // null: the step holds single tokens only
    const int pos = positions[t];
    const int* table = block_table + (size_t)token_slot[t] * table_stride;
    const int kend = pos + 1;
    const int kstart = (window > 0 && pos - window + 1 > 0) ? pos - window + 1 : 0;
    // The launch has nsplit splits of at most split_chunk keys, laid out for the longest context
    // it may meet (a recorded step serves every context of its bucket).  This request's keys are
    // dealt to the splits evenly: runs of a multiple of 32 keys, at least 128 (shorter runs only
    // add merge work), never more than split_chunk (the page ids of a run are staged in LDS).
    // nsplit * split_chunk covers the longest context, so the runs cover this one.
    const int first = kstart & ~31;
    int run = ((kend - first + nsplit - 1) / nsplit + 31) & ~31;
    run = min(max(run, 128), split_chunk);
    const int lo = first + split * run;
    const int hi = min(kend, lo + run);

    const int hh = hc * 16 + col;  // head within the group
    const bool head_ok = hh < G;
    const int head = hk * G + (head_ok ? hh : 0);
    const size_t slot_index = ((size_t)seq * nq + head) * nsplit + split;

    float m = -INFINITY, l = 0.f;
    f32x4 acc[DB];
#pragma unroll
    for (int b = 0; b < DB; ++b) acc[b] = (f32x4){0.f, 0.f, 0.f, 0.f};

    if (lo < hi) {  // the same for every thread of the workgroup
        // page ids of the split, once: the loop's loads then depend on nothing but LDS
        const int last_key = kend - 1;
        const int page0 = lo / page_size;
        {
            const int npages = last_key / page_size - page0 + 1;
            for (int i = threadIdx.x; i < npages && i < DEC_MAX_PAGES + 2; i += DEC_WAVES * RL_WAVE)
                lds_pages[i] = table[page0 + i];
        }
        const bf16_t* qrow = q + (size_t)t * ex.qkv_stride + (size_t)head * D;
        // Q^T as B operand: lane (row col, group g) holds channels 32c + 8g .. + 7
        bf16x8 qf[DC];
        if (FUSED) {
            prepared_query(qf, qrow, head_ok, pos, g, ex);
            // the token's own key and value: written by the split that holds its position
            // (with more than 16 heads on a kv head every chunk of heads writes the same bytes:
            // each reads them back after its own barrier only)
            if (ex.k_write && pos >= lo && pos < hi) {
                const size_t page = (size_t)table[pos / page_size];
                const int off = pos % page_size;
                const bf16_t* krow = q + (size_t)t * ex.qkv_stride + (size_t)(nq + hk) * D;
                const bf16_t* vrow = q + (size_t)t * ex.qkv_stride + (size_t)(nq + nkv + hk) * D;
                if (wave == 0) {
                    // lane handles the pairs (i, i + D/2) for i = lane, lane + 64
                    constexpr int half = D / 2;
                    float x1[2], x2[2];
                    float ks = 0.f;
#pragma unroll
                    for (int r = 0; r < 2; ++r) {
                        const int i = lane + r * RL_WAVE;
                        x1[r] = x2[r] = 0.f;
                        if (i < half) {
                            x1[r] = bf16_to_float(krow[i]);
                            x2[r] = bf16_to_float(krow[i + half]);
                            ks += x1[r] * x1[r] + x2[r] * x2[r];
                        }
                    }
                    float rrms = 1.f;
                    if (ex.k_norm_w) rrms = rsqrtf(wave_sum(ks) / (float)D + ex.eps);
                    bf16_t* dst = ex.k_write + ((page * nkv + hk) * page_size + off) * D;
#pragma unroll
                    for (int r = 0; r < 2; ++r) {
                        const int i = lane + r * RL_WAVE;
                        if (i < half) {
                            float a = x1[r], bb = x2[r];
                            if (ex.k_norm_w) {
                                a = a * rrms * ex.k_norm_w[i];
                                bb = bb * rrms * ex.k_norm_w[i + half];
                            }
                            if (ex.cos_tab) {
                                const float cs = ex.cos_tab[(size_t)pos * half + i];
                                const float sn = ex.sin_tab[(size_t)pos * half + i];
                                const float ra = a * cs - bb * sn;
                                bb = bb * cs + a * sn;
                                a = ra;
                            }
                            dst[i] = float_to_bf16(a);
                            dst[i + half] = float_to_bf16(bb);
                        }
                    }
                } else if (wave == 1) {
                    bf16_t* dst = ex.v_write + ((page * nkv + hk) * D) * page_size + off;
                    for (int i = lane; i < D; i += RL_WAVE) dst[(size_t)i * page_size] = vrow[i];
                }
                __threadfence_block();  // the loop below reads them back from the cache
            }
        } else {
#pragma unroll
            for (int c = 0; c < DC; ++c) {
                const bool chan_ok = !(D_TAIL && c == DC - 1 && g >= 2);
                qf[c] = (head_ok && chan_ok) ? load16(qrow + 32 * c + 8 * g) : zero8();
            }
        }
        __syncthreads();

        // A wave asks for one step's keys and values, waits for them and multiplies; what hides
        // the wait is the other waves of the compute unit.  Keeping the next step's loads in
        // flight as well (a second set of 64 registers) left room for two waves a SIMD instead of
        // three and was 2 to 5% slower at every batch size and context length measured (256
        // requests of 64 to 1,152 keys 182.7 -> 174.3 us, 64 of 2,100 keys 107.5 -> 103.6, 8 of
        // 16,000 keys 95.5 -> 94.0); forcing four waves a SIMD spills and loses again.
        DecodeFrags cur;
        int base = lo + 32 * wave;
        for (; base < hi; base += 32 * DEC_WAVES) {
            decode_load<V16>(cur, k_cache, v_cache, lds_pages, page0, page_size, nkv, hk, base,
                             last_key, col, g);
            // ---- S^T = K Q^T for two blocks of 16 keys --------------------------------
            f32x4 s[2];
#pragma unroll
            for (int kb = 0; kb < 2; ++kb) {
                s[kb] = (f32x4){0.f, 0.f, 0.f, 0.f};
#pragma unroll
                for (int c = 0; c < DC; ++c) s[kb] = mfma(cur.k[kb][c], qf[c], s[kb]);
            }
            // ---- which of this lane's keys (base + 8g + 4kb + i) are visible ------------
            unsigned ok[2];
#pragma unroll
            for (int kb = 0; kb < 2; ++kb) {
                ok[kb] = 0;
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    const int key = base + 8 * g + 4 * kb + i;
                    ok[kb] |= (key >= kstart && key < kend) ? (1u << i) : 0u;
                }
            }
            const bf16x8 p = softmax_step(s[0], s[1], ok[0], ok[1], scale_log2, m, l, acc);
            // ---- O^T += V^T P^T ---------------------------------------------------------
            const bool partial = (base + 32 > kend) || (base < kstart);
#pragma unroll
            for (int b = 0; b < DB; ++b) {
                bf16x8 v = cur.v[b];
                if (partial) {
                    // 0 * stale data must be 0: a page used before may hold anything
#pragma unroll
                    for (int i = 0; i < 4; ++i) {
                        if (!((ok[0] >> i) & 1u)) v[i] = (__bf16)0.f;
                        if (!((ok[1] >> i) & 1u)) v[4 + i] = (__bf16)0.f;
                    }
                }
                acc[b] = mfma(v, p, acc[b]);
            }
        }

        // ---- combine the waves pairwise, in the accumulators' own layout --------------------
        l = row_sum4(l);
        auto put = [&](int slot) {
            if (g == 0) {
                lds_m[slot][col] = m;
                lds_l[slot][col] = l;
            }
#pragma unroll
            for (int b = 0; b < DB; ++b)
#pragma unroll
                for (int i = 0; i < 4; ++i)
                    lds_o[slot][(16 * b + 4 * g + i) * 16 + col] = acc[b][i];
        };
        auto take = [&](int slot) {
            const float m_o = lds_m[slot][col], l_o = lds_l[slot][col];
            const float mm = fmaxf(m, m_o);
            const float ms = (mm == -INFINITY) ? 0.f : mm;  // a wave without keys has m = -inf
            const float f1 = exp2f(m - ms), f2 = exp2f(m_o - ms);
#pragma unroll
            for (int b = 0; b < DB; ++b)
#pragma unroll
                for (int i = 0; i < 4; ++i)
                    acc[b][i] =
                        acc[b][i] * f1 + lds_o[slot][(16 * b + 4 * g + i) * 16 + col] * f2;
            l = l * f1 + l_o * f2;
            m = mm;
        };
        // waves [s, 2s) hand their state to waves [0, s), for s = DEC_WAVES / 2, .., 1
#pragma unroll
        for (int s = DEC_WAVES / 2; s >= 1; s >>= 1) {
            if (wave >= s && wave < 2 * s) put(wave - s);
            __syncthreads();
            if (wave < s) take(wave);
            if (s > 1) __syncthreads();
        }
        if (wave != 0) return;
    } else if (wave != 0) {
        return;
    }
    // ---- wave 0: this split's result (m = -inf, l = 0 if the split holds no key) -------------
    const float inv = l > 0.f ? 1.f / l : 0.f;
    if (nsplit == 1) {
        if (!head_ok) return;
        bf16_t* orow = out + ((size_t)t * nq + head) * D;
#pragma unroll
        for (int b = 0; b < DB; ++b) {
            struct {
                bf16_t v[4];
            } o;
#pragma unroll
            for (int i = 0; i < 4; ++i) o.v[i] = float_to_bf16(acc[b][i] * inv);
            *reinterpret_cast<uint2*>(orow + 16 * b + 4 * g) = __builtin_bit_cast(uint2, o);
        }
        return;
    }
    if (head_ok) {
        float* orow = part_o + slot_index * D;
        if (l > 0.f) {
#pragma unroll
            for (int b = 0; b < DB; ++b)
                *reinterpret_cast<float4*>(orow + 16 * b + 4 * g) = make_float4(
                    acc[b][0] * inv, acc[b][1] * inv, acc[b][2] * inv, acc[b][3] * inv);
        }
        if (g == 0) {
            part_ml[slot_index * 2] = m;
            part_ml[slot_index * 2 + 1] = l;
        }
    }
}

// merge of the splits: out = sum_s w_s o_s / sum_s w_s with w_s = l_s * 2^(m_s - max m).
// One thread per channel; the loads of MERGE_STEP splits are issued together and folded into a
// running (max, weight, output), in the order of the splits.
#define MERGE_STEP 8
// by_token: the partial results lie at the token's place in the step, not at the launch's own
// count of its rows (the prefill kernel's splits).
__global__ void attn_merge_kernel(const float* __restrict__ part_o,
                                  const float* __restrict__ part_ml, bf16_t* __restrict__ out,
                                  const int* __restrict__ seq_token, int nq, int nsplit,
                                  int by_token) {
    const int seq = blockIdx.x, head = blockIdx.y;
    const int t = seq_token ? seq_token[seq] : seq;
    const size_t slot0 = ((size_t)(by_token ? t : seq) * nq + head) * nsplit;
    const int d = threadIdx.x;
    if (d >= D) return;
    float mm = -INFINITY, wsum = 0.f, o = 0.f;
    for (int s0 = 0; s0 < nsplit; s0 += MERGE_STEP) {
        float ms[MERGE_STEP], ls[MERGE_STEP], os[MERGE_STEP];
#pragma unroll
        for (int j = 0; j < MERGE_STEP; ++j) {
            const bool in = s0 + j < nsplit;
            const size_t slot = slot0 + (in ? s0 + j : 0);
            ms[j] = in ? part_ml[slot * 2] : -INFINITY;
            ls[j] = part_ml[slot * 2 + 1];
            os[j] = part_o[slot * D + d];
        }
#pragma unroll
        for (int j = 0; j < MERGE_STEP; ++j) {
            if (ms[j] == -INFINITY) continue;  // an empty split wrote no output
            const float mn = fmaxf(mm, ms[j]);
            const float keep = exp2f(mm - mn);  // 0 while nothing has been folded in
            const float w = ls[j] * exp2f(ms[j] - mn);
            o = o * keep + os[j] * w;
            wsum = wsum * keep + w;
            mm = mn;
        }
    }
    out[((size_t)t * nq + head) * D + d] = float_to_bf16(o / wsum);
}

extern "C" int rl_attn_head_dim() { return D; }

// Fused form (`fused` != 0): `q` is the packed [q | k | v] row, norm weights and rotation
// tables may be null, `k_write` / `v_write` null for a layer that writes no cache.  The splits
// are merged by a second kernel: letting the split that finishes last merge (a counter and
// device-wide fences) was measured and lost, 226 us against 108 us at 64 requests of 2,048
// keys in four splits, because every workgroup's fence writes the L2 back.
extern "C" int rl_attn_decode(const void* q, const void* k_cache, const void* v_cache, void* out,
                              float* part_o, float* part_ml, const int* seq_token,
                              const int* seq_order, const int* positions, const int* token_slot,
                              const int* block_table, int table_stride, int page_size,
                              int num_seqs, int nq, int nkv, int window, float scale,
                              int split_chunk, int nsplit, int fused, const float* q_norm_w,
                              const float* k_norm_w, const float* cos_tab, const float* sin_tab,
                              void* k_write, void* v_write, float eps, hipStream_t stream) {
    if (num_seqs <= 0) return RL_OK;
    if (nkv < 1 || nq % nkv || page_size < 4 || page_size % 4 || split_chunk < 32 ||
        split_chunk % 32 || nsplit < 1 || nsplit > 65535)
        return RL_ERR_ARG;
    // a split's pages are staged in LDS (its keys may start up to 31 before a page's first)
    if ((split_chunk + 31) / page_size + 1 > DEC_MAX_PAGES) return RL_ERR_ARG;
    if (nsplit > 1 && (!part_o || !part_ml)) return RL_ERR_ARG;
    if (fused && (D % 64 != 0 || (cos_tab && !sin_tab) || (k_write && !v_write))) return RL_ERR_ARG;
    const int G = nq / nkv;
    const int head_chunks = (G + 15) / 16;
    if (num_seqs > 65535) return RL_ERR_ARG;  // the requests are the grid's y
    const float scale_log2 = scale * 1.4426950408889634f;
    DecodeExtra ex;
    ex.q_norm_w = fused ? q_norm_w : nullptr;
    ex.k_norm_w = fused ? k_norm_w : nullptr;
    ex.cos_tab = fused ? cos_tab : nullptr;
    ex.sin_tab = fused ? sin_tab : nullptr;
    ex.k_write = fused ? (bf16_t*)k_write : nullptr;
    ex.v_write = fused ? (bf16_t*)v_write : nullptr;
    ex.eps = eps;
    ex.qkv_stride = fused ? (nq + 2 * nkv) * D : nq * D;
    dim3 grid(nkv * head_chunks, num_seqs, nsplit), block(DEC_WAVES * RL_WAVE);
#define RL_DECODE(V16, FUSED)                                                                  \
    hipLaunchKernelGGL((attn_decode_kernel<V16, FUSED>), grid, block, 0, stream,               \
                       (const bf16_t*)q, (const bf16_t*)k_cache, (const bf16_t*)v_cache,       \
                       (bf16_t*)out, part_o, part_ml, seq_token, seq_order, positions,         \
                       token_slot,                                                             \
                       block_table, table_stride, page_size, nq, nkv, window, scale_log2,      \
                       split_chunk, nsplit, ex)
    if (fused) {
        if constexpr (D % 64 == 0) {
            if (page_size % 8 == 0)
                RL_DECODE(true, true);
            else
                RL_DECODE(false, true);
        }
    } else {
        if (page_size % 8 == 0)
            RL_DECODE(true, false);
        else
            RL_DECODE(false, false);
    }
#undef RL_DECODE
    if (hipGetLastError() != hipSuccess) return RL_ERR_LAUNCH;
    if (nsplit > 1) {
        hipLaunchKernelGGL(attn_merge_kernel, dim3(num_seqs, nq), dim3(D < 64 ? 64 : D), 0,
                           stream, part_o, part_ml, (bf16_t*)out, seq_token, nq, nsplit, 0);
    }
    return rl_launch_status();
}

extern "C" int rl_attn_decode_fusable() { return D % 64 == 0 ? 1 : 0; }

// =========================================================================== //
// prefill
// =========================================================================== //
#ifndef RL_PF_NQ
#define RL_PF_NQ 2
#endif
#define PF_WAVES 4                       // waves that share the rows of a tile
#define PF_NQ RL_PF_NQ                   // 16-row blocks per wave
#define PF_ROWS (PF_WAVES * PF_NQ * 16)  // rows per workgroup
#define PF_KEYS 64                       // keys per LDS tile and per softmax step
#define PF_THREADS (PF_WAVES * RL_WAVE)  // threads of one wave group
#define K_LD (D + 8)                     // padded row of the K tile (bfloat16 elements)
#define V_LD (PF_KEYS + 16)              // padded row of the V^T tile (16 measured 3% faster than 8, 24 or 40)
#define PF_TILE_ELEMS (PF_KEYS * K_LD + D * V_LD)  // one group's K and V^T tiles in LDS

// Softmax is the arithmetic that competes with the matrix cores here, so a step covers 64
// keys (one maximum, one rescale and one sum for 16 scores per lane), scores are masked only
// in tiles that the diagonal, a window's edge or the end of the sequence crosses, and the
// accumulators are rescaled only when some row's maximum moved.
//
// tile_info[4 * tile + {0,1,2,3}] = {first token of the request's portion in the flat batch,
//   tokens of the request already in the cache, tokens in this portion, first row of the tile};
// work_order (optional): workgroup b takes (tile, kv head) = (work_order[b] / nkv, % nkv), so
// that the host decides which workgroups start together.
// Two waves per SIMD at most: the accumulators then live in ordinary vector registers, which
// the rescale and the epilogue read directly (at the default budget of 128 the compiler parks
// them in accumulation registers and moves them back and forth around every rescale).
//
// GROUPS == 2: the two waves of a SIMD belong to one workgroup.  Two groups of four waves hold
// the same rows and take the 64-key steps of the tile alternately (group 0 the even ones), each
// with K and V^T tiles of its own in LDS; at the end group 1 hands its softmax state and
// accumulators to group 0 through LDS.  A tile is then walked in half as many steps, which
// pays when the longest tile bounds the launch's time (one prompt from its start: every
// workgroup is resident at once and the last rows see the most keys).  GROUPS == 1: the two
// waves of a SIMD belong to two workgroups with tiles of their own, which drift apart so that
// one's matrix products overlap the other's softmax; better when there is enough work to keep
// every unit busy (2,048 tokens of Qwen3-8B from the start: 78 against 86 us; 8,192 tokens:
// 819 against 731 us).
//
// DIRECT (head size 128, pages of a multiple of eight keys): a step's keys and values go from
// memory straight into LDS (the loads that name an LDS address, 16 bytes a lane), into one of two
// sets of tiles in turn, so that a step has one barrier, no wave holds a tile's share in
// registers and none stores it.  Such a load writes a wave's 64 x 16 bytes side by side, so the
// tiles have no padding: instead, 16-byte unit u of row r lies at unit u ^ (r % 16) of a key row
// and u ^ (r / 2 % 8) of a value row (two to 256 bytes), which spreads an operand read's sixteen
// rows over the banks; a lane asks memory for the unit that belongs at its place.
typedef __attribute__((address_space(3))) void* rl_lds_ptr;
typedef const __attribute__((address_space(1))) void* rl_global_ptr;
constexpr bool PF_DIRECT_OK = (D == 128);
constexpr int PF_DIRECT_TILE = PF_KEYS * D * 2;      // bytes of a key tile and of a value tile
constexpr int PF_DIRECT_SET = 2 * PF_DIRECT_TILE;    // one step's tiles
constexpr int PF_DIRECT_GROUP = 2 * PF_DIRECT_SET;   // a wave group's two sets

template <int GROUPS, bool DIRECT>
__global__ __launch_bounds__(GROUPS* PF_THREADS) __attribute__((amdgpu_waves_per_eu(1, 2))) void
attn_prefill_kernel(
    const bf16_t* __restrict__ q, const bf16_t* __restrict__ k_cache,
    const bf16_t* __restrict__ v_cache, bf16_t* __restrict__ out,
    const int* __restrict__ tile_info, const int* __restrict__ work_order,
    const int* __restrict__ token_slot, const int* __restrict__ block_table, int table_stride,
    int page_size, unsigned page_magic, int nq, int nkv, int window, float scale_log2, int nsplit,
    float* __restrict__ part_o, float* __restrict__ part_ml, int prep_q, DecodeExtra ex) {
    constexpr int GROUP_ELEMS = DIRECT ? PF_DIRECT_GROUP / 2 : PF_TILE_ELEMS;  // bfloat16 elements
    __shared__ __attribute__((aligned(1024))) bf16_t tiles[GROUPS * GROUP_ELEMS];
    __shared__ float fold_ml[GROUPS > 1 ? PF_WAVES * PF_NQ * 2 * RL_WAVE : 1];

    const int G = nq / nkv;
    // nsplit > 1: the keys of every tile are cut into nsplit runs of whole 64-key steps, one
    // workgroup each; the runs' results go to part_o / part_ml (indexed by the token's place in
    // the step) and are folded by the merge kernel, as the decode kernel's splits are
    const int split = blockIdx.x % nsplit;
    const int wg = blockIdx.x / nsplit;
    const int item = work_order ? work_order[wg] : wg;
    const int tile = item / nkv;
    const int hk = item % nkv;
    const int tok0 = tile_info[4 * tile + 0];
    const int start = tile_info[4 * tile + 1];
    const int qlen = tile_info[4 * tile + 2];
    const int row0 = tile_info[4 * tile + 3];
    const int rows = qlen * G;
    const int seq_end = start + qlen;  // keys at or beyond this were never written
    const int* table = block_table + (size_t)token_slot[tok0] * table_stride;

    const int grp = GROUPS > 1 ? threadIdx.x / PF_THREADS : 0;  // wave group: which steps
    const int tid = threadIdx.x - grp * PF_THREADS;             // thread within the group
    const int lane = tid & (RL_WAVE - 1);
    const int wave = tid / RL_WAVE;
    const int col = lane & 15;
    const int g = lane >> 4;
    bf16_t* const Ks = tiles + grp * GROUP_ELEMS;
    bf16_t* const Vs = Ks + PF_KEYS * K_LD;  // (the padded layout's; DIRECT: see direct_issue)
    unsigned char* const dtiles = reinterpret_cast<unsigned char*>(tiles) + grp * (GROUP_ELEMS * 2);

    // rows of this lane: one per 16-row block
    int r_tok[PF_NQ], r_head[PF_NQ], r_pos[PF_NQ];
    bool r_ok[PF_NQ];
    bf16x8 qf[PF_NQ][DC];
#pragma unroll
    for (int n = 0; n < PF_NQ; ++n) {
        const int row = row0 + (wave * PF_NQ + n) * 16 + col;
        r_ok[n] = row < rows;
        const int rr = r_ok[n] ? row : rows - 1;
        r_tok[n] = tok0 + rr / G;
        r_head[n] = hk * G + rr % G;
        r_pos[n] = start + rr / G;
    }
    // prep_q: `q` holds the raw packed [q | k | v] rows, and the workgroup norms and rotates its
    // rows' heads itself, as the decode kernel does (the host asks for it only where
    // D % 64 == 0); else `q` holds finished queries.  Called once the first tile has been asked
    // for: finishing a query waits for its channels, and the tile travels meanwhile.
    auto load_queries = [&]() {
#pragma unroll
        for (int n = 0; n < PF_NQ; ++n) {
            const bf16_t* qrow = q + (size_t)r_tok[n] * ex.qkv_stride + (size_t)r_head[n] * D;
            if (prep_q) {
                prepared_query(qf[n], qrow, r_ok[n], r_pos[n], g, ex);
            } else {
#pragma unroll
                for (int c = 0; c < DC; ++c) {
                    const bool chan_ok = !(D_TAIL && c == DC - 1 && g >= 2);
                    qf[n][c] = (r_ok[n] && chan_ok) ? load16(qrow + 32 * c + 8 * g) : zero8();
                }
            }
        }
    };
    // keys the tile needs: up to the position of its last row; from the window of its first
    const int last_row = min(row0 + PF_ROWS, rows) - 1;
    const int tile_kend = start + last_row / G + 1;
    const int first_pos = start + row0 / G;
    const int tile_kstart = (window > 0 && first_pos - window + 1 > 0) ? first_pos - window + 1 : 0;
    // positions of this wave's rows (rows ascend with the position)
    const int w_first = min(row0 + wave * PF_NQ * 16, rows - 1);
    const int w_last = min(row0 + (wave + 1) * PF_NQ * 16, rows) - 1;
    const int wave_min_pos = start + w_first / G;
    const int wave_max_pos = start + (w_last > w_first ? w_last : w_first) / G;

    float m[PF_NQ], l[PF_NQ];
    f32x4 acc[PF_NQ][DB];
#pragma unroll
    for (int n = 0; n < PF_NQ; ++n) {
        m[n] = -INFINITY;
        l[n] = 0.f;
#pragma unroll
        for (int b = 0; b < DB; ++b) acc[n][b] = (f32x4){0.f, 0.f, 0.f, 0.f};
    }

    // The next tile's keys and values travel from memory into registers while this tile is
    // multiplied; they reach LDS after the barrier that ends this tile's reads.
    constexpr int TPK = PF_THREADS / PF_KEYS;  // threads sharing one key row
    constexpr int KCH = (D / 8 + TPK - 1) / TPK;
    constexpr int KG = PF_KEYS / 4;  // groups of four keys
    constexpr int VCH = (D + PF_THREADS / KG - 1) / (PF_THREADS / KG);
    // native vector types: an array of them is taken apart into registers, whereas an array
    // of uint4 structs stayed in memory and each tile's keys were waited for as soon as asked for
    bf16x8 kreg[KCH];
    u32x2 vreg[VCH];
    // The page ids of a step are asked for one step before its keys and values, so that no
    // wave waits for a table entry in front of its products.  key / page_size is a multiply
    // by page_magic = ceil(2^32 / page_size), exact for key < 2^32 / page_size (host-checked).
    int k_key = 0, k_page = 0, v_key = 0, v_page = 0;
    auto stage_pages = [&](int base) {
        k_key = min(base + tid / TPK, seq_end - 1);  // clamped; masked by position below
        k_page = table[__umulhi((unsigned)k_key, page_magic)];
        v_key = min(base + 4 * (tid % KG), (seq_end - 1) & ~3);
        v_page = table[__umulhi((unsigned)v_key, page_magic)];
    };
    // a page of one layer's keys (or values) is nkv * page_size * D elements, a count that fits
    // 32 bits (host-checked), so an address is one 32 x 32 -> 64 bit multiply-add of the page id
    // and an offset of 32 bits within the page
    const unsigned page_elems = (unsigned)nkv * (unsigned)page_size * (unsigned)D;
    const unsigned head_off = (unsigned)hk * (unsigned)page_size * (unsigned)D;
    auto stage_load = [&]() {
        {
            const unsigned in_page = (unsigned)k_key - __umulhi((unsigned)k_key, page_magic) * (unsigned)page_size;
            const bf16_t* krow =
                k_cache + ((unsigned long long)(unsigned)k_page * page_elems + (head_off + in_page * (unsigned)D));
#pragma unroll
            for (int i = 0; i < KCH; ++i) {
                const int ch = tid % TPK + i * TPK;
                if (ch < D / 8) kreg[i] = load16(krow + 8 * ch);
            }
        }
        {
            const unsigned in_page = (unsigned)v_key - __umulhi((unsigned)v_key, page_magic) * (unsigned)page_size;
            const bf16_t* vbase = v_cache + ((unsigned long long)(unsigned)v_page * page_elems + (head_off + in_page));
#pragma unroll
            for (int i = 0; i < VCH; ++i) {
                const int d = tid / KG + i * (PF_THREADS / KG);
                if (d < D) vreg[i] = *reinterpret_cast<const u32x2*>(vbase + (unsigned)d * (unsigned)page_size);
            }
        }
    };
    auto stage_store = [&](int base) {
        {
            // key kk of the tile goes to the LDS row from which the first product reads it:
            // row 32 hf + 16 kb + i holds key 32 hf + 8 (i / 4) + 4 kb + i % 4, so that the
            // sixteen lanes of an operand read consecutive rows (no bank conflicts)
            const int kk = tid / TPK;
            const int r = kk & 31;
            const int lrow = (kk & 32) + 16 * ((r >> 2) & 1) + 4 * (r >> 3) + (r & 3);
#pragma unroll
            for (int i = 0; i < KCH; ++i) {
                const int ch = tid % TPK + i * TPK;
                if (ch < D / 8) *reinterpret_cast<bf16x8*>(&Ks[lrow * K_LD + 8 * ch]) = kreg[i];
            }
        }
        {
            const int kg = tid % KG;
            // keys that may be multiplied: written ones (below seq_end) that no row's window has
            // left behind (their pages may have been given back already).  Most steps hold such
            // keys only (the same for every thread): their values go to LDS as they came
            if (base >= tile_kstart && base + PF_KEYS <= seq_end) {
#pragma unroll
                for (int i = 0; i < VCH; ++i) {
                    const int d = tid / KG + i * (PF_THREADS / KG);
                    if (d < D) *reinterpret_cast<u32x2*>(&Vs[d * V_LD + 4 * kg]) = vreg[i];
                }
            } else {
                const int key = base + 4 * kg;
                const int lo_cut = tile_kstart - key;  // keys i < lo_cut are out
                const int hi_cut = seq_end - key;      // keys i >= hi_cut are out
                unsigned keep_x = 0, keep_y = 0;  // never multiply stale data, not even by zero
                if (0 >= lo_cut && 0 < hi_cut) keep_x |= 0x0000ffffu;
                if (1 >= lo_cut && 1 < hi_cut) keep_x |= 0xffff0000u;
                if (2 >= lo_cut && 2 < hi_cut) keep_y |= 0x0000ffffu;
                if (3 >= lo_cut && 3 < hi_cut) keep_y |= 0xffff0000u;
#pragma unroll
                for (int i = 0; i < VCH; ++i) {
                    const int d = tid / KG + i * (PF_THREADS / KG);
                    if (d < D) {
                        u32x2 v = vreg[i];
                        v.x &= keep_x;
                        v.y &= keep_y;
                        *reinterpret_cast<u32x2*>(&Vs[d * V_LD + 4 * kg]) = v;
                    }
                }
            }
        }
    };

    // ---- DIRECT: the loads of a step, and the repair of a step at the sequence's or window's edge
    // Instruction i of wave w fills rows 4 (4 i + w) .. + 3 of the key tile (a lane: row lane / 16,
    // unit lane % 16) and rows 8 (4 i + w) .. + 7 of the value tile (row lane / 8, unit lane % 8).
    // Key row r holds key 32 (r / 32) + 8 (r % 16 / 4) + 4 (r / 16 % 2) + r % 4 of the step (see
    // stage_store): an instruction's four rows are four consecutive keys of one page, whose id is
    // the same for the wave.  A lane's value unit is the same in all four instructions.
    const int wave_u = __builtin_amdgcn_readfirstlane(wave);
    int d_kpage[4] = {0, 0, 0, 0}, d_kin[4] = {0, 0, 0, 0};  // wave-uniform: page id, first key's place in it
    int d_vpage = 0, d_vin = 0;
    const int d_vunit = (lane & 7) ^ ((4 * wave + (lane >> 4)) & 7);  // keys 8 d_vunit .. + 7 of the step
    auto direct_pages = [&](int base) {
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const int r = 4 * (4 * i + wave_u);
            const int key = min(base + 32 * (r >> 5) + 8 * ((r & 15) >> 2) + 4 * ((r >> 4) & 1), (seq_end - 1) & ~3);
            const int pg = (int)__umulhi((unsigned)key, page_magic);
            d_kpage[i] = table[pg];
            d_kin[i] = key - pg * page_size;
        }
        const int key = min(base + 8 * d_vunit, (seq_end - 1) & ~7);
        const int pg = (int)__umulhi((unsigned)key, page_magic);
        d_vpage = table[pg];
        d_vin = key - pg * page_size;
    };
    auto direct_issue = [&](int set) {
        unsigned char* kt = dtiles + set * PF_DIRECT_SET;
        unsigned char* vt = kt + PF_DIRECT_TILE;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const int r = 4 * (4 * i + wave_u) + (lane >> 4);  // this lane's row
            const bf16_t* src = k_cache + ((unsigned long long)(unsigned)d_kpage[i] * page_elems +
                                           (head_off + (unsigned)(d_kin[i] + (lane >> 4)) * (unsigned)D)) +
                                8 * ((lane & 15) ^ (r & 15));
            __builtin_amdgcn_global_load_lds((rl_global_ptr)src, (rl_lds_ptr)(kt + 1024 * (4 * i + wave_u)), 16, 0, 0);
        }
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const int d = 8 * (4 * i + wave_u) + (lane >> 3);
            const bf16_t* src = v_cache + ((unsigned long long)(unsigned)d_vpage * page_elems +
                                           (head_off + (unsigned)d * (unsigned)page_size + (unsigned)d_vin));
            __builtin_amdgcn_global_load_lds((rl_global_ptr)src, (rl_lds_ptr)(vt + 1024 * (4 * i + wave_u)), 16, 0, 0);
        }
    };
    // values of keys that no row may see (never written, or behind every row's window: their
    // pages may hold anything) are zeroed where they lie: each lane repairs what it asked for
    auto direct_repair = [&](int set, int base) {
        unsigned char* vt = dtiles + set * PF_DIRECT_SET + PF_DIRECT_TILE;
        const int key0 = base + 8 * d_vunit;
        unsigned keep[4];
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            keep[j] = 0;
            if (key0 + 2 * j >= tile_kstart && key0 + 2 * j < seq_end) keep[j] |= 0x0000ffffu;
            if (key0 + 2 * j + 1 >= tile_kstart && key0 + 2 * j + 1 < seq_end) keep[j] |= 0xffff0000u;
        }
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            uint4* at = reinterpret_cast<uint4*>(vt + 1024 * (4 * i + wave_u) + 16 * lane);
            uint4 v = *at;
            v.x &= keep[0];
            v.y &= keep[1];
            v.z &= keep[2];
            v.w &= keep[3];
            *at = v;
        }
    };

    int first_base = tile_kstart & ~(PF_KEYS - 1);
    int run_end = tile_kend;
    if (nsplit > 1) {
        const int steps = (tile_kend - first_base + PF_KEYS - 1) / PF_KEYS;
        const int per = (steps + nsplit - 1) / nsplit;
        run_end = min(tile_kend, first_base + (split + 1) * per * PF_KEYS);
        first_base += split * per * PF_KEYS;
    }
    constexpr int STRIDE = GROUPS * PF_KEYS;  // the groups advance together
    if (first_base + grp * PF_KEYS < run_end) {
        if constexpr (DIRECT) {
            direct_pages(first_base + grp * PF_KEYS);
            direct_issue(0);
            if (first_base + grp * PF_KEYS + STRIDE < run_end) direct_pages(first_base + grp * PF_KEYS + STRIDE);
        } else {
            stage_pages(first_base + grp * PF_KEYS);
            stage_load();
            if (first_base + grp * PF_KEYS + STRIDE < run_end) stage_pages(first_base + grp * PF_KEYS + STRIDE);
        }
    }
    load_queries();
    // q has arrived before the loop starts: inside it, waiting for q would mean waiting for
    // everything asked for since, the next step's keys and values included
#pragma unroll
    for (int n = 0; n < PF_NQ; ++n)
#pragma unroll
        for (int c = 0; c < DC; ++c) asm volatile("" : "+v"(qf[n][c]));
    int set = 0;  // DIRECT: the set of tiles this step reads
    for (int both = first_base; both < run_end; both += STRIDE, set ^= 1) {
        const int base = both + grp * PF_KEYS;  // this group's step
        const bool live = base < run_end;       // group 1 may have no last step
        if constexpr (DIRECT) {
            // what this wave asked for has arrived in LDS (such loads count as loads from memory)
            asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
            if (live && (base < tile_kstart || base + PF_KEYS > seq_end)) direct_repair(set, base);
            __syncthreads();  // every wave's share is there, and the other set has been consumed
            if (base + STRIDE < run_end) {
                direct_issue(set ^ 1);  // of the step whose page ids were asked for a step ago
                if (base + 2 * STRIDE < run_end) direct_pages(base + 2 * STRIDE);
            }
        } else {
            __syncthreads();  // the previous tile has been consumed
            if (live) stage_store(base);
            __syncthreads();
            if (base + STRIDE < run_end) {
                stage_load();  // of the step whose page ids were asked for a step ago
                if (base + 2 * STRIDE < run_end) stage_pages(base + 2 * STRIDE);
            }
        }
        if (!live || base > wave_max_pos) continue;  // no key of the step is visible to this wave's rows
        const unsigned char* const kt = dtiles + set * PF_DIRECT_SET;
        const unsigned char* const vt = kt + PF_DIRECT_TILE;
        // masks are needed where the diagonal or a window's edge crosses the tile
        const bool need_mask =
            (base + PF_KEYS - 1 > wave_min_pos) || (window > 0 && base < wave_max_pos - window + 1);

        // ---- S^T = K Q^T: tile row i of key block (hf, kb) is key 32 hf + 8 (i / 4) + 4 kb + i % 4,
        // so that a lane ends up with the scores of keys 32 hf + 8 g .. + 7 (see DecodeFrags)
        f32x4 s[PF_NQ][4];
#pragma unroll
        for (int hb = 0; hb < 4; ++hb) {
            const int krow = 16 * hb + col;  // see stage_store for the key it holds
            bf16x8 kf[DC];
#pragma unroll
            for (int c = 0; c < DC; ++c) {
                const bool chan_ok = !(D_TAIL && c == DC - 1 && g >= 2);
                if constexpr (DIRECT)
                    kf[c] = *reinterpret_cast<const bf16x8*>(kt + krow * (2 * D) + 16 * ((4 * c + g) ^ col));
                else
                    kf[c] = chan_ok ? load16(&Ks[krow * K_LD + 32 * c + 8 * g]) : zero8();
            }
#pragma unroll
            for (int n = 0; n < PF_NQ; ++n) {
                s[n][hb] = (f32x4){0.f, 0.f, 0.f, 0.f};
#pragma unroll
                for (int c = 0; c < DC; ++c) s[n][hb] = mfma(kf[c], qf[n][c], s[n][hb]);
            }
        }
        // ---- softmax of 64 keys per row: maxima first, for both row blocks ---------------------
        bf16x8 p[PF_NQ][2];
        float m_safe_n[PF_NQ];
#pragma unroll
        for (int n = 0; n < PF_NQ; ++n) {
            if (need_mask) {
                const int pos = r_pos[n];
                const int wlo = (window > 0) ? pos - window + 1 : 0;
#pragma unroll
                for (int e = 0; e < 16; ++e) {
                    const int key = base + 32 * (e >> 3) + 8 * g + (e & 7);
                    if (!(key <= pos && key >= wlo)) s[n][e >> 2][e & 3] = -INFINITY;
                }
            }
            float mx = s[n][0][0];
#pragma unroll
            for (int e = 1; e < 16; ++e) mx = fmaxf(mx, s[n][e >> 2][e & 3]);
            mx = row_max4(mx) * scale_log2;  // the scale is positive: max commutes with it
            const float m_new = fmaxf(m[n], mx);
            // a row that has seen no visible key yet keeps m = -inf; exp2 of (-inf) - 0 is 0
            const float m_safe = (m_new == -INFINITY) ? 0.f : m_new;
            if (__any(m_new > m[n])) {
                const float alpha = __builtin_amdgcn_exp2f(m[n] - m_safe);
                l[n] *= alpha;
#pragma unroll
                for (int b = 0; b < DB; ++b) {
                    acc[n][b][0] *= alpha;
                    acc[n][b][1] *= alpha;
                    acc[n][b][2] *= alpha;
                    acc[n][b][3] *= alpha;
                }
                m[n] = m_new;
            }
            m_safe_n[n] = m_safe;
        }
        // ---- the weights of the first 32 keys, then of the last 32; the products follow half by
        // half, so that the first half's matrix instructions run beside the second half's
        // exponentials (8,192 tokens: 701 -> 681 us) ---------------------------------------------
        float psum[PF_NQ];
#pragma unroll
        for (int n = 0; n < PF_NQ; ++n) {
            psum[n] = 0.f;
#pragma unroll
            for (int e = 0; e < 8; ++e) {
                const float pe = __builtin_amdgcn_exp2f(fmaf(s[n][e >> 2][e & 3], scale_log2, -m_safe_n[n]));
                psum[n] += pe;
                p[n][0][e] = (__bf16)pe;
            }
        }
#pragma unroll
        for (int n = 0; n < PF_NQ; ++n) {
#pragma unroll
            for (int e = 8; e < 16; ++e) {
                const float pe = __builtin_amdgcn_exp2f(fmaf(s[n][e >> 2][e & 3], scale_log2, -m_safe_n[n]));
                psum[n] += pe;
                p[n][1][e & 7] = (__bf16)pe;
            }
            l[n] += psum[n];  // per-lane partial sum; the four groups are added at the end
        }
#pragma unroll
        for (int hf = 0; hf < 2; ++hf) {
#pragma unroll
            for (int b = 0; b < DB; ++b) {
                bf16x8 v;
                if constexpr (DIRECT)
                    v = *reinterpret_cast<const bf16x8*>(vt + (16 * b + col) * (2 * PF_KEYS) +
                                                         16 * ((4 * hf + g) ^ ((col >> 1) & 7)));
                else
                    v = load16(&Vs[(16 * b + col) * V_LD + 32 * hf + 8 * g]);
#pragma unroll
                for (int n = 0; n < PF_NQ; ++n) acc[n][b] = mfma(v, p[n][hf], acc[n][b]);
            }
        }
    }
    if (GROUPS > 1) {
        // group 1's state travels through the LDS that held the tiles: element j of a lane at
        // [wave][j][lane]; group 0 folds it into its own
        float* fold_acc = reinterpret_cast<float*>(tiles);
        constexpr int PER_LANE = PF_NQ * DB * 4;
        static_assert(GROUPS == 1 || sizeof(float) * PF_WAVES * PER_LANE * RL_WAVE <= sizeof(tiles),
                      "the accumulators of one group fit where the tiles were");
        __syncthreads();  // every wave has read its last tile
        if (grp == 1) {
#pragma unroll
            for (int n = 0; n < PF_NQ; ++n) {
                fold_ml[((wave * PF_NQ + n) * 2 + 0) * RL_WAVE + lane] = m[n];
                fold_ml[((wave * PF_NQ + n) * 2 + 1) * RL_WAVE + lane] = l[n];
#pragma unroll
                for (int b = 0; b < DB; ++b)
#pragma unroll
                    for (int i = 0; i < 4; ++i)
                        fold_acc[(wave * PER_LANE + (n * DB + b) * 4 + i) * RL_WAVE + lane] = acc[n][b][i];
            }
        }
        __syncthreads();
        if (grp == 1) return;
#pragma unroll
        for (int n = 0; n < PF_NQ; ++n) {
            const float m1 = fold_ml[((wave * PF_NQ + n) * 2 + 0) * RL_WAVE + lane];
            const float l1 = fold_ml[((wave * PF_NQ + n) * 2 + 1) * RL_WAVE + lane];
            const float m_new = fmaxf(m[n], m1);
            const float m_safe = (m_new == -INFINITY) ? 0.f : m_new;
            const float a0 = __builtin_amdgcn_exp2f(m[n] - m_safe);
            const float a1 = __builtin_amdgcn_exp2f(m1 - m_safe);
            m[n] = m_new;
            l[n] = l[n] * a0 + l1 * a1;
#pragma unroll
            for (int b = 0; b < DB; ++b)
#pragma unroll
                for (int i = 0; i < 4; ++i)
                    acc[n][b][i] = acc[n][b][i] * a0 +
                                   fold_acc[(wave * PER_LANE + (n * DB + b) * 4 + i) * RL_WAVE + lane] * a1;
        }
    }
#pragma unroll
    for (int n = 0; n < PF_NQ; ++n) {
        const float lt = row_sum4(l[n]);
        const float inv = lt > 0.f ? 1.f / lt : 0.f;
        if (!r_ok[n]) continue;
        if (nsplit > 1) {
            const size_t slot = ((size_t)r_tok[n] * nq + r_head[n]) * nsplit + split;
            if (lt > 0.f) {
                float* prow = part_o + slot * D;
#pragma unroll
                for (int b = 0; b < DB; ++b)
                    *reinterpret_cast<float4*>(prow + 16 * b + 4 * g) =
                        make_float4(acc[n][b][0] * inv, acc[n][b][1] * inv, acc[n][b][2] * inv,
                                    acc[n][b][3] * inv);
            }
            if (g == 0) {
                part_ml[slot * 2] = lt > 0.f ? m[n] : -INFINITY;
                part_ml[slot * 2 + 1] = lt;
            }
            continue;
        }
        bf16_t* orow = out + ((size_t)r_tok[n] * nq + r_head[n]) * D;
#pragma unroll
        for (int b = 0; b < DB; ++b) {
            struct {
                bf16_t v[4];
            } o;
#pragma unroll
            for (int i = 0; i < 4; ++i) o.v[i] = float_to_bf16(acc[n][b][i] * inv);
            *reinterpret_cast<uint2*>(orow + 16 * b + 4 * g) = __builtin_bit_cast(uint2, o);
        }
    }
}

extern "C" int rl_attn_prefill_rows() { return PF_ROWS; }

// groups: 1 or 2 wave groups per workgroup (a compute unit then holds 2 or 1 workgroups).
// nsplit > 1 cuts every tile's keys into that many runs (for launches of few, long tiles);
// part_o [tokens of the step, nq, nsplit, D] and part_ml [.., 2] then hold the runs' results
// and prefill_tokens [num_prefill_tokens] names the tokens the merge kernel writes.
// prep_q != 0: `q` is the packed [q | k | v] row of every token; the kernel norms (q_norm_w, eps;
// null: no norm) and rotates (cos_tab, sin_tab; null: no rotation) the query heads it reads.
extern "C" int rl_attn_prefill(const void* q, const void* k_cache, const void* v_cache, void* out,
                               const int* tile_info, const int* work_order, int num_tiles,
                               const int* token_slot,
                               const int* block_table, int table_stride, int page_size, int nq,
                               int nkv, int window, float scale, int groups, int nsplit, float* part_o,
                               float* part_ml, const int* prefill_tokens, int num_prefill_tokens,
                               int prep_q, const float* q_norm_w, const float* cos_tab,
                               const float* sin_tab, float eps, hipStream_t stream) {
    if (num_tiles <= 0) return RL_OK;
    if (nkv < 1 || nq % nkv || page_size < 4 || page_size % 4 || nkv > 65535 || nsplit < 1 ||
        (groups != 1 && groups != 2))
        return RL_ERR_ARG;
    if (nsplit > 1 && (!part_o || !part_ml || !prefill_tokens || num_prefill_tokens < 1 || nq > 65535))
        return RL_ERR_ARG;
    if (prep_q && (D % 64 != 0 || (cos_tab && !sin_tab))) return RL_ERR_ARG;
    DecodeExtra ex;
    ex.q_norm_w = prep_q ? q_norm_w : nullptr;
    ex.k_norm_w = nullptr;
    ex.cos_tab = prep_q ? cos_tab : nullptr;
    ex.sin_tab = prep_q ? sin_tab : nullptr;
    ex.k_write = ex.v_write = nullptr;
    ex.eps = eps;
    ex.qkv_stride = prep_q ? (nq + 2 * nkv) * D : nq * D;
    const float scale_log2 = scale * 1.4426950408889634f;
    const unsigned page_magic = (unsigned)(((1ull << 32) + page_size - 1) / page_size);
    if ((long)num_tiles * nkv * nsplit > 0x7fffffffL) return RL_ERR_ARG;
    // the kernel's addresses are page id x elements of a page (32 bits) + an offset in the page
    if ((long)nkv * page_size * D > 0x7fffffffL) return RL_ERR_ARG;
    dim3 grid(num_tiles * nkv * nsplit), block(groups * PF_THREADS);
    auto kernel = groups == 2 ? attn_prefill_kernel<2, false> : attn_prefill_kernel<1, false>;
    if constexpr (PF_DIRECT_OK) {
        if (page_size % 8 == 0)
            kernel = groups == 2 ? attn_prefill_kernel<2, true> : attn_prefill_kernel<1, true>;
    }
    hipLaunchKernelGGL(kernel, grid, block, 0, stream, (const bf16_t*)q, (const bf16_t*)k_cache,
                       (const bf16_t*)v_cache, (bf16_t*)out, tile_info, work_order, token_slot,
                       block_table, table_stride, page_size, page_magic, nq, nkv, window, scale_log2,
                       nsplit, part_o, part_ml, prep_q ? 1 : 0, ex);
    if (hipGetLastError() != hipSuccess) return RL_ERR_LAUNCH;
    if (nsplit > 1)
        hipLaunchKernelGGL(attn_merge_kernel, dim3(num_prefill_tokens, nq), dim3(D < 64 ? 64 : D), 0,
                           stream, part_o, part_ml, (bf16_t*)out, prefill_tokens, nq, nsplit, 1);
    return rl_launch_status();
}
