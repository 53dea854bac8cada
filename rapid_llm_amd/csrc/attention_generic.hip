// Paged causal attention, one workgroup per (token, query head), float32 arithmetic for
// any element type.  This is the whole attention of the float32 path and the fallback of
// the bfloat16 path for shapes the matrix-core kernels refuse.  It serves every token of a
// mixed batch alike: a token at absolute position pos of a request reads the keys
// [max(0, pos - window + 1), pos] of that request through its block table
// (window 0: all keys), which were written before this kernel runs.
//
// Scores (q . k) / sqrt(d) (rapid_llm/modules/attention.py:62), online softmax over tiles
// of 256 keys in ascending order (rapid_llm/kernels/ops/attention/flashattention2_nopad.py:
// 138-168), query head h reads kv head h / (nq / nkv) (:85).  Masked keys contribute
// exactly zero (-inf scores, as in rapid_llm/kernels/ops/attention/flashdecoding.py:223-237).
#include "common.h"

#define ATT_THREADS 256

template <typename T>
__global__ __launch_bounds__(ATT_THREADS) void attention_generic_kernel(
    const T* __restrict__ q, const T* __restrict__ k_cache, const T* __restrict__ v_cache,
    T* __restrict__ out, const int* __restrict__ positions, const int* __restrict__ token_slot,
    const int* __restrict__ block_table, int table_stride, int page_size, int nq, int nkv, int d,
    int window, float scale) {
    __shared__ float qs[256];
    __shared__ float ps[ATT_THREADS];
    __shared__ int key_page[ATT_THREADS];  // page * nkv + kv head of each key of the tile
    __shared__ int key_off[ATT_THREADS];
    __shared__ float scratch[16];

    const int t = blockIdx.x;
    const int h = blockIdx.y;
    const int hk = h / (nq / nkv);
    const int tid = threadIdx.x;
    const int pos = positions[t];
    const int* table = block_table + (size_t)token_slot[t] * table_stride;
    const int kend = pos + 1;
    const int kstart = (window > 0 && pos - window + 1 > 0) ? pos - window + 1 : 0;

    const T* qrow = q + ((size_t)t * nq + h) * d;
    if (tid < d) qs[tid] = to_float(qrow[tid]);
    __syncthreads();

    float m = -INFINITY, l = 0.f, acc = 0.f;
    for (int base = kstart; base < kend; base += ATT_THREADS) {
        const int j = base + tid;
        float s = -INFINITY;
        if (j < kend) {
            const int page = table[j / page_size];
            const int off = j % page_size;
            key_page[tid] = page * nkv + hk;
            key_off[tid] = off;
            const T* krow = k_cache + ((size_t)(page * nkv + hk) * page_size + off) * d;
            float dot = 0.f;
            for (int i = 0; i < d; ++i) dot = fmaf(qs[i], to_float(krow[i]), dot);
            s = dot * scale;
        }
        const float tile_max = block_max(s, scratch);  // finite: the tile holds >= 1 key
        const float m_new = fmaxf(m, tile_max);
        const float p = (j < kend) ? expf(s - m_new) : 0.f;
        ps[tid] = p;
        const float tile_sum = block_sum(p, scratch);  // syncs: ps, key_page, key_off visible
        const float alpha = expf(m - m_new);           // m = -inf on the first tile: 0
        l = l * alpha + tile_sum;
        m = m_new;
        if (tid < d) {
            acc *= alpha;
            const int n = min(ATT_THREADS, kend - base);
            for (int jj = 0; jj < n; ++jj) {
                const T* vrow = v_cache + ((size_t)key_page[jj] * d + tid) * page_size;
                acc = fmaf(ps[jj], to_float(vrow[key_off[jj]]), acc);
            }
        }
        __syncthreads();  // ps / key_* are rewritten by the next tile
    }
    if (tid < d) out[((size_t)t * nq + h) * d + tid] = from_float<T>(acc / l);
}

extern "C" int rl_attention_generic(const void* q, const void* k_cache, const void* v_cache,
                                    void* out, const int* positions, const int* token_slot,
                                    const int* block_table, int table_stride, int page_size,
                                    int tokens, int nq, int nkv, int d, int window, float scale,
                                    int act_type, hipStream_t stream) {
    if (tokens <= 0) return RL_OK;
    if (d < 1 || d > 256 || nkv < 1 || nq % nkv || page_size < 1 || nq > 65535)
        return RL_ERR_ARG;
    dim3 grid(tokens, nq), block(ATT_THREADS);
    if (act_type == RL_F32)
        hipLaunchKernelGGL(attention_generic_kernel<float>, grid, block, 0, stream,
                           (const float*)q, (const float*)k_cache, (const float*)v_cache,
                           (float*)out, positions, token_slot, block_table, table_stride,
                           page_size, nq, nkv, d, window, scale);
    else if (act_type == RL_BF16)
        hipLaunchKernelGGL(attention_generic_kernel<bf16_t>, grid, block, 0, stream,
                           (const bf16_t*)q, (const bf16_t*)k_cache, (const bf16_t*)v_cache,
                           (bf16_t*)out, positions, token_slot, block_table, table_stride,
                           page_size, nq, nkv, d, window, scale);
    else
        return RL_ERR_ARG;
    return rl_launch_status();
}
