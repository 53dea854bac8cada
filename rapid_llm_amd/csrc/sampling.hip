// Token selection from float32 logits.  Greedy rows take the arg-max (the lowest index
// among equal maxima, as torch.argmax does on one device).
#include "common.h"
#include "static_entry.h"

#include <mutex>

// row_index (optional, in every kernel of this file): the row of `logits` that output row b
// reads; without it output row b reads row b.
__device__ inline const float* logits_row(const float* logits, const int* row_index, int b,
                                          int vocab) {
    return logits + (size_t)(row_index ? row_index[b] : b) * vocab;
}

__global__ void argmax_kernel(const float* __restrict__ logits, const int* __restrict__ row_index,
                              int* __restrict__ out, int vocab) {
    __shared__ float best_v[1024 / RL_WAVE];
    __shared__ int best_i[1024 / RL_WAVE];
    const float* row = logits_row(logits, row_index, blockIdx.x, vocab);
    float bv = -INFINITY;
    int bi = 0x7fffffff;
    for (int i = threadIdx.x; i < vocab; i += blockDim.x) {
        const float v = row[i];
        // NaN never wins; ties keep the lower index (i ascends within a thread)
        if (v > bv || (v == bv && i < bi)) {
            bv = v;
            bi = i;
        }
    }
#pragma unroll
    for (int off = RL_WAVE / 2; off > 0; off >>= 1) {
        const float ov = __shfl_xor(bv, off, RL_WAVE);
        const int oi = __shfl_xor(bi, off, RL_WAVE);
        if (ov > bv || (ov == bv && oi < bi)) {
            bv = ov;
            bi = oi;
        }
    }
    const int lane = threadIdx.x & (RL_WAVE - 1), wave = threadIdx.x / RL_WAVE;
    if (lane == 0) {
        best_v[wave] = bv;
        best_i[wave] = bi;
    }
    __syncthreads();
    if (threadIdx.x == 0) {
        const int nwaves = blockDim.x / RL_WAVE;
        for (int w = 1; w < nwaves; ++w)
            if (best_v[w] > bv || (best_v[w] == bv && best_i[w] < bi)) {
                bv = best_v[w];
                bi = best_i[w];
            }
        out[blockIdx.x] = (bi == 0x7fffffff) ? 0 : bi;
    }
}

// Wide rows in two stages, so that a handful of rows still fills the chip: stage one finds
// the best (value, index) of each slice of a row, stage two the best of the slices.  Ties
// keep the lower index in both, so the result is the one-stage kernel's.
#define ARGMAX_SLICE 4096

__global__ __launch_bounds__(256) void argmax_slices_kernel(const float* __restrict__ logits,
                                                           const int* __restrict__ row_index,
                                                           float* __restrict__ part_v,
                                                           int* __restrict__ part_i, int vocab,
                                                           int slices) {
    __shared__ float best_v[4];
    __shared__ int best_i[4];
    const float* row = logits_row(logits, row_index, blockIdx.y, vocab);
    const int lo = blockIdx.x * ARGMAX_SLICE;
    const int hi = min(vocab, lo + ARGMAX_SLICE);
    float bv = -INFINITY;
    int bi = 0x7fffffff;
    for (int i = lo + threadIdx.x; i < hi; i += 256) {
        const float v = row[i];
        if (v > bv || (v == bv && i < bi)) {
            bv = v;
            bi = i;
        }
    }
#pragma unroll
    for (int off = RL_WAVE / 2; off > 0; off >>= 1) {
        const float ov = __shfl_xor(bv, off, RL_WAVE);
        const int oi = __shfl_xor(bi, off, RL_WAVE);
        if (ov > bv || (ov == bv && oi < bi)) {
            bv = ov;
            bi = oi;
        }
    }
    const int lane = threadIdx.x & (RL_WAVE - 1), wave = threadIdx.x / RL_WAVE;
    if (lane == 0) {
        best_v[wave] = bv;
        best_i[wave] = bi;
    }
    __syncthreads();
    if (threadIdx.x == 0) {
        for (int w = 1; w < 4; ++w)
            if (best_v[w] > bv || (best_v[w] == bv && best_i[w] < bi)) {
                bv = best_v[w];
                bi = best_i[w];
            }
        part_v[(size_t)blockIdx.y * slices + blockIdx.x] = bv;
        part_i[(size_t)blockIdx.y * slices + blockIdx.x] = bi;
    }
}

__global__ __launch_bounds__(RL_WAVE) void argmax_merge_kernel(const float* __restrict__ part_v,
                                                              const int* __restrict__ part_i,
                                                              int* __restrict__ out, int slices) {
    float bv = -INFINITY;
    int bi = 0x7fffffff;
    for (int s = threadIdx.x; s < slices; s += RL_WAVE) {
        const float v = part_v[(size_t)blockIdx.x * slices + s];
        const int i = part_i[(size_t)blockIdx.x * slices + s];
        if (v > bv || (v == bv && i < bi)) {
            bv = v;
            bi = i;
        }
    }
#pragma unroll
    for (int off = RL_WAVE / 2; off > 0; off >>= 1) {
        const float ov = __shfl_xor(bv, off, RL_WAVE);
        const int oi = __shfl_xor(bi, off, RL_WAVE);
        if (ov > bv || (ov == bv && oi < bi)) {
            bv = ov;
            bi = oi;
        }
    }
    if (threadIdx.x == 0) out[blockIdx.x] = (bi == 0x7fffffff) ? 0 : bi;
}

extern "C" int rl_argmax_slices(int vocab) { return (vocab + ARGMAX_SLICE - 1) / ARGMAX_SLICE; }

// part_v / part_i: [rows, rl_argmax_slices(vocab)] scratch of the caller; without it (null)
// the one-stage kernel runs.
extern "C" int rl_argmax(const float* logits, const int* row_index, int* out, float* part_v,
                         int* part_i, int rows, int vocab, hipStream_t stream) {
    if (rows <= 0) return RL_OK;
    if (vocab < 1) return RL_ERR_ARG;
    const int slices = (vocab + ARGMAX_SLICE - 1) / ARGMAX_SLICE;
    if (part_v && part_i && slices > 1 && rows <= 65535) {
        hipLaunchKernelGGL(argmax_slices_kernel, dim3(slices, rows), dim3(256), 0, stream, logits,
                           row_index, part_v, part_i, vocab, slices);
        if (hipGetLastError() != hipSuccess) return RL_ERR_LAUNCH;
        hipLaunchKernelGGL(argmax_merge_kernel, dim3(rows), dim3(RL_WAVE), 0, stream, part_v,
                           part_i, out, slices);
        return rl_launch_status();
    }
    hipLaunchKernelGGL(argmax_kernel, dim3(rows), dim3(1024), 0, stream, logits, row_index,
                       out, vocab);
    return rl_launch_status();
}

// The two-stage arg-max for callers that cannot allocate (static_entry.h): stage one's results
// live in this array, of which every GPU holds its own copy at its own address.  In host code
// the array's name is only a handle for hipGetSymbolAddress; kernels and every other host use
// take the address that call returned for the current device.
static __device__ __align__(256) unsigned char argmax_static_scratch[RL_ARGMAX_STATIC_ENTRIES * 8];

#define RL_MAX_DEVICES 64
static void* argmax_static_ptr[RL_MAX_DEVICES];
static std::mutex argmax_static_mutex;

// The address of the current device's copy of the array; looked up once per device.
static int argmax_static_address(void** ptr) {
    int device = -1;
    if (hipGetDevice(&device) != hipSuccess || device < 0 || device >= RL_MAX_DEVICES)
        return RL_ERR_SETUP;
    std::lock_guard<std::mutex> guard(argmax_static_mutex);
    if (!argmax_static_ptr[device]) {
        void* found = nullptr;
        if (hipGetSymbolAddress(&found, HIP_SYMBOL(argmax_static_scratch)) != hipSuccess || !found)
            return RL_ERR_SETUP;
        argmax_static_ptr[device] = found;
    }
    *ptr = argmax_static_ptr[device];
    return RL_OK;
}

extern "C" int rl_argmax_static_prepare() {
    void* ptr = nullptr;
    return argmax_static_address(&ptr);
}

extern "C" int rl_argmax_static_limit() { return RL_ARGMAX_STATIC_ENTRIES; }

extern "C" int rl_argmax_static(const float* logits, const int* row_index, int* out, int rows,
                                int vocab, hipStream_t stream) {
    if (rows <= 0) return RL_OK;
    if (vocab < 1 || rows > 65535) return RL_ERR_ARG;
    const int slices = (vocab + ARGMAX_SLICE - 1) / ARGMAX_SLICE;
    if ((long)rows * slices > RL_ARGMAX_STATIC_ENTRIES) return RL_ERR_ARG;
    void* base = nullptr;
    const int rc = argmax_static_address(&base);
    if (rc != RL_OK) return rc;
    float* part_v = reinterpret_cast<float*>(base);
    int* part_i = reinterpret_cast<int*>(static_cast<unsigned char*>(base) + RL_ARGMAX_STATIC_ENTRIES * 4);
    hipLaunchKernelGGL(argmax_slices_kernel, dim3(slices, rows), dim3(256), 0, stream, logits,
                       row_index, part_v, part_i, vocab, slices);
    if (hipGetLastError() != hipSuccess) return RL_ERR_LAUNCH;
    hipLaunchKernelGGL(argmax_merge_kernel, dim3(rows), dim3(RL_WAVE), 0, stream, part_v, part_i,
                       out, slices);
    return rl_launch_status();
}

// --------------------------------------------------------------------------- //
// General token selection, one workgroup of 1024 threads per row.
//
// In the order of rapid_llm/engine/sampler.py:641-718:
//   1. repetition penalty over the tokens the request has generated so far, each token once:
//      a negative logit is multiplied by the penalty, any other divided (:134-179);
//   2. temperature 0: arg-max, lowest index among equals; done;
//   3. probabilities softmax(logits / temperature) in float32;
//   4. top_p == 1: one draw from the whole distribution (:218);
//      otherwise the pool is the POOL most likely tokens in descending order, a token is
//      dropped when the mass before it exceeds top_p, but only in a row whose pool reaches
//      top_p at all (:234-244); the rest is renormalised and one token drawn.
// The draw is the inverse of the cumulative distribution at u * (kept mass), with u in
// [0, 1) a counter-based hash of (seed, counter): the same request draws the same tokens
// whatever else is in the batch and however often it is recomputed.
//
// Per-row parameters, 8 int32 words: temperature, top_p, penalty (float bits), seed low,
// seed high, counter, first and one-past-last index of its generated tokens in `history`.
// A negative entry -(r + 1) of the history stands for a token the host has not read yet:
// what sampling row r of the step before chose, kept in `fed` [fed_rows].  `fed` must not
// be the buffer this launch writes its own choices to.
// --------------------------------------------------------------------------- //
#define SMP_THREADS 1024
#define SMP_WAVES (SMP_THREADS / RL_WAVE)
#define SMP_POOL 1024  // candidates of nucleus sampling (rapid_llm/engine/sampler.py:186)

__device__ inline int history_token(int tok, const int* __restrict__ fed, int fed_rows) {
    if (tok >= 0) return tok;
    const int r = -tok - 1;
    return (fed && r < fed_rows) ? fed[r] : -1;
}

__device__ inline uint32_t float_key(float v) {
    // order-preserving map float -> uint32 (NaN sorts lowest)
    if (v != v) return 0u;
    const uint32_t u = __float_as_uint(v);
    return (u & 0x80000000u) ? ~u : (u | 0x80000000u);
}
__device__ inline float key_float(uint32_t k) {
    const uint32_t u = (k & 0x80000000u) ? (k & 0x7fffffffu) : ~k;
    return __uint_as_float(u);
}

// splitmix64 of (seed + counter * golden ratio); the top 24 bits make u in [0, 1)
__device__ __host__ inline float sample_uniform(uint32_t seed_lo, uint32_t seed_hi,
                                                uint32_t counter) {
    uint64_t z = (((uint64_t)seed_hi << 32) | seed_lo) +
                 ((uint64_t)counter + 1ull) * 0x9E3779B97F4A7C15ull;
    z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
    z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
    z = z ^ (z >> 31);
    return (float)(z >> 40) * (1.0f / 16777216.0f);
}

__device__ inline float wave_inclusive_scan(float v) {
    const int lane = threadIdx.x & (RL_WAVE - 1);
#pragma unroll
    for (int off = 1; off < RL_WAVE; off <<= 1) {
        const float o = __shfl_up(v, off, RL_WAVE);
        if (lane >= off) v += o;
    }
    return v;
}

__global__ __launch_bounds__(SMP_THREADS) void sample_kernel(
    const float* __restrict__ logits, const int* __restrict__ row_index,
    const int* __restrict__ row_params, const int* __restrict__ history,
    const int* __restrict__ fed, int fed_rows, int* __restrict__ out,
    float* __restrict__ out_logprob, int vocab, int bitmap_words) {
    extern __shared__ uint32_t seen[];  // one bit per token id, when the row has a penalty
    __shared__ unsigned long long cand[SMP_POOL];
    __shared__ float cum[SMP_POOL];
    __shared__ unsigned int hist[256];
    __shared__ float scratch[16];
    __shared__ float wave_tot[SMP_WAVES];
    __shared__ float best_v[SMP_WAVES];
    __shared__ int best_i[SMP_WAVES];
    __shared__ unsigned int sh_u[4];
    __shared__ int sh_i[2];

    const int tid = threadIdx.x;
    const int lane = tid & (RL_WAVE - 1), wave = tid / RL_WAVE;
    const int* rp = row_params + 8 * blockIdx.x;
    const float temperature = __int_as_float(rp[0]);
    const float top_p = __int_as_float(rp[1]);
    const float penalty = __int_as_float(rp[2]);
    const bool penalise = bitmap_words > 0 && penalty != 1.0f && rp[7] > rp[6];
    const bool greedy = !(temperature > 0.f);
    const float inv_t = greedy ? 1.f : 1.f / temperature;
    const float* row = logits_row(logits, row_index, blockIdx.x, vocab);

    if (penalise) {
        for (int i = tid; i < bitmap_words; i += SMP_THREADS) seen[i] = 0u;
        __syncthreads();
        for (int i = rp[6] + tid; i < rp[7]; i += SMP_THREADS) {
            const int tok = history_token(history[i], fed, fed_rows);
            if (tok >= 0 && tok < vocab) atomicOr(&seen[tok >> 5], 1u << (tok & 31));
        }
        __syncthreads();
    }
    // z(i): penalised logit over temperature
    auto zval = [&](int i) -> float {
        float x = row[i];
        if (penalise && ((seen[i >> 5] >> (i & 31)) & 1u)) x = x < 0.f ? x * penalty : x / penalty;
        return x * inv_t;
    };

    // ---- maximum and arg-max (lowest index among equals; NaN never wins) -----------------
    float bv = -INFINITY;
    int bi = 0x7fffffff;
    for (int i = tid; i < vocab; i += SMP_THREADS) {
        const float v = zval(i);
        if (v > bv || (v == bv && i < bi)) {
            bv = v;
            bi = i;
        }
    }
#pragma unroll
    for (int off = RL_WAVE / 2; off > 0; off >>= 1) {
        const float ov = __shfl_xor(bv, off, RL_WAVE);
        const int oi = __shfl_xor(bi, off, RL_WAVE);
        if (ov > bv || (ov == bv && oi < bi)) {
            bv = ov;
            bi = oi;
        }
    }
    if (lane == 0) {
        best_v[wave] = bv;
        best_i[wave] = bi;
    }
    __syncthreads();
    bv = best_v[0];
    bi = best_i[0];
    for (int w = 1; w < SMP_WAVES; ++w)
        if (best_v[w] > bv || (best_v[w] == bv && best_i[w] < bi)) {
            bv = best_v[w];
            bi = best_i[w];
        }
    if (bi == 0x7fffffff) bi = 0;  // a row of NaN or -inf
    const float zmax = bv;

    // ---- sum of exp, in a fixed order: wave w owns a contiguous segment -------------------
    // (needed for the probabilities and for the logprob of the chosen token)
    const int seg = ((vocab + SMP_WAVES - 1) / SMP_WAVES + RL_WAVE - 1) / RL_WAVE * RL_WAVE;
    const int seg_lo = min(vocab, wave * seg), seg_hi = min(vocab, seg_lo + seg);
    float wsum = 0.f;
    if (!greedy || out_logprob) {
        for (int base = seg_lo; base < seg_hi; base += RL_WAVE) {
            const int i = base + lane;
            wsum += (i < seg_hi) ? expf(zval(i) - zmax) : 0.f;
        }
        wsum = wave_sum(wsum);
        if (lane == 0) wave_tot[wave] = wsum;
    }
    __syncthreads();
    float total = 0.f;
    if (!greedy || out_logprob)
        for (int w = 0; w < SMP_WAVES; ++w) total += wave_tot[w];

    if (greedy) {
        if (tid == 0) {
            out[blockIdx.x] = bi;
            if (out_logprob) out_logprob[blockIdx.x] = -logf(total);  // z - zmax = 0
        }
        return;
    }
    const float u = sample_uniform((uint32_t)rp[3], (uint32_t)rp[4], (uint32_t)rp[5]);

    if (top_p >= 1.0f) {
        // ---- one draw from the whole distribution: first i with cumsum(i) >= u * total ----
        const float target = u * total;
        float before = 0.f;
        int owner = SMP_WAVES - 1;
        for (int w = 0; w < SMP_WAVES; ++w) {
            if (before + wave_tot[w] >= target && wave_tot[w] > 0.f) {
                owner = w;
                break;
            }
            before += wave_tot[w];
        }
        // rounding may leave the target just beyond the last wave with mass: fall back to it
        while (owner > 0 && !(wave_tot[owner] > 0.f)) --owner;
        if (wave != owner) return;
        float run = 0.f;
        for (int w = 0; w < owner; ++w) run += wave_tot[w];
        int chosen = -1, last_mass = -1;
        for (int base = seg_lo; base < seg_hi && chosen < 0; base += RL_WAVE) {
            const int i = base + lane;
            const float e = (i < seg_hi) ? expf(zval(i) - zmax) : 0.f;
            const float inc = wave_inclusive_scan(e) + run;
            const unsigned long long hit = __ballot(e > 0.f && inc >= target);
            const unsigned long long mass = __ballot(e > 0.f);
            if (mass) last_mass = base + 63 - __clzll(mass);
            if (hit) chosen = base + __ffsll((long long)hit) - 1;
            run = __shfl(inc, RL_WAVE - 1, RL_WAVE);
        }
        if (chosen < 0) chosen = last_mass >= 0 ? last_mass : bi;
        if (lane == 0) {
            out[blockIdx.x] = chosen;
            if (out_logprob) out_logprob[blockIdx.x] = zval(chosen) - zmax - logf(total);
        }
        return;
    }

    // ---- the pool: the k = min(POOL, vocab) largest z, by radix select on their keys ------
    const int k = min(SMP_POOL, vocab);
    uint32_t prefix = 0;
    int k_rem = k;
    if (vocab > SMP_POOL) {
        for (int shift = 24; shift >= 0; shift -= 8) {
            if (tid < 256) hist[tid] = 0u;
            __syncthreads();
            for (int i = tid; i < vocab; i += SMP_THREADS) {
                const uint32_t key = float_key(zval(i));
                if (shift == 24 || (key >> (shift + 8)) == prefix)
                    atomicAdd(&hist[(key >> shift) & 255u], 1u);
            }
            __syncthreads();
            if (tid == 0) {
                int acc = 0, b = 255;
                for (; b > 0; --b) {
                    if (acc + (int)hist[b] >= k_rem) break;
                    acc += (int)hist[b];
                }
                sh_u[0] = (prefix << 8) | (uint32_t)b;
                sh_i[0] = k_rem - acc;
                sh_i[1] = (int)hist[b];  // elements sharing the digits chosen so far
            }
            __syncthreads();
            prefix = sh_u[0];
            k_rem = sh_i[0];
            __syncthreads();
        }
    }
    const int equal_total = (vocab > SMP_POOL) ? sh_i[1] : 0;
    // gather: keys above the threshold in any order (they are sorted afterwards); keys equal
    // to it by ascending index until the pool is full
    cand[tid] = 0ull;
    if (tid == 0) sh_u[1] = 0u;
    __syncthreads();
    if (vocab <= SMP_POOL) {
        if (tid < vocab)
            cand[tid] = ((unsigned long long)float_key(zval(tid)) << 32) | (0xffffffffu - (uint32_t)tid);
    } else {
        const bool all_equal_fit = equal_total == k_rem;
        for (int i = tid; i < vocab; i += SMP_THREADS) {
            const uint32_t key = float_key(zval(i));
            if (key > prefix || (all_equal_fit && key == prefix)) {
                const unsigned int at = atomicAdd(&sh_u[1], 1u);
                if (at < SMP_POOL)
                    cand[at] = ((unsigned long long)key << 32) | (0xffffffffu - (uint32_t)i);
            }
        }
        __syncthreads();
        if (!all_equal_fit) {
            // more equal keys than places: the lowest indices take them
            int base_count = 0;
            const int first_free = k - k_rem;
            for (int base = 0; base < vocab && base_count < k_rem; base += SMP_THREADS) {
                const int i = base + tid;
                const bool eq = i < vocab && float_key(zval(i)) == prefix;
                const unsigned long long bal = __ballot(eq);
                if (lane == 0) hist[wave] = (unsigned int)__popcll(bal);
                __syncthreads();
                int before = base_count;
                for (int w = 0; w < wave; ++w) before += (int)hist[w];
                int tile_total = 0;
                for (int w = 0; w < SMP_WAVES; ++w) tile_total += (int)hist[w];
                const int rank = before + __popcll(bal & ((1ull << lane) - 1ull));
                if (eq && rank < k_rem)
                    cand[first_free + rank] =
                        ((unsigned long long)prefix << 32) | (0xffffffffu - (uint32_t)i);
                base_count += tile_total;
                __syncthreads();
            }
        }
    }
    __syncthreads();
    // ---- bitonic sort, descending (key, then lower index first) -----------------------------
    for (int size = 2; size <= SMP_POOL; size <<= 1) {
        for (int stride = size >> 1; stride > 0; stride >>= 1) {
            if (tid < SMP_POOL / 2) {
                const int lo = 2 * tid - (tid & (stride - 1));
                const int hi = lo + stride;
                const bool desc = (lo & size) == 0;
                const unsigned long long a = cand[lo], b = cand[hi];
                if ((a < b) == desc) {
                    cand[lo] = b;
                    cand[hi] = a;
                }
            }
            __syncthreads();
        }
    }
    // ---- probabilities of the pool, their cumulative sums, the nucleus ----------------------
    const float p = (tid < k) ? expf(key_float((uint32_t)(cand[tid] >> 32)) - zmax) / total : 0.f;
    float inc = wave_inclusive_scan(p);
    if (lane == RL_WAVE - 1) scratch[wave] = inc;
    __syncthreads();
    float off = 0.f;
    for (int w = 0; w < wave; ++w) off += scratch[w];
    inc += off;
    cum[tid] = inc;
    __syncthreads();
    const float pool_mass = cum[SMP_POOL - 1];
    const bool dropped = tid >= k || (pool_mass > top_p && inc - p > top_p);
    // the kept tokens are a prefix of the pool (the mass before a token never decreases)
    const unsigned long long kb = __ballot(!dropped);
    if (lane == 0) hist[wave] = (unsigned int)__popcll(kb);
    __syncthreads();
    int n_keep = 0;
    for (int w = 0; w < SMP_WAVES; ++w) n_keep += (int)hist[w];
    if (n_keep < 1) n_keep = 1;
    const float target = u * cum[n_keep - 1];
    __syncthreads();
    const unsigned long long below = __ballot(tid < n_keep && cum[tid] < target);
    if (lane == 0) hist[wave] = (unsigned int)__popcll(below);
    __syncthreads();
    if (tid == 0) {
        int j = 0;
        for (int w = 0; w < SMP_WAVES; ++w) j += (int)hist[w];
        if (j > n_keep - 1) j = n_keep - 1;
        const int chosen = (int)(0xffffffffu - (uint32_t)(cand[j] & 0xffffffffull));
        out[blockIdx.x] = chosen;
        if (out_logprob)
            out_logprob[blockIdx.x] =
                key_float((uint32_t)(cand[j] >> 32)) - zmax - logf(total);
    }
}

// the uniform draw of (seed, counter), for tests and for callers that mirror the draw
extern "C" float rl_sample_uniform(unsigned int seed_lo, unsigned int seed_hi,
                                   unsigned int counter) {
    return sample_uniform(seed_lo, seed_hi, counter);
}

extern "C" int rl_sample_pool() { return SMP_POOL; }

// history may be null when no row has a penalty, fed when the history names no row of the
// step before.  out_logprob (optional): log-probability of the chosen token under the
// penalised, temperature-scaled distribution.
extern "C" int rl_sample(const float* logits, const int* row_index, const int* row_params,
                         const int* history, const int* fed, int fed_rows, int* out,
                         float* out_logprob, int rows, int vocab, int any_penalty,
                         hipStream_t stream) {
    if (rows <= 0) return RL_OK;
    if (vocab < 1) return RL_ERR_ARG;
    int words = 0;
    if (any_penalty) {
        words = (vocab + 31) / 32;
        if ((size_t)words * 4 > 40 * 1024) return RL_ERR_ARG;  // the bitmap lives in LDS
        if (!history) return RL_ERR_ARG;
    }
    if (fed && (fed == out || fed_rows < 0)) return RL_ERR_ARG;
    hipLaunchKernelGGL(sample_kernel, dim3(rows), dim3(SMP_THREADS), (size_t)words * 4, stream,
                       logits, row_index, row_params, history, fed, fed_rows, out, out_logprob, vocab,
                       words);
    return rl_launch_status();
}

// --------------------------------------------------------------------------- //
// Log-probability records (rapid_llm/engine/sampler.py:343-369): for every row the
// log-probability of a given token (the one chosen, or the prompt's own next token) and the
// k most likely tokens with theirs, in descending order, equal values by ascending id.
//
// The distribution is the one the row is sampled from: log_softmax of the penalised logits
// over the temperature, a greedy row counting as temperature 1 (:708-712).  Without
// row_params it is log_softmax of the raw logits, as prompt positions are scored (:425-447).
//
// One workgroup per row; the k tokens are found one after the other, each as the largest
// (value, lowest id) that comes after the previous one in that order: k + 2 passes over a
// row that stays in cache, no memory beyond the outputs, and a fixed result.
// --------------------------------------------------------------------------- //
__global__ __launch_bounds__(SMP_THREADS) void logprobs_kernel(
    const float* __restrict__ logits, const int* __restrict__ row_index,
    const int* __restrict__ row_params, const int* __restrict__ history,
    const int* __restrict__ fed, int fed_rows,
    const int* __restrict__ targets, float* __restrict__ out_target, int* __restrict__ out_top_ids,
    float* __restrict__ out_top_lp, int vocab, int k, int bitmap_words) {
    extern __shared__ uint32_t seen[];
    __shared__ float wave_tot[SMP_WAVES];
    __shared__ float best_v[SMP_WAVES];
    __shared__ int best_i[SMP_WAVES];

    const int tid = threadIdx.x;
    const int lane = tid & (RL_WAVE - 1), wave = tid / RL_WAVE;
    const int* rp = row_params ? row_params + 8 * blockIdx.x : nullptr;
    const float temperature = rp ? __int_as_float(rp[0]) : 1.f;
    const float penalty = rp ? __int_as_float(rp[2]) : 1.f;
    const bool penalise = rp && bitmap_words > 0 && penalty != 1.0f && rp[7] > rp[6];
    const float inv_t = temperature > 0.f ? 1.f / temperature : 1.f;
    const float* row = logits_row(logits, row_index, blockIdx.x, vocab);

    if (penalise) {
        for (int i = tid; i < bitmap_words; i += SMP_THREADS) seen[i] = 0u;
        __syncthreads();
        for (int i = rp[6] + tid; i < rp[7]; i += SMP_THREADS) {
            const int tok = history_token(history[i], fed, fed_rows);
            if (tok >= 0 && tok < vocab) atomicOr(&seen[tok >> 5], 1u << (tok & 31));
        }
        __syncthreads();
    }
    auto zval = [&](int i) -> float {
        float x = row[i];
        if (penalise && ((seen[i >> 5] >> (i & 31)) & 1u)) x = x < 0.f ? x * penalty : x / penalty;
        return x * inv_t;
    };
    // the largest (value, lowest id) after (pv, pi) in descending order; first: no bound
    auto next_best = [&](bool first, float pv, int pi, float& rv, int& ri) {
        float bv = -INFINITY;
        int bi = 0x7fffffff;
        for (int i = tid; i < vocab; i += SMP_THREADS) {
            const float v = zval(i);
            const bool after = first || v < pv || (v == pv && i > pi);
            if (after && (v > bv || (v == bv && i < bi))) {
                bv = v;
                bi = i;
            }
        }
#pragma unroll
        for (int off = RL_WAVE / 2; off > 0; off >>= 1) {
            const float ov = __shfl_xor(bv, off, RL_WAVE);
            const int oi = __shfl_xor(bi, off, RL_WAVE);
            if (ov > bv || (ov == bv && oi < bi)) {
                bv = ov;
                bi = oi;
            }
        }
        __syncthreads();  // the previous round's readers are done
        if (lane == 0) {
            best_v[wave] = bv;
            best_i[wave] = bi;
        }
        __syncthreads();
        bv = best_v[0];
        bi = best_i[0];
        for (int w = 1; w < SMP_WAVES; ++w)
            if (best_v[w] > bv || (best_v[w] == bv && best_i[w] < bi)) {
                bv = best_v[w];
                bi = best_i[w];
            }
        rv = bv;
        ri = bi;
    };

    float top_v;
    int top_i;
    next_best(true, 0.f, 0, top_v, top_i);
    const float zmax = top_v;

    // sum of exp in a fixed order: wave w owns a contiguous segment
    const int seg = ((vocab + SMP_WAVES - 1) / SMP_WAVES + RL_WAVE - 1) / RL_WAVE * RL_WAVE;
    const int seg_lo = min(vocab, wave * seg), seg_hi = min(vocab, seg_lo + seg);
    float wsum = 0.f;
    for (int base = seg_lo; base < seg_hi; base += RL_WAVE) {
        const int i = base + lane;
        wsum += (i < seg_hi) ? expf(zval(i) - zmax) : 0.f;
    }
    wsum = wave_sum(wsum);
    if (lane == 0) wave_tot[wave] = wsum;
    __syncthreads();
    float total = 0.f;
    for (int w = 0; w < SMP_WAVES; ++w) total += wave_tot[w];
    const float log_z = zmax + logf(total);

    if (tid == 0) {
        const int t = targets[blockIdx.x];
        out_target[blockIdx.x] = (t >= 0 && t < vocab) ? zval(t) - log_z : NAN;
    }
    for (int j = 0; j < k; ++j) {
        if (j > 0 && top_i != 0x7fffffff) next_best(false, top_v, top_i, top_v, top_i);
        if (tid == 0) {
            // fewer than k values that can be ordered (NaN cannot): the rest is marked empty
            const bool none = top_i == 0x7fffffff;
            out_top_ids[(size_t)blockIdx.x * k + j] = none ? -1 : top_i;
            out_top_lp[(size_t)blockIdx.x * k + j] = none ? -INFINITY : top_v - log_z;
        }
    }
}

// targets [rows]: the token whose log-probability goes to out_target [rows] (NaN for an id
// outside the vocabulary).  out_top_ids / out_top_lp [rows, k]; k may be 0.  row_params and
// history and fed as for rl_sample, or null for the raw distribution.
extern "C" int rl_logprobs(const float* logits, const int* row_index, const int* row_params,
                           const int* history, const int* fed, int fed_rows,
                           const int* targets, float* out_target,
                           int* out_top_ids, float* out_top_lp, int rows, int vocab, int k,
                           int any_penalty, hipStream_t stream) {
    if (rows <= 0) return RL_OK;
    if (vocab < 1 || k < 0 || k > vocab || !targets || !out_target) return RL_ERR_ARG;
    if (k > 0 && (!out_top_ids || !out_top_lp)) return RL_ERR_ARG;
    int words = 0;
    if (any_penalty) {
        words = (vocab + 31) / 32;
        if ((size_t)words * 4 > 40 * 1024) return RL_ERR_ARG;
        if (!history || !row_params) return RL_ERR_ARG;
    }
    if (fed && fed_rows < 0) return RL_ERR_ARG;
    hipLaunchKernelGGL(logprobs_kernel, dim3(rows), dim3(SMP_THREADS), (size_t)words * 4, stream,
                       logits, row_index, row_params, history, fed, fed_rows, targets, out_target,
                       out_top_ids,
                       out_top_lp, vocab, k, words);
    return rl_launch_status();
}
