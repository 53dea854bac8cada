// Row-wise kernels of the decoder: embedding gather, residual-add + RMSNorm, SwiGLU,
// rotation tables, the fused per-head norm + rotation + cache write, and a type cast.
// All arithmetic is float32; the element type only decides loads and stores.
#include "common.h"

// --------------------------------------------------------------------------- //
// embedding: residual[t, :] = table[ids[t], :]   (float32 residual stream)
// rapid_llm/modules/vocab_parallel.py:102-103
// --------------------------------------------------------------------------- //
// A negative id -(r + 1) stands for "the token chosen in row r of the previous step", which
// the host may not have seen yet: it is read from `fed` (the sampling kernels' output)
// (rapid_llm/engine/scheduler.py:241-249: the placeholder a device-side gather replaces).
template <typename W>
__global__ void embed_kernel(const int* __restrict__ ids, const int* __restrict__ fed, int fed_rows,
                             const W* __restrict__ table, float* __restrict__ out, int hidden,
                             int vocab) {
    const int t = blockIdx.x;
    int id = ids[t];
    if (id < 0 && fed && -id - 1 < fed_rows) id = fed[-id - 1];
    // ids are validated on the host; an id outside the table reads row 0 rather than faulting
    if (id < 0 || id >= vocab) id = 0;
    const W* row = table + (size_t)id * hidden;
    float* dst = out + (size_t)t * hidden;
    constexpr int VEC = 16 / sizeof(W);  // elements of one 16-byte read
    if (hidden % VEC == 0) {
        struct alignas(16) Pack {
            W v[VEC];
        };
        for (int i = threadIdx.x * VEC; i < hidden; i += blockDim.x * VEC) {
            const Pack p = *reinterpret_cast<const Pack*>(row + i);
#pragma unroll
            for (int j = 0; j < VEC; j += 4)
                *reinterpret_cast<float4*>(dst + i + j) = make_float4(
                    to_float(p.v[j]), to_float(p.v[j + 1]), to_float(p.v[j + 2]), to_float(p.v[j + 3]));
        }
        return;
    }
    for (int i = threadIdx.x; i < hidden; i += blockDim.x) dst[i] = to_float(row[i]);
}

extern "C" int rl_embed(const int* ids, const int* fed, int fed_rows, const void* table,
                        int table_type, float* out, int tokens, int hidden, int vocab,
                        hipStream_t stream) {
    if (tokens <= 0) return RL_OK;
    dim3 grid(tokens), block(256);
    if (table_type == RL_F32)
        hipLaunchKernelGGL(embed_kernel<float>, grid, block, 0, stream, ids, fed, fed_rows,
                           (const float*)table, out, hidden, vocab);
    else if (table_type == RL_BF16)
        hipLaunchKernelGGL(embed_kernel<bf16_t>, grid, block, 0, stream, ids, fed, fed_rows,
                           (const bf16_t*)table, out, hidden, vocab);
    else
        return RL_ERR_ARG;
    return rl_launch_status();
}

// --------------------------------------------------------------------------- //
// residual += delta (float32, in place); out = residual * rsqrt(mean(residual^2)+eps) * w
// One block per produced row; `rows` (optional) selects which residual rows are produced,
// packed in order.  rapid_llm/kernels/ops/layernorm/skip_rmsnorm.py:51-85: the sum is
// formed in float32 and the norm reads the unrounded sum.
// --------------------------------------------------------------------------- //
template <typename T>
__global__ void add_rmsnorm_kernel(float* __restrict__ residual, const T* __restrict__ delta,
                                   const float* __restrict__ weight, T* __restrict__ out,
                                   const int* __restrict__ rows, int hidden, float eps) {
    __shared__ float scratch[16];
    const int r = blockIdx.x;
    const int row = rows ? rows[r] : r;
    float* res = residual + (size_t)row * hidden;
    const T* dl = delta ? delta + (size_t)row * hidden : nullptr;
    float ss = 0.f;
    for (int i = threadIdx.x; i < hidden; i += blockDim.x) {
        float v = res[i];
        if (dl) {
            v += to_float(dl[i]);
            res[i] = v;
        }
        ss += v * v;
    }
    ss = block_sum(ss, scratch);
    const float rrms = rsqrtf(ss / (float)hidden + eps);
    T* o = out + (size_t)r * hidden;
    // each thread re-reads exactly the elements it wrote above
    for (int i = threadIdx.x; i < hidden; i += blockDim.x)
        o[i] = from_float<T>(res[i] * rrms * weight[i]);
}

// The same with four elements per thread and load: a row of up to 16 * blockDim elements
// stays in registers between the two passes, so a row costs one round trip to memory.  With
// few rows (decode) the kernel's time is that latency, not bandwidth.
template <typename T>
struct alignas(sizeof(T) * 4) Vec4 {
    T v[4];
};

template <typename T, int CHUNKS>
__global__ void add_rmsnorm_vec_kernel(float* __restrict__ residual, const T* __restrict__ delta,
                                       const float* __restrict__ weight, T* __restrict__ out,
                                       const int* __restrict__ rows, int hidden, float eps) {
    __shared__ float scratch[16];
    const int r = blockIdx.x;
    const int row = rows ? rows[r] : r;
    float4* res = reinterpret_cast<float4*>(residual + (size_t)row * hidden);
    const Vec4<T>* dl = delta ? reinterpret_cast<const Vec4<T>*>(delta + (size_t)row * hidden) : nullptr;
    const int nvec = hidden >> 2;
    const float4* w4 = reinterpret_cast<const float4*>(weight);
    float4 val[CHUNKS], wt[CHUNKS];
    float ss = 0.f;
    // the weights are read before the sum, not after its barrier: one wait less in a kernel
    // that is all latency when it has a handful of rows
#pragma unroll
    for (int c = 0; c < CHUNKS; ++c) {
        const int i = threadIdx.x + c * blockDim.x;
        if (i < nvec) wt[c] = w4[i];
    }
#pragma unroll
    for (int c = 0; c < CHUNKS; ++c) {
        const int i = threadIdx.x + c * blockDim.x;
        if (i < nvec) {
            float4 v = res[i];
            if (dl) {
                const Vec4<T> d = dl[i];
                v.x += to_float(d.v[0]);
                v.y += to_float(d.v[1]);
                v.z += to_float(d.v[2]);
                v.w += to_float(d.v[3]);
                res[i] = v;
            }
            val[c] = v;
            ss += v.x * v.x + v.y * v.y + v.z * v.z + v.w * v.w;
        }
    }
    ss = block_sum(ss, scratch);
    const float rrms = rsqrtf(ss / (float)hidden + eps);
    Vec4<T>* o = reinterpret_cast<Vec4<T>*>(out + (size_t)r * hidden);
#pragma unroll
    for (int c = 0; c < CHUNKS; ++c) {
        const int i = threadIdx.x + c * blockDim.x;
        if (i < nvec) {
            const float4 w = wt[c];
            Vec4<T> y;
            y.v[0] = from_float<T>(val[c].x * rrms * w.x);
            y.v[1] = from_float<T>(val[c].y * rrms * w.y);
            y.v[2] = from_float<T>(val[c].z * rrms * w.z);
            y.v[3] = from_float<T>(val[c].w * rrms * w.w);
            o[i] = y;
        }
    }
}

template <typename T>
static void launch_add_rmsnorm(float* residual, const T* delta, const float* weight, T* out,
                               const int* rows, int out_rows, int hidden, float eps,
                               hipStream_t stream) {
    dim3 grid(out_rows);
    if (hidden % 4 == 0 && hidden <= 16 * 1024) {
        const int nvec = hidden / 4;
        // one chunk per thread while the block stays within 1024 threads, then up to four
        int threads = ((nvec + RL_WAVE - 1) / RL_WAVE) * RL_WAVE;
        if (threads <= 1024) {
            hipLaunchKernelGGL((add_rmsnorm_vec_kernel<T, 1>), grid, dim3(threads), 0, stream,
                               residual, delta, weight, out, rows, hidden, eps);
        } else {
            hipLaunchKernelGGL((add_rmsnorm_vec_kernel<T, 4>), grid, dim3(1024), 0, stream,
                               residual, delta, weight, out, rows, hidden, eps);
        }
        return;
    }
    int threads = hidden >= 2048 ? 512 : (hidden >= 512 ? 256 : 64);
    hipLaunchKernelGGL(add_rmsnorm_kernel<T>, grid, dim3(threads), 0, stream, residual, delta,
                       weight, out, rows, hidden, eps);
}

extern "C" int rl_add_rmsnorm(float* residual, const void* delta, const float* weight, void* out,
                              const int* rows, int out_rows, int hidden, float eps, int act_type,
                              hipStream_t stream) {
    if (out_rows <= 0) return RL_OK;
    if (act_type == RL_F32)
        launch_add_rmsnorm<float>(residual, (const float*)delta, weight, (float*)out, rows,
                                  out_rows, hidden, eps, stream);
    else if (act_type == RL_BF16)
        launch_add_rmsnorm<bf16_t>(residual, (const bf16_t*)delta, weight, (bf16_t*)out, rows,
                                   out_rows, hidden, eps, stream);
    else
        return RL_ERR_ARG;
    return rl_launch_status();
}

// The same norm where the delta arrives as `nparts` float32 runs of a product's K
// (parts[run][row][hidden], see rl_gemm_mid_parts): the runs are added in order, the sum is
// rounded to the activation type as a stored product would be, then added to the residual.
template <typename T, int CHUNKS>
__global__ void add_parts_rmsnorm_kernel(float* __restrict__ residual, const float* __restrict__ parts,
                                         int nparts, size_t part_stride,
                                         const float* __restrict__ weight, T* __restrict__ out,
                                         int hidden, float eps) {
    __shared__ float scratch[16];
    const int row = blockIdx.x;
    float4* res = reinterpret_cast<float4*>(residual + (size_t)row * hidden);
    const int nvec = hidden >> 2;
    const float4* w4 = reinterpret_cast<const float4*>(weight);
    float4 val[CHUNKS], wt[CHUNKS];
    float ss = 0.f;
#pragma unroll
    for (int c = 0; c < CHUNKS; ++c) {
        const int i = threadIdx.x + c * blockDim.x;
        if (i < nvec) wt[c] = w4[i];
    }
#pragma unroll
    for (int c = 0; c < CHUNKS; ++c) {
        const int i = threadIdx.x + c * blockDim.x;
        if (i < nvec) {
            const float4* pr = reinterpret_cast<const float4*>(parts + (size_t)row * hidden) + i;
            float4 d = *pr;
            for (int r = 1; r < nparts; ++r) {
                const float4 e = *reinterpret_cast<const float4*>(
                    reinterpret_cast<const float*>(pr) + (size_t)r * part_stride);
                d.x += e.x;
                d.y += e.y;
                d.z += e.z;
                d.w += e.w;
            }
            float4 v = res[i];
            v.x += to_float(from_float<T>(d.x));
            v.y += to_float(from_float<T>(d.y));
            v.z += to_float(from_float<T>(d.z));
            v.w += to_float(from_float<T>(d.w));
            res[i] = v;
            val[c] = v;
            ss += v.x * v.x + v.y * v.y + v.z * v.z + v.w * v.w;
        }
    }
    ss = block_sum(ss, scratch);
    const float rrms = rsqrtf(ss / (float)hidden + eps);
    Vec4<T>* o = reinterpret_cast<Vec4<T>*>(out + (size_t)row * hidden);
#pragma unroll
    for (int c = 0; c < CHUNKS; ++c) {
        const int i = threadIdx.x + c * blockDim.x;
        if (i < nvec) {
            const float4 w = wt[c];
            Vec4<T> y;
            y.v[0] = from_float<T>(val[c].x * rrms * w.x);
            y.v[1] = from_float<T>(val[c].y * rrms * w.y);
            y.v[2] = from_float<T>(val[c].z * rrms * w.z);
            y.v[3] = from_float<T>(val[c].w * rrms * w.w);
            o[i] = y;
        }
    }
}

// parts [nparts, rows, hidden] float32, contiguous; bfloat16 rows out; hidden a multiple of 4 up to 16 K
extern "C" int rl_add_rmsnorm_parts(float* residual, const float* parts, int nparts,
                                    const float* weight, void* out, int rows, int hidden, float eps,
                                    hipStream_t stream) {
    if (rows <= 0) return RL_OK;
    if (nparts < 1 || hidden % 4 || hidden > 16 * 1024) return RL_ERR_ARG;
    const int nvec = hidden / 4;
    const int threads = ((nvec + RL_WAVE - 1) / RL_WAVE) * RL_WAVE;
    const size_t stride = (size_t)rows * hidden;
    if (threads <= 1024)
        hipLaunchKernelGGL((add_parts_rmsnorm_kernel<bf16_t, 1>), dim3(rows), dim3(threads), 0, stream,
                           residual, parts, nparts, stride, weight, (bf16_t*)out, hidden, eps);
    else
        hipLaunchKernelGGL((add_parts_rmsnorm_kernel<bf16_t, 4>), dim3(rows), dim3(1024), 0, stream,
                           residual, parts, nparts, stride, weight, (bf16_t*)out, hidden, eps);
    return rl_launch_status();
}

// --------------------------------------------------------------------------- //
// SwiGLU on the packed [gate | up] row: out[:, j] = silu(x[:, j]) * x[:, I + j]
// rapid_llm/kernels/ops/activation/swiglu.py:91-121
// --------------------------------------------------------------------------- //
template <typename T>
__global__ void swiglu_kernel(const T* __restrict__ gate_up, T* __restrict__ out, int inter,
                              size_t total) {
    size_t idx = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    const size_t step = (size_t)gridDim.x * blockDim.x;
    for (; idx < total; idx += step) {
        const size_t t = idx / inter;
        const int j = (int)(idx - t * inter);
        const T* row = gate_up + t * 2 * (size_t)inter;
        const float g = to_float(row[j]);
        const float u = to_float(row[inter + j]);
        const float s = g / (1.f + expf(-g));
        out[idx] = from_float<T>(s * u);
    }
}

// eight elements per thread (16-byte loads for bfloat16) when the width allows it
template <typename T>
struct alignas(sizeof(T) * 8) Vec8 {
    T v[8];
};

template <typename T>
__global__ void swiglu_vec_kernel(const T* __restrict__ gate_up, T* __restrict__ out, int inter,
                                  size_t total_vec) {
    size_t idx = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    const size_t step = (size_t)gridDim.x * blockDim.x;
    const int per_row = inter >> 3;
    for (; idx < total_vec; idx += step) {
        const size_t t = idx / per_row;
        const int j = (int)(idx - t * per_row) << 3;
        const T* row = gate_up + t * 2 * (size_t)inter;
        const Vec8<T> g = *reinterpret_cast<const Vec8<T>*>(row + j);
        const Vec8<T> u = *reinterpret_cast<const Vec8<T>*>(row + inter + j);
        Vec8<T> y;
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            const float gf = to_float(g.v[i]);
            y.v[i] = from_float<T>(gf / (1.f + expf(-gf)) * to_float(u.v[i]));
        }
        *reinterpret_cast<Vec8<T>*>(out + t * (size_t)inter + j) = y;
    }
}

template <typename T>
static void launch_swiglu(const T* gate_up, T* out, int tokens, int inter, hipStream_t stream) {
    if (inter % 8 == 0) {
        const size_t total = (size_t)tokens * (inter / 8);
        size_t blocks = (total + 255) / 256;
        if (blocks > 65536) blocks = 65536;
        hipLaunchKernelGGL(swiglu_vec_kernel<T>, dim3((unsigned)blocks), dim3(256), 0, stream,
                           gate_up, out, inter, total);
        return;
    }
    const size_t total = (size_t)tokens * inter;
    size_t blocks = (total + 255) / 256;
    if (blocks > 65536) blocks = 65536;
    hipLaunchKernelGGL(swiglu_kernel<T>, dim3((unsigned)blocks), dim3(256), 0, stream, gate_up, out,
                       inter, total);
}

extern "C" int rl_swiglu(const void* gate_up, void* out, int tokens, int inter, int act_type,
                         hipStream_t stream) {
    if (tokens <= 0) return RL_OK;
    if (act_type == RL_F32)
        launch_swiglu<float>((const float*)gate_up, (float*)out, tokens, inter, stream);
    else if (act_type == RL_BF16)
        launch_swiglu<bf16_t>((const bf16_t*)gate_up, (bf16_t*)out, tokens, inter, stream);
    else
        return RL_ERR_ARG;
    return rl_launch_status();
}

// --------------------------------------------------------------------------- //
// cast between float32 and bfloat16 (either direction, or a copy)
// --------------------------------------------------------------------------- //
template <typename S, typename D>
__global__ void cast_kernel(const S* __restrict__ src, D* __restrict__ dst, size_t total) {
    size_t idx = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    const size_t step = (size_t)gridDim.x * blockDim.x;
    for (; idx < total; idx += step) dst[idx] = from_float<D>(to_float(src[idx]));
}

extern "C" int rl_cast(const void* src, int src_type, void* dst, int dst_type, size_t total,
                       hipStream_t stream) {
    if (total == 0) return RL_OK;
    size_t blocks = (total + 255) / 256;
    if (blocks > 65536) blocks = 65536;
    dim3 grid((unsigned)blocks), block(256);
    if (src_type == RL_F32 && dst_type == RL_BF16)
        hipLaunchKernelGGL((cast_kernel<float, bf16_t>), grid, block, 0, stream,
                           (const float*)src, (bf16_t*)dst, total);
    else if (src_type == RL_BF16 && dst_type == RL_F32)
        hipLaunchKernelGGL((cast_kernel<bf16_t, float>), grid, block, 0, stream,
                           (const bf16_t*)src, (float*)dst, total);
    else if (src_type == RL_F32 && dst_type == RL_F32)
        hipLaunchKernelGGL((cast_kernel<float, float>), grid, block, 0, stream,
                           (const float*)src, (float*)dst, total);
    else if (src_type == RL_BF16 && dst_type == RL_BF16)
        hipLaunchKernelGGL((cast_kernel<bf16_t, bf16_t>), grid, block, 0, stream,
                           (const bf16_t*)src, (bf16_t*)dst, total);
    else
        return RL_ERR_ARG;
    return rl_launch_status();
}

// --------------------------------------------------------------------------- //
// bias of a product: y[r, c] += bias[c], the sum rounded once to y's type
// (rapid_llm/modules/linear.py adds the bias inside F.linear; Qwen3 has none, other
// architectures' projections do)
// --------------------------------------------------------------------------- //
template <typename T>
__global__ void add_bias_kernel(T* __restrict__ y, const float* __restrict__ bias, size_t total,
                                int cols) {
    size_t idx = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    const size_t step = (size_t)gridDim.x * blockDim.x;
    for (; idx < total; idx += step) y[idx] = from_float<T>(to_float(y[idx]) + bias[idx % cols]);
}

extern "C" int rl_add_bias(void* y, const float* bias, int rows, int cols, int act_type,
                           hipStream_t stream) {
    if (rows <= 0 || cols <= 0) return RL_OK;
    const size_t total = (size_t)rows * cols;
    size_t blocks = (total + 255) / 256;
    if (blocks > 65536) blocks = 65536;
    dim3 grid((unsigned)blocks), block(256);
    if (act_type == RL_F32)
        hipLaunchKernelGGL(add_bias_kernel<float>, grid, block, 0, stream, (float*)y, bias, total, cols);
    else if (act_type == RL_BF16)
        hipLaunchKernelGGL(add_bias_kernel<bf16_t>, grid, block, 0, stream, (bf16_t*)y, bias, total, cols);
    else
        return RL_ERR_ARG;
    return rl_launch_status();
}

// --------------------------------------------------------------------------- //
// rotation tables: cos/sin[p, i] of the float32 product p * inv_freq[i]
// rapid_llm/modules/rotary_embedding.py:194-202 (float32 outer product, then cos/sin)
// --------------------------------------------------------------------------- //
__global__ void rope_table_kernel(const float* __restrict__ inv_freq, float* __restrict__ cos_out,
                                  float* __restrict__ sin_out, int half, size_t total) {
    size_t idx = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    const size_t step = (size_t)gridDim.x * blockDim.x;
    for (; idx < total; idx += step) {
        const size_t p = idx / half;
        const int i = (int)(idx - p * half);
        const float ang = (float)p * inv_freq[i];
        // the angle is the float32 product; its cosine and sine are taken in double so
        // that range reduction of large angles costs nothing in accuracy
        cos_out[idx] = (float)cos((double)ang);
        sin_out[idx] = (float)sin((double)ang);
    }
}

extern "C" int rl_rope_table(const float* inv_freq, float* cos_out, float* sin_out,
                             int positions, int half, hipStream_t stream) {
    const size_t total = (size_t)positions * half;
    if (total == 0) return RL_OK;
    size_t blocks = (total + 255) / 256;
    if (blocks > 65536) blocks = 65536;
    hipLaunchKernelGGL(rope_table_kernel, dim3((unsigned)blocks), dim3(256), 0, stream, inv_freq,
                       cos_out, sin_out, half, total);
    return rl_launch_status();
}

// --------------------------------------------------------------------------- //
// Fused per-head RMSNorm (optional) + rotation (optional) of q and k, and the write of k and v
// into the paged cache.  One wave per (token, head); a workgroup of four waves takes four
// heads of a token.
//
// qkv row layout: [q heads | k heads | v heads], heads adjacent (rapid_llm/modules/linear.py:
// 236-251).  Norm over head_dim before the rotation (rapid_llm/models/base.py:134-140).
// Rotation of a pair (x1, x2) by the position's angle of that pair: o1 = x1*c - x2*s,
// o2 = x2*c + x1*s (rapid_llm/kernels/ops/rope/rope_emb.py:47-82).  Which channels pair, and
// how many of a head's channels rotate, is the position encoding's to say: the first
// 2 * rotary_half channels rotate, pair p of them being channels (p, p + rotary_half) with the
// half-split pairing (the reference's) and (2p, 2p + 1) with the interleaved one; the channels
// beyond pass with the norm alone.  This kernel takes every such case; the vectorised ones
// below take the half-split rotation of the whole head.
//
// Cache layout of one layer, page p, kv head h:
//   keys   K[p][h][slot_in_page][d]      (row-major, d contiguous)
//   values V[p][h][d][slot_in_page]      (transposed: the page's positions contiguous)
// A token at position pos of a request lies in page table[slot_of_request][pos / P] at
// slot_in_page = pos % P.
// --------------------------------------------------------------------------- //
template <typename T>
__global__ void qknorm_rope_kvwrite_kernel(
    const T* __restrict__ qkv, T* __restrict__ q_out, T* __restrict__ k_cache,
    T* __restrict__ v_cache, const float* __restrict__ q_norm_w,
    const float* __restrict__ k_norm_w, const float* __restrict__ cos_tab,
    const float* __restrict__ sin_tab, const int* __restrict__ positions,
    const int* __restrict__ token_slot, const int* __restrict__ block_table, int table_stride,
    int page_size, int nq, int nkv, int d, int rotary_half, int interleaved, float eps,
    int write_cache, int write_values, int head0) {
    const int t = blockIdx.x;
    const int lane = threadIdx.x & (RL_WAVE - 1);
    const int wave = threadIdx.x / RL_WAVE;
    const int nwaves = blockDim.x / RL_WAVE;
    const int half = d / 2;
    const int pos = positions[t];
    const int total_heads = nq + 2 * nkv;
    const T* row = qkv + (size_t)t * total_heads * d;

    size_t page = 0;
    int off = 0;
    if (write_cache) {
        page = (size_t)block_table[(size_t)token_slot[t] * table_stride + pos / page_size];
        off = pos % page_size;
    }

    // head0: the first head to work on (the number of query heads where the attention kernels
    // finish the queries themselves)
    for (int head = head0 + blockIdx.y * nwaves + wave; head < total_heads; head += nwaves * gridDim.y) {
        const T* x = row + (size_t)head * d;
        if (head >= nq + nkv) {
            // value head: copy into the transposed page (unless the tile kernel below does it)
            if (!write_cache || !write_values) continue;
            const int h = head - nq - nkv;
            T* dst = v_cache + ((page * nkv + h) * d) * page_size + off;
            for (int i = lane; i < d; i += RL_WAVE) dst[(size_t)i * page_size] = x[i];
            continue;
        }
        const bool is_q = head < nq;
        if (!is_q && !write_cache) continue;
        const float* w = is_q ? q_norm_w : k_norm_w;
        // lane handles the pairs p = lane, lane + 64 (half <= 128) of channels (e1, e2): the
        // pairs that rotate first, as the pairing says, then the channels beyond two by two
        const int rot = cos_tab ? rotary_half : 0;
        int e1[2], e2[2];
        float x1[2], x2[2];
        float ss = 0.f;
#pragma unroll
        for (int r = 0; r < 2; ++r) {
            const int p = lane + r * RL_WAVE;
            const bool split = p < rot && !interleaved;
            e1[r] = split ? p : 2 * p;
            e2[r] = split ? p + rot : 2 * p + 1;
            x1[r] = 0.f;
            x2[r] = 0.f;
            if (p < half) {
                x1[r] = to_float(x[e1[r]]);
                x2[r] = to_float(x[e2[r]]);
                ss += x1[r] * x1[r] + x2[r] * x2[r];
            }
        }
        float rrms = 1.f;
        if (w) {
            ss = wave_sum(ss);
            rrms = rsqrtf(ss / (float)d + eps);
        }
        T* dst;
        if (is_q)
            dst = q_out + ((size_t)t * nq + head) * d;
        else
            dst = k_cache + ((page * nkv + (head - nq)) * page_size + off) * d;
#pragma unroll
        for (int r = 0; r < 2; ++r) {
            const int p = lane + r * RL_WAVE;
            if (p < half) {
                float a = x1[r], b = x2[r];
                if (w) {
                    a = a * rrms * w[e1[r]];
                    b = b * rrms * w[e2[r]];
                }
                if (p < rot) {
                    const float c = cos_tab[(size_t)pos * rotary_half + p];
                    const float s = sin_tab[(size_t)pos * rotary_half + p];
                    const float ra = a * c - b * s;
                    const float rb = b * c + a * s;
                    a = ra;
                    b = rb;
                }
                dst[e1[r]] = from_float<T>(a);
                dst[e2[r]] = from_float<T>(b);
            }
        }
    }
}

// The same with four consecutive channels of each half per lane: LPH lanes (16 for heads up to
// 128, else 32) take one head, a wave takes 64 / LPH heads, and every load and store moves 8
// or 16 bytes.  Needs d % 8 == 0.
template <typename T, int LPH>
__device__ inline void qknorm_rope_kvwrite_vec(
    int t, int head_group, const T* __restrict__ qkv, T* __restrict__ q_out, T* __restrict__ k_cache,
    T* __restrict__ v_cache, const float* __restrict__ q_norm_w,
    const float* __restrict__ k_norm_w, const float* __restrict__ cos_tab,
    const float* __restrict__ sin_tab, const int* __restrict__ positions,
    const int* __restrict__ token_slot, const int* __restrict__ block_table, int table_stride,
    int page_size, int nq, int nkv, int d, float eps, int write_cache, int write_values, int head0) {
    constexpr int HPW = RL_WAVE / LPH;  // heads per wave
    const int lane = threadIdx.x & (RL_WAVE - 1);
    const int wave = threadIdx.x / RL_WAVE;
    const int sub = lane / LPH;  // which of the wave's heads
    const int li = lane % LPH;   // channels 4 li .. 4 li + 3 of each half
    const int half = d / 2;
    const int pos = positions[t];
    const int total_heads = nq + (write_values ? 2 * nkv : nkv);
    const T* row = qkv + (size_t)t * (nq + 2 * nkv) * d;
    size_t page = 0;
    int off = 0;
    if (write_cache) {
        page = (size_t)block_table[(size_t)token_slot[t] * table_stride + pos / page_size];
        off = pos % page_size;
    }
    const int head = head0 + (head_group * (blockDim.x / RL_WAVE) + wave) * HPW + sub;
    if (head >= total_heads) return;  // whole groups of LPH lanes leave together
    const T* x = row + (size_t)head * d;
    const bool active = 4 * li < half;
    if (head >= nq + nkv) {
        if (!write_cache) return;
        const int h = head - nq - nkv;
        T* dst = v_cache + ((page * nkv + h) * d) * page_size + off;
        for (int i = li; i < d; i += LPH) dst[(size_t)i * page_size] = x[i];
        return;
    }
    const bool is_q = head < nq;
    if (!is_q && !write_cache) return;
    const float* w = is_q ? q_norm_w : k_norm_w;
    float a[4] = {0.f, 0.f, 0.f, 0.f}, b[4] = {0.f, 0.f, 0.f, 0.f};
    float ss = 0.f;
    if (active) {
        const Vec4<T> va = *reinterpret_cast<const Vec4<T>*>(x + 4 * li);
        const Vec4<T> vb = *reinterpret_cast<const Vec4<T>*>(x + half + 4 * li);
#pragma unroll
        for (int k = 0; k < 4; ++k) {
            a[k] = to_float(va.v[k]);
            b[k] = to_float(vb.v[k]);
            ss += a[k] * a[k] + b[k] * b[k];
        }
    }
    if (w) {
        // sum over the LPH lanes of the head (a power of two, aligned in the wave)
#pragma unroll
        for (int o = LPH / 2; o > 0; o >>= 1) ss += __shfl_xor(ss, o, RL_WAVE);
        const float rrms = rsqrtf(ss / (float)d + eps);
        if (active) {
            const float4 wa = *reinterpret_cast<const float4*>(w + 4 * li);
            const float4 wb = *reinterpret_cast<const float4*>(w + half + 4 * li);
            a[0] *= rrms * wa.x; a[1] *= rrms * wa.y; a[2] *= rrms * wa.z; a[3] *= rrms * wa.w;
            b[0] *= rrms * wb.x; b[1] *= rrms * wb.y; b[2] *= rrms * wb.z; b[3] *= rrms * wb.w;
        }
    }
    if (!active) return;
    if (cos_tab) {
        const float4 c4 = *reinterpret_cast<const float4*>(cos_tab + (size_t)pos * half + 4 * li);
        const float4 s4 = *reinterpret_cast<const float4*>(sin_tab + (size_t)pos * half + 4 * li);
        const float cs[4] = {c4.x, c4.y, c4.z, c4.w}, sn[4] = {s4.x, s4.y, s4.z, s4.w};
#pragma unroll
        for (int k = 0; k < 4; ++k) {
            const float ra = a[k] * cs[k] - b[k] * sn[k];
            b[k] = b[k] * cs[k] + a[k] * sn[k];
            a[k] = ra;
        }
    }
    T* dst = is_q ? q_out + ((size_t)t * nq + head) * d
                  : k_cache + ((page * nkv + (head - nq)) * page_size + off) * d;
    Vec4<T> oa, ob;
#pragma unroll
    for (int k = 0; k < 4; ++k) {
        oa.v[k] = from_float<T>(a[k]);
        ob.v[k] = from_float<T>(b[k]);
    }
    *reinterpret_cast<Vec4<T>*>(dst + 4 * li) = oa;
    *reinterpret_cast<Vec4<T>*>(dst + half + 4 * li) = ob;
}

template <typename T, int LPH>
__global__ __launch_bounds__(256) void qknorm_rope_kvwrite_vec_kernel(
    const T* __restrict__ qkv, T* __restrict__ q_out, T* __restrict__ k_cache,
    T* __restrict__ v_cache, const float* __restrict__ q_norm_w,
    const float* __restrict__ k_norm_w, const float* __restrict__ cos_tab,
    const float* __restrict__ sin_tab, const int* __restrict__ positions,
    const int* __restrict__ token_slot, const int* __restrict__ block_table, int table_stride,
    int page_size, int nq, int nkv, int d, float eps, int write_cache, int write_values, int head0) {
    qknorm_rope_kvwrite_vec<T, LPH>(blockIdx.x, blockIdx.y, qkv, q_out, k_cache, v_cache, q_norm_w, k_norm_w,
                                    cos_tab, sin_tab, positions, token_slot, block_table, table_stride,
                                    page_size, nq, nkv, d, eps, write_cache, write_values, head0);
}

template <typename T>
static void launch_qknorm(const T* qkv, T* q_out, T* k_cache, T* v_cache, const float* q_norm_w,
                          const float* k_norm_w, const float* cos_tab, const float* sin_tab,
                          const int* positions, const int* token_slot, const int* block_table,
                          int table_stride, int page_size, int tokens, int nq, int nkv, int d,
                          int rotary_half, int interleaved, float eps, int write_cache,
                          int write_values, int head0, hipStream_t stream) {
    const int total_heads = nq + (write_values ? 2 * nkv : nkv) - head0;  // heads to work on
    // the vectorised kernel: head sizes in steps of 8, the half-split rotation of the whole head
    if (d % 8 == 0 && (!cos_tab || (rotary_half == d / 2 && !interleaved))) {
        const int lph = d <= 128 ? 16 : 32;
        const int heads_per_block = 4 * (RL_WAVE / lph);
        const int groups = (total_heads + heads_per_block - 1) / heads_per_block;
        dim3 grid(tokens, groups), block(256);
        if (lph == 16)
            hipLaunchKernelGGL((qknorm_rope_kvwrite_vec_kernel<T, 16>), grid, block, 0, stream, qkv,
                               q_out, k_cache, v_cache, q_norm_w, k_norm_w, cos_tab, sin_tab,
                               positions, token_slot, block_table, table_stride, page_size, nq, nkv,
                               d, eps, write_cache, write_values, head0);
        else
            hipLaunchKernelGGL((qknorm_rope_kvwrite_vec_kernel<T, 32>), grid, block, 0, stream, qkv,
                               q_out, k_cache, v_cache, q_norm_w, k_norm_w, cos_tab, sin_tab,
                               positions, token_slot, block_table, table_stride, page_size, nq, nkv,
                               d, eps, write_cache, write_values, head0);
        return;
    }
    const int head_groups = (total_heads + 3) / 4;
    dim3 grid(tokens, head_groups > 65535 ? 65535 : head_groups), block(256);
    hipLaunchKernelGGL(qknorm_rope_kvwrite_kernel<T>, grid, block, 0, stream, qkv, q_out, k_cache,
                       v_cache, q_norm_w, k_norm_w, cos_tab, sin_tab, positions, token_slot,
                       block_table, table_stride, page_size, nq, nkv, d, rotary_half, interleaved, eps,
                       write_cache, write_values, head0);
}

// Values of 16 consecutive tokens of the batch and one kv head, written by one workgroup.
// The cache stores values transposed, V[page][head][channel][slot]: the sixteen slots of a
// channel are one 32-byte row (at a page of 16), and consecutive tokens of a request fill
// consecutive slots of it.  Written token by token those rows are completed by sixteen
// different workgroups, 2 bytes at a time; here a thread writes the four slots of four
// consecutive tokens at once where they line up, and the four threads of a row sit in
// adjacent lanes.
#define VT_TOKENS 16

template <typename T>
__device__ inline void v_tile_write(
    int tile, int h, const T* __restrict__ qkv, T* __restrict__ v_cache, const int* __restrict__ positions,
    const int* __restrict__ token_slot, const int* __restrict__ block_table, int table_stride,
    int page_size, int tokens, int nq, int nkv, int d) {
    __shared__ T vt[VT_TOKENS][256 + 8];
    __shared__ int s_page[VT_TOKENS];
    __shared__ int s_off[VT_TOKENS];
    const int t0 = tile * VT_TOKENS;
    const int row_width = (nq + 2 * nkv) * d;
    if (threadIdx.x < VT_TOKENS) {
        const int t = t0 + threadIdx.x;
        int page = -1, off = 0;
        if (t < tokens) {
            const int pos = positions[t];
            page = block_table[(size_t)token_slot[t] * table_stride + pos / page_size];
            off = pos % page_size;
        }
        s_page[threadIdx.x] = page;
        s_off[threadIdx.x] = off;
    }
    for (int idx = threadIdx.x; idx < VT_TOKENS * d; idx += 256) {
        const int i = idx / d, c = idx - i * d;
        if (t0 + i < tokens)
            vt[i][c] = qkv[(size_t)(t0 + i) * row_width + (size_t)(nq + nkv + h) * d + c];
    }
    __syncthreads();
    for (int idx = threadIdx.x; idx < 4 * d; idx += 256) {
        const int quarter = idx & 3, c = idx >> 2;
        const int i0 = 4 * quarter;
        const int page = s_page[i0], off = s_off[i0];
        bool lined_up = page >= 0 && (off & 3) == 0 && (page_size & 3) == 0;
#pragma unroll
        for (int k = 1; k < 4; ++k)
            lined_up = lined_up && s_page[i0 + k] == page && s_off[i0 + k] == off + k;
        if (lined_up) {
            Vec4<T> v;
#pragma unroll
            for (int k = 0; k < 4; ++k) v.v[k] = vt[i0 + k][c];
            *reinterpret_cast<Vec4<T>*>(v_cache + (((size_t)page * nkv + h) * d + c) * page_size + off) = v;
        } else {
#pragma unroll
            for (int k = 0; k < 4; ++k) {
                const int pg = s_page[i0 + k];
                if (pg >= 0)
                    v_cache[(((size_t)pg * nkv + h) * d + c) * page_size + s_off[i0 + k]] = vt[i0 + k][c];
            }
        }
    }
}

// One launch for a step of many tokens: the first tokens * head_groups workgroups norm, rotate
// and write the query and key heads of one token each, the rest write the values of 16 tokens
// and one kv head each.  A workgroup is wholly one or the other.
template <typename T, int LPH>
__global__ __launch_bounds__(256) void qkv_prepare_kernel(
    const T* __restrict__ qkv, T* __restrict__ q_out, T* __restrict__ k_cache,
    T* __restrict__ v_cache, const float* __restrict__ q_norm_w,
    const float* __restrict__ k_norm_w, const float* __restrict__ cos_tab,
    const float* __restrict__ sin_tab, const int* __restrict__ positions,
    const int* __restrict__ token_slot, const int* __restrict__ block_table, int table_stride,
    int page_size, int tokens, int head_groups, int nq, int nkv, int d, float eps, int head0) {
    const int qk_blocks = tokens * head_groups;
    if ((int)blockIdx.x < qk_blocks) {
        qknorm_rope_kvwrite_vec<T, LPH>(blockIdx.x / head_groups, blockIdx.x % head_groups, qkv, q_out, k_cache,
                                        v_cache, q_norm_w, k_norm_w, cos_tab, sin_tab, positions, token_slot,
                                        block_table, table_stride, page_size, nq, nkv, d, eps, 1, 0, head0);
    } else {
        const int b = blockIdx.x - qk_blocks;
        v_tile_write<T>(b / nkv, b % nkv, qkv, v_cache, positions, token_slot, block_table, table_stride,
                        page_size, tokens, nq, nkv, d);
    }
}

template <typename T>
__global__ __launch_bounds__(256) void v_tile_write_kernel(
    const T* __restrict__ qkv, T* __restrict__ v_cache, const int* __restrict__ positions,
    const int* __restrict__ token_slot, const int* __restrict__ block_table, int table_stride,
    int page_size, int tokens, int nq, int nkv, int d) {
    v_tile_write<T>(blockIdx.x, blockIdx.y, qkv, v_cache, positions, token_slot, block_table, table_stride,
                    page_size, tokens, nq, nkv, d);
}

// true if it launched: head sizes in steps of 8, and a grid that fits
template <typename T>
static bool launch_qkv_prepare(const T* qkv, T* q_out, T* k_cache, T* v_cache, const float* q_norm_w,
                               const float* k_norm_w, const float* cos_tab, const float* sin_tab,
                               const int* positions, const int* token_slot, const int* block_table,
                               int table_stride, int page_size, int tokens, int nq, int nkv, int d,
                               float eps, int head0, hipStream_t stream) {
    if (d % 8) return false;
    const int lph = d <= 128 ? 16 : 32;
    const int heads_per_block = 4 * (RL_WAVE / lph);
    const int head_groups = (nq + nkv - head0 + heads_per_block - 1) / heads_per_block;
    const long blocks = (long)tokens * head_groups + (long)((tokens + VT_TOKENS - 1) / VT_TOKENS) * nkv;
    if (blocks > 0x7fffffffL) return false;
    dim3 grid((unsigned)blocks), block(256);
    if (lph == 16)
        hipLaunchKernelGGL((qkv_prepare_kernel<T, 16>), grid, block, 0, stream, qkv, q_out, k_cache, v_cache,
                           q_norm_w, k_norm_w, cos_tab, sin_tab, positions, token_slot, block_table,
                           table_stride, page_size, tokens, head_groups, nq, nkv, d, eps, head0);
    else
        hipLaunchKernelGGL((qkv_prepare_kernel<T, 32>), grid, block, 0, stream, qkv, q_out, k_cache, v_cache,
                           q_norm_w, k_norm_w, cos_tab, sin_tab, positions, token_slot, block_table,
                           table_stride, page_size, tokens, head_groups, nq, nkv, d, eps, head0);
    return true;
}

extern "C" int rl_qknorm_rope_kvwrite(const void* qkv, void* q_out, void* k_cache, void* v_cache,
                                      const float* q_norm_w, const float* k_norm_w,
                                      const float* cos_tab, const float* sin_tab,
                                      const int* positions, const int* token_slot,
                                      const int* block_table, int table_stride, int page_size,
                                      int tokens, int nq, int nkv, int d, int rotary_half,
                                      int interleaved, float eps, int write_cache, int act_type,
                                      hipStream_t stream) {
    if (tokens <= 0) return RL_OK;
    if (d % 2 || d > 256) return RL_ERR_ARG;
    // q_out null: the attention kernels finish the query heads themselves, and the work here
    // starts at the first key head
    const int head0 = q_out ? 0 : nq;
    if (!q_out && !write_cache) return RL_OK;  // nothing to write at all
    // the first 2 * rotary_half channels of a head rotate: at least one pair, at most all
    if (cos_tab && (rotary_half < 1 || rotary_half > d / 2)) return RL_ERR_ARG;
    const bool whole_split = !cos_tab || (rotary_half == d / 2 && !interleaved);
    // with enough tokens the values go through the tile kernel, and the per-head kernel
    // covers the query and key heads only
    const int tile_values = write_cache && tokens >= 8 && nkv <= 65535;
    if ((long)nq + 2 * nkv > 65535 * 4) return RL_ERR_ARG;
    dim3 block(256);
    dim3 vgrid((tokens + VT_TOKENS - 1) / VT_TOKENS, nkv);
    if (tile_values && whole_split && act_type == RL_F32 &&
        launch_qkv_prepare<float>((const float*)qkv, (float*)q_out, (float*)k_cache, (float*)v_cache, q_norm_w,
                                  k_norm_w, cos_tab, sin_tab, positions, token_slot, block_table,
                                  table_stride, page_size, tokens, nq, nkv, d, eps, head0, stream))
        return rl_launch_status();
    if (tile_values && whole_split && act_type == RL_BF16 &&
        launch_qkv_prepare<bf16_t>((const bf16_t*)qkv, (bf16_t*)q_out, (bf16_t*)k_cache, (bf16_t*)v_cache,
                                   q_norm_w, k_norm_w, cos_tab, sin_tab, positions, token_slot, block_table,
                                   table_stride, page_size, tokens, nq, nkv, d, eps, head0, stream))
        return rl_launch_status();
    if (act_type == RL_F32) {
        launch_qknorm<float>((const float*)qkv, (float*)q_out, (float*)k_cache, (float*)v_cache,
                             q_norm_w, k_norm_w, cos_tab, sin_tab, positions, token_slot,
                             block_table, table_stride, page_size, tokens, nq, nkv, d, rotary_half,
                             interleaved, eps, write_cache, !tile_values, head0, stream);
        if (tile_values)
            hipLaunchKernelGGL(v_tile_write_kernel<float>, vgrid, block, 0, stream,
                               (const float*)qkv, (float*)v_cache, positions, token_slot,
                               block_table, table_stride, page_size, tokens, nq, nkv, d);
    } else if (act_type == RL_BF16) {
        launch_qknorm<bf16_t>((const bf16_t*)qkv, (bf16_t*)q_out, (bf16_t*)k_cache,
                              (bf16_t*)v_cache, q_norm_w, k_norm_w, cos_tab, sin_tab, positions,
                              token_slot, block_table, table_stride, page_size, tokens, nq, nkv, d,
                              rotary_half, interleaved, eps, write_cache, !tile_values, head0, stream);
        if (tile_values)
            hipLaunchKernelGGL(v_tile_write_kernel<bf16_t>, vgrid, block, 0, stream,
                               (const bf16_t*)qkv, (bf16_t*)v_cache, positions, token_slot,
                               block_table, table_stride, page_size, tokens, nq, nkv, d);
    } else {
        return RL_ERR_ARG;
    }
    return rl_launch_status();
}

// --------------------------------------------------------------------------- //
// order[r] = the single-token request with the r-th longest context of the step: request i's
// last position is positions[seq_token ? seq_token[i] : i]; equal lengths keep their order.
// Every thread counts the requests that come before its own (n^2 comparisons through LDS:
// a step has hundreds of requests, not millions).  The decode attention hands its workgroups
// out in this order.
// --------------------------------------------------------------------------- //
__global__ __launch_bounds__(256) void order_by_length_kernel(const int* __restrict__ positions,
                                                              const int* __restrict__ seq_token,
                                                              int n, int* __restrict__ order) {
    __shared__ __attribute__((aligned(16))) int keys[256];
    const int i = blockIdx.x * 256 + threadIdx.x;
    const int mine = i < n ? positions[seq_token ? seq_token[i] : i] : 0;
    int rank = 0;
    for (int base = 0; base < n; base += 256) {  // the same trips for every thread
        const int j = base + threadIdx.x;
        __syncthreads();
        // beyond the last request: shorter than any (positions are never negative)
        keys[threadIdx.x] = j < n ? positions[seq_token ? seq_token[j] : j] : -1;
        __syncthreads();
        // requests base + k before mine: longer ones, and equal ones with a smaller index
        const int before = i - base;  // k < before: a smaller index
#pragma unroll 8
        for (int k4 = 0; k4 < 256; k4 += 4) {
            const int4 o = *reinterpret_cast<const int4*>(&keys[k4]);
            rank += (o.x > mine || (o.x == mine && k4 + 0 < before)) ? 1 : 0;
            rank += (o.y > mine || (o.y == mine && k4 + 1 < before)) ? 1 : 0;
            rank += (o.z > mine || (o.z == mine && k4 + 2 < before)) ? 1 : 0;
            rank += (o.w > mine || (o.w == mine && k4 + 3 < before)) ? 1 : 0;
        }
    }
    if (i < n) order[rank] = i;
}

extern "C" int rl_order_by_length(const int* positions, const int* seq_token, int n, int* order,
                                  hipStream_t stream) {
    if (n <= 0) return RL_OK;
    if (!positions || !order) return RL_ERR_ARG;
    hipLaunchKernelGGL(order_by_length_kernel, dim3((n + 255) / 256), dim3(256), 0, stream,
                       positions, seq_token, n, order);
    return rl_launch_status();
}

// --------------------------------------------------------------------------- //
// A plain read of a buffer, for measuring what the memory system delivers: every thread
// keeps eight 16-byte loads in flight; nothing is written unless the data match a pattern
// that never occurs (so that the loads cannot be dropped).
// --------------------------------------------------------------------------- //
__global__ __launch_bounds__(256) void read_kernel(const uint4* __restrict__ src, size_t n16,
                                                   unsigned* __restrict__ sink) {
    size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    const size_t stride = (size_t)gridDim.x * blockDim.x;
    unsigned acc = 0;
    for (; i + 7 * stride < n16; i += 8 * stride) {
        uint4 v[8];
#pragma unroll
        for (int u = 0; u < 8; ++u) v[u] = src[i + u * stride];
#pragma unroll
        for (int u = 0; u < 8; ++u) acc += v[u].x ^ v[u].y ^ v[u].z ^ v[u].w;
    }
    for (; i < n16; i += stride) acc += src[i].x;
    if (acc == 0x9e3779b9u) sink[0] = acc;
}

extern "C" int rl_read_buffer(const void* src, size_t bytes, unsigned* sink, int blocks,
                              hipStream_t stream) {
    if (bytes < 16 || blocks < 1 || (reinterpret_cast<uintptr_t>(src) & 15)) return RL_ERR_ARG;
    hipLaunchKernelGGL(read_kernel, dim3(blocks), dim3(256), 0, stream, (const uint4*)src,
                       bytes / 16, sink);
    return rl_launch_status();
}
