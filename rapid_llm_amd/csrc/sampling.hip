// Token selection from float32 logits.  Greedy rows take the arg-max (the lowest index
// among equal maxima, as torch.argmax does on one device).
#include "common.h"

__global__ void argmax_kernel(const float* __restrict__ logits, int* __restrict__ out, int vocab) {
    __shared__ float best_v[1024 / RL_WAVE];
    __shared__ int best_i[1024 / RL_WAVE];
    const float* row = logits + (size_t)blockIdx.x * vocab;
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

extern "C" int rl_argmax(const float* logits, int* out, int rows, int vocab, hipStream_t stream) {
    if (rows <= 0) return RL_OK;
    if (vocab < 1) return RL_ERR_ARG;
    hipLaunchKernelGGL(argmax_kernel, dim3(rows), dim3(1024), 0, stream, logits, out, vocab);
    return rl_launch_status();
}
