// Token selection on the device, one block per row of logits.
//  - argmax: first maximum wins (reference: Daisi.Llogos/Inference/Sampler.cs:234-247).
//  - the sampling pipeline of Daisi.Llogos/Inference/Sampler.cs:26-85: penalties,
//    temperature, top-k, min-p, softmax over the candidates, typical-p, top-p and the
//    draw, which walks the candidates in descending order of their scaled logit (the
//    order in which the reference's top-k collection leaves them, :249-276) and takes
//    the first whose cumulative probability exceeds the uniform number (:334-345).
#include "common.h"

constexpr int kSampleThreads = 1024;

// ---------------------------------------------------------------- argmax
__global__ __launch_bounds__(kSampleThreads) void argmax_kernel(int* __restrict__ out,
                                                                const float* __restrict__ logits, int V) {
    __shared__ float s_val[kSampleThreads / kWave];
    __shared__ int s_idx[kSampleThreads / kWave];
    const float* row = logits + (size_t)blockIdx.x * V;
    float best = -INFINITY;
    int best_i = 0x7fffffff;
    for (int i = threadIdx.x; i < V; i += blockDim.x) {
        const float v = row[i];
        if (v > best || best_i == 0x7fffffff) { best = v; best_i = i; }
    }
#pragma unroll
    for (int o = kWave / 2; o > 0; o >>= 1) {
        const float ov = __shfl_xor(best, o, kWave);
        const int oi = __shfl_xor(best_i, o, kWave);
        if (ov > best || (ov == best && oi < best_i)) { best = ov; best_i = oi; }
    }
    const int lane = threadIdx.x & (kWave - 1), wave = threadIdx.x / kWave;
    if (lane == 0) { s_val[wave] = best; s_idx[wave] = best_i; }
    __syncthreads();
    if (threadIdx.x == 0) {
        for (int wv = 1; wv < kSampleThreads / kWave; ++wv)
            if (s_val[wv] > best || (s_val[wv] == best && s_idx[wv] < best_i)) { best = s_val[wv]; best_i = s_idx[wv]; }
        out[blockIdx.x] = best_i;
    }
}

LLOGOS_EXPORT int llogos_argmax(int* out, const float* logits, int R, int V, hipStream_t stream) {
    if (R <= 0 || V <= 0) return LLOGOS_BAD_ARGUMENT;
    argmax_kernel<<<R, kSampleThreads, 0, stream>>>(out, logits, V);
    return LLOGOS_LAUNCH_CHECK();
}
