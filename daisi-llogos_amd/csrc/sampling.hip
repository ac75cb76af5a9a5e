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
    if ((V & 3) == 0 && ((uintptr_t)row & 15) == 0) {
        // four values per load, several loads in flight; a thread visits its indices in
        // ascending order, so the strict comparison keeps the first maximum
        const float4* row4 = reinterpret_cast<const float4*>(row);
        const int n4 = V >> 2;
#pragma unroll 4
        for (int i = threadIdx.x; i < n4; i += blockDim.x) {
            const float4 v = row4[i];
            const float e[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
            for (int j = 0; j < 4; ++j)
                if (e[j] > best || best_i == 0x7fffffff) { best = e[j]; best_i = 4 * i + j; }
        }
    } else {
        for (int i = threadIdx.x; i < V; i += blockDim.x) {
            const float v = row[i];
            if (v > best || best_i == 0x7fffffff) { best = v; best_i = i; }
        }
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

// ---------------------------------------------------------------- penalties and temperature
// work[r, :] = logits[r, :] with the repetition / frequency / presence penalties of the
// last `hist_len[r]` tokens applied (Sampler.cs:89-143: per occurrence l/p or l*p by sign,
// then - frequency * count - presence once per distinct token; tokens 10 and 13 are spared
// unless penalize_newline), the given ids set to -inf (PreventEOS, :49-53), then times
// 1 / temperature (:60-62).
struct PenaltyParams {
    float repetition, frequency, presence, inv_temperature;
    int penalize_newline;
    int n_banned;
    int banned[8];
};

__global__ __launch_bounds__(kSampleThreads) void sample_prepare_kernel(
        float* __restrict__ work, const float* __restrict__ logits, int V,
        const int* __restrict__ hist, const int* __restrict__ hist_len, int hist_stride, PenaltyParams pp) {
    const int r = blockIdx.x;
    const float* row = logits + (size_t)r * V;
    float* w = work + (size_t)r * V;
    for (int i = threadIdx.x; i < V; i += blockDim.x) w[i] = row[i];
    __syncthreads();
    const bool penalties = pp.repetition != 1.0f || pp.frequency != 0.f || pp.presence != 0.f;
    if (penalties && hist) {
        const int* h = hist + (size_t)r * hist_stride;
        const int n = hist_len[r];
        // one thread per window position; the first occurrence of a token does the work
        for (int i = threadIdx.x; i < n; i += blockDim.x) {
            const int tok = h[i];
            if (tok < 0 || tok >= V) continue;
            if (!pp.penalize_newline && (tok == 10 || tok == 13)) continue;
            bool first = true;
            for (int j = 0; j < i; ++j) if (h[j] == tok) { first = false; break; }
            if (!first) continue;
            int count = 0;
            for (int j = i; j < n; ++j) count += (h[j] == tok);
            float l = w[tok];
            if (pp.repetition != 1.0f)
                for (int c = 0; c < count; ++c) l = l > 0.f ? l / pp.repetition : l * pp.repetition;
            if (pp.frequency != 0.f || pp.presence != 0.f) {
                l -= pp.frequency * (float)count;
                l -= pp.presence;
            }
            w[tok] = l;
        }
        __syncthreads();
    }
    if (threadIdx.x < pp.n_banned) {
        const int tok = pp.banned[threadIdx.x];
        if (tok >= 0 && tok < V) w[tok] = -INFINITY;
    }
    __syncthreads();
    if (pp.inv_temperature != 1.0f)
        for (int i = threadIdx.x; i < V; i += blockDim.x) w[i] *= pp.inv_temperature;
}

LLOGOS_EXPORT int llogos_sample_prepare(float* work, const float* logits, int R, int V,
                                        const int* hist, const int* hist_len, int hist_stride,
                                        float repetition, float frequency, float presence, float inv_temperature,
                                        int penalize_newline, const int* banned, int n_banned, hipStream_t stream) {
    if (R <= 0 || V <= 0 || n_banned < 0 || n_banned > 8) return LLOGOS_BAD_ARGUMENT;
    PenaltyParams pp{repetition, frequency, presence, inv_temperature, penalize_newline, n_banned, {}};
    for (int i = 0; i < n_banned; ++i) pp.banned[i] = banned[i];
    sample_prepare_kernel<<<R, kSampleThreads, 0, stream>>>(work, logits, V, hist, hist_len, hist_stride, pp);
    return LLOGOS_LAUNCH_CHECK();
}

// ---------------------------------------------------------------- the candidate pipeline
// Order-preserving map of a float onto an unsigned integer (larger float, larger integer).
__device__ __forceinline__ uint32_t ordered_bits(float f) {
    const uint32_t u = __float_as_uint(f);
    return (u & 0x80000000u) ? ~u : (u | 0x80000000u);
}
// ascending sort of these puts the larger value first and, among equals, the lower id
__device__ __forceinline__ uint64_t desc_key(float v, int id) {
    return ((uint64_t)(~ordered_bits(v)) << 32) | (uint32_t)id;
}
__device__ __forceinline__ uint64_t asc_key(float v, int id) {
    return ((uint64_t)ordered_bits(v) << 32) | (uint32_t)id;
}
__device__ __forceinline__ int key_id(uint64_t k) { return (int)(uint32_t)k; }

// In-place ascending bitonic sort of n_pad (a power of two) keys by one block.
__device__ void bitonic_sort(uint64_t* d, int n_pad) {
    for (int k = 2; k <= n_pad; k <<= 1) {
        for (int j = k >> 1; j > 0; j >>= 1) {
            for (int i = threadIdx.x; i < n_pad; i += blockDim.x) {
                const int p = i ^ j;
                if (p > i) {
                    const uint64_t a = d[i], b = d[p];
                    const bool up = (i & k) == 0;
                    if ((a > b) == up) { d[i] = b; d[p] = a; }
                }
            }
            __syncthreads();
        }
    }
}

// Sum of f(i) for i < n over the block; f is evaluated in chunks of consecutive i per thread.
template <typename F>
__device__ float block_sum_over(int n, float* red, F f) {
    const int chunk = (n + blockDim.x - 1) / blockDim.x;
    const int lo = min(n, (int)threadIdx.x * chunk), hi = min(n, lo + chunk);
    float s = 0.f;
    for (int i = lo; i < hi; ++i) s += f(i);
    return block_sum(s, red);
}

// First i < n (and i >= from) whose running sum of f exceeds `target` (or reaches it when
// `reach`); -1 when none does.  `scan` holds blockDim.x floats, `found` one int.
template <typename F>
__device__ int first_crossing(int n, int from, float target, bool reach, float* scan, int* found, F f) {
    const int chunk = (n + blockDim.x - 1) / blockDim.x;
    const int lo = min(n, (int)threadIdx.x * chunk), hi = min(n, lo + chunk);
    float s = 0.f;
    for (int i = lo; i < hi; ++i) s += f(i);
    __syncthreads();
    scan[threadIdx.x] = s;
    if (threadIdx.x == 0) *found = 0x7fffffff;
    __syncthreads();
    for (int o = 1; o < blockDim.x; o <<= 1) {          // inclusive scan over the threads' sums
        float add = threadIdx.x >= o ? scan[threadIdx.x - o] : 0.f;
        __syncthreads();
        scan[threadIdx.x] += add;
        __syncthreads();
    }
    float run = scan[threadIdx.x] - s;                   // sum before this thread's chunk
    for (int i = lo; i < hi; ++i) {
        run += f(i);
        const bool hit = reach ? run >= target : run > target;
        if (hit && i >= from) { atomicMin(found, i); break; }
    }
    __syncthreads();
    const int first = *found;
    return first == 0x7fffffff ? -1 : first;
}

struct SampleParams {
    int top_k;          // 0 = off
    float top_p;        // >= 1 = off
    float min_p;        // 0 = off
    float typical_p;    // >= 1 = off
    int min_keep;
};

// One block per row.  `work` holds the penalised, temperature-scaled logits and is turned
// into probabilities of the candidates; `list` is this row's scratch of n_pad keys.
__global__ __launch_bounds__(kSampleThreads) void sample_pipeline_kernel(
        int* __restrict__ out, float* __restrict__ work_all, int V, uint64_t* __restrict__ list_all,
        int n_pad, const float* __restrict__ uniforms, SampleParams sp) {
    __shared__ float red[16];
    __shared__ float scan[kSampleThreads];
    __shared__ int found;
    const int r = blockIdx.x;
    float* work = work_all + (size_t)r * V;
    uint64_t* list = list_all + (size_t)r * n_pad;

    // 1. all tokens in descending order of their scaled logit, lower id first among equals;
    //    the first k of them are the candidates (Sampler.cs:249-276)
    for (int i = threadIdx.x; i < n_pad; i += blockDim.x)
        list[i] = i < V ? desc_key(work[i], i) : ~(uint64_t)0;
    __syncthreads();
    bitonic_sort(list, n_pad);
    int n = (sp.top_k > 0 && sp.top_k < V) ? sp.top_k : V;
    const int keep = max(sp.min_keep, 1);

    // 2. min-p on the scaled logits (Sampler.cs:157-174): the kept ones are a prefix
    const float top = work[key_id(list[0])];
    if (sp.min_p > 0.f && sp.min_p < 1.f && n > keep) {
        const float thr = top + logf(sp.min_p);
        const float cnt = block_sum_over(n, red, [&](int i) { return work[key_id(list[i])] >= thr ? 1.f : 0.f; });
        n = max(keep, (int)cnt);
    }
    __syncthreads();

    // 3. softmax over the candidates (Sampler.cs:278-295)
    const float esum = block_sum_over(n, red, [&](int i) { return expf(work[key_id(list[i])] - top); });
    const float inv = 1.0f / esum;
    __syncthreads();
    for (int i = threadIdx.x; i < n; i += blockDim.x) {
        const int t = key_id(list[i]);
        work[t] = expf(work[t] - top) * inv;
    }
    __syncthreads();

    // 4. typical-p (Sampler.cs:182-230): by |(-log p) - entropy| ascending, keep until the
    //    cumulative probability reaches typical_p, renormalise
    bool resorted = false;
    if (sp.typical_p > 0.f && sp.typical_p < 1.f && n > keep) {
        const float ent = block_sum_over(n, red, [&](int i) {
            const float p = work[key_id(list[i])];
            return p > 0.f ? -p * logf(p) : 0.f; });
        __syncthreads();
        int np2 = 1;
        while (np2 < n) np2 <<= 1;
        for (int i = threadIdx.x; i < np2; i += blockDim.x) {
            uint64_t k = ~(uint64_t)0;
            if (i < n) {
                const int t = key_id(list[i]);
                const float p = work[t];
                const float lp = p > 0.f ? -logf(p) : 3.4028235e38f;
                k = asc_key(fabsf(lp - ent), t);
            }
            list[i] = k;
        }
        __syncthreads();
        bitonic_sort(list, np2);
        int cut = first_crossing(n, keep - 1, sp.typical_p, true, scan, &found,
                                 [&](int i) { return work[key_id(list[i])]; });
        if (cut >= 0) n = cut + 1;
        const float s = block_sum_over(n, red, [&](int i) { return work[key_id(list[i])]; });
        __syncthreads();
        if (s > 0.f)
            for (int i = threadIdx.x; i < n; i += blockDim.x) work[key_id(list[i])] *= 1.0f / s;
        __syncthreads();
        resorted = true;
    }

    // 5. top-p (Sampler.cs:297-332): by probability descending, cut after the first whose
    //    cumulative probability exceeds p, renormalise
    if (sp.top_p > 0.f && sp.top_p < 1.f) {
        if (resorted) {
            int np2 = 1;
            while (np2 < n) np2 <<= 1;
            for (int i = threadIdx.x; i < np2; i += blockDim.x) {
                uint64_t k = ~(uint64_t)0;
                if (i < n) { const int t = key_id(list[i]); k = desc_key(work[t], t); }
                list[i] = k;
            }
            __syncthreads();
            bitonic_sort(list, np2);
        }
        int cut = first_crossing(n, keep - 1, sp.top_p, false, scan, &found,
                                 [&](int i) { return work[key_id(list[i])]; });
        if (cut >= 0) n = cut + 1;
        const float s = block_sum_over(n, red, [&](int i) { return work[key_id(list[i])]; });
        __syncthreads();
        if (s > 0.f)
            for (int i = threadIdx.x; i < n; i += blockDim.x) work[key_id(list[i])] *= 1.0f / s;
        __syncthreads();
    }

    // 6. the draw (Sampler.cs:334-345): first candidate whose cumulative probability exceeds u
    const float u = uniforms[r];
    int pick = first_crossing(n, 0, u, false, scan, &found, [&](int i) { return work[key_id(list[i])]; });
    if (threadIdx.x == 0) out[r] = key_id(list[pick >= 0 ? pick : 0]);
}

LLOGOS_EXPORT int llogos_sample_pipeline(int* out, float* work, int R, int V, void* list, int n_pad,
                                         const float* uniforms, int top_k, float top_p, float min_p,
                                         float typical_p, int min_keep, hipStream_t stream) {
    if (R <= 0 || V <= 0 || n_pad < V || (n_pad & (n_pad - 1))) return LLOGOS_BAD_ARGUMENT;
    SampleParams sp{top_k, top_p, min_p, typical_p, min_keep};
    sample_pipeline_kernel<<<R, kSampleThreads, 0, stream>>>(out, work, V, (uint64_t*)list, n_pad, uniforms, sp);
    return LLOGOS_LAUNCH_CHECK();
}
