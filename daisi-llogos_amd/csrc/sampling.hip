// Token selection on the device, one block per row of logits.
//  - argmax: first maximum wins (reference: Daisi.Llogos/Inference/Sampler.cs:234-247).
//  - the sampling pipeline of Daisi.Llogos/Inference/Sampler.cs:26-85: penalties,
//    temperature, top-k, min-p, softmax over the candidates, typical-p, top-p and the
//    draw, which walks the candidates in descending order of their scaled logit (the
//    order in which the reference's top-k collection leaves them, :249-276) and takes
//    the first whose cumulative probability exceeds the uniform number (:334-345).
#include "common.h"

constexpr int kSampleThreads = 1024;

// f(i, row[i]) for every i < V, the block's threads together, in no particular order: eight
// 16-byte loads in flight per thread where the row allows them (one block reads a row of
// 10^5 values from the L2 in a few microseconds this way; one 4-byte load at a time, each
// waiting for the last, takes thirty).
template <typename F>
__device__ __forceinline__ void for_each_value(const float* __restrict__ row, int V, F f) {
    constexpr int U = 8;
    if ((V & 3) == 0 && ((uintptr_t)row & 15) == 0) {
        const float4* row4 = reinterpret_cast<const float4*>(row);
        const int n4 = V >> 2;
        for (int i0 = threadIdx.x; i0 < n4; i0 += U * blockDim.x) {
            float4 v[U];
#pragma unroll
            for (int j = 0; j < U; ++j) {
                const int i = i0 + j * blockDim.x;
                v[j] = i < n4 ? row4[i] : float4{0.f, 0.f, 0.f, 0.f};
            }
#pragma unroll
            for (int j = 0; j < U; ++j) {
                const int i = i0 + j * blockDim.x;
                if (i < n4) { f(4 * i, v[j].x); f(4 * i + 1, v[j].y); f(4 * i + 2, v[j].z); f(4 * i + 3, v[j].w); }
            }
        }
    } else {
        for (int i0 = threadIdx.x; i0 < V; i0 += U * blockDim.x) {
            float v[U];
#pragma unroll
            for (int j = 0; j < U; ++j) {
                const int i = i0 + j * blockDim.x;
                v[j] = i < V ? row[i] : 0.f;
            }
#pragma unroll
            for (int j = 0; j < U; ++j) {
                const int i = i0 + j * blockDim.x;
                if (i < V) f(i, v[j]);
            }
        }
    }
}

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
constexpr int kMaxBanned = 64;           // ids that a call can ban (a model's stop tokens)
struct PenaltyParams {
    float repetition, frequency, presence, inv_temperature;
    int penalize_newline;
    int n_banned;
    int banned[kMaxBanned];
};

__global__ __launch_bounds__(kSampleThreads) void sample_prepare_kernel(
        float* __restrict__ work, const float* __restrict__ logits, int V,
        const int* __restrict__ hist, const int* __restrict__ hist_len, int hist_stride, PenaltyParams pp) {
    const int r = blockIdx.x;
    const float* row = logits + (size_t)r * V;
    float* w = work + (size_t)r * V;
    const float inv_t = pp.inv_temperature;
    const bool scaled = inv_t != 1.0f;
    for_each_value(row, V, [&](int i, float x) { w[i] = scaled ? x * inv_t : x; });
    __syncthreads();
    // the few tokens that penalties touch are made again from the logits: penalty first, then the scale
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
            float l = row[tok];
            if (pp.repetition != 1.0f)
                for (int c = 0; c < count; ++c) l = l > 0.f ? l / pp.repetition : l * pp.repetition;
            if (pp.frequency != 0.f || pp.presence != 0.f) {
                l -= pp.frequency * (float)count;
                l -= pp.presence;
            }
            w[tok] = scaled ? l * inv_t : l;
        }
        __syncthreads();
    }
    if (threadIdx.x < pp.n_banned) {
        const int tok = pp.banned[threadIdx.x];
        if (tok >= 0 && tok < V) w[tok] = -INFINITY;
    }
}

LLOGOS_EXPORT int llogos_sample_prepare(float* work, const float* logits, int R, int V,
                                        const int* hist, const int* hist_len, int hist_stride,
                                        float repetition, float frequency, float presence, float inv_temperature,
                                        int penalize_newline, const int* banned, int n_banned, hipStream_t stream) {
    if (R <= 0 || V <= 0 || n_banned < 0 || n_banned > kMaxBanned) return LLOGOS_BAD_ARGUMENT;
    PenaltyParams pp{repetition, frequency, presence, inv_temperature, penalize_newline, n_banned, {}};
    for (int i = 0; i < n_banned; ++i) pp.banned[i] = banned[i];
    sample_prepare_kernel<<<R, kSampleThreads, 0, stream>>>(work, logits, V, hist, hist_len, hist_stride, pp);
    return LLOGOS_LAUNCH_CHECK();
}

// ---------------------------------------------------------------- the candidate pipeline
// Order-preserving map of a float onto an unsigned integer (larger float, larger integer).
__device__ __forceinline__ uint32_t ordered_bits(float f) {
    uint32_t u = __float_as_uint(f);
    if (u == 0x80000000u) u = 0;          // -0 equals +0: the lower id decides between them, as between other equals
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
#pragma unroll 8
    for (int i = lo; i < hi; ++i) s += f(i);
    return block_sum(s, red);
}

// Sum of f(row[i]) for i < V over the block, each thread adding the values it visits.
template <typename F>
__device__ float block_sum_values(const float* row, int V, float* red, F f) {
    float s = 0.f;
    for_each_value(row, V, [&](int, float x) { s += f(x); });
    return block_sum(s, red);
}

// First i < n (and i >= from) whose running sum of f exceeds `target` (or reaches it when
// `reach`); -1 when none does.  `scan` holds blockDim.x floats, `found` one int.
template <typename F>
__device__ int first_crossing(int n, int from, float target, bool reach, float* scan, int* found, F f) {
    const int chunk = (n + blockDim.x - 1) / blockDim.x;
    const int lo = min(n, (int)threadIdx.x * chunk), hi = min(n, lo + chunk);
    float s = 0.f;
#pragma unroll 8
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

// Steps 2 to 6 on a list whose first n_list keys are the row's tokens in descending order of
// their scaled logit (lower id first among equals); n of the row's V tokens are candidates
// after top-k.  With n_list < n the list is only the head of that order: the steps that look
// at every candidate (the count of min-p, the sum of the softmax) then walk the row itself,
// and -1 comes back when a cut or the draw lies beyond the head.  `src` holds the scaled
// logits; the candidates' probabilities go to `dst` (indexed by token; src itself or another
// row of V floats).  Returns the token drawn.
__device__ int pipeline_on_sorted(uint64_t* list, int n_list, int n, const float* src, float* dst, int V,
                                  const SampleParams& sp, float u, float* red, float* scan, int* found) {
    const int keep = max(sp.min_keep, 1);
    // 2. min-p on the scaled logits (Sampler.cs:157-174): the kept ones are a prefix
    const float top = src[key_id(list[0])];
    float thr = -INFINITY;
    if (sp.min_p > 0.f && sp.min_p < 1.f && n > keep) {
        thr = top + logf(sp.min_p);
        const float cnt = n <= n_list
            ? block_sum_over(n, red, [&](int i) { return src[key_id(list[i])] >= thr ? 1.f : 0.f; })
            : block_sum_values(src, V, red, [&](float x) { return x >= thr ? 1.f : 0.f; });
        n = max(keep, (int)cnt);
    }
    __syncthreads();

    // 3. softmax over the candidates (Sampler.cs:278-295)
    const float esum = n <= n_list
        ? block_sum_over(n, red, [&](int i) { return expf(src[key_id(list[i])] - top); })
        : block_sum_values(src, V, red, [&](float x) { return x >= thr ? expf(x - top) : 0.f; });
    const float inv = 1.0f / esum;
    __syncthreads();
    const int head = min(n, n_list);
    for (int i = threadIdx.x; i < head; i += blockDim.x) {
        const int t = key_id(list[i]);
        dst[t] = expf(src[t] - top) * inv;
    }
    __syncthreads();

    // 4. typical-p (Sampler.cs:182-230): by |(-log p) - entropy| ascending, keep until the
    //    cumulative probability reaches typical_p, renormalise
    bool resorted = false;
    if (sp.typical_p > 0.f && sp.typical_p < 1.f && n > keep) {
        if (n > n_list) return -1;
        const float ent = block_sum_over(n, red, [&](int i) {
            const float p = dst[key_id(list[i])];
            return p > 0.f ? -p * logf(p) : 0.f; });
        __syncthreads();
        int np2 = 1;
        while (np2 < n) np2 <<= 1;
        for (int i = threadIdx.x; i < np2; i += blockDim.x) {
            uint64_t k = ~(uint64_t)0;
            if (i < n) {
                const int t = key_id(list[i]);
                const float p = dst[t];
                const float lp = p > 0.f ? -logf(p) : 3.4028235e38f;
                k = asc_key(fabsf(lp - ent), t);
            }
            list[i] = k;
        }
        __syncthreads();
        bitonic_sort(list, np2);
        int cut = first_crossing(n, keep - 1, sp.typical_p, true, scan, found,
                                 [&](int i) { return dst[key_id(list[i])]; });
        if (cut >= 0) n = cut + 1;
        const float s = block_sum_over(n, red, [&](int i) { return dst[key_id(list[i])]; });
        __syncthreads();
        if (s > 0.f)
            for (int i = threadIdx.x; i < n; i += blockDim.x) dst[key_id(list[i])] *= 1.0f / s;
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
                if (i < n) { const int t = key_id(list[i]); k = desc_key(dst[t], t); }
                list[i] = k;
            }
            __syncthreads();
            bitonic_sort(list, np2);
        }
        int cut = first_crossing(min(n, n_list), keep - 1, sp.top_p, false, scan, found,
                                 [&](int i) { return dst[key_id(list[i])]; });
        if (cut >= 0) n = cut + 1;
        else if (n > n_list) return -1;
        const float s = block_sum_over(n, red, [&](int i) { return dst[key_id(list[i])]; });
        __syncthreads();
        if (s > 0.f)
            for (int i = threadIdx.x; i < n; i += blockDim.x) dst[key_id(list[i])] *= 1.0f / s;
        __syncthreads();
    }

    // 6. the draw (Sampler.cs:334-345): first candidate whose cumulative probability exceeds u
    int pick = first_crossing(min(n, n_list), 0, u, false, scan, found, [&](int i) { return dst[key_id(list[i])]; });
    if (pick < 0 && n > n_list) return -1;
    return key_id(list[pick >= 0 ? pick : 0]);
}

// The head of the descending order without sorting the row.  A histogram of the distance to
// the largest logit says which bins hold the first `want` tokens; those bins' tokens are
// gathered into LDS (any order) and sorted there by their full keys.  The distance is
// monotonic in the logit, so a bin boundary never separates equal values.  Bins are 1/64 wide
// down to 24 units below the largest and 1/4 wide from there to 151.75 units below; the last
// bin takes everything beyond, whose exp(logit - largest) is exactly 0 in float32, and NaN.
// Returns how many sorted keys `head` then holds (each at least as large as every token left
// out), or 0 when more than kHeadMax would be needed or the largest is not finite.
// *complete: the head holds every token outside the last bin, that is every token whose
// probability is not exactly 0.
constexpr int kHeadMax = 4096, kHeadBins = 2048, kFineBins = 1536;
constexpr float kFinePerUnit = 64.f, kCoarsePerUnit = 4.f;

__device__ __forceinline__ int head_bin(float top, float x) {
    const float d = top - x;
    if (d < (float)kFineBins / kFinePerUnit) return (int)(d * kFinePerUnit);
    const float e = (d - (float)kFineBins / kFinePerUnit) * kCoarsePerUnit;
    return e < (float)(kHeadBins - 1 - kFineBins) ? kFineBins + (int)e : kHeadBins - 1;   // NaN, -inf: the last bin
}

__device__ int sorted_head(uint64_t* head, const float* row, int V, int want, float* red, float* scan, int* bins,
                           int* counter, bool* complete) {
    float m = -INFINITY;
    for_each_value(row, V, [&](int, float x) { m = fmaxf(m, x); });
    const float top = block_max(m, red);
    if (!(top > -INFINITY && top < INFINITY)) return 0;
    for (int i = threadIdx.x; i < kHeadBins; i += blockDim.x) bins[i] = 0;
    if (threadIdx.x == 0) *counter = 0;
    __syncthreads();
    for_each_value(row, V, [&](int, float x) {
        const int b = head_bin(top, x);
        if (b < kHeadBins - 1) atomicAdd(&bins[b], 1);
    });
    __syncthreads();
    // last bin needed: the first whose running count reaches `want`, or the last one in use when
    // there are fewer tokens than that (thread t adds bins 2 t and 2 t + 1, a scan over the
    // threads gives the running counts; the last bin's counter is still 0 and takes the answer)
    static_assert(kHeadBins == 2 * kSampleThreads, "two bins a thread");
    int* run = reinterpret_cast<int*>(scan);
    const int a = bins[2 * threadIdx.x], b = bins[2 * threadIdx.x + 1];
    run[threadIdx.x] = a + b;
    __syncthreads();
    for (int o = 1; o < blockDim.x; o <<= 1) {
        const int add = threadIdx.x >= o ? run[threadIdx.x - o] : 0;
        __syncthreads();
        run[threadIdx.x] += add;
        __syncthreads();
    }
    const int incl = run[threadIdx.x], excl = incl - (a + b);
    const int outside_last = run[blockDim.x - 1];                        // >= 1: the largest itself
    want = min(want, outside_last);
    if (threadIdx.x == 0) bins[kHeadBins - 1] = -1;
    __syncthreads();
    if (excl < want && incl >= want) {
        const bool in_first = excl + a >= want;
        const int total = in_first ? excl + a : incl;
        bins[kHeadBins - 1] = total <= kHeadMax ? 2 * (int)threadIdx.x + (in_first ? 0 : 1) : -1;
    }
    __syncthreads();
    const int last = bins[kHeadBins - 1];
    if (last < 0) return 0;
    for_each_value(row, V, [&](int i, float x) {
        if (head_bin(top, x) <= last) head[atomicAdd(counter, 1)] = desc_key(x, i);
    });
    __syncthreads();
    const int n = *counter;
    *complete = n == outside_last;
    int np2 = 1;
    while (np2 < n) np2 <<= 1;
    for (int i = n + threadIdx.x; i < np2; i += blockDim.x) head[i] = ~(uint64_t)0;
    __syncthreads();
    bitonic_sort(head, np2);
    return n;
}

// One block per row.  `work` holds the penalised, temperature-scaled logits.
//  - try_head: the block tries with the sorted head of the row alone (in LDS; probabilities go
//    to `prob`, the logits stay as they are): all candidates when top-k leaves at most
//    kHeadMax / 2, else the first kHeadMax / 2 of the whole row.
//  - where that cannot decide (see pipeline_on_sorted and sorted_head), or without try_head:
//    with sort_here the block sorts the whole row into `list`, this row's scratch of n_pad
//    keys, and turns `work` into probabilities in place (slow: one compute unit sorts 10^5
//    keys in milliseconds); without sort_here it leaves out[row] = -1 for sample_sorted_kernel.
__global__ __launch_bounds__(kSampleThreads) void sample_pipeline_kernel(
        int* __restrict__ out, float* __restrict__ work_all, float* __restrict__ prob_all, int V,
        uint64_t* __restrict__ list_all, int n_pad, const float* __restrict__ uniforms, SampleParams sp,
        int try_head, int sort_here) {
    __shared__ float red[16];
    __shared__ float scan[kSampleThreads];
    __shared__ int found;
    __shared__ int counter;
    __shared__ int bins[kHeadBins];
    __shared__ uint64_t head[kHeadMax];
    const int r = blockIdx.x;
    float* work = work_all + (size_t)r * V;
    const float u = uniforms[r];
    const int n = (sp.top_k > 0 && sp.top_k < V) ? sp.top_k : V;

    if (try_head && (n <= kHeadMax / 2 || n == V)) {
        bool complete = false;
        const int n_head = sorted_head(head, work, V, min(n, kHeadMax / 2), red, scan, bins, &counter, &complete);
        if (n_head > 0) {
            // a complete head holds every candidate that can be drawn: the rest count for nothing
            const int token = pipeline_on_sorted(head, n_head, complete ? min(n, n_head) : n, work,
                                                 prob_all + (size_t)r * V, V, sp, u, red, scan, &found);
            if (token >= 0) {
                if (threadIdx.x == 0) out[r] = token;
                return;
            }
        }
        __syncthreads();
    }
    if (!sort_here) {
        if (threadIdx.x == 0) out[r] = -1;
        return;
    }
    // 1. all tokens in descending order of their scaled logit, lower id first among equals;
    //    the first k of them are the candidates (Sampler.cs:249-276)
    uint64_t* list = list_all + (size_t)r * n_pad;
    for (int i = threadIdx.x; i < n_pad; i += blockDim.x)
        list[i] = i < V ? desc_key(work[i], i) : ~(uint64_t)0;
    __syncthreads();
    bitonic_sort(list, n_pad);
    const int token = pipeline_on_sorted(list, V, n, work, work, V, sp, u, red, scan, &found);
    if (threadIdx.x == 0) out[r] = token;
}

// ---- whole rows sorted by many blocks: the bitonic network over n_pad keys, cut into chunks
// of kSortChunk keys that a block sorts or merges in LDS, and passes over global memory for the
// exchanges between chunks.  grid (chunks or blocks of pairs, rows); rows that already have
// their token (out[row] >= 0) are left alone.
constexpr int kSortChunk = 8192;

// the t-th pair (i, i + j) of an exchange at distance j: t with a zero bit put in at j's place
__device__ __forceinline__ int pair_low(int t, int j) { return ((t & ~(j - 1)) << 1) | (t & (j - 1)); }   // j: a power of two

__device__ __forceinline__ void exchange(uint64_t* d, int i, int p, bool up) {
    const uint64_t a = d[i], b = d[p];
    if ((a > b) == up) { d[i] = b; d[p] = a; }
}

// stage 0: makes the chunk's keys from the row and sorts it (network stages 2 .. chunk);
// stage k > chunk: the exchanges at distances chunk / 2 .. 1 of network stage k.
__global__ __launch_bounds__(kSampleThreads) void sort_chunk_kernel(
        uint64_t* __restrict__ list_all, const float* __restrict__ work_all, const int* __restrict__ out,
        int V, int n_pad, int stage) {
    __shared__ uint64_t d[kSortChunk];
    const int r = blockIdx.y;
    if (out[r] >= 0) return;
    const int m = min(kSortChunk, n_pad), base = blockIdx.x * m;
    uint64_t* list = list_all + (size_t)r * n_pad + base;
    if (stage == 0) {
        const float* work = work_all + (size_t)r * V;
        for (int i = threadIdx.x; i < m; i += blockDim.x)
            d[i] = base + i < V ? desc_key(work[base + i], base + i) : ~(uint64_t)0;
    } else {
        for (int i = threadIdx.x; i < m; i += blockDim.x) d[i] = list[i];
    }
    __syncthreads();
    for (int k = stage == 0 ? 2 : stage; k <= (stage == 0 ? m : stage); k <<= 1)
        for (int j = min(k, m) >> 1; j > 0; j >>= 1) {
            for (int t = threadIdx.x; t < m / 2; t += blockDim.x) {
                const int i = pair_low(t, j);
                exchange(d, i, i + j, ((base + i) & k) == 0);
            }
            __syncthreads();
        }
    for (int i = threadIdx.x; i < m; i += blockDim.x) list[i] = d[i];
}

// the exchanges at distance j >= chunk of network stage k
__global__ __launch_bounds__(kSampleThreads) void sort_exchange_kernel(
        uint64_t* __restrict__ list_all, const int* __restrict__ out, int n_pad, int k, int j) {
    const int r = blockIdx.y;
    if (out[r] >= 0) return;
    const int t = blockIdx.x * blockDim.x + threadIdx.x;
    if (t >= n_pad / 2) return;
    const int i = pair_low(t, j);
    exchange(list_all + (size_t)r * n_pad, i, i + j, (i & k) == 0);
}

// steps 2 to 6 for the rows sorted so; `work` becomes probabilities in place
__global__ __launch_bounds__(kSampleThreads) void sample_sorted_kernel(
        int* __restrict__ out, float* __restrict__ work_all, int V, uint64_t* __restrict__ list_all, int n_pad,
        const float* __restrict__ uniforms, SampleParams sp) {
    __shared__ float red[16];
    __shared__ float scan[kSampleThreads];
    __shared__ int found;
    const int r = blockIdx.x;
    if (out[r] >= 0) return;
    float* work = work_all + (size_t)r * V;
    const int n = (sp.top_k > 0 && sp.top_k < V) ? sp.top_k : V;
    const int token = pipeline_on_sorted(list_all + (size_t)r * n_pad, V, n, work, work, V, sp, uniforms[r], red, scan,
                                         &found);
    if (threadIdx.x == 0) out[r] = token;
}

// mode: 0 = every row sorted whole by its own block (the plain form); 1 = the head of the order
// first, rows it cannot decide sorted whole by many blocks; 2 = every row sorted by many blocks.
// In mode 1 the kernels of the many-block sort are launched only where an ordinary row can need
// them (no top-k, or one beyond the head's size); a row whose head is undecided although top-k
// is small (thousands of tokens within 1/64 of the k-th) is sorted by its own block.
LLOGOS_EXPORT int llogos_sample_pipeline(int* out, float* work, float* prob, int R, int V, void* list, int n_pad,
                                         const float* uniforms, int top_k, float top_p, float min_p,
                                         float typical_p, int min_keep, int mode, hipStream_t stream) {
    if (R <= 0 || V <= 0 || n_pad < V || (n_pad & (n_pad - 1)) || mode < 0 || mode > 2 || (mode == 1 && prob == nullptr))
        return LLOGOS_BAD_ARGUMENT;
    SampleParams sp{top_k, top_p, min_p, typical_p, min_keep};
    const int n = (top_k > 0 && top_k < V) ? top_k : V;
    const bool head_fits = n <= kHeadMax / 2 || n == V;
    const bool many_blocks = mode == 2 || (mode == 1 && (n == V || !head_fits));
    sample_pipeline_kernel<<<R, kSampleThreads, 0, stream>>>(out, work, prob, V, (uint64_t*)list, n_pad, uniforms, sp,
                                                             mode == 1, !many_blocks);
    if (many_blocks) {
        uint64_t* keys = (uint64_t*)list;
        const int m = n_pad < kSortChunk ? n_pad : kSortChunk;
        const dim3 chunks(n_pad / m, R), pairs((n_pad / 2 + kSampleThreads - 1) / kSampleThreads, R);
        sort_chunk_kernel<<<chunks, kSampleThreads, 0, stream>>>(keys, work, out, V, n_pad, 0);
        for (int k = 2 * m; k <= n_pad; k <<= 1) {
            for (int j = k >> 1; j >= m; j >>= 1)
                sort_exchange_kernel<<<pairs, kSampleThreads, 0, stream>>>(keys, out, n_pad, k, j);
            sort_chunk_kernel<<<chunks, kSampleThreads, 0, stream>>>(keys, work, out, V, n_pad, k);
        }
        sample_sorted_kernel<<<R, kSampleThreads, 0, stream>>>(out, work, V, keys, n_pad, uniforms, sp);
    }
    return LLOGOS_LAUNCH_CHECK();
}
