// Attention over the paged cache for any step shape (whole prompts, single tokens, a
// mixture), any head size up to 512 and any grouping, float or bfloat16 storage with
// all arithmetic in 32-bit floats.  One block per (token, query head); keys are visited
// in tiles of 256 that start at key 0, with a running maximum and sum, so the order of
// the additions for a query depends on its position alone and not on how the tokens
// were cut into steps or on what else is in the batch.
// (reference: gated_attention / batched_gated_attention,
//  Daisi.Llogos.Cuda/kernels/composite_ops.cu:275-387, 396-512: kv head = head / group,
//  scale after the dot, tiles of 256 keys, running max and sum; the sigmoid gate of that
//  kernel is identically 1 for this architecture and is left out.)
#include "common.h"

constexpr int kTileKeys = 256;
constexpr int kMaxHeadDimGeneric = 512;

template <typename T>
__global__ __launch_bounds__(256) void attn_generic_kernel(
        T* __restrict__ out, const T* __restrict__ q, int q_stride,
        const T* __restrict__ k_pool, const T* __restrict__ v_pool, PagedKV cache,
        const int* __restrict__ tok_seq, const int* __restrict__ tok_pos,
        int n_heads, int group, int head_dim, float scale, int window, int sinks) {
    extern __shared__ float smem[];
    float* qf = smem;                    // [head_dim]
    float* p_lds = smem + head_dim;      // [kTileKeys]
    float* red = p_lds + kTileKeys;      // [16]
    const int t = blockIdx.x, h = blockIdx.y, tid = threadIdx.x;
    const int seq = tok_seq[t], pos = tok_pos[t];
    const int kvh = h / group;

    const T* qrow = q + (size_t)t * q_stride + (size_t)h * head_dim;
    for (int d = tid; d < head_dim; d += blockDim.x) qf[d] = load_f32(qrow + d);
    __syncthreads();

    float m_run = -INFINITY, l_run = 0.f;
    float acc[kMaxHeadDimGeneric / 256] = {};

    for (int j0 = 0; j0 <= pos; j0 += kTileKeys) {
        if (window > 0 && j0 >= sinks && j0 + kTileKeys - 1 <= pos - window) continue;   // nothing visible
        const int j = j0 + tid;
        const bool vis = key_visible(pos, j, window, sinks);
        float s = -INFINITY;
        if (vis) {
            const T* kpage = k_pool + paged_base(cache, seq, kvh, j);
            float dot = 0.f;
            for (int d = 0; d < head_dim; ++d)
                dot = fmaf(qf[d], load_f32(kpage + page_key_offset(j % kPageTokens, d, head_dim)), dot);
            s = dot * scale;
        }
        const float tile_max = block_max(s, red);
        if (tile_max == -INFINITY) continue;
        const float m_new = fmaxf(m_run, tile_max);
        const float p = vis ? expf(s - m_new) : 0.f;
        __syncthreads();
        p_lds[tid] = p;
        const float tile_sum = block_sum(p, red);   // its barriers also publish p_lds
        const float corr = (m_run == -INFINITY) ? 0.f : expf(m_run - m_new);
        const int n_keys = min(kTileKeys, pos - j0 + 1);
#pragma unroll
        for (int r = 0; r < kMaxHeadDimGeneric / 256; ++r) {
            const int d = tid + r * 256;
            if (d < head_dim) {
                float a = acc[r] * corr;
                for (int jj = 0; jj < n_keys; ++jj) {
                    const float pj = p_lds[jj];
                    if (pj != 0.f)
                        a = fmaf(pj, load_f32(v_pool + paged_base(cache, seq, kvh, j0 + jj)
                                              + page_value_offset((j0 + jj) % kPageTokens, d)), a);
                }
                acc[r] = a;
            }
        }
        l_run = l_run * corr + tile_sum;
        m_run = m_new;
    }
    const float inv = l_run > 0.f ? 1.0f / l_run : 0.f;
    T* orow = out + ((size_t)t * n_heads + h) * head_dim;
#pragma unroll
    for (int r = 0; r < kMaxHeadDimGeneric / 256; ++r) {
        const int d = tid + r * 256;
        if (d < head_dim) store_f32(orow + d, acc[r] * inv);
    }
}

LLOGOS_EXPORT int llogos_attention_generic(void* out, const void* q, int dtype, int q_stride,
                                           const void* k_pool, const void* v_pool,
                                           const int* table, int table_stride,
                                           const int* tok_seq, const int* tok_pos,
                                           int T, int n_heads, int n_kv_heads, int head_dim,
                                           float scale, int window, int sinks, hipStream_t stream) {
    if (T <= 0 || n_heads <= 0 || n_kv_heads <= 0 || n_heads % n_kv_heads != 0) return LLOGOS_BAD_ARGUMENT;
    if (head_dim <= 0 || head_dim > kMaxHeadDimGeneric || window < 0 || sinks < 0) return LLOGOS_BAD_ARGUMENT;
    PagedKV cache{table, table_stride, n_kv_heads, head_dim};
    dim3 grid(T, n_heads);
    const size_t smem = (size_t)(head_dim + kTileKeys + 16) * sizeof(float);
    const int group = n_heads / n_kv_heads;
    if (dtype == DT_F32)
        attn_generic_kernel<float><<<grid, 256, smem, stream>>>(
            (float*)out, (const float*)q, q_stride, (const float*)k_pool, (const float*)v_pool, cache,
            tok_seq, tok_pos, n_heads, group, head_dim, scale, window, sinks);
    else if (dtype == DT_BF16)
        attn_generic_kernel<bf16_t><<<grid, 256, smem, stream>>>(
            (bf16_t*)out, (const bf16_t*)q, q_stride, (const bf16_t*)k_pool, (const bf16_t*)v_pool, cache,
            tok_seq, tok_pos, n_heads, group, head_dim, scale, window, sinks);
    else
        return LLOGOS_BAD_ARGUMENT;
    return LLOGOS_LAUNCH_CHECK();
}
