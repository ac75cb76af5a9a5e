// Row-wise kernels around the matrix products: embedding gather, RMSNorm with the
// residual sum fused in, the rotary table, the fused per-head norm + rotation + cache
// write, and SwiGLU.  All arithmetic is in 32-bit floats (angles in double); storage
// is float or bfloat16.
#include "common.h"

// what the host side checks its own page size against when it loads the library
LLOGOS_EXPORT int llogos_page_tokens(void) { return kPageTokens; }
// where element (token, d) of a kv head's part of a page lies (for checks of the host's copy of the rule)
LLOGOS_EXPORT int llogos_page_key_offset(int token, int d, int head_dim) { return page_key_offset(token, d, head_dim); }
LLOGOS_EXPORT int llogos_page_value_offset(int token, int d) { return page_value_offset(token, d); }
LLOGOS_EXPORT int llogos_wave_size(void) { return kWave; }

// ---------------------------------------------------------------- embedding
// out[t, :] = table[ids[t], :] as float.  One block per token.
// (reference: Daisi.Llogos.Cuda/kernels/elementwise.cu:402-457, one row per call)
template <typename T>
__global__ void embed_kernel(float* __restrict__ out, const T* __restrict__ table,
                             const int* __restrict__ ids, int H, float scale) {
    const int t = blockIdx.x;
    const T* row = table + (size_t)ids[t] * H;
    float* o = out + (size_t)t * H;
    if (scale == 1.0f) {
        for (int i = threadIdx.x; i < H; i += blockDim.x) o[i] = load_f32(row + i);
    } else {
        for (int i = threadIdx.x; i < H; i += blockDim.x) o[i] = load_f32(row + i) * scale;
    }
}

// out[t, :] = table[ids[t], :] * scale (scale 1: a row copy)
LLOGOS_EXPORT int llogos_embed(float* out, const void* table, int table_dtype, const int* ids,
                               int T, int H, float scale, hipStream_t stream) {
    if (T <= 0 || H <= 0) return LLOGOS_BAD_ARGUMENT;
    if (table_dtype == DT_F32)
        embed_kernel<float><<<T, 256, 0, stream>>>(out, (const float*)table, ids, H, scale);
    else if (table_dtype == DT_BF16)
        embed_kernel<bf16_t><<<T, 256, 0, stream>>>(out, (const bf16_t*)table, ids, H, scale);
    else
        return LLOGOS_BAD_ARGUMENT;
    return LLOGOS_LAUNCH_CHECK();
}

// x = x * scale, then, with cap > 0, x = cap * tanh(x / cap): scaled and soft-capped logits
__global__ void scale_softcap_kernel(float* __restrict__ x, long long n, float scale, float cap) {
    const long long i = (long long)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= n) return;
    float v = x[i] * scale;
    if (cap > 0.f) v = cap * tanhf(v / cap);
    x[i] = v;
}

LLOGOS_EXPORT int llogos_scale_softcap(float* x, long long n, float scale, float cap, hipStream_t stream) {
    if (n <= 0 || cap < 0.f) return LLOGOS_BAD_ARGUMENT;
    scale_softcap_kernel<<<(unsigned)((n + 255) / 256), 256, 0, stream>>>(x, n, scale, cap);
    return LLOGOS_LAUNCH_CHECK();
}

// dst[i] = src[rows[i]] for int32 values: a step's token ids picked from the ids another
// step's sampler left on the device.  rows outside 0..n_src-1 give 0.
__global__ void gather_i32_kernel(int* __restrict__ dst, const int* __restrict__ src,
                                  const int* __restrict__ rows, int n, int n_src) {
    const int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= n) return;
    const int r = rows[i];
    dst[i] = (r >= 0 && r < n_src) ? src[r] : 0;
}

LLOGOS_EXPORT int llogos_gather_i32(int* dst, const int* src, const int* rows, int n, int n_src,
                                    hipStream_t stream) {
    if (n <= 0 || n_src <= 0) return LLOGOS_BAD_ARGUMENT;
    gather_i32_kernel<<<(n + 255) / 256, 256, 0, stream>>>(dst, src, rows, n, n_src);
    return LLOGOS_LAUNCH_CHECK();
}

// ---------------------------------------------------------------- RMSNorm (+ residual add)
// For output row r (source row s = rows ? rows[r] : r):
//   v = x[s] + delta[s]   (delta optional; written back to x when write_back)
//   out[r] = v * rsqrt(mean(v^2) + eps) * w
// The residual stream x stays in float; out has the matrix products' input type.
// (reference: rms_norm / add_rms_norm_residual, Daisi.Llogos.Cuda/kernels/elementwise.cu:18-171,
//  668-733; eps inside the root, weight multiplies as it is.)
// sum of the `parts` partial products of element i (parts lie part_stride elements apart),
// added in ascending order
template <typename TD>
__device__ __forceinline__ float sum_parts(const TD* p, size_t i, int parts, size_t part_stride) {
    float v = load_f32(p + i);
    for (int q = 1; q < parts; ++q) v += load_f32(p + q * part_stride + i);
    return v;
}

template <typename TO, typename TD>
__global__ void rmsnorm_kernel(TO* __restrict__ out, float* __restrict__ x, const TD* __restrict__ delta,
                               int parts, size_t part_stride,
                               const int* __restrict__ rows, const float* __restrict__ w,
                               float eps, int H, int write_back) {
    __shared__ float red[16];
    const int r = blockIdx.x;
    const size_t s = rows ? (size_t)rows[r] : (size_t)r;
    float* xr = x + s * H;
    const TD* dr = delta ? delta + s * H : nullptr;
    float ss = 0.f;
    for (int i = threadIdx.x; i < H; i += blockDim.x) {
        float v = xr[i];
        if (dr) {
            v += sum_parts(dr, i, parts, part_stride);
            if (write_back) xr[i] = v;
        }
        ss += v * v;
    }
    const float total = block_sum(ss, red);
    const float inv = 1.0f / sqrtf(total / (float)H + eps);
    TO* o = out + (size_t)r * H;
    for (int i = threadIdx.x; i < H; i += blockDim.x) {
        float v = xr[i];
        if (dr && !write_back) v += sum_parts(dr, i, parts, part_stride);
        store_f32(o + i, v * inv * w[i]);
    }
}

// The same with the row held in registers: each thread owns ITEMS groups of 4 consecutive
// values, all loads (the row and every part of delta) are issued before the first sum, and
// the row is read from memory once.  For H % 4 == 0 and H <= 4 * ITEMS * blockDim.
__device__ __forceinline__ float4 load4_f32(const float* p) { return *reinterpret_cast<const float4*>(p); }
__device__ __forceinline__ float4 load4_f32(const bf16_t* p) {
    const uint2 u = *reinterpret_cast<const uint2*>(p);
    return make_float4(__uint_as_float(u.x << 16), __uint_as_float(u.x & 0xffff0000u),
                       __uint_as_float(u.y << 16), __uint_as_float(u.y & 0xffff0000u));
}
__device__ __forceinline__ void store4_f32(float* p, float4 v) { *reinterpret_cast<float4*>(p) = v; }
__device__ __forceinline__ void store4_f32(bf16_t* p, float4 v) {
    uint2 u;
    u.x = (uint32_t)f32_to_bf16(v.x) | ((uint32_t)f32_to_bf16(v.y) << 16);
    u.y = (uint32_t)f32_to_bf16(v.z) | ((uint32_t)f32_to_bf16(v.w) << 16);
    *reinterpret_cast<uint2*>(p) = u;
}

constexpr int kMaxNormParts = 8;

template <typename TO, typename TD, int ITEMS, int MAXP>
__global__ __launch_bounds__(1024) void rmsnorm_vec_kernel(TO* __restrict__ out, float* __restrict__ x, const TD* __restrict__ delta,
                                   int parts, size_t part_stride,
                                   const int* __restrict__ rows, const float* __restrict__ w,
                                   float eps, int H, int write_back) {
    __shared__ float red[16];
    const int r = blockIdx.x;
    const size_t s = rows ? (size_t)rows[r] : (size_t)r;
    float* xr = x + s * H;
    const TD* dr = delta ? delta + s * H : nullptr;
    float4 v[ITEMS], wv[ITEMS];
    float4 dv[ITEMS][MAXP];
#pragma unroll
    for (int it = 0; it < ITEMS; ++it) {
        const int i = 4 * (it * blockDim.x + threadIdx.x);
        const bool ok = i < H;
        v[it] = ok ? load4_f32(xr + i) : make_float4(0.f, 0.f, 0.f, 0.f);
        wv[it] = ok ? load4_f32(w + i) : make_float4(0.f, 0.f, 0.f, 0.f);
#pragma unroll
        for (int q = 0; q < MAXP; ++q)
            dv[it][q] = (ok && dr && q < parts) ? load4_f32(dr + q * part_stride + i) : make_float4(0.f, 0.f, 0.f, 0.f);
    }
    float ss = 0.f;
#pragma unroll
    for (int it = 0; it < ITEMS; ++it) {
        if (dr) {
            float4 d = dv[it][0];
#pragma unroll
            for (int q = 1; q < MAXP; ++q) {                // ascending order, as sum_parts
                d.x += dv[it][q].x; d.y += dv[it][q].y; d.z += dv[it][q].z; d.w += dv[it][q].w;
            }
            v[it].x += d.x; v[it].y += d.y; v[it].z += d.z; v[it].w += d.w;
            const int i = 4 * (it * blockDim.x + threadIdx.x);
            if (write_back && i < H) store4_f32(xr + i, v[it]);
        }
        ss += v[it].x * v[it].x + v[it].y * v[it].y + v[it].z * v[it].z + v[it].w * v[it].w;
    }
    const float total = block_sum(ss, red);
    const float inv = 1.0f / sqrtf(total / (float)H + eps);
    TO* o = out + (size_t)r * H;
#pragma unroll
    for (int it = 0; it < ITEMS; ++it) {
        const int i = 4 * (it * blockDim.x + threadIdx.x);
        if (i < H)
            store4_f32(o + i, make_float4(v[it].x * inv * wv[it].x, v[it].y * inv * wv[it].y,
                                          v[it].z * inv * wv[it].z, v[it].w * inv * wv[it].w));
    }
}

// delta: `parts` partial products [parts][T][H] (part_stride elements apart) that are summed
// on the way; parts = 1 for a plain delta.
LLOGOS_EXPORT int llogos_rmsnorm(void* out, int out_dtype, float* x, const void* delta, int delta_dtype,
                                 int parts, long long part_stride,
                                 const int* rows, const float* w, float eps, int R, int H,
                                 int write_back, hipStream_t stream) {
    if (R <= 0 || H <= 0 || parts < 1) return LLOGOS_BAD_ARGUMENT;
    const bool aligned = (H % 4 == 0) && ((uintptr_t)x % 16 == 0) && ((uintptr_t)w % 16 == 0) &&
                         ((uintptr_t)out % 16 == 0) && (!delta || ((uintptr_t)delta % 16 == 0 && part_stride % 4 == 0));
    if (aligned && parts <= kMaxNormParts && H <= (parts == 1 ? 4 : 2) * 4 * 1024) {
        const int groups = H / 4;
        // few rows: one group per thread, so that the row's loads are all in flight at once;
        // many rows: four groups per thread, fewer and fuller waves
        int items = groups <= 1024 ? 1 : (groups <= 2048 ? 2 : 4);
        if (R >= 256 && groups >= 256 && parts == 1) items = 4;
        int threads = (groups + items - 1) / items;
        threads = (threads + kWave - 1) / kWave * kWave;
#define LAUNCHV(TO, TD, IT, MP) rmsnorm_vec_kernel<TO, TD, IT, MP><<<R, threads, 0, stream>>>( \
        (TO*)out, x, (const TD*)delta, parts, (size_t)part_stride, rows, w, eps, H, write_back)
#define PICK(TO, TD) do { \
        if (parts == 1) { if (items == 1) LAUNCHV(TO, TD, 1, 1); else if (items == 2) LAUNCHV(TO, TD, 2, 1); else LAUNCHV(TO, TD, 4, 1); } \
        else { if (items == 1) LAUNCHV(TO, TD, 1, kMaxNormParts); else LAUNCHV(TO, TD, 2, kMaxNormParts); } } while (0)
        if (out_dtype == DT_F32 && delta_dtype == DT_F32) PICK(float, float);
        else if (out_dtype == DT_BF16 && delta_dtype == DT_BF16) PICK(bf16_t, bf16_t);
        else if (out_dtype == DT_BF16 && delta_dtype == DT_F32) PICK(bf16_t, float);
        else if (out_dtype == DT_F32 && delta_dtype == DT_BF16) PICK(float, bf16_t);
        else return LLOGOS_BAD_ARGUMENT;
#undef PICK
#undef LAUNCHV
        return LLOGOS_LAUNCH_CHECK();
    }
    const int threads = H >= 1024 ? 256 : (H >= 256 ? 128 : 64);
#define LAUNCH(TO, TD) rmsnorm_kernel<TO, TD><<<R, threads, 0, stream>>>( \
        (TO*)out, x, (const TD*)delta, parts, (size_t)part_stride, rows, w, eps, H, write_back)
    if (out_dtype == DT_F32 && delta_dtype == DT_F32) LAUNCH(float, float);
    else if (out_dtype == DT_BF16 && delta_dtype == DT_BF16) LAUNCH(bf16_t, bf16_t);
    else if (out_dtype == DT_BF16 && delta_dtype == DT_F32) LAUNCH(bf16_t, float);
    else if (out_dtype == DT_F32 && delta_dtype == DT_BF16) LAUNCH(float, bf16_t);
    else return LLOGOS_BAD_ARGUMENT;
#undef LAUNCH
    return LLOGOS_LAUNCH_CHECK();
}

// x[s] += delta[s] for all rows (the last residual sum, when no norm follows).
template <typename TD>
__global__ void residual_add_kernel(float* __restrict__ x, const TD* __restrict__ delta, size_t n) {
    size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) x[i] += load_f32(delta + i);
}

LLOGOS_EXPORT int llogos_residual_add(float* x, const void* delta, int delta_dtype, long long n,
                                      hipStream_t stream) {
    if (n <= 0) return LLOGOS_BAD_ARGUMENT;
    const unsigned blocks = (unsigned)((n + 255) / 256);
    if (delta_dtype == DT_F32) residual_add_kernel<float><<<blocks, 256, 0, stream>>>(x, (const float*)delta, (size_t)n);
    else if (delta_dtype == DT_BF16) residual_add_kernel<bf16_t><<<blocks, 256, 0, stream>>>(x, (const bf16_t*)delta, (size_t)n);
    else return LLOGOS_BAD_ARGUMENT;
    return LLOGOS_LAUNCH_CHECK();
}

// ---------------------------------------------------------------- rotary table
// cs[t, i] = (cos, sin)(pos[t] * inv_freq[i]) with the angle, cosine and sine in double
// (reference: Daisi.Llogos.Cpu/Rope.cs:147-152; Daisi.Llogos.Cuda/kernels/elementwise.cu:258-261).
// One table serves every layer that shares the rotary parameters.
__global__ void rope_table_kernel(float2* __restrict__ cs, const int* __restrict__ pos,
                                  const double* __restrict__ inv_freq, int T, int half) {
    const int idx = blockIdx.x * blockDim.x + threadIdx.x;
    if (idx >= T * half) return;
    const int t = idx / half, i = idx % half;
    const double a = (double)pos[t] * inv_freq[i];
    cs[idx] = make_float2((float)cos(a), (float)sin(a));
}

LLOGOS_EXPORT int llogos_rope_table(void* cs, const int* pos, const double* inv_freq, int T, int half,
                                    hipStream_t stream) {
    if (T <= 0 || half <= 0) return LLOGOS_BAD_ARGUMENT;
    const int n = T * half;
    rope_table_kernel<<<(n + 255) / 256, 256, 0, stream>>>((float2*)cs, pos, inv_freq, T, half);
    return LLOGOS_LAUNCH_CHECK();
}

// ---------------------------------------------------------------- per-head norm + rotation + cache write
// One wave per (token, head) of the fused projection row [q heads | k heads | v heads]:
//   q, k heads: optional RMSNorm over head_dim with a shared weight, then rotation of the
//               first `rot` dimensions; q goes back in place, k goes to its cache page;
//   v heads:    copied to the cache.
// pairing 0: (i, i + rot/2) for checkpoints that are not row-permuted; 1: (2i, 2i+1), the
// reference's default (Daisi.Llogos.Cuda/kernels/elementwise.cu:243-349; per_head_rms_norm
// composite_ops.cu:106-136; kv_cache_write composite_ops.cu:198-264).
constexpr int kHeadsPerBlock = 4;
constexpr int kMaxHeadDim = 512;

template <typename TI, typename T>
__global__ void qk_rope_cache_kernel(const TI* __restrict__ qkv, int parts, size_t part_stride, int row_stride,
                                     const float* __restrict__ bias, T* __restrict__ q_out,
                                     int n_heads, int n_kv_heads, int head_dim, int rot, int pairing,
                                     const float* __restrict__ q_norm_w, const float* __restrict__ k_norm_w,
                                     float eps, const float2* __restrict__ cs,
                                     T* __restrict__ k_pool, T* __restrict__ v_pool, PagedKV cache,
                                     const int* __restrict__ tok_seq, const int* __restrict__ tok_pos) {
    extern __shared__ float smem[];
    const int t = blockIdx.x;
    const int head = blockIdx.y * kHeadsPerBlock + threadIdx.y;
    const int lane = threadIdx.x;
    const int total_heads = n_heads + 2 * n_kv_heads;
    const bool active = head < total_heads;
    float* buf = smem + threadIdx.y * head_dim;
    const int half = rot / 2;

    const size_t col0 = (size_t)(active ? head : 0) * head_dim;
    const TI* src = qkv + (size_t)t * row_stride + col0;
    const bool is_q = head < n_heads;
    const bool is_k = !is_q && head < n_heads + n_kv_heads;
    const float* norm_w = is_q ? q_norm_w : (is_k ? k_norm_w : nullptr);

    float ss = 0.f;
    if (active) {
        for (int d = lane; d < head_dim; d += kWave) {
            float v = sum_parts(src, (size_t)d, parts, part_stride);
            if (bias) v += bias[col0 + d];
            buf[d] = v;
            ss += v * v;
        }
    }
    ss = wave_sum(ss);
    __syncthreads();
    if (active && norm_w) {
        const float inv = 1.0f / sqrtf(ss / (float)head_dim + eps);
        for (int d = lane; d < head_dim; d += kWave) buf[d] = buf[d] * inv * norm_w[d];
    }
    __syncthreads();
    if (!active) return;

    const int in_page = tok_pos[t] % kPageTokens;
    T* dst;
    if (is_q) {
        dst = q_out + ((size_t)t * n_heads + head) * head_dim;
    } else if (is_k) {
        dst = k_pool + paged_base(cache, tok_seq[t], head - n_heads, tok_pos[t]);
    } else {
        T* vdst = v_pool + paged_base(cache, tok_seq[t], head - n_heads - n_kv_heads, tok_pos[t]);
        for (int d = lane; d < head_dim; d += kWave) store_f32(vdst + page_value_offset(in_page, d), buf[d]);
        return;
    }
    const float2* c = cs + (size_t)t * half;
    for (int d = lane; d < head_dim; d += kWave) {
        float v = buf[d];
        if (d < rot) {
            if (pairing == 0) {
                if (d < half) v = buf[d] * c[d].x - buf[d + half] * c[d].y;
                else          v = buf[d - half] * c[d - half].y + buf[d] * c[d - half].x;
            } else {
                const int i = d >> 1;
                if ((d & 1) == 0) v = buf[d] * c[i].x - buf[d + 1] * c[i].y;
                else              v = buf[d - 1] * c[i].y + buf[d] * c[i].x;
            }
        }
        store_f32(dst + (is_q ? d : page_key_offset(in_page, d, head_dim)), v);
    }
}

// The same for head_dim = rot = 128 with split-half pairing, without LDS or block barriers, for
// prompts.  With one (token, head) a wave and two values a lane this kernel took 29.5 us for 2,048
// tokens of the 8B head shape (2.6 TB/s) and 20 us of that with every store left out: its time
// was the number of its load instructions (five a token and head, of 4 and 8 bytes a lane), not
// bytes or latency.  So a lane takes four consecutive dimensions (one 16-byte load), half a
// wave a head (the rotation partner, 64 dimensions away, sits 16 lanes away), and a wave its two
// heads for kRopeTokens tokens in a row, all of whose values it asks for before it works on the
// first.  Values of eight consecutive positions are neighbours in a value page, so when the
// wave's tokens are such a run its value stores are 16 bytes (otherwise one element each).
constexpr int kRopeTokens = 8;
constexpr int kRopeHeadsPerBlock = 8;                 // four waves of two heads

template <typename TI> __device__ __forceinline__ float4 load4_f32(const TI* p);
template <> __device__ __forceinline__ float4 load4_f32<float>(const float* p) { return *reinterpret_cast<const float4*>(p); }
template <> __device__ __forceinline__ float4 load4_f32<bf16_t>(const bf16_t* p) {
    const uint2 v = *reinterpret_cast<const uint2*>(p);
    return make_float4(__uint_as_float(v.x << 16), __uint_as_float(v.x & 0xffff0000u),
                       __uint_as_float(v.y << 16), __uint_as_float(v.y & 0xffff0000u));
}
template <typename T> __device__ __forceinline__ void store4_f32(T* p, float a, float b, float c, float d);
template <> __device__ __forceinline__ void store4_f32<float>(float* p, float a, float b, float c, float d) {
    *reinterpret_cast<float4*>(p) = make_float4(a, b, c, d);
}
template <> __device__ __forceinline__ void store4_f32<bf16_t>(bf16_t* p, float a, float b, float c, float d) {
    uint2 v;
    v.x = (uint32_t)f32_to_bf16(a) | ((uint32_t)f32_to_bf16(b) << 16);
    v.y = (uint32_t)f32_to_bf16(c) | ((uint32_t)f32_to_bf16(d) << 16);
    *reinterpret_cast<uint2*>(p) = v;
}

template <typename TI, typename T>
__global__ __launch_bounds__(kWave * kRopeHeadsPerBlock / 2) void qk_rope_cache_hd128_kernel(
        const TI* __restrict__ qkv, int parts, size_t part_stride, int row_stride,
        const float* __restrict__ bias, T* __restrict__ q_out, int n_heads, int n_kv_heads,
        const float* __restrict__ q_norm_w, const float* __restrict__ k_norm_w,
        float eps, const float2* __restrict__ cs, T* __restrict__ k_pool, T* __restrict__ v_pool, PagedKV cache,
        const int* __restrict__ tok_seq, const int* __restrict__ tok_pos, int n_tokens) {
    constexpr int HD = 128;
    const int t0 = blockIdx.x * kRopeTokens;
    const int lane = threadIdx.x & (kWave - 1), wave = threadIdx.x / kWave;
    const int l = lane & 31;
    const int head = blockIdx.y * kRopeHeadsPerBlock + 2 * wave + (lane >> 5);
    const int total_heads = n_heads + 2 * n_kv_heads;
    const bool live = head < total_heads;              // (a wave's second head may lie past the last one)
    const int hsafe = live ? head : total_heads - 1;
    const int d = 4 * l;
    const size_t col = (size_t)hsafe * HD + d;
    const bool is_q = hsafe < n_heads;
    const bool is_k = !is_q && hsafe < n_heads + n_kv_heads;
    const bool is_v = !is_q && !is_k;
    float4 x[kRopeTokens], ca[kRopeTokens], cb[kRopeTokens];
    int seq[kRopeTokens], pos[kRopeTokens];
#pragma unroll
    for (int i = 0; i < kRopeTokens; ++i) {
        const int t = min(t0 + i, n_tokens - 1);       // (tokens past the end: the last one again, not stored)
        const TI* src = qkv + (size_t)t * row_stride + col;
        x[i] = load4_f32<TI>(src);
        for (int q = 1; q < parts; ++q) {
            const float4 more = load4_f32<TI>(src + q * part_stride);
            x[i].x += more.x; x[i].y += more.y; x[i].z += more.z; x[i].w += more.w;
        }
        // (cos, sin) of dimensions d & 63 .. + 3: two 16-byte loads
        const float4* c4 = reinterpret_cast<const float4*>(cs + (size_t)t * 64 + (d & 63));
        ca[i] = c4[0];
        cb[i] = c4[1];
        seq[i] = tok_seq[t];
        pos[i] = tok_pos[t];
    }
    float4 b = make_float4(0.f, 0.f, 0.f, 0.f), w = make_float4(1.f, 1.f, 1.f, 1.f);
    if (bias) b = *reinterpret_cast<const float4*>(bias + col);
    const float* norm_w = is_q ? q_norm_w : (is_k ? k_norm_w : nullptr);
    if (norm_w) w = *reinterpret_cast<const float4*>(norm_w + d);
    // whether the wave's tokens are eight consecutive positions of one sequence that start at a multiple of eight
    bool run = t0 + kRopeTokens <= n_tokens && (pos[0] & 7) == 0;
#pragma unroll
    for (int i = 1; i < kRopeTokens; ++i) run = run && seq[i] == seq[0] && pos[i] == pos[0] + i;
#pragma unroll
    for (int i = 0; i < kRopeTokens; ++i) {
        x[i].x += b.x; x[i].y += b.y; x[i].z += b.z; x[i].w += b.w;
    }
    if (is_v) {
        if (!live) return;
        if (run) {
            T* vdst = v_pool + paged_base(cache, seq[0], hsafe - n_heads - n_kv_heads, pos[0]);
            const int at = pos[0] % kPageTokens;
            // eight positions of one dimension lie side by side
            T* p0 = vdst + page_value_offset(at, d);
            store4_f32<T>(p0, x[0].x, x[1].x, x[2].x, x[3].x);       store4_f32<T>(p0 + 4, x[4].x, x[5].x, x[6].x, x[7].x);
            T* p1 = vdst + page_value_offset(at, d + 1);
            store4_f32<T>(p1, x[0].y, x[1].y, x[2].y, x[3].y);       store4_f32<T>(p1 + 4, x[4].y, x[5].y, x[6].y, x[7].y);
            T* p2 = vdst + page_value_offset(at, d + 2);
            store4_f32<T>(p2, x[0].z, x[1].z, x[2].z, x[3].z);       store4_f32<T>(p2 + 4, x[4].z, x[5].z, x[6].z, x[7].z);
            T* p3 = vdst + page_value_offset(at, d + 3);
            store4_f32<T>(p3, x[0].w, x[1].w, x[2].w, x[3].w);       store4_f32<T>(p3 + 4, x[4].w, x[5].w, x[6].w, x[7].w);
            return;
        }
#pragma unroll
        for (int i = 0; i < kRopeTokens; ++i) {
            if (t0 + i >= n_tokens) break;
            T* vdst = v_pool + paged_base(cache, seq[i], hsafe - n_heads - n_kv_heads, pos[i]);
            const int at = pos[i] % kPageTokens;
            store_f32(vdst + page_value_offset(at, d), x[i].x);
            store_f32(vdst + page_value_offset(at, d + 1), x[i].y);
            store_f32(vdst + page_value_offset(at, d + 2), x[i].z);
            store_f32(vdst + page_value_offset(at, d + 3), x[i].w);
        }
        return;
    }
    // (both heads of a wave take the same path from here on, or the other one is a value head and has left:
    // the exchanges below stay within a head's 32 lanes)
#pragma unroll
    for (int i = 0; i < kRopeTokens; ++i) {
        const int t = t0 + i;
        if (t >= n_tokens) break;
        float4 a = x[i];
        if (norm_w) {
            float ss = a.x * a.x + a.y * a.y + a.z * a.z + a.w * a.w;
#pragma unroll
            for (int o = 16; o > 0; o >>= 1) ss += __shfl_xor(ss, o, kWave);
            const float inv = 1.0f / sqrtf(ss / (float)HD + eps);
            a.x = a.x * inv * w.x; a.y = a.y * inv * w.y; a.z = a.z * inv * w.z; a.w = a.w * inv * w.w;
        }
        float4 p;
        p.x = __shfl_xor(a.x, 16, kWave); p.y = __shfl_xor(a.y, 16, kWave);
        p.z = __shfl_xor(a.z, 16, kWave); p.w = __shfl_xor(a.w, 16, kWave);
        float4 y;
        if (l < 16) {
            y.x = a.x * ca[i].x - p.x * ca[i].y; y.y = a.y * ca[i].z - p.y * ca[i].w;
            y.z = a.z * cb[i].x - p.z * cb[i].y; y.w = a.w * cb[i].z - p.w * cb[i].w;
        } else {
            y.x = p.x * ca[i].y + a.x * ca[i].x; y.y = p.y * ca[i].w + a.y * ca[i].z;
            y.z = p.z * cb[i].y + a.z * cb[i].x; y.w = p.w * cb[i].w + a.w * cb[i].z;
        }
        if (!live) continue;
        // (four consecutive dimensions are neighbours in a key page too)
        T* dst = is_q ? q_out + ((size_t)t * n_heads + hsafe) * HD + d
                      : k_pool + paged_base(cache, seq[i], hsafe - n_heads, pos[i])
                               + page_key_offset(pos[i] % kPageTokens, d, HD);
        store4_f32<T>(dst, y.x, y.y, y.z, y.w);
    }
}

// qkv: the fused projection [parts][T][row_stride] in float32 or in the cache's type (parts are
// summed, then `bias` [width] is added); q_out [T, n_heads * head_dim] and the pools have the
// cache's type `dtype`.
LLOGOS_EXPORT int llogos_qk_rope_cache(const void* qkv, int in_dtype, int parts, long long part_stride,
                                       int row_stride, const float* bias, void* q_out, int dtype,
                                       int n_heads, int n_kv_heads, int head_dim, int rot, int pairing,
                                       const float* q_norm_w, const float* k_norm_w, float eps,
                                       const void* cs, void* k_pool, void* v_pool,
                                       const int* table, int table_stride,
                                       const int* tok_seq, const int* tok_pos, int T, hipStream_t stream) {
    if (T <= 0 || n_heads <= 0 || n_kv_heads < 0 || head_dim <= 0 || head_dim > kMaxHeadDim) return LLOGOS_BAD_ARGUMENT;
    if (rot < 0 || rot > head_dim || (rot & 1) || parts < 1) return LLOGOS_BAD_ARGUMENT;
    if (n_kv_heads > 0 && (!k_pool || !v_pool || !table)) return LLOGOS_BAD_ARGUMENT;
    if (row_stride < (n_heads + 2 * n_kv_heads) * head_dim) return LLOGOS_BAD_ARGUMENT;
    PagedKV cache{table, table_stride, n_kv_heads, head_dim};
    const int total_heads = n_heads + 2 * n_kv_heads;
    dim3 grid(T, (total_heads + kHeadsPerBlock - 1) / kHeadsPerBlock), block(kWave, kHeadsPerBlock);
    dim3 grid128((T + kRopeTokens - 1) / kRopeTokens, (total_heads + kRopeHeadsPerBlock - 1) / kRopeHeadsPerBlock);
    // (the wide form takes 16-byte steps through rows, tables and pools)
    const bool wide = head_dim == 128 && rot == 128 && pairing == 0 && (row_stride % 4) == 0 && (part_stride % 4) == 0 &&
                      ((uintptr_t)qkv % 16) == 0 && ((uintptr_t)q_out % 16) == 0 && ((uintptr_t)cs % 16) == 0 &&
                      ((uintptr_t)bias % 16) == 0 && ((uintptr_t)k_pool % 16) == 0 && ((uintptr_t)v_pool % 16) == 0 &&
                      ((uintptr_t)q_norm_w % 16) == 0 && ((uintptr_t)k_norm_w % 16) == 0;
    const size_t smem = (size_t)kHeadsPerBlock * head_dim * sizeof(float);
#define LAUNCH(TI, T_) do { \
        if (wide) \
            qk_rope_cache_hd128_kernel<TI, T_><<<grid128, kWave * kRopeHeadsPerBlock / 2, 0, stream>>>( \
                (const TI*)qkv, parts, (size_t)part_stride, row_stride, bias, (T_*)q_out, n_heads, n_kv_heads, \
                q_norm_w, k_norm_w, eps, (const float2*)cs, (T_*)k_pool, (T_*)v_pool, cache, tok_seq, tok_pos, T); \
        else \
            qk_rope_cache_kernel<TI, T_><<<grid, block, smem, stream>>>( \
                (const TI*)qkv, parts, (size_t)part_stride, row_stride, bias, (T_*)q_out, n_heads, n_kv_heads, head_dim, \
                rot, pairing, q_norm_w, k_norm_w, eps, (const float2*)cs, (T_*)k_pool, (T_*)v_pool, cache, tok_seq, tok_pos); \
    } while (0)
    if (dtype == DT_F32 && in_dtype == DT_F32) LAUNCH(float, float);
    else if (dtype == DT_BF16 && in_dtype == DT_BF16) LAUNCH(bf16_t, bf16_t);
    else if (dtype == DT_BF16 && in_dtype == DT_F32) LAUNCH(float, bf16_t);
    else return LLOGOS_BAD_ARGUMENT;
#undef LAUNCH
    return LLOGOS_LAUNCH_CHECK();
}

// ---------------------------------------------------------------- SwiGLU
// out[t, i] = silu(gu[t, i]) * gu[t, I + i] from the fused row [gate | up].
// (reference: split_swiglu, Daisi.Llogos.Cuda/kernels/elementwise.cu:1084-1110; silu(z) = z / (1 + exp(-z)))
template <typename TI, typename T>
__global__ void swiglu_kernel(T* __restrict__ out, const TI* __restrict__ gu, int parts, size_t part_stride,
                              int I, size_t n) {
    const size_t idx = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (idx >= n) return;
    const size_t t = idx / I;
    const int i = (int)(idx % I);
    const float g = sum_parts(gu, t * 2 * I + i, parts, part_stride);
    const float u = sum_parts(gu, t * 2 * I + I + i, parts, part_stride);
    store_f32(out + idx, g / (1.0f + expf(-g)) * u);
}

// the same for one bfloat16 part and I % 8 == 0: eight values per thread, 16-byte loads and stores
__global__ void swiglu_bf16x8_kernel(bf16_t* __restrict__ out, const bf16_t* __restrict__ gu, int I, size_t n8) {
    const size_t idx = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (idx >= n8) return;
    const int per_row = I / 8;
    const size_t t = idx / per_row;
    const int i = (int)(idx % per_row) * 8;
    const uint4 gv = *reinterpret_cast<const uint4*>(gu + t * 2 * I + i);
    const uint4 uv = *reinterpret_cast<const uint4*>(gu + t * 2 * I + I + i);
    const uint32_t gw[4] = {gv.x, gv.y, gv.z, gv.w}, uw[4] = {uv.x, uv.y, uv.z, uv.w};
    uint32_t o[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        const float g0 = __uint_as_float(gw[j] << 16), g1 = __uint_as_float(gw[j] & 0xffff0000u);
        const float u0 = __uint_as_float(uw[j] << 16), u1 = __uint_as_float(uw[j] & 0xffff0000u);
        o[j] = (uint32_t)f32_to_bf16(g0 / (1.0f + expf(-g0)) * u0) |
               ((uint32_t)f32_to_bf16(g1 / (1.0f + expf(-g1)) * u1) << 16);
    }
    *reinterpret_cast<uint4*>(out + t * I + i) = make_uint4(o[0], o[1], o[2], o[3]);
}

// gu: [parts][T][2 I] in float32 or in the output's type; parts are summed on the way.
LLOGOS_EXPORT int llogos_swiglu(void* out, int dtype, const void* gu, int in_dtype, int parts,
                                long long part_stride, int T, int I, hipStream_t stream) {
    if (T <= 0 || I <= 0 || parts < 1) return LLOGOS_BAD_ARGUMENT;
    const size_t n = (size_t)T * I;
    if (dtype == DT_BF16 && in_dtype == DT_BF16 && parts == 1 && I % 8 == 0 &&
        (uintptr_t)gu % 16 == 0 && (uintptr_t)out % 16 == 0) {
        const size_t n8 = n / 8;
        swiglu_bf16x8_kernel<<<(unsigned)((n8 + 255) / 256), 256, 0, stream>>>((bf16_t*)out, (const bf16_t*)gu, I, n8);
        return LLOGOS_LAUNCH_CHECK();
    }
    const unsigned blocks = (unsigned)((n + 255) / 256);
#define LAUNCH(TI, T_) swiglu_kernel<TI, T_><<<blocks, 256, 0, stream>>>( \
        (T_*)out, (const TI*)gu, parts, (size_t)part_stride, I, n)
    if (dtype == DT_F32 && in_dtype == DT_F32) LAUNCH(float, float);
    else if (dtype == DT_BF16 && in_dtype == DT_BF16) LAUNCH(bf16_t, bf16_t);
    else if (dtype == DT_BF16 && in_dtype == DT_F32) LAUNCH(float, bf16_t);
    else return LLOGOS_BAD_ARGUMENT;
#undef LAUNCH
    return LLOGOS_LAUNCH_CHECK();
}

// out[T, N] = sum of parts (+ bias): for consumers that want one plain tensor.
template <typename TI, typename TO>
__global__ void sum_parts_kernel(TO* __restrict__ out, const TI* __restrict__ in, int parts, size_t part_stride,
                                 const float* __restrict__ bias, int N, size_t n) {
    const size_t idx = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (idx >= n) return;
    float v = sum_parts(in, idx, parts, part_stride);
    if (bias) v += bias[idx % N];
    store_f32(out + idx, v);
}

LLOGOS_EXPORT int llogos_sum_parts(void* out, int out_dtype, const void* in, int in_dtype, int parts,
                                   long long part_stride, const float* bias, int T, int N, hipStream_t stream) {
    if (T <= 0 || N <= 0 || parts < 1) return LLOGOS_BAD_ARGUMENT;
    const size_t n = (size_t)T * N;
    const unsigned blocks = (unsigned)((n + 255) / 256);
#define LAUNCH(TI, TO) sum_parts_kernel<TI, TO><<<blocks, 256, 0, stream>>>( \
        (TO*)out, (const TI*)in, parts, (size_t)part_stride, bias, N, n)
    if (in_dtype == DT_F32 && out_dtype == DT_F32) LAUNCH(float, float);
    else if (in_dtype == DT_F32 && out_dtype == DT_BF16) LAUNCH(float, bf16_t);
    else if (in_dtype == DT_BF16 && out_dtype == DT_F32) LAUNCH(bf16_t, float);
    else if (in_dtype == DT_BF16 && out_dtype == DT_BF16) LAUNCH(bf16_t, bf16_t);
    else return LLOGOS_BAD_ARGUMENT;
#undef LAUNCH
    return LLOGOS_LAUNCH_CHECK();
}
