// bfloat16 attention over the paged cache on the matrix cores (gfx950,
// v_mfma_f32_16x16x32_bf16), for head sizes 64 and 128 and up to 16 query heads per
// key/value head.  Softmax statistics, scores and the output sums are float32.
//
// One wave works on 16 "columns" and one page of 64 keys at a time:
//   decode  (one token per sequence): the columns are the query heads of one kv head;
//           a block of 4 waves takes a run of pages of one (sequence, kv head), each wave
//           every fourth of them in turn; the waves' running (max, sum, output) are merged
//           through LDS, blocks along the context write partial results that a second small
//           kernel merges;
//   prefill (many tokens per sequence): the columns are 16 consecutive tokens of one
//           sequence for one query head; each wave walks the pages up to its last row.
// Scores are computed transposed, S^T[key][column] = K . Q^T, so that the lane that holds
// the scores of a column for 16 keys is the lane that must supply them as the second
// operand of O^T[d][column] = V^T[d][key] . P^T[key][column]; no shuffle or LDS pass sits
// between the two products.  Pages are stored in the order of these operands (common.h): a
// fragment is 1 KB of consecutive memory, a lane's eight values 16 bytes of it; a value
// fragment holds eight consecutive tokens of one dimension per lane, and the rows of a key
// fragment are the keys 16 * (i / 4) + 4 * rb + i % 4 (i = operand row, rb = block of 16),
// which makes lane group g own keys 16 g .. 16 g + 15.
// (reference: gated_attention / batched_gated_attention, Daisi.Llogos.Cuda/kernels/
//  composite_ops.cu:275-512: tiles of keys with running maximum and sum, kv head = head /
//  group, scale after the dot, query m of a prompt sees keys 0 .. start + m.)
#include "common.h"
#include "llogos_api.h"
#include <algorithm>
#include <mutex>

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float f32x4 __attribute__((ext_vector_type(4)));

constexpr int kAttnWaves = 4;

__device__ __forceinline__ bf16x8 ld_frag(const bf16_t* p) {
    return __builtin_bit_cast(bf16x8, *reinterpret_cast<const uint4*>(p));
}

// A fragment of a page, read once: 64 lanes x 16 bytes of consecutive memory, past the caches'
// keeping (a step reads every page once and the next step comes after all other layers).
typedef unsigned u32x4 __attribute__((ext_vector_type(4)));
__device__ __forceinline__ bf16x8 ld_frag_once(const bf16_t* p) {
    return __builtin_bit_cast(bf16x8, __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(p)));
}

__device__ __forceinline__ bf16x8 zero_frag() {
    return __builtin_bit_cast(bf16x8, make_uint4(0, 0, 0, 0));
}

typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
typedef float f32x2 __attribute__((ext_vector_type(2)));

// two floats to packed bfloat16, round to nearest even (one v_cvt_pk_bf16_f32)
__device__ __forceinline__ uint32_t pack_bf16(float lo, float hi) {
    const f32x2 v = {lo, hi};
    return __builtin_bit_cast(uint32_t, __builtin_convertvector(v, bf16x2));
}

constexpr float kLog2e = 1.4426950408889634f;

// Maximum and sum over the four lanes l, l ^ 16, l ^ 32, l ^ 48 (one column of an MFMA result),
// left in all four.  v_permlane16_swap exchanges the odd rows of 16 lanes of its first operand
// with the even rows of its second, v_permlane32_swap the upper half of the first with the
// lower half of the second: fed the same value twice, the two results hold a lane's own value
// and its partner's.  (A shuffle would go through the LDS pipeline and cost its latency.)
typedef unsigned u32x2 __attribute__((ext_vector_type(2)));
__device__ __forceinline__ float quad_max(float x) {
    u32x2 r = __builtin_amdgcn_permlane16_swap(__float_as_uint(x), __float_as_uint(x), false, false);
    x = fmaxf(__uint_as_float(r[0]), __uint_as_float(r[1]));
    r = __builtin_amdgcn_permlane32_swap(__float_as_uint(x), __float_as_uint(x), false, false);
    return fmaxf(__uint_as_float(r[0]), __uint_as_float(r[1]));
}
__device__ __forceinline__ float quad_sum(float x) {
    u32x2 r = __builtin_amdgcn_permlane16_swap(__float_as_uint(x), __float_as_uint(x), false, false);
    x = __uint_as_float(r[0]) + __uint_as_float(r[1]);
    r = __builtin_amdgcn_permlane32_swap(__float_as_uint(x), __float_as_uint(x), false, false);
    return __uint_as_float(r[0]) + __uint_as_float(r[1]);
}

// Keeps the first n (0..8) of a fragment's eight values and zeroes the rest.
__device__ __forceinline__ bf16x8 keep_first(bf16x8 f, int n) {
    uint4 u = __builtin_bit_cast(uint4, f);
    uint32_t* w = reinterpret_cast<uint32_t*>(&u);
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        const uint32_t mask = (2 * j + 1 < n) ? 0xffffffffu : ((2 * j < n) ? 0x0000ffffu : 0u);
        w[j] &= mask;
    }
    return __builtin_bit_cast(bf16x8, u);
}

// Running softmax state of one wave: per column (lane & 15) the maximum and the sum, and
// the output sums O^T[d][column] with d = 16 db + 4 g + r in acc[db][r].  The maximum is kept
// in units of log2: m = max(score * scale) * log2(e), so that exp(x - max) is one
// multiply-add and one v_exp_f32.
template <int HD>
struct WaveState {
    float m, l;
    f32x4 acc[HD / 16];
    __device__ void init() {
        m = -INFINITY;
        l = 0.f;
#pragma unroll
        for (int db = 0; db < HD / 16; ++db) acc[db] = f32x4{0.f, 0.f, 0.f, 0.f};
    }
};

// Softmax of one page for one block of 16 columns.  s[rb][r]: raw dot products of this lane's
// column with key key0 + g * GS + rb * RS + r.  Returns the probabilities as the two second
// operands of O^T += V^T . P^T (step t, slot e <-> s[2 t + e / 4][e % 4]) and the factor by
// which the running sums shrink.  MASKED = false when every key of the page is visible to
// every column of the wave.
template <bool MASKED, int GS, int RS, int HD>
__device__ __forceinline__ void softmax_page(f32x4 (&s)[4], WaveState<HD>& st, float scale_log2, int q_pos,
                                             int key0, int window, int sinks, bf16x8 (&pf)[2], float& corr) {
    const int g = (threadIdx.x & (kWave - 1)) >> 4;
    float tile_max = -INFINITY;
#pragma unroll
    for (int rb = 0; rb < 4; ++rb)
#pragma unroll
        for (int r = 0; r < 4; ++r) {
            if (MASKED) {
                const int key = key0 + g * GS + rb * RS + r;
                if (!(q_pos >= 0 && key_visible(q_pos, key, window, sinks))) s[rb][r] = -INFINITY;
            }
            tile_max = fmaxf(tile_max, s[rb][r]);
        }
    tile_max = quad_max(tile_max);
    const float m_new = fmaxf(st.m, tile_max * scale_log2);              // scale > 0: the maximum commutes
    // a column that has seen no key yet keeps m = -inf; exp2(-inf - (-inf)) must not be taken
    const float m_use = (m_new == -INFINITY) ? 0.f : m_new;
    corr = __builtin_amdgcn_exp2f(st.m - m_use);                          // exp2(-inf) = 0 for the first page
    float p[16], sum = 0.f;
#pragma unroll
    for (int rb = 0; rb < 4; ++rb)
#pragma unroll
        for (int r = 0; r < 4; ++r) {
            const float e = __builtin_amdgcn_exp2f(fmaf(s[rb][r], scale_log2, -m_use));   // masked: exp2(-inf) = 0
            p[4 * rb + r] = e;
            sum += e;
        }
    sum = quad_sum(sum);
    st.l = st.l * corr + sum;
    st.m = m_new;
#pragma unroll
    for (int t = 0; t < 2; ++t) {
        uint4 u;
        u.x = pack_bf16(p[8 * t + 0], p[8 * t + 1]);
        u.y = pack_bf16(p[8 * t + 2], p[8 * t + 3]);
        u.z = pack_bf16(p[8 * t + 4], p[8 * t + 5]);
        u.w = pack_bf16(p[8 * t + 6], p[8 * t + 7]);
        pf[t] = __builtin_bit_cast(bf16x8, u);
    }
}

// Whether every key of the page [key0, key0 + 63] is visible to every query at first_pos .. last_pos.
__device__ __forceinline__ bool page_fully_visible(int first_pos, int last_pos, int key0, int window, int sinks) {
    if (key0 + kPageTokens - 1 > first_pos) return false;
    if (window <= 0) return true;
    return key0 + kPageTokens - 1 < sinks || key0 > last_pos - window;
}

// The parts of a page's work.  kpage, vpage: one kv head's part of a page, in fragment order
// (common.h): fragment f of either is the 512 elements from 512 f on, lane l's eight at 8 l.
template <int HD>
__device__ __forceinline__ void load_keys(bf16x8 (&kf)[4][HD / 32], const bf16_t* __restrict__ kpage) {
    const bf16_t* mine = kpage + 8 * (threadIdx.x & (kWave - 1));
#pragma unroll
    for (int rb = 0; rb < 4; ++rb)
#pragma unroll
        for (int sk = 0; sk < HD / 32; ++sk) kf[rb][sk] = ld_frag_once(mine + 512 * (rb * (HD / 32) + sk));
}

template <int HD>
__device__ __forceinline__ void load_values(bf16x8 (&vf)[HD / 16][2], const bf16_t* __restrict__ vpage) {
    const bf16_t* mine = vpage + 8 * (threadIdx.x & (kWave - 1));
#pragma unroll
    for (int db = 0; db < HD / 16; ++db) {
        vf[db][0] = ld_frag_once(mine + 512 * (2 * db));
        vf[db][1] = ld_frag_once(mine + 512 * (2 * db + 1));
    }
}

// S^T = K . Q^T, four blocks of 16 keys; this lane: column lane & 15, keys 16 g + 4 rb + r in s[rb][r]
template <int HD>
__device__ __forceinline__ void page_scores(f32x4 (&s)[4], const bf16x8 (&kf)[4][HD / 32], const bf16x8 (&qf)[HD / 32]) {
#pragma unroll
    for (int rb = 0; rb < 4; ++rb) {
        s[rb] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int sk = 0; sk < HD / 32; ++sk)
            s[rb] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(kf[rb][sk], qf[sk], s[rb], 0, 0, 0);
    }
}

// O^T = O^T * corr + V^T . P^T; slot (g, e) of step t is key 16 g + 8 t + e.  Values of keys
// that have not been written (valid_keys and on) are zeroed: 0 * NaN is NaN.
template <int HD>
__device__ __forceinline__ void weigh_values(WaveState<HD>& st, const bf16x8 (&vf)[HD / 16][2], const bf16x8 (&pf)[2],
                                             float corr, int valid_keys) {
    const int g = (threadIdx.x & (kWave - 1)) >> 4;
    const bool rescale = __ballot(corr != 1.0f) != 0;
#pragma unroll
    for (int db = 0; db < HD / 16; ++db) {
        f32x4 a = st.acc[db];
        if (rescale) {
#pragma unroll
            for (int r = 0; r < 4; ++r) a[r] *= corr;
        }
        bf16x8 v0 = vf[db][0], v1 = vf[db][1];
        if (valid_keys < kPageTokens) {
            v0 = keep_first(v0, valid_keys - 16 * g);
            v1 = keep_first(v1, valid_keys - 16 * g - 8);
        }
        a = __builtin_amdgcn_mfma_f32_16x16x32_bf16(v0, pf[0], a, 0, 0, 0);
        a = __builtin_amdgcn_mfma_f32_16x16x32_bf16(v1, pf[1], a, 0, 0, 0);
        st.acc[db] = a;
    }
}

// One page of 64 keys.  qf: the columns' queries as second operands (lane (c, g) holds
// Q[c][32 s + 8 g ..]); kpage, vpage: one kv head's part of a page; q_pos: position of this lane's column
// (-1: the column is not in use); key0: position of the page's first key; valid_keys: how
// many of the page's keys have been written (the rest of the page holds whatever was there
// before: such scores are masked, and such values are zeroed because 0 * NaN is NaN).
template <int HD>
__device__ __forceinline__ void attend_page(WaveState<HD>& st, const bf16x8 (&qf)[HD / 32],
                                            const bf16_t* __restrict__ kpage, const bf16_t* __restrict__ vpage,
                                            int q_pos, int key0, int valid_keys, bool all_visible,
                                            float scale_log2, int window, int sinks) {
    // all of the page's loads are issued before the first product
    bf16x8 kf[4][HD / 32], vf[HD / 16][2];
    load_keys<HD>(kf, kpage);
    load_values<HD>(vf, vpage);
    f32x4 s[4];
    page_scores<HD>(s, kf, qf);
    bf16x8 pf[2];
    float corr;
    if (all_visible) softmax_page<false, 16, 4, HD>(s, st, scale_log2, q_pos, key0, window, sinks, pf, corr);
    else             softmax_page<true, 16, 4, HD>(s, st, scale_log2, q_pos, key0, window, sinks, pf, corr);
    weigh_values<HD>(st, vf, pf, corr, valid_keys);
}

// Whether any key of the page [key0, key0 + 63] can be visible to a query at q_pos.
__device__ __forceinline__ bool page_may_be_visible(int q_pos, int key0, int window, int sinks) {
    if (key0 > q_pos) return false;
    if (window <= 0) return true;
    return key0 < sinks || key0 + kPageTokens - 1 > q_pos - window;
}

// The same for queries at positions first_pos .. last_pos: the causal bound is loosest for the
// last of them, the window's for the first.
__device__ __forceinline__ bool page_may_be_visible_to_range(int first_pos, int last_pos, int key0,
                                                             int window, int sinks) {
    if (key0 > last_pos) return false;
    if (window <= 0) return true;
    return key0 < sinks || key0 + kPageTokens - 1 > first_pos - window;
}

// ---------------------------------------------------------------- decode
// grid (batch, kv heads, blocks along the context); a block of WAVES waves covers WAVES * ppw
// consecutive pages, wave w taking pages w, w + WAVES, ... of them one after the other.  (Asking
// for the next page's keys and values while a wave works on this one takes twice the registers
// and was slower: what hides the latency is the other waves.)  With one block
// along the context (gridDim.z == 1) the block writes the attention output itself; otherwise
// partial: [batch][heads][grid.z][HD + 2] floats (max, sum, unnormalised output) for the merge
// kernel.  Dynamic LDS: decode_lds_bytes(WAVES, group, HD).
__host__ __device__ constexpr size_t decode_lds_bytes(int waves, int group, int hd) {
    return (size_t)waves * (group * (hd + 1) + 32) * sizeof(float);
}

// The fused form (FUSED, head size 64 or 128 rotated whole with split-half pairing) starts from the
// projection itself: a block first makes its queries (sum of the projection's partial products,
// bias, per-head norm, rotation) into LDS, and the block whose pages hold the step's position
// also makes the step's key and value and writes them to their page, which the rotation kernel
// does otherwise.  One token a sequence: token b is sequence b.
struct QkvSource {
    const float* qkv;          // [parts][batch][row_stride]: partial sums of the fused rows [q | k | v]
    int parts;
    size_t part_stride;
    int row_stride;
    const float* bias;         // [(heads + 2 kv heads) * head size] or null
    const float* q_norm_w;     // [head size] or null
    const float* k_norm_w;
    float eps;
    const float2* cs;          // [batch][head size / 2] (cos, sin) of each sequence's position
    bf16_t* k_pool;            // the pools, writable
    bf16_t* v_pool;
};

template <int HD, int WAVES, bool FUSED>
__global__ __launch_bounds__(WAVES * kWave) void attn_decode_kernel(
        bf16_t* __restrict__ out, float* __restrict__ partial, const bf16_t* __restrict__ q, int q_stride,
        QkvSource src, const bf16_t* k_pool, const bf16_t* v_pool,
        const int* __restrict__ table, int table_stride, const int* __restrict__ tok_pos,
        int n_heads, int n_kv_heads, int group, float scale, int window, int sinks, int ppw) {
    extern __shared__ float lds[];
    float* lds_m = lds;                                   // [WAVES][16]
    float* lds_l = lds + WAVES * 16;                      // [WAVES][16]
    float* lds_o = lds + WAVES * 32;                      // [WAVES][group][HD + 1]
    __shared__ __attribute__((aligned(16))) bf16_t q_lds[FUSED ? 16 : 1][HD];
    const int b = blockIdx.x, kvh = blockIdx.y, z = blockIdx.z;
    const int lane = threadIdx.x & (kWave - 1), wave = threadIdx.x / kWave;
    const int c = lane & 15, g = lane >> 4;
    const int pos = tok_pos[b];
    const int n_pages = pos / kPageTokens + 1;
    const int first_page = z * WAVES * ppw;
    if (first_page >= n_pages) return;                           // nothing of this sequence here
    const int* row = table + (size_t)b * table_stride;

    // this wave's pages: first_page + wave + WAVES j, j < ppw, as far as the sequence goes and a
    // query at pos can see any of their keys (a page outside the window may have been given back)
    auto page_at = [&](int j) { return first_page + wave + WAVES * j; };
    auto next_from = [&](int j) {
        while (j < ppw && page_at(j) < n_pages && !page_may_be_visible(pos, page_at(j) * kPageTokens, window, sinks)) ++j;
        return (j < ppw && page_at(j) < n_pages) ? j : -1;
    };
    auto page_base = [&](int j) { return ((size_t)row[page_at(j)] * n_kv_heads + kvh) * kPageTokens * HD; };
    int j = next_from(0);

    if (FUSED) {
        // items 0 .. group - 1: the kv head's query heads; then, in the block that holds the
        // step's position, its key and its value.  A wave takes an item; lane l holds
        // dimensions PER l .. PER l + PER - 1 (two for head size 128, one for 64), and the
        // rotation partner, HD / 2 dimensions away, is lane l ^ 32.
        constexpr int PER = HD / kWave;
        static_assert(PER == 1 || PER == 2, "head sizes 64 and 128");
        const bool writer = (n_pages - 1) / (WAVES * ppw) == z;
        const int items = group + (writer ? 2 : 0);
        const int d = PER * lane;
        const size_t wbase = writer ? ((size_t)row[n_pages - 1] * n_kv_heads + kvh) * kPageTokens * HD : 0;
        for (int item = wave; item < items; item += WAVES) {
            const bool is_q = item < group, is_k = item == group;
            const int head = is_q ? kvh * group + item : (is_k ? n_heads + kvh : n_heads + n_kv_heads + kvh);
            const size_t col = (size_t)head * HD + d;
            const float* p = src.qkv + (size_t)b * src.row_stride + col;
            float x[PER];
#pragma unroll
            for (int e = 0; e < PER; ++e) x[e] = p[e];
            for (int part0 = 1; part0 < src.parts; part0 += 8) {     // eight loads in flight, added in ascending order
                float y[8][PER];
#pragma unroll
                for (int jj = 0; jj < 8; ++jj)
#pragma unroll
                    for (int e = 0; e < PER; ++e)
                        y[jj][e] = part0 + jj < src.parts ? p[(part0 + jj) * src.part_stride + e] : 0.f;
#pragma unroll
                for (int jj = 0; jj < 8; ++jj)
                    if (part0 + jj < src.parts) {
#pragma unroll
                        for (int e = 0; e < PER; ++e) x[e] += y[jj][e];
                    }
            }
            if (src.bias) {
#pragma unroll
                for (int e = 0; e < PER; ++e) x[e] += src.bias[col + e];
            }
            if (!is_q && !is_k) {
                bf16_t* vdst = src.v_pool + wbase;
#pragma unroll
                for (int e = 0; e < PER; ++e) vdst[page_value_offset(pos % kPageTokens, d + e)] = f32_to_bf16(x[e]);
                continue;
            }
            const float* norm_w = is_q ? src.q_norm_w : src.k_norm_w;
            if (norm_w) {
                float sq = 0.f;
#pragma unroll
                for (int e = 0; e < PER; ++e) sq += x[e] * x[e];
                const float inv = 1.0f / sqrtf(wave_sum(sq) / (float)HD + src.eps);
#pragma unroll
                for (int e = 0; e < PER; ++e) x[e] = x[e] * inv * norm_w[d + e];
            }
            bf16_t y[PER];
#pragma unroll
            for (int e = 0; e < PER; ++e) {
                const float partner = __shfl_xor(x[e], 32, kWave);
                const float2 cs = src.cs[(size_t)b * (HD / 2) + ((d + e) & (HD / 2 - 1))];
                y[e] = f32_to_bf16(lane < 32 ? x[e] * cs.x - partner * cs.y : partner * cs.y + x[e] * cs.x);
            }
            // (a lane's one or two dimensions are neighbours in a key page too)
            bf16_t* dst = is_q ? &q_lds[item][d] : src.k_pool + wbase + page_key_offset(pos % kPageTokens, d, HD);
#pragma unroll
            for (int e = 0; e < PER; ++e) dst[e] = y[e];
        }
        __syncthreads();          // the queries in LDS, and the key and value in memory, for every wave of the block
    }

    WaveState<HD> st;
    st.init();
    if (j >= 0) {
        bf16x8 qf[HD / 32];
        const bool col_ok = c < group;
        const bf16_t* qrow = FUSED ? &q_lds[col_ok ? c : 0][8 * g]
                                   : q + (size_t)b * q_stride + (size_t)(kvh * group + (col_ok ? c : 0)) * HD + 8 * g;
#pragma unroll
        for (int sk = 0; sk < HD / 32; ++sk) qf[sk] = col_ok ? ld_frag(qrow + 32 * sk) : zero_frag();
        // unused columns (c >= group) have zero queries and are never stored: they may run unmasked
        for (; j >= 0; j = next_from(j + 1)) {
            const int key0 = page_at(j) * kPageTokens;
            const size_t base = page_base(j);
            attend_page<HD>(st, qf, k_pool + base, v_pool + base, col_ok ? pos : -1, key0,
                            min(kPageTokens, pos - key0 + 1), page_fully_visible(pos, pos, key0, window, sinks),
                            scale * kLog2e, window, sinks);
        }
    }
    // merge the waves
    if (g == 0) { lds_m[wave * 16 + c] = st.m; lds_l[wave * 16 + c] = st.l; }
    if (c < group) {
        float* dst = lds_o + ((size_t)wave * group + c) * (HD + 1);
#pragma unroll
        for (int db = 0; db < HD / 16; ++db)
#pragma unroll
            for (int r = 0; r < 4; ++r) dst[16 * db + 4 * g + r] = st.acc[db][r];
    }
    __syncthreads();
    const int n_z = gridDim.z;
    for (int idx = threadIdx.x; idx < group * HD; idx += blockDim.x) {
        const int col = idx / HD, d = idx % HD;
        float m = -INFINITY;
#pragma unroll
        for (int w = 0; w < WAVES; ++w) m = fmaxf(m, lds_m[w * 16 + col]);
        float l = 0.f, o = 0.f;
#pragma unroll
        for (int w = 0; w < WAVES; ++w) {
            const float mw = lds_m[w * 16 + col];
            const float f = (mw == -INFINITY) ? 0.f : __builtin_amdgcn_exp2f(mw - m);
            l += lds_l[w * 16 + col] * f;
            o += lds_o[((size_t)w * group + col) * (HD + 1) + d] * f;
        }
        if (n_z == 1) {
            out[((size_t)b * n_heads + kvh * group + col) * HD + d] = f32_to_bf16(l > 0.f ? o / l : 0.f);
        } else {
            float* dst = partial + (((size_t)b * n_heads + kvh * group + col) * n_z + z) * (HD + 2);
            dst[2 + d] = o;
            if (d == 0) { dst[0] = m; dst[1] = l; }
        }
    }
}

// grid (batch, heads); kMergeLanes x HD threads.  Adds the partial results of the blocks along
// the context, each of which covered pages_per_block pages: thread (j, d) takes blocks j,
// j + kMergeLanes, ... of dimension d, and LDS adds the kMergeLanes sums in ascending j, so the
// order depends on the sequence's own length alone.  (One thread per dimension walking all
// blocks took 17 us at 33 blocks: a chain of dependent L2 latencies.  Letting the last block
// to finish add them, behind a device-wide fence and a ticket counter, was measured too: the
// fence writes back whatever earlier kernels left dirty in the L2 and cost 20 us a layer at
// batch 8; this kernel costs 4.6.)
constexpr int kMergeLanes = 4;

template <int HD>
__global__ __launch_bounds__(kMergeLanes * HD) void attn_decode_merge_kernel(
        bf16_t* __restrict__ out, const float* __restrict__ partial, const int* __restrict__ tok_pos,
        int n_heads, int n_z, int pages_per_block) {
    __shared__ float lds_m[kMergeLanes], lds_l[kMergeLanes], lds_o[kMergeLanes][HD];
    const int b = blockIdx.x, h = blockIdx.y, d = threadIdx.x % HD, j = threadIdx.x / HD;
    const int n_pages = tok_pos[b] / kPageTokens + 1;
    const int used = min(n_z, (n_pages + pages_per_block - 1) / pages_per_block);
    const float* src = partial + ((size_t)b * n_heads + h) * n_z * (HD + 2);
    float m = -INFINITY;
#pragma unroll 4
    for (int z = j; z < used; z += kMergeLanes) m = fmaxf(m, src[(size_t)z * (HD + 2)]);
    if (d == 0) lds_m[j] = m;
    __syncthreads();
#pragma unroll
    for (int i = 0; i < kMergeLanes; ++i) m = fmaxf(m, lds_m[i]);
    float l = 0.f, o = 0.f;
#pragma unroll 4
    for (int z = j; z < used; z += kMergeLanes) {
        const float* p = src + (size_t)z * (HD + 2);
        const float f = (p[0] == -INFINITY) ? 0.f : __builtin_amdgcn_exp2f(p[0] - m);
        l += p[1] * f;
        o += p[2 + d] * f;
    }
    lds_o[j][d] = o;
    if (d == 0) lds_l[j] = l;
    __syncthreads();
    if (j != 0) return;
    l = lds_l[0]; o = lds_o[0][d];
#pragma unroll
    for (int i = 1; i < kMergeLanes; ++i) { l += lds_l[i]; o += lds_o[i][d]; }
    out[((size_t)b * n_heads + h) * HD + d] = f32_to_bf16(l > 0.f ? o / l : 0.f);
}

// ---------------------------------------------------------------- prefill
// grid (tiles of 64 tokens over all sequences, heads); wave w of a block takes rows
// 16 w .. 16 w + 15 of the tile.  cu: token offsets of the sequences [batch + 1];
// starts: position of each sequence's first token in this step.
template <int HD>
__global__ __launch_bounds__(kAttnWaves * kWave) void attn_prefill_kernel(
        bf16_t* __restrict__ out, const bf16_t* __restrict__ q, int q_stride,
        const bf16_t* __restrict__ k_pool, const bf16_t* __restrict__ v_pool,
        const int* __restrict__ table, int table_stride, const int* __restrict__ cu,
        const int* __restrict__ tok_pos, int batch, int n_heads, int n_kv_heads, int group,
        float scale, int window, int sinks) {
    // which sequence does this tile belong to?
    int tile = blockIdx.x, b = 0, first = 0;
    for (; b < batch; ++b) {
        const int len = cu[b + 1] - cu[b];
        const int tiles = (len + 63) / 64;
        if (tile < tiles) { first = cu[b] + tile * 64; break; }
        tile -= tiles;
    }
    if (b >= batch) return;
    const int h = blockIdx.y, kvh = h / group;
    const int lane = threadIdx.x & (kWave - 1), wave = threadIdx.x / kWave;
    const int c = lane & 15, g = lane >> 4;
    const int row0 = first + 16 * wave;                          // this wave's first token row
    const int seq_end = cu[b + 1];
    if (row0 >= seq_end) return;
    const int rows = min(16, seq_end - row0);
    const bool col_ok = c < rows;
    const int my_row = row0 + (col_ok ? c : 0);
    const int q_pos = col_ok ? tok_pos[my_row] : -1;
    const int last_pos = tok_pos[row0 + rows - 1];
    const int first_pos = tok_pos[row0];
    const int written = tok_pos[seq_end - 1] + 1;                // positions of this sequence that hold keys

    bf16x8 qf[HD / 32];
    const bf16_t* qrow = q + (size_t)my_row * q_stride + (size_t)h * HD + 8 * g;
#pragma unroll
    for (int sk = 0; sk < HD / 32; ++sk) qf[sk] = col_ok ? ld_frag(qrow + 32 * sk) : zero_frag();

    WaveState<HD> st;
    st.init();
    const int n_pages = last_pos / kPageTokens + 1;
    for (int pi = 0; pi < n_pages; ++pi) {
        const int key0 = pi * kPageTokens;
        if (!page_may_be_visible_to_range(first_pos, last_pos, key0, window, sinks)) continue;
        const int page = table[(size_t)b * table_stride + pi];
        const size_t base = ((size_t)page * n_kv_heads + kvh) * kPageTokens * HD;
        attend_page<HD>(st, qf, k_pool + base, v_pool + base, q_pos, key0, min(kPageTokens, written - key0),
                        rows == 16 && page_fully_visible(first_pos, last_pos, key0, window, sinks),
                        scale * kLog2e, window, sinks);
    }
    if (!col_ok) return;
    const float inv = st.l > 0.f ? 1.0f / st.l : 0.f;
    bf16_t* orow = out + ((size_t)my_row * n_heads + h) * HD;
#pragma unroll
    for (int db = 0; db < HD / 16; ++db) {
        uint2 u;
        u.x = pack_bf16(st.acc[db][0] * inv, st.acc[db][1] * inv);
        u.y = pack_bf16(st.acc[db][2] * inv, st.acc[db][3] * inv);
        *reinterpret_cast<uint2*>(orow + 16 * db + 4 * g) = u;
    }
}

constexpr int kTileRows = 128;

// ---------------------------------------------------------------- prefill, pages shared through LDS
// grid: one block per (tile of 128 tokens over all sequences, head), in the order given in the
// kernel; the 4 waves of a block take 32 rows each (two blocks of 16 columns) and walk the same
// pages: a page is copied to LDS once per block (two buffers, the copy of the next page is in
// flight while the current one is used), and every key and value fragment a wave reads serves
// both of its column blocks.  A page's keys and values go from global memory into LDS without
// passing through registers (16 bytes a lane, a wave's 64 lanes to 1 KB of consecutive LDS),
// which frees the 32 registers of the copy and the time of the stores.  Pages are in fragment
// order in memory, and so they are in LDS: a wave's read of a fragment is 64 x 16 consecutive
// bytes, which LDS serves without a bank conflict; no padding and no swizzle.
template <int HD>
struct DirectPageLds {
    bf16_t k[HD / 8][512];               // fragment (rb, sk) at rb * (HD / 32) + sk
    bf16_t v[HD / 8][512];               // fragment (db, half) at 2 db + half
};

// HALVES = 2: a block of 8 waves, two sets of 4 with page buffers of their own, takes the same
// 128 rows; the sets take the tile's pages in turn and add their results through LDS at the end.
// One such block fills a compute unit (two waves a SIMD, as two blocks of 4 do), and a tile's
// pages take half as long: with HALVES = 1 a block left alone on its unit goes no faster (one
// wave a SIMD cannot overlap its matrix and its vector instructions), so a prompt of few tiles
// took as long as the pages of its last tile, one after the other.
template <int HD, int HALVES>
__global__ __launch_bounds__(HALVES * kAttnWaves * kWave) __attribute__((amdgpu_waves_per_eu(2, 2)))
void attn_prefill_direct_kernel(
        bf16_t* __restrict__ out, const bf16_t* __restrict__ q, int q_stride,
        const bf16_t* __restrict__ k_pool, const bf16_t* __restrict__ v_pool,
        const int* __restrict__ table, int table_stride, const int* __restrict__ cu,
        const int* __restrict__ tok_pos, int batch, int n_tiles, int n_heads, int n_kv_heads, int group,
        float scale, int window, int sinks) {
    extern __shared__ __attribute__((aligned(16))) unsigned char smem_raw[];
    const int set = HALVES == 2 ? __builtin_amdgcn_readfirstlane(threadIdx.x / (kAttnWaves * kWave)) : 0;
    DirectPageLds<HD>* lds = reinterpret_cast<DirectPageLds<HD>*>(smem_raw) + 2 * set;   // two buffers a set
    // Blocks start in the order of their index, round-robin over the 8 XCDs.  Block L is the
    // m-th block of XCD x (L = 8 m + x); an XCD takes the `group` query heads of one (tile, kv
    // head) pair one after the other, so that the pair's pages stay in its L2, and the pairs go
    // from the last tile to the first: late tiles of a causal prompt see the most keys, and
    // starting with them keeps the compute units evenly busy to the end.
    // A grid of at most two blocks per compute unit starts all at once, and the m-th and the
    // (m + 32)-th block of an XCD share a compute unit: the second half runs in rising order
    // then, so that the longest block shares with the shortest.
    int m_xcd = blockIdx.x / 8;
    const int xcd = blockIdx.x % 8, per_xcd = gridDim.x / 8;
    if (HALVES == 1 && per_xcd > 32 && per_xcd <= 64 && m_xcd >= 32) m_xcd = per_xcd - 1 - (m_xcd - 32);
    const int pair = (m_xcd / group) * 8 + xcd;
    if (pair >= n_tiles * n_kv_heads) return;
    const int kvh = pair % n_kv_heads, h = kvh * group + m_xcd % group;
    int tile = n_tiles - 1 - pair / n_kv_heads, b = 0, first = 0;
    for (; b < batch; ++b) {
        const int len = cu[b + 1] - cu[b];
        const int tiles = (len + kTileRows - 1) / kTileRows;
        if (tile < tiles) { first = cu[b] + tile * kTileRows; break; }
        tile -= tiles;
    }
    if (b >= batch) return;
    const int lane = threadIdx.x & (kWave - 1);
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / kWave) % kAttnWaves;   // within its set
    const int c = lane & 15, g = lane >> 4;
    const int seq_end = cu[b + 1];
    const int tile_rows = min(kTileRows, seq_end - first);
    const int tile_last_pos = tok_pos[first + tile_rows - 1];
    const int tile_first_pos = tok_pos[first];
    const int written = tok_pos[seq_end - 1] + 1;
    const int row0 = first + 32 * wave;
    const int wave_rows = max(0, min(32, seq_end - row0));
    const bool ok0 = c < wave_rows, ok1 = 16 + c < wave_rows;
    const int q_pos0 = ok0 ? tok_pos[row0 + c] : -1, q_pos1 = ok1 ? tok_pos[row0 + 16 + c] : -1;
    bf16x8 qf0[HD / 32], qf1[HD / 32];
    {
        const bf16_t* qrow0 = q + (size_t)(row0 + (ok0 ? c : 0)) * q_stride + (size_t)h * HD + 8 * g;
        const bf16_t* qrow1 = q + (size_t)(row0 + (ok1 ? 16 + c : 0)) * q_stride + (size_t)h * HD + 8 * g;
#pragma unroll
        for (int sk = 0; sk < HD / 32; ++sk) {
            qf0[sk] = ok0 ? ld_frag(qrow0 + 32 * sk) : zero_frag();
            qf1[sk] = ok1 ? ld_frag(qrow1 + 32 * sk) : zero_frag();
        }
    }
    WaveState<HD> st0, st1;
    st0.init();
    st1.init();
    const int wave_first_pos = wave_rows > 0 ? tok_pos[row0] : 0;
    const int wave_last_pos = wave_rows > 0 ? tok_pos[row0 + wave_rows - 1] : -1;
    const float scale_log2 = scale * kLog2e;

    const int n_pages = tile_last_pos / kPageTokens + 1;
    auto page_needed = [&](int pi) {
        return page_may_be_visible_to_range(tile_first_pos, tile_last_pos, pi * kPageTokens, window, sinks);
    };
    auto next_needed = [&](int pi) {
        ++pi;
        while (pi < n_pages && !page_needed(pi)) ++pi;
        return pi;
    };
    auto page_id = [&](int pi) { return table[(size_t)b * table_stride + pi]; };
    auto page_base = [&](int id) { return ((size_t)id * n_kv_heads + kvh) * kPageTokens * HD; };
    // This wave's share of a page's copy, in instructions of 1 KB (64 lanes x 16 bytes, a fragment):
    // the block's instructions go to its waves in turn.
    auto copy_page = [&](int id, DirectPageLds<HD>& pg) {
        const bf16_t* kpage = k_pool + page_base(id);
        const bf16_t* vpage = v_pool + page_base(id);
#pragma unroll
        for (int j = 0; j < HD / 8 / kAttnWaves; ++j) {
            const int f = kAttnWaves * j + wave;
            __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)(kpage + 512 * f + 8 * lane),
                                             (__attribute__((address_space(3))) void*)&pg.k[f][0], 16, 0, 0);
        }
#pragma unroll
        for (int j = 0; j < HD / 8 / kAttnWaves; ++j) {
            const int f = kAttnWaves * j + wave;
            __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)(vpage + 512 * f + 8 * lane),
                                             (__attribute__((address_space(3))) void*)&pg.v[f][0], 16, 0, 0);
        }
    };
    // The values of tokens that have not been written may be anything, also NaN, and 0 * NaN is
    // NaN: in the one page of a sequence that is not full they are zeroed in LDS after the copy.
    // Every lane does so with the pieces it copied itself, once they have arrived and before the
    // block's barrier (one barrier a page, whatever the page: the two sets of HALVES = 2 are at
    // different pages and must meet the same barriers).
    auto zero_unwritten = [&](DirectPageLds<HD>& pg, int valid_keys) {
#pragma unroll
        for (int j = 0; j < HD / 8 / kAttnWaves; ++j) {
            const int f = kAttnWaves * j + wave;
            const int keep = valid_keys - 16 * (lane >> 4) - 8 * (f & 1);          // of the tokens this piece holds
            if (keep >= 8) continue;
            uint4* at = reinterpret_cast<uint4*>(&pg.v[f][8 * lane]);
            *at = __builtin_bit_cast(uint4, keep_first(__builtin_bit_cast(bf16x8, *at), keep));
        }
    };
    auto land = [&](int pi, DirectPageLds<HD>& pg) {                        // the copy of page pi is complete and visible
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        const int valid_keys = written - pi * kPageTokens;
        if (pi < n_pages && valid_keys < kPageTokens) zero_unwritten(pg, valid_keys);
        __syncthreads();
    };
    // The pages that are needed go to the sets in turn.  `lead` is the first set's page: every
    // wave follows it, so that both sets go round the loop, and through its barriers, equally often.
    auto advance = [&](int pi) {
        pi = next_needed(pi);
        return HALVES == 2 ? next_needed(pi) : pi;
    };
    int lead = next_needed(-1);
    if (lead >= n_pages) return;                                         // cannot happen: a row sees itself
    int cur = set ? next_needed(lead) : lead;
    int nxt = advance(cur);
    int nxt_id = nxt < n_pages ? page_id(nxt) : 0;
    if (cur < n_pages) copy_page(page_id(cur), lds[0]);
    land(cur, lds[0]);
    int buf = 0;
    while (lead < n_pages) {
        const int nxt2 = advance(nxt);
        if (nxt < n_pages) copy_page(nxt_id, lds[buf ^ 1]);
        const int nxt2_id = nxt2 < n_pages ? page_id(nxt2) : 0;
        do {
        const int key0 = cur * kPageTokens;
        if (cur >= n_pages) break;                                        // the second set, after an odd number of pages
        if (wave_rows <= 0 || key0 > wave_last_pos) break;                // nothing of this page for this wave
        if (!page_may_be_visible_to_range(wave_first_pos, wave_last_pos, key0, window, sinks)) break;
        const DirectPageLds<HD>& pg = lds[buf];
        f32x4 s0[4], s1[4];
#pragma unroll
        for (int rb = 0; rb < 4; ++rb) {
            s0[rb] = f32x4{0.f, 0.f, 0.f, 0.f};
            s1[rb] = f32x4{0.f, 0.f, 0.f, 0.f};
        }
#pragma unroll
        for (int sk = 0; sk < HD / 32; ++sk) {
#pragma unroll
            for (int rb = 0; rb < 4; ++rb) {
                const bf16x8 kf = __builtin_bit_cast(bf16x8, *reinterpret_cast<const uint4*>(
                    &pg.k[rb * (HD / 32) + sk][8 * lane]));
                s0[rb] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(kf, qf0[sk], s0[rb], 0, 0, 0);
                s1[rb] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(kf, qf1[sk], s1[rb], 0, 0, 0);
            }
        }
        auto read_v = [&](int db, int t) {
            return __builtin_bit_cast(bf16x8, *reinterpret_cast<const uint4*>(&pg.v[2 * db + t][8 * lane]));
        };
        constexpr int kEarly = 2;
        bf16x8 vf[HD / 16][2];
#pragma unroll
        for (int db = 0; db < kEarly; ++db) { vf[db][0] = read_v(db, 0); vf[db][1] = read_v(db, 1); }
        bf16x8 pf0[2], pf1[2];
        float corr0, corr1;
        const bool all_visible = wave_rows == 32 &&
                                 page_fully_visible(wave_first_pos, wave_last_pos, key0, window, sinks);
        if (all_visible) {
            softmax_page<false, 16, 4, HD>(s0, st0, scale_log2, q_pos0, key0, window, sinks, pf0, corr0);
            softmax_page<false, 16, 4, HD>(s1, st1, scale_log2, q_pos1, key0, window, sinks, pf1, corr1);
        } else {
            softmax_page<true, 16, 4, HD>(s0, st0, scale_log2, q_pos0, key0, window, sinks, pf0, corr0);
            softmax_page<true, 16, 4, HD>(s1, st1, scale_log2, q_pos1, key0, window, sinks, pf1, corr1);
        }
        const bool rescale = __ballot(corr0 != 1.0f || corr1 != 1.0f) != 0;
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int db = 0; db < HD / 16; ++db) {
            if (db + kEarly < HD / 16) {
                vf[db + kEarly][0] = read_v(db + kEarly, 0);
                vf[db + kEarly][1] = read_v(db + kEarly, 1);
            }
            f32x4 a0 = st0.acc[db], a1 = st1.acc[db];
            if (rescale) {
#pragma unroll
                for (int r = 0; r < 4; ++r) { a0[r] *= corr0; a1[r] *= corr1; }
            }
#pragma unroll
            for (int t = 0; t < 2; ++t) {
                a0 = __builtin_amdgcn_mfma_f32_16x16x32_bf16(vf[db][t], pf0[t], a0, 0, 0, 0);
                a1 = __builtin_amdgcn_mfma_f32_16x16x32_bf16(vf[db][t], pf1[t], a1, 0, 0, 0);
            }
            st0.acc[db] = a0;
            st1.acc[db] = a1;
        }
        } while (0);
        land(nxt, lds[buf ^ 1]);
        cur = nxt;
        nxt = nxt2;
        nxt_id = nxt2_id;
        buf ^= 1;
        lead = advance(lead);
    }
    if (HALVES == 2) {
        // The second set's running maxima, sums and outputs go through LDS (lane by lane: the two
        // sets hold the same rows in the same lanes) and are added to the first set's.  The loop's
        // last barrier came after the last read of a page.
        constexpr int kStateFloats = 2 + HD / 4;
        float* state = reinterpret_cast<float*>(smem_raw) + (size_t)wave * (2 * kStateFloats * kWave) + lane;
        auto put = [&](const WaveState<HD>& st, float* at) {
            at[0] = st.m;
            at[kWave] = st.l;
#pragma unroll
            for (int db = 0; db < HD / 16; ++db)
#pragma unroll
                for (int r = 0; r < 4; ++r) at[(2 + 4 * db + r) * kWave] = st.acc[db][r];
        };
        auto add = [&](WaveState<HD>& st, const float* at) {
            const float m_other = at[0], l_other = at[kWave];
            const float m = fmaxf(st.m, m_other);
            const float mine = st.m == -INFINITY ? 0.f : __builtin_amdgcn_exp2f(st.m - m);
            const float theirs = m_other == -INFINITY ? 0.f : __builtin_amdgcn_exp2f(m_other - m);
            st.l = st.l * mine + l_other * theirs;
            st.m = m;
#pragma unroll
            for (int db = 0; db < HD / 16; ++db)
#pragma unroll
                for (int r = 0; r < 4; ++r) st.acc[db][r] = st.acc[db][r] * mine + at[(2 + 4 * db + r) * kWave] * theirs;
        };
        if (set == 1) {
            put(st0, state);
            put(st1, state + kStateFloats * kWave);
        }
        __syncthreads();
        if (set == 1) return;
        add(st0, state);
        add(st1, state + kStateFloats * kWave);
    }
    auto write_out = [&](const WaveState<HD>& st, int rr) {
        if (rr >= wave_rows) return;
        const float inv = st.l > 0.f ? 1.0f / st.l : 0.f;
        bf16_t* orow = out + ((size_t)(row0 + rr) * n_heads + h) * HD;
#pragma unroll
        for (int db = 0; db < HD / 16; ++db) {
            uint2 u;
            u.x = pack_bf16(st.acc[db][0] * inv, st.acc[db][1] * inv);
            u.y = pack_bf16(st.acc[db][2] * inv, st.acc[db][3] * inv);
            *reinterpret_cast<uint2*>(orow + 16 * db + 4 * g) = u;
        }
    };
    write_out(st0, c);
    write_out(st1, 16 + c);
}

// ---------------------------------------------------------------- entry points
static bool mfma_shape_ok(int n_heads, int n_kv_heads, int head_dim) {
    if (n_kv_heads <= 0 || n_heads % n_kv_heads) return false;
    return (head_dim == 64 || head_dim == 128) && n_heads / n_kv_heads <= 16;
}

// The classes of batch sizes: the sizes at which single-token steps are captured (a batch in
// between runs padded to the next of them).  Whatever a kernel's shape takes from the batch it
// takes from the class, or a sequence's sums would come in another order alone than beside
// others of its class.
LLOGOS_EXPORT int llogos_batch_class(int batch) {
    static const int classes[] = {1, 2, 3, 4, 5, 6, 7, 8, 12, 16, 24, 32, 48, 64};
    for (int c : classes) if (batch <= c) return c;
    return (batch + 63) / 64 * 64;
}

// compute units of the current device, asked for once per device
static int compute_units() {
    static int cached[64];
    int device = 0;
    if (hipGetDevice(&device) != hipSuccess || device < 0 || device >= 64) return 256;
    if (cached[device] == 0) {
        int n = 0;
        if (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, device) != hipSuccess || n <= 0) n = 256;
        cached[device] = n;
    }
    return cached[device];
}

constexpr int kDecodeWaves = 4;
constexpr int kMaxPagesPerWave = 16;

// Pages per wave.  A wave's pages come one after the other, a "step" each; a CU works on one
// block's waves at a time as far as timings show, so a launch takes about as many steps as the
// blocks that fall to the busiest CU have together: blocks of ppw steps go round by round over
// the CUs, the shorter last block of each sequence after them.  Every round of blocks costs a
// quarter of a step more (queries, merge through LDS), the merge kernel three quarters.  The
// count of steps is what 26 shapes measured at the 8B head shape (32 query heads, 8 kv heads of
// 128; batch 1 to 64, 640 to 131,000 positions) order by.  Against one page a wave in blocks of
// up to 16 waves: batch 64 at 640 positions 42.5 us from 46.2, at 8,192 361 from 417; batch 8
// at 32,768 192 from 211; batch 1 at 131,000 102 from 117; batch 32 at 640 25.1 from 23.6.
static int decode_pages_per_wave(int table_width, int batch, int n_kv_heads) {
    const long long pairs = (long long)llogos_batch_class(batch) * n_kv_heads;
    const long long units = compute_units();
    int best = 1;
    double best_cost = 0;
    for (int ppw = 1; ppw <= kMaxPagesPerWave; ++ppw) {
        const int chunk = kDecodeWaves * ppw;
        const long long full = table_width / chunk;                       // whole blocks of a sequence
        const int rest = table_width % chunk;                             // pages of its last, shorter block
        const long long full_rounds = (pairs * full + units - 1) / units;
        double steps = (double)full_rounds * ppw, rounds = (double)full_rounds;
        if (rest > 0) {
            const long long room = full_rounds * units - pairs * full;    // places the last round of whole blocks leaves
            const long long more = pairs > room ? (pairs - room + units - 1) / units : 0;
            // (blocks a quarter as long as the whole ones, or less, run beside the last of those: half a step each)
            const int rest_steps = (rest + kDecodeWaves - 1) / kDecodeWaves;
            steps += (double)more * rest_steps * (full > 0 && 4 * rest_steps <= ppw ? 0.5 : 1.0);
            rounds += (double)more;
        }
        const double cost = steps + 0.25 * rounds + (full + (rest > 0) > 1 ? 0.75 : 0.0);
        if (ppw == 1 || cost < best_cost - 1e-9) { best = ppw; best_cost = cost; }
    }
    return best;
}

// floats the decode workspace needs
LLOGOS_EXPORT long long llogos_attn_decode_workspace(int batch, int n_heads, int n_kv_heads, int head_dim,
                                                     int table_width) {
    if (n_kv_heads <= 0 || n_heads % n_kv_heads) return 0;
    const int ppw = decode_pages_per_wave(table_width, batch, n_kv_heads);
    const int n_z = (table_width + kDecodeWaves * ppw - 1) / (kDecodeWaves * ppw);
    return n_z == 1 ? 0 : (long long)batch * n_heads * n_z * (head_dim + 2);
}

static int launch_decode(void* out, const void* q, int q_stride, const QkvSource* src, const void* k_pool,
                         const void* v_pool, const int* table, int table_stride, int table_width,
                         const int* tok_pos, int batch, int n_heads, int n_kv_heads, int head_dim,
                         float scale, int window, int sinks, float* workspace, long long workspace_floats,
                         hipStream_t stream) {
    if (batch <= 0 || table_width <= 0 || window < 0 || sinks < 0) return LLOGOS_BAD_ARGUMENT;
    if (!mfma_shape_ok(n_heads, n_kv_heads, head_dim)) return LLOGOS_UNSUPPORTED;
    if (workspace_floats < llogos_attn_decode_workspace(batch, n_heads, n_kv_heads, head_dim, table_width))
        return LLOGOS_BAD_ARGUMENT;
    const int group = n_heads / n_kv_heads;
    const int waves = kDecodeWaves, ppw = decode_pages_per_wave(table_width, batch, n_kv_heads);
    const int n_z = (table_width + waves * ppw - 1) / (waves * ppw);
    if (n_z > 1 && workspace == nullptr) return LLOGOS_BAD_ARGUMENT;
    dim3 grid(batch, n_kv_heads, n_z), mgrid(batch, n_heads);
    const size_t smem = decode_lds_bytes(waves, group, head_dim);
    const QkvSource none{};
#define GO(HD, FUSED) do { \
    attn_decode_kernel<HD, kDecodeWaves, FUSED><<<grid, kDecodeWaves * kWave, smem, stream>>>( \
        (bf16_t*)out, workspace, (const bf16_t*)q, q_stride, FUSED ? *src : none, (const bf16_t*)k_pool, \
        (const bf16_t*)v_pool, table, table_stride, tok_pos, n_heads, n_kv_heads, group, scale, window, sinks, ppw); \
    if (n_z > 1) attn_decode_merge_kernel<HD><<<mgrid, kMergeLanes * HD, 0, stream>>>((bf16_t*)out, workspace, tok_pos, n_heads, \
                                                                        n_z, kDecodeWaves * ppw); } while (0)
    if (src != nullptr && head_dim == 64) GO(64, true);
    else if (src != nullptr) GO(128, true);
    else if (head_dim == 64) GO(64, false);
    else GO(128, false);
#undef GO
    return LLOGOS_LAUNCH_CHECK();
}

LLOGOS_EXPORT int llogos_attn_decode_bf16(void* out, const void* q, int q_stride, const void* k_pool,
                                          const void* v_pool, const int* table, int table_stride, int table_width,
                                          const int* tok_pos, int batch, int n_heads, int n_kv_heads, int head_dim,
                                          float scale, int window, int sinks, float* workspace,
                                          long long workspace_floats, hipStream_t stream) {
    if ((q_stride % 8) || ((uintptr_t)q % 16)) return LLOGOS_UNSUPPORTED;
    return launch_decode(out, q, q_stride, nullptr, k_pool, v_pool, table, table_stride, table_width, tok_pos, batch,
                         n_heads, n_kv_heads, head_dim, scale, window, sinks, workspace, workspace_floats, stream);
}

// ---------------------------------------------------------------- decode without allocation
// The decode attention for callers that cannot allocate (see llogos_api.h).  The partial
// results of the blocks along the context, which llogos_attn_decode_bf16 takes in a workspace
// from its caller, live in a file-scope device array here.  In host code the array's name is
// only a stand-in for the symbol: its device address is asked for once per device, with that
// device current, and that pointer is what the kernels, and anything else on the host, get.
constexpr long long kStaticScratchFloats = 4ll << 20;                  // 16 MiB on each GPU the library runs on
static __device__ __align__(256) float scratch[kStaticScratchFloats];
constexpr int kMaxDevices = 64;
static float* scratch_ptr[kMaxDevices];                                // per device; null until asked for
static std::mutex scratch_mutex;

// The current device's copy of the array, through *ptr.
static int static_scratch(float** ptr) {
    int device = -1;
    hipError_t e = hipGetDevice(&device);
    if (e != hipSuccess) return (int)e;
    if (device < 0 || device >= kMaxDevices) return LLOGOS_BAD_ARGUMENT;
    std::lock_guard<std::mutex> hold(scratch_mutex);
    if (scratch_ptr[device] == nullptr) {
        float* p = nullptr;
        e = hipGetSymbolAddress((void**)&p, HIP_SYMBOL(scratch));
        if (e != hipSuccess) return (int)e;
        if (p == nullptr) return (int)hipErrorInvalidSymbol;
        scratch_ptr[device] = p;
    }
    *ptr = scratch_ptr[device];
    return 0;
}

LLOGOS_EXPORT long long llogos_attn_decode_static_capacity(void) { return kStaticScratchFloats; }

LLOGOS_EXPORT int llogos_attn_decode_static_init(void) {
    float* p = nullptr;
    return static_scratch(&p);
}

LLOGOS_EXPORT int llogos_attn_decode_static_bf16(void* out, const void* q, int q_stride, const void* k_pool,
                                                 const void* v_pool, const int* table, int table_stride,
                                                 int table_width, const int* tok_pos, int batch, int n_heads,
                                                 int n_kv_heads, int head_dim, float scale, int window, int sinks,
                                                 hipStream_t stream) {
    if ((q_stride % 8) || ((uintptr_t)q % 16)) return LLOGOS_UNSUPPORTED;
    if (batch <= 0 || table_width <= 0) return LLOGOS_BAD_ARGUMENT;
    if (!mfma_shape_ok(n_heads, n_kv_heads, head_dim)) return LLOGOS_UNSUPPORTED;
    // Nothing in the array has to start at zero: the merge kernel reads only the partial results
    // that this call's blocks have written (blocks z < ceil(pages / pages per block) of each
    // sequence), so what an earlier call left is never looked at.
    const long long need = llogos_attn_decode_workspace(batch, n_heads, n_kv_heads, head_dim, table_width);
    if (need > kStaticScratchFloats) return LLOGOS_TOO_LARGE;
    float* ws = nullptr;
    const int code = static_scratch(&ws);
    if (code != 0) return code;
    return launch_decode(out, q, q_stride, nullptr, k_pool, v_pool, table, table_stride, table_width, tok_pos, batch,
                         n_heads, n_kv_heads, head_dim, scale, window, sinks, ws, kStaticScratchFloats, stream);
}

// The same from the fused projection (see QkvSource): head sizes 64 and 128; also writes the
// step's keys and values to their pages.  cs: [batch][head size / 2][2] floats.
LLOGOS_EXPORT int llogos_attn_decode_fused_bf16(void* out, const float* qkv, int parts, long long part_stride,
                                                int row_stride, const float* bias, const float* q_norm_w,
                                                const float* k_norm_w, float eps, const void* cs, void* k_pool,
                                                void* v_pool, const int* table, int table_stride, int table_width,
                                                const int* tok_pos, int batch, int n_heads, int n_kv_heads,
                                                int head_dim, float scale, int window, int sinks, float* workspace,
                                                long long workspace_floats, hipStream_t stream) {
    if (head_dim != 128 && head_dim != 64) return LLOGOS_UNSUPPORTED;
    if (parts < 1 || (row_stride % 2) || (part_stride % 2) || ((uintptr_t)qkv % 8) ||
        row_stride < (n_heads + 2 * n_kv_heads) * head_dim)
        return LLOGOS_BAD_ARGUMENT;
    const QkvSource src{qkv, parts, (size_t)part_stride, row_stride, bias, q_norm_w, k_norm_w, eps,
                        (const float2*)cs, (bf16_t*)k_pool, (bf16_t*)v_pool};
    return launch_decode(out, nullptr, 0, &src, k_pool, v_pool, table, table_stride, table_width, tok_pos, batch,
                         n_heads, n_kv_heads, head_dim, scale, window, sinks, workspace, workspace_floats, stream);
}

// tile_rows: 64 for the kernel whose waves read pages from global memory, 128 for the kernel
// that shares pages through LDS (n_tiles counts tiles of that many tokens per sequence).
LLOGOS_EXPORT int llogos_attn_prefill_bf16(void* out, const void* q, int q_stride, const void* k_pool,
                                           const void* v_pool, const int* table, int table_stride,
                                           const int* cu, const int* tok_pos, int batch, int n_tiles, int tile_rows,
                                           int n_heads, int n_kv_heads, int head_dim,
                                           float scale, int window, int sinks, int halves, hipStream_t stream) {
    if (batch <= 0 || n_tiles <= 0 || window < 0 || sinks < 0 || (halves != 1 && halves != 2)) return LLOGOS_BAD_ARGUMENT;
    if (tile_rows != 64 && tile_rows != kTileRows) return LLOGOS_BAD_ARGUMENT;
    if (!mfma_shape_ok(n_heads, n_kv_heads, head_dim) || (q_stride % 8) || ((uintptr_t)q % 16)) return LLOGOS_UNSUPPORTED;
    const int group = n_heads / n_kv_heads;
    dim3 grid(n_tiles, n_heads);
    if (tile_rows == kTileRows) {
        const long long pairs = (long long)n_tiles * n_kv_heads;
        const dim3 lgrid((unsigned)((pairs + 7) / 8 * 8 * group));
#define GOD(HD, HALVES) do { \
        const size_t smem = HALVES * 2 * sizeof(DirectPageLds<HD>); \
        hipError_t e = hipFuncSetAttribute((const void*)attn_prefill_direct_kernel<HD, HALVES>, \
                                           hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem); \
        if (e != hipSuccess) return (int)e; \
        attn_prefill_direct_kernel<HD, HALVES><<<lgrid, HALVES * kAttnWaves * kWave, smem, stream>>>( \
            (bf16_t*)out, (const bf16_t*)q, q_stride, (const bf16_t*)k_pool, (const bf16_t*)v_pool, table, table_stride, \
            cu, tok_pos, batch, n_tiles, n_heads, n_kv_heads, group, scale, window, sinks); \
        return LLOGOS_LAUNCH_CHECK(); } while (0)
        if (halves == 2) { if (head_dim == 64) GOD(64, 2); else GOD(128, 2); }
        if (head_dim == 64) GOD(64, 1); else GOD(128, 1);
#undef GOD
    }
#define GO(HD) attn_prefill_kernel<HD><<<grid, kAttnWaves * kWave, 0, stream>>>( \
        (bf16_t*)out, (const bf16_t*)q, q_stride, (const bf16_t*)k_pool, (const bf16_t*)v_pool, table, table_stride, \
        cu, tok_pos, batch, n_heads, n_kv_heads, group, scale, window, sinks)
    if (head_dim == 64) { GO(64); } else { GO(128); }
#undef GO
    return LLOGOS_LAUNCH_CHECK();
}
