// Shared device helpers for the gfx950 kernels: storage types, 64-wide wave
// reductions, the paged cache's address arithmetic.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#define LLOGOS_EXPORT extern "C" __attribute__((visibility("default")))

// element type codes shared with the Python side
enum { DT_F32 = 0, DT_BF16 = 1 };

// error codes returned by entry points (positive values are hipError_t)
enum { LLOGOS_BAD_ARGUMENT = -1, LLOGOS_UNSUPPORTED = -2, LLOGOS_TOO_LARGE = -3 };

constexpr int kWave = 64;        // CDNA wavefront
constexpr int kPageTokens = 64;  // tokens per cache page

typedef uint16_t bf16_t;

__device__ __forceinline__ float bf16_to_f32(bf16_t v) {
    return __uint_as_float(((uint32_t)v) << 16);
}

// round to nearest even; NaN stays NaN
__device__ __forceinline__ bf16_t f32_to_bf16(float f) {
    uint32_t u = __float_as_uint(f);
    if ((u & 0x7fffffffu) > 0x7f800000u) return (bf16_t)((u >> 16) | 0x40u);
    u += 0x7fffu + ((u >> 16) & 1u);
    return (bf16_t)(u >> 16);
}

template <typename T> __device__ __forceinline__ float load_f32(const T* p);
template <> __device__ __forceinline__ float load_f32<float>(const float* p) { return *p; }
template <> __device__ __forceinline__ float load_f32<bf16_t>(const bf16_t* p) { return bf16_to_f32(*p); }

template <typename T> __device__ __forceinline__ void store_f32(T* p, float v);
template <> __device__ __forceinline__ void store_f32<float>(float* p, float v) { *p = v; }
template <> __device__ __forceinline__ void store_f32<bf16_t>(bf16_t* p, float v) { *p = f32_to_bf16(v); }

__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
    for (int o = kWave / 2; o > 0; o >>= 1) v += __shfl_xor(v, o, kWave);
    return v;
}

__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
    for (int o = kWave / 2; o > 0; o >>= 1) v = fmaxf(v, __shfl_xor(v, o, kWave));
    return v;
}

// Sum over a block of up to 1024 threads; `red` holds at least 16 floats of LDS.
// Every thread gets the result.  The order of the additions is fixed by the block
// shape alone, so a row gives the same sum whatever else is in the batch.
__device__ __forceinline__ float block_sum(float v, float* red) {
    const int lane = threadIdx.x & (kWave - 1), wave = threadIdx.x / kWave;
    const int nwaves = (blockDim.x + kWave - 1) / kWave;
    v = wave_sum(v);
    __syncthreads();
    if (lane == 0) red[wave] = v;
    __syncthreads();
    float t = 0.f;
    for (int i = 0; i < nwaves; ++i) t += red[i];
    return t;
}

__device__ __forceinline__ float block_max(float v, float* red) {
    const int lane = threadIdx.x & (kWave - 1), wave = threadIdx.x / kWave;
    const int nwaves = (blockDim.x + kWave - 1) / kWave;
    v = wave_max(v);
    __syncthreads();
    if (lane == 0) red[wave] = v;
    __syncthreads();
    float t = red[0];
    for (int i = 1; i < nwaves; ++i) t = fmaxf(t, red[i]);
    return t;
}

// A layer's keys and values live in pages of kPageTokens tokens.  A sequence's pages are
// listed in its row of the step's page table.  pool[page][kv_head] is one kv head's part of a
// page: kPageTokens * head_dim elements, keys in one pool and values in another, laid out in
// the order in which the matrix cores take them as operands, so that a wave's load of a
// fragment (64 lanes x 8 elements) is one run of consecutive memory and every cache line that
// is fetched is used whole:
//   keys:   [block of 4 tokens rb = (t >> 2) & 3][8 dimensions d >> 3][row i = 4 (t >> 4) + (t & 3)][d & 7]
//           fragment (rb, d >> 5) holds, for lane (i, g), dimensions 32 (d >> 5) + 8 g .. + 7 of
//           token 16 (i >> 2) + 4 rb + (i & 3): after the four blocks' products S^T = K . Q^T, lane
//           group g holds the scores of tokens 16 g .. 16 g + 15.
//   values: [16 dimensions d >> 4][half (t >> 3) & 1][tokens t >> 4][d & 15][t & 7]
//           fragment (d >> 4, half) holds, for lane (i, g), tokens 16 g + 8 half .. + 7 of
//           dimension 16 (d >> 4) + i: the first operand of O^T += V^T . P^T.
// head_dim is a multiple of 16.
__host__ __device__ __forceinline__ int page_key_offset(int token, int d, int head_dim) {
    return ((((token >> 2) & 3) * (head_dim >> 3) + (d >> 3)) * 16 + (((token >> 4) << 2) | (token & 3))) * 8 + (d & 7);
}

__host__ __device__ __forceinline__ int page_value_offset(int token, int d) {
    return ((((d >> 4) * 2 + ((token >> 3) & 1)) * 4 + (token >> 4)) * 16 + (d & 15)) * 8 + (token & 7);
}

struct PagedKV {
    const int* table;      // [batch, table_stride] page ids of this step's sequences
    int table_stride;
    int n_kv_heads;
    int head_dim;
};

// offset of the kv head's part of the page that holds position pos of sequence seq
__device__ __forceinline__ size_t paged_base(const PagedKV& c, int seq, int kv_head, int pos) {
    const int page = c.table[(size_t)seq * c.table_stride + pos / kPageTokens];
    return ((size_t)page * c.n_kv_heads + kv_head) * kPageTokens * c.head_dim;
}

// A query at q_pos sees key k_pos when it is not in the future and, with a window,
// is one of the first `sinks` positions or one of the last `window` ones.
__device__ __forceinline__ bool key_visible(int q_pos, int k_pos, int window, int sinks) {
    if (k_pos > q_pos) return false;
    if (window <= 0) return true;
    return k_pos < sinks || k_pos > q_pos - window;
}

#define LLOGOS_LAUNCH_CHECK() (int)hipGetLastError()
