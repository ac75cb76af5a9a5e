// What this GPU does at best, measured: reading a buffer from memory, and issuing bfloat16
// MFMAs (16x16x32 and 32x32x16) back to back.  The bench reports its kernels against these
// figures beside the published peaks.
#include "common.h"

typedef __attribute__((__vector_size__(8 * sizeof(__bf16)))) __bf16 bf16x8_m;
typedef __attribute__((__vector_size__(4 * sizeof(float)))) float f32x4_m;

// A block reads 4 KB of consecutive memory per load slot (16 bytes a thread), eight slots in
// flight (32 KB of consecutive memory a round), with loads that do not stay in the caches; blocks
// stride over the buffer.  Of the patterns tried on the MI355X this one reads fastest (4 GiB:
// 7.2 TB/s; cached loads 6.4; loads a whole grid apart 5.7).  Nothing is written unless the data
// has a value it cannot have, which keeps the loads alive.
typedef unsigned u32x4_m __attribute__((ext_vector_type(4)));
constexpr int kReadSlots = 8;

__global__ __launch_bounds__(256) void read_stream_kernel(const u32x4_m* __restrict__ src, long long n16,
                                                          unsigned* __restrict__ sink) {
    u32x4_m acc = {0, 0, 0, 0};
    const long long round = 256ll * kReadSlots;
    for (long long base = (long long)blockIdx.x * round; base < n16; base += (long long)gridDim.x * round) {
        u32x4_m v[kReadSlots];
#pragma unroll
        for (int u = 0; u < kReadSlots; ++u) {
            const long long i = base + 256ll * u + threadIdx.x;
            v[u] = i < n16 ? __builtin_nontemporal_load(src + i) : u32x4_m{0, 0, 0, 0};
        }
#pragma unroll
        for (int u = 0; u < kReadSlots; ++u) acc ^= v[u];
    }
    if ((acc.x & acc.y & acc.z & acc.w) == 0xFFFFFFFFu && acc.x + acc.y == 12345u) sink[0] = acc.x;
}

// blocks: how many blocks of 256 threads read (a few per compute unit)
LLOGOS_EXPORT int llogos_measure_read(const void* src, long long bytes, int blocks, unsigned* sink, hipStream_t stream) {
    if (src == nullptr || sink == nullptr || bytes < 16 || blocks <= 0 || ((uintptr_t)src % 16)) return LLOGOS_BAD_ARGUMENT;
    read_stream_kernel<<<blocks, 256, 0, stream>>>((const u32x4_m*)src, bytes / 16, sink);
    return LLOGOS_LAUNCH_CHECK();
}

// Each wave keeps eight independent accumulators and issues `iters` rounds of eight MFMAs
// (2 * 16 * 16 * 32 flops each) on operands that never change.
// noisy: operands of pseudo-random values in (-1, 1) (every bit of the mantissas toggles from lane to
// lane, as in real data) instead of a few small constants: the matrix cores' rate depends on it,
// the chip lowers its clock under the power of real data.
__device__ __forceinline__ float measure_value(unsigned seed, int noisy) {
    unsigned x = seed * 2654435761u + 12345u;
    x ^= x >> 15; x *= 2246822519u; x ^= x >> 13;
    return noisy ? ((float)(x & 0xffff) / 32768.0f - 1.0f) : 0.001f * (float)(seed % 7);
}

__global__ __launch_bounds__(256) void mfma_peak_kernel(float* __restrict__ out, int iters, int noisy) {
    bf16x8_m a, b;
#pragma unroll
    for (int i = 0; i < 8; ++i) {
        a[i] = (__bf16)measure_value(threadIdx.x * 16 + i, noisy);
        b[i] = (__bf16)measure_value(threadIdx.x * 16 + 8 + i + blockIdx.x * 4096, noisy);
    }
    f32x4_m acc[8];
#pragma unroll
    for (int j = 0; j < 8; ++j) acc[j] = f32x4_m{0.f, 0.f, 0.f, 0.f};
    for (int it = 0; it < iters; ++it) {
#pragma unroll
        for (int j = 0; j < 8; ++j) acc[j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b, acc[j], 0, 0, 0);
    }
    float s = 0.f;
#pragma unroll
    for (int j = 0; j < 8; ++j) s += acc[j][0] + acc[j][1] + acc[j][2] + acc[j][3];
    out[(size_t)blockIdx.x * 256 + threadIdx.x] = s;
}

// The same with v_mfma_f32_32x32x16_bf16 (2 * 32 * 32 * 16 flops each, four accumulators of 16 floats).
typedef __attribute__((__vector_size__(16 * sizeof(float)))) float f32x16_m;

__global__ __launch_bounds__(256) void mfma32_peak_kernel(float* __restrict__ out, int iters, int noisy) {
    bf16x8_m a, b;
#pragma unroll
    for (int i = 0; i < 8; ++i) {
        a[i] = (__bf16)measure_value(threadIdx.x * 16 + i, noisy);
        b[i] = (__bf16)measure_value(threadIdx.x * 16 + 8 + i + blockIdx.x * 4096, noisy);
    }
    f32x16_m acc[4];
#pragma unroll
    for (int j = 0; j < 4; ++j)
#pragma unroll
        for (int e = 0; e < 16; ++e) acc[j][e] = 0.f;
    for (int it = 0; it < iters; ++it) {
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, acc[j], 0, 0, 0);
    }
    float s = 0.f;
#pragma unroll
    for (int j = 0; j < 4; ++j) s += acc[j][0] + acc[j][5] + acc[j][10] + acc[j][15];
    out[(size_t)blockIdx.x * 256 + threadIdx.x] = s;
}

// out: blocks * 256 floats.  shape 16: v_mfma_f32_16x16x32_bf16, flops = blocks * 4 waves * iters * 8 * 16384;
// shape 32: v_mfma_f32_32x32x16_bf16, flops = blocks * 4 waves * iters * 4 * 32768.
LLOGOS_EXPORT int llogos_measure_mfma(float* out, int blocks, int iters, int shape, int noisy, hipStream_t stream) {
    if (out == nullptr || blocks <= 0 || iters <= 0 || (shape != 16 && shape != 32)) return LLOGOS_BAD_ARGUMENT;
    if (shape == 16) mfma_peak_kernel<<<blocks, 256, 0, stream>>>(out, iters, noisy);
    else mfma32_peak_kernel<<<blocks, 256, 0, stream>>>(out, iters, noisy);
    return LLOGOS_LAUNCH_CHECK();
}
