// What this GPU does at best, measured: reading a buffer from memory, and issuing
// v_mfma_f32_16x16x32_bf16 back to back.  The bench reports its kernels against these
// figures beside the published peaks.
#include "common.h"

typedef __attribute__((__vector_size__(8 * sizeof(__bf16)))) __bf16 bf16x8_m;
typedef __attribute__((__vector_size__(4 * sizeof(float)))) float f32x4_m;

// Every thread reads 16 bytes at a time, a block a contiguous 4 KiB, blocks striding over the
// buffer; four loads in flight per thread.  Nothing is written unless the data has a value it
// cannot have, which keeps the loads alive.
__global__ __launch_bounds__(256) void read_stream_kernel(const uint4* __restrict__ src, long long n16,
                                                          unsigned* __restrict__ sink) {
    const long long stride = (long long)gridDim.x * 256;
    long long i = (long long)blockIdx.x * 256 + threadIdx.x;
    uint4 acc = make_uint4(0, 0, 0, 0);
    for (; i + 3 * stride < n16; i += 4 * stride) {
        const uint4 a = src[i], b = src[i + stride], c = src[i + 2 * stride], d = src[i + 3 * stride];
        acc.x ^= a.x ^ b.x ^ c.x ^ d.x; acc.y ^= a.y ^ b.y ^ c.y ^ d.y;
        acc.z ^= a.z ^ b.z ^ c.z ^ d.z; acc.w ^= a.w ^ b.w ^ c.w ^ d.w;
    }
    for (; i < n16; i += stride) {
        const uint4 a = src[i];
        acc.x ^= a.x; acc.y ^= a.y; acc.z ^= a.z; acc.w ^= a.w;
    }
    if ((acc.x & acc.y & acc.z & acc.w) == 0xFFFFFFFFu && acc.x + acc.y == 12345u) sink[0] = acc.x;
}

// blocks: how many blocks of 256 threads read (a few per compute unit)
LLOGOS_EXPORT int llogos_measure_read(const void* src, long long bytes, int blocks, unsigned* sink, hipStream_t stream) {
    if (src == nullptr || sink == nullptr || bytes < 16 || blocks <= 0 || ((uintptr_t)src % 16)) return LLOGOS_BAD_ARGUMENT;
    read_stream_kernel<<<blocks, 256, 0, stream>>>((const uint4*)src, bytes / 16, sink);
    return LLOGOS_LAUNCH_CHECK();
}

// Each wave keeps eight independent accumulators and issues `iters` rounds of eight MFMAs
// (2 * 16 * 16 * 32 flops each) on operands that never change.
__global__ __launch_bounds__(256) void mfma_peak_kernel(float* __restrict__ out, int iters) {
    bf16x8_m a, b;
#pragma unroll
    for (int i = 0; i < 8; ++i) { a[i] = (__bf16)(0.001f * (float)(threadIdx.x % 7)); b[i] = (__bf16)(0.002f * (float)(threadIdx.x % 5)); }
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

// out: blocks * 256 floats.  flops done = blocks * 4 waves * iters * 8 * 16384.
LLOGOS_EXPORT int llogos_measure_mfma(float* out, int blocks, int iters, hipStream_t stream) {
    if (out == nullptr || blocks <= 0 || iters <= 0) return LLOGOS_BAD_ARGUMENT;
    mfma_peak_kernel<<<blocks, 256, 0, stream>>>(out, iters);
    return LLOGOS_LAUNCH_CHECK();
}
