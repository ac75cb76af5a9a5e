// out[M, N] = a[M, K] . w[N, K]^T (+ bias) for few rows (M <= 64) of bfloat16 activations:
// the decode step's matrix products, which are bound by streaming w from HBM once.
//
// Mapping to the hardware (gfx950, 64-wide waves, v_mfma_f32_16x16x32_bf16):
//  * a wave owns a strip of RB * 16 rows of w and a range of k.  Each lane loads 16 bytes of
//    a row straight from global memory into the matrix-core operand layout (lane = row +
//    16 * k-group), several loads in flight before the first MFMA;
//  * the activations are the other operand (M padded to MB * 16 columns); they are small,
//    come from L2, and one activation fragment serves the RB row blocks of the strip;
//  * the 4 waves of a block split the block's k range and add their sums through LDS;
//  * when k is split over blocks as well, each block writes its float32 partial sums to
//    out[split][M][N] and the kernel that consumes the product adds the parts in a fixed
//    order (a fence between blocks would cost a write-back of the whole L2 on this chip).
// Every output element sums k in an order that depends on N and K alone, never on M.
// (reference: one-row dequant_matmul_bf16, Daisi.Llogos.Cuda/kernels/dequant_matmul.cu:593-619,
//  one row of w per block with FP32 accumulation.)
#include "common.h"

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float f32x4 __attribute__((ext_vector_type(4)));

constexpr int kSkinnyWaves = 4;
constexpr int kStepK = 32;

__device__ __forceinline__ bf16x8 load_frag(const bf16_t* p, bool ok) {
    uint4 v = make_uint4(0, 0, 0, 0);
    if (ok) v = *reinterpret_cast<const uint4*>(p);
    return __builtin_bit_cast(bf16x8, v);
}

template <int RB, int MB, int U, typename TO>
__global__ __launch_bounds__(kSkinnyWaves * kWave) void gemm_skinny_kernel(
        TO* __restrict__ out, const bf16_t* __restrict__ a, const bf16_t* __restrict__ w,
        const float* __restrict__ bias, int M, int N, int K, int lda, int ldo, size_t part_stride,
        int k_per_block) {
    __shared__ float red[kSkinnyWaves][RB * MB][kWave][4];
    const int lane = threadIdx.x & (kWave - 1), wave = threadIdx.x / kWave;
    const int r = lane & 15, g = lane >> 4;
    const int split = blockIdx.y;
    const int n0 = blockIdx.x * (16 * RB);
    const int k_per_wave = k_per_block / kSkinnyWaves;
    const int k_begin = split * k_per_block + wave * k_per_wave;
    const int k_end = min(K, k_begin + k_per_wave);

    const bf16_t* wrow[RB];
#pragma unroll
    for (int rb = 0; rb < RB; ++rb)                        // rows past N read a valid row, never stored
        wrow[rb] = w + (size_t)min(n0 + rb * 16 + r, N - 1) * K + g * 8;
    const bf16_t* arow[MB];
    bool a_ok[MB];
#pragma unroll
    for (int mb = 0; mb < MB; ++mb) {
        const int m = mb * 16 + r;
        a_ok[mb] = m < M;
        arow[mb] = a + (size_t)min(m, M - 1) * lda + g * 8;
    }
    f32x4 acc[RB][MB];
#pragma unroll
    for (int rb = 0; rb < RB; ++rb)
#pragma unroll
        for (int mb = 0; mb < MB; ++mb) acc[rb][mb] = f32x4{0.f, 0.f, 0.f, 0.f};

    // two register buffers of U steps each: the loads of the next U steps are in flight while
    // the matrix cores work on the current ones
    bf16x8 wf0[U][RB], af0[U][MB], wf1[U][RB], af1[U][MB];
    auto load = [&](bf16x8 (&wf)[U][RB], bf16x8 (&af)[U][MB], int k) {
#pragma unroll
        for (int u = 0; u < U; ++u) {
            const int kk = k + u * kStepK;
            const bool ok = kk + g * 8 < k_end;           // K % 8 == 0: a 16-byte load is in or out as a whole
#pragma unroll
            for (int rb = 0; rb < RB; ++rb) wf[u][rb] = load_frag(wrow[rb] + kk, ok);
#pragma unroll
            for (int mb = 0; mb < MB; ++mb) af[u][mb] = load_frag(arow[mb] + kk, ok && a_ok[mb]);
        }
    };
    auto multiply = [&](const bf16x8 (&wf)[U][RB], const bf16x8 (&af)[U][MB]) {
#pragma unroll
        for (int u = 0; u < U; ++u)
#pragma unroll
            for (int rb = 0; rb < RB; ++rb)
#pragma unroll
                for (int mb = 0; mb < MB; ++mb)
                    acc[rb][mb] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wf[u][rb], af[u][mb], acc[rb][mb], 0, 0, 0);
    };
    constexpr int kChunk = kStepK * U;
    if (k_begin < k_end) load(wf0, af0, k_begin);
    for (int k = k_begin; k < k_end; k += 2 * kChunk) {
        const bool second = k + kChunk < k_end;
        if (second) load(wf1, af1, k + kChunk);
        multiply(wf0, af0);
        if (k + 2 * kChunk < k_end) load(wf0, af0, k + 2 * kChunk);
        if (second) multiply(wf1, af1);
    }

    // acc[rb][mb][i] = sum for row n0 + rb * 16 + 4 g + i of w and activation row mb * 16 + r
#pragma unroll
    for (int rb = 0; rb < RB; ++rb)
#pragma unroll
        for (int mb = 0; mb < MB; ++mb)
#pragma unroll
            for (int i = 0; i < 4; ++i) red[wave][rb * MB + mb][lane][i] = acc[rb][mb][i];
    __syncthreads();

    const int t_lane = threadIdx.x & (kWave - 1), t_i = threadIdx.x / kWave;   // 256 threads: one (lane, i) each
    TO* dst = out + (size_t)split * part_stride;
#pragma unroll
    for (int rb = 0; rb < RB; ++rb) {
        const int n = n0 + rb * 16 + 4 * (t_lane >> 4) + t_i;
#pragma unroll
        for (int mb = 0; mb < MB; ++mb) {
            float s = 0.f;
#pragma unroll
            for (int wv = 0; wv < kSkinnyWaves; ++wv) s += red[wv][rb * MB + mb][t_lane][t_i];
            const int m = mb * 16 + (t_lane & 15);
            if (m < M && n < N) store_f32(dst + (size_t)m * ldo + n, s + (bias ? bias[n] : 0.f));
        }
    }
}

// Third form, for up to 16 activation rows and very many rows of w (gate/up, the output head):
// the activations stay in registers.  The WAVES waves of a block split k; each wave loads its
// share of the activation fragments once (STEPS steps of 32 values of k = 4 STEPS registers)
// and then streams `strips` strips of 16 rows of w past them, so that the activations cost
// 1 / strips of what they cost when every strip fetches its own.  The waves' sums of a strip
// are added through LDS in wave order, as in the first form.  K <= 32 * STEPS * WAVES:
// 4 waves x 32 steps for K <= 4096, 8 x 20 for K <= 5120, 8 x 32 for K <= 8192.
constexpr int kStatU = 4;               // steps per prefetched chunk

template <typename TO, int WAVES, int STEPS>
__global__ __launch_bounds__(WAVES * kWave) void gemm_skinny_stationary_kernel(
        TO* __restrict__ out, const bf16_t* __restrict__ a, const bf16_t* __restrict__ w,
        const float* __restrict__ bias, int M, int N, int K, int lda, int ldo, int strips_per_block) {
    static_assert(STEPS % kStatU == 0, "whole chunks");
    __shared__ float red[WAVES][kWave][4];
    const int lane = threadIdx.x & (kWave - 1), wave = threadIdx.x / kWave;
    const int r = lane & 15, g = lane >> 4;
    const int k_per_wave = (((K + 31) / 32 + WAVES - 1) / WAVES) * 32;               // <= 32 * STEPS
    const int k_begin = wave * k_per_wave;
    const int k_end = min(K, k_begin + k_per_wave);
    constexpr int kChunks = STEPS / kStatU;

    // this wave's activation fragments, once
    bf16x8 af[STEPS];
    {
        const bool row_ok = r < M;
        const bf16_t* arow = a + (size_t)min(r, M - 1) * lda + g * 8;
#pragma unroll
        for (int s = 0; s < STEPS; ++s) {
            const int kk = k_begin + s * kStepK;
            af[s] = load_frag(arow + kk, row_ok && kk + g * 8 < k_end);
        }
    }
    const int n_strips = (N + 15) / 16;
    const int strip0 = blockIdx.x * strips_per_block;
    const int my_strips = min(strips_per_block, n_strips - strip0);
    if (my_strips <= 0) return;
    const int total = my_strips * kChunks;                               // chunks of kStatU steps to stream

    auto load_chunk = [&](bf16x8 (&wf)[kStatU], int gc) {
        const int strip = strip0 + gc / kChunks, c = gc % kChunks;
        const bf16_t* wrow = w + (size_t)min(strip * 16 + r, N - 1) * K + g * 8;
#pragma unroll
        for (int u = 0; u < kStatU; ++u) {
            const int kk = k_begin + (c * kStatU + u) * kStepK;
            wf[u] = load_frag(wrow + kk, gc < total && kk + g * 8 < k_end);
        }
    };
    f32x4 acc = f32x4{0.f, 0.f, 0.f, 0.f};
    auto multiply = [&](const bf16x8 (&wf)[kStatU], int c) {
        // the fragment index must be a constant for the registers: one case per chunk of the strip
#pragma unroll
        for (int cc = 0; cc < kChunks; ++cc)
            if (cc == c) {
#pragma unroll
                for (int u = 0; u < kStatU; ++u)
                    acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wf[u], af[cc * kStatU + u], acc, 0, 0, 0);
            }
    };
    auto finish_strip = [&](int strip) {
#pragma unroll
        for (int i = 0; i < 4; ++i) red[wave][lane][i] = acc[i];
        acc = f32x4{0.f, 0.f, 0.f, 0.f};
        __syncthreads();
        if (threadIdx.x < 4 * kWave) {                                   // one thread per value of the strip
            const int t_lane = threadIdx.x & (kWave - 1), t_i = threadIdx.x / kWave;
            float sum = 0.f;
#pragma unroll
            for (int wv = 0; wv < WAVES; ++wv) sum += red[wv][t_lane][t_i];
            const int n = strip * 16 + 4 * (t_lane >> 4) + t_i, m = t_lane & 15;
            if (m < M && n < N) store_f32(out + (size_t)m * ldo + n, sum + (bias ? bias[n] : 0.f));
        }
        __syncthreads();
    };

    bf16x8 wf0[kStatU], wf1[kStatU];
    load_chunk(wf0, 0);
    for (int gc = 0; gc < total; gc += 2) {
        load_chunk(wf1, gc + 1);
        multiply(wf0, gc % kChunks);
        if ((gc + 1) % kChunks == 0) finish_strip(strip0 + gc / kChunks);
        load_chunk(wf0, gc + 2);
        if (gc + 1 < total) {
            multiply(wf1, (gc + 1) % kChunks);
            if ((gc + 2) % kChunks == 0) finish_strip(strip0 + (gc + 1) / kChunks);
        }
    }
}

template <int WAVES, int STEPS>
static int launch_stationary(void* out, int out_dtype, const void* a, const void* w, const float* bias, int M, int N,
                             int K, int lda, int ldo, int strips_per_block, hipStream_t stream) {
    const int n_strips = (N + 15) / 16;
    const int blocks = (n_strips + strips_per_block - 1) / strips_per_block;
    if (out_dtype == DT_BF16)
        gemm_skinny_stationary_kernel<bf16_t, WAVES, STEPS><<<blocks, WAVES * kWave, 0, stream>>>(
            (bf16_t*)out, (const bf16_t*)a, (const bf16_t*)w, bias, M, N, K, lda, ldo, strips_per_block);
    else
        gemm_skinny_stationary_kernel<float, WAVES, STEPS><<<blocks, WAVES * kWave, 0, stream>>>(
            (float*)out, (const bf16_t*)a, (const bf16_t*)w, bias, M, N, K, lda, ldo, strips_per_block);
    return LLOGOS_LAUNCH_CHECK();
}

// The few-row product with stationary activations: M <= 16, K <= 8192.  One part, bias allowed.
LLOGOS_EXPORT int llogos_gemm_skinny_stationary_bf16(void* out, int out_dtype, const void* a, const void* w,
                                                     const float* bias, int M, int N, int K, int lda, int ldo,
                                                     int strips_per_block, hipStream_t stream) {
    if (M <= 0 || N <= 0 || K <= 0 || lda < K || ldo < N || strips_per_block < 1) return LLOGOS_BAD_ARGUMENT;
    if (out_dtype != DT_BF16 && out_dtype != DT_F32) return LLOGOS_BAD_ARGUMENT;
    if (M > 16 || K > 8192 || (K % 8) || (lda % 8) || ((uintptr_t)a % 16) || ((uintptr_t)w % 16))
        return LLOGOS_UNSUPPORTED;
    if (K <= 4096) return launch_stationary<4, 32>(out, out_dtype, a, w, bias, M, N, K, lda, ldo, strips_per_block, stream);
    if (K <= 5120) return launch_stationary<8, 20>(out, out_dtype, a, w, bias, M, N, K, lda, ldo, strips_per_block, stream);
    return launch_stationary<8, 32>(out, out_dtype, a, w, bias, M, N, K, lda, ldo, strips_per_block, stream);
}

template <int RB, int MB, int U>
static int launch_skinny(void* out, int out_dtype, const bf16_t* a, const bf16_t* w, const float* bias,
                         int M, int N, int K, int lda, int ldo, size_t part_stride, int k_per_block,
                         int k_splits, hipStream_t stream) {
    dim3 grid((N + 16 * RB - 1) / (16 * RB), k_splits);
    if (out_dtype == DT_BF16)
        gemm_skinny_kernel<RB, MB, U, bf16_t><<<grid, kSkinnyWaves * kWave, 0, stream>>>(
            (bf16_t*)out, a, w, bias, M, N, K, lda, ldo, part_stride, k_per_block);
    else
        gemm_skinny_kernel<RB, MB, U, float><<<grid, kSkinnyWaves * kWave, 0, stream>>>(
            (float*)out, a, w, bias, M, N, K, lda, ldo, part_stride, k_per_block);
    return LLOGOS_LAUNCH_CHECK();
}

// k range of one block for `splits` blocks along k: a multiple of 4 waves * 32.
static int k_per_block_for(int K, int splits) {
    const int unit = kSkinnyWaves * kStepK;
    return ((K + splits - 1) / splits + unit - 1) / unit * unit;
}

// The number of parts the product is written in for `splits` requested blocks along k
// (rounding k per block up can need fewer blocks than asked for).
LLOGOS_EXPORT int llogos_gemm_skinny_parts(int K, int splits) {
    if (K <= 0 || splits <= 1) return 1;
    const int kpb = k_per_block_for(K, splits);
    return (K + kpb - 1) / kpb;
}

// out: [parts][M][ldo] with parts = llogos_gemm_skinny_parts(K, splits); float32 when parts > 1
// (bias must then be left to the consumer).  row_blocks: 16-row blocks of w per wave (1, 2, 4).
// Returns LLOGOS_UNSUPPORTED for shapes this kernel does not take.
LLOGOS_EXPORT int llogos_gemm_skinny_bf16(void* out, int out_dtype, const void* a, const void* w,
                                          const float* bias, int M, int N, int K, int lda, int ldo,
                                          long long part_stride, int splits, int row_blocks,
                                          hipStream_t stream) {
    if (M <= 0 || N <= 0 || K <= 0 || lda < K || ldo < N || splits < 1) return LLOGOS_BAD_ARGUMENT;
    if (out_dtype != DT_BF16 && out_dtype != DT_F32) return LLOGOS_BAD_ARGUMENT;
    if (M > 64 || (K % 8) || (lda % 8) || ((uintptr_t)a % 16) || ((uintptr_t)w % 16)) return LLOGOS_UNSUPPORTED;
    const int parts = llogos_gemm_skinny_parts(K, splits);
    if (parts > 1 && (out_dtype != DT_F32 || bias != nullptr || part_stride < (long long)M * ldo))
        return LLOGOS_BAD_ARGUMENT;
    const int kpb = k_per_block_for(K, parts);
    const bf16_t* A = (const bf16_t*)a;
    const bf16_t* W = (const bf16_t*)w;
    const int mb = (M + 15) / 16;
#define GO(RB, MB, U) return launch_skinny<RB, MB, U>(out, out_dtype, A, W, bias, M, N, K, lda, ldo, \
                                                      (size_t)part_stride, kpb, parts, stream)
    if (mb == 1) {
        if (row_blocks >= 4) GO(4, 1, 2);
        if (row_blocks == 2) GO(2, 1, 4);
        GO(1, 1, 4);
    } else if (mb == 2) {
        if (row_blocks >= 4) GO(4, 2, 2);
        if (row_blocks == 2) GO(2, 2, 2);
        GO(1, 2, 4);
    } else {
        if (row_blocks >= 4) GO(4, 4, 1);
        if (row_blocks == 2) GO(2, 4, 2);
        GO(1, 4, 2);
    }
#undef GO
}
