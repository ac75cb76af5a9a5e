// out[M, N] = a[M, K] . w[N, K]^T for few rows (M <= 128), second form: the activations are
// staged in LDS and shared by all waves of a block.
//
// The address path of a compute unit handles a fixed number of lanes per clock, so in the
// first form (gemm_skinny_bf16.hip), where every wave fetches its own copy of the activation
// fragments, those fetches take up to as many slots as the weights themselves.  Here
//  * the 4 waves of a block own 4 * RB * 16 different rows of w and walk the same range of k;
//  * the block copies the activations of that range, 256 values of k at a time, with full
//    16-byte-per-lane loads into LDS (two buffers; the copy of the next chunk is in flight
//    while the current one is multiplied), and the waves read their second MFMA operand
//    from LDS (rows are padded by 32 bytes: with a row stride of 32 bytes modulo 64 a wave's
//    16-byte reads of 16 rows take 4 clocks, free of bank conflicts by the hardware's counters;
//    a stride of 16 modulo 32 takes 8);
//  * each wave loads its weights straight from global memory into the MFMA operand layout,
//    a whole chunk ahead;
//  * an activation "producer" can be fused into the copy: SwiGLU of the (partial) gate/up
//    product, so that silu(g) * u never goes to memory.
// Outputs are written as [parts][M][N] like the first form's (parts = blocks along k).
// The order of a row's additions depends on N and K alone.
#include "common.h"

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef float f32x2 __attribute__((ext_vector_type(2)));
typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));

constexpr int kLdsWaves = 4;                 // waves per block (8 measured no faster)
constexpr int kChunkK = 256;                 // values of k per LDS chunk (128 and 512 measured no faster)
constexpr int kChunkSteps = kChunkK / 32;    // MFMA steps per chunk
constexpr int kLdsMaxRows = 128;            // rows of activations (64 with a fused producer)
constexpr int kRowPad = 16;                  // bf16 of padding per LDS row (32 bytes)

enum { PRODUCE_PLAIN = 0, PRODUCE_SWIGLU_F32 = 1, PRODUCE_SWIGLU_BF16 = 2 };

struct ActSource {
    const void* ptr;        // plain: bf16 [M][lda]; swiglu: [parts][M][2 K] float32 or bf16
    int lda;                // plain: row stride in elements; swiglu: 2 K
    int parts;              // swiglu: partial products to add
    size_t part_stride;     // elements between parts
};

// eight consecutive activations (k .. k + 7 of row m) as bf16
template <int MODE>
__device__ __forceinline__ uint4 produce8(const ActSource& src, int m, int k, int K) {
    if (MODE == PRODUCE_PLAIN) {
        return *reinterpret_cast<const uint4*>((const bf16_t*)src.ptr + (size_t)m * src.lda + k);
    } else {
        float g[8], u[8];
        if (MODE == PRODUCE_SWIGLU_F32) {
            const float* base = (const float*)src.ptr + (size_t)m * src.lda + k;
#pragma unroll
            for (int e = 0; e < 8; ++e) { g[e] = 0.f; u[e] = 0.f; }
            for (int p = 0; p < src.parts; ++p) {
                const float4* gp = reinterpret_cast<const float4*>(base + p * src.part_stride);
                const float4* up = reinterpret_cast<const float4*>(base + p * src.part_stride + K);
                const float4 g0 = gp[0], g1 = gp[1], u0 = up[0], u1 = up[1];
                g[0] += g0.x; g[1] += g0.y; g[2] += g0.z; g[3] += g0.w;
                g[4] += g1.x; g[5] += g1.y; g[6] += g1.z; g[7] += g1.w;
                u[0] += u0.x; u[1] += u0.y; u[2] += u0.z; u[3] += u0.w;
                u[4] += u1.x; u[5] += u1.y; u[6] += u1.z; u[7] += u1.w;
            }
        } else {
            const bf16_t* base = (const bf16_t*)src.ptr + (size_t)m * src.lda + k;
            const uint4 gv = *reinterpret_cast<const uint4*>(base);
            const uint4 uv = *reinterpret_cast<const uint4*>(base + K);
            const uint32_t gw[4] = {gv.x, gv.y, gv.z, gv.w}, uw[4] = {uv.x, uv.y, uv.z, uv.w};
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                g[2 * j] = __uint_as_float(gw[j] << 16); g[2 * j + 1] = __uint_as_float(gw[j] & 0xffff0000u);
                u[2 * j] = __uint_as_float(uw[j] << 16); u[2 * j + 1] = __uint_as_float(uw[j] & 0xffff0000u);
            }
        }
        // silu(g) * u with the hardware's exp2 and reciprocal (about 1 ulp each, far below the
        // rounding to bfloat16 that follows); every block of a column of blocks repeats this work,
        // so it has to be cheap
        uint32_t o[4];
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const float a = g[2 * j] * __builtin_amdgcn_rcpf(1.0f + __builtin_amdgcn_exp2f(-1.4426950408889634f * g[2 * j])) * u[2 * j];
            const float b = g[2 * j + 1] * __builtin_amdgcn_rcpf(1.0f + __builtin_amdgcn_exp2f(-1.4426950408889634f * g[2 * j + 1])) * u[2 * j + 1];
            const f32x2 ab = {a, b};
            o[j] = __builtin_bit_cast(uint32_t, __builtin_convertvector(ab, bf16x2));
        }
        return make_uint4(o[0], o[1], o[2], o[3]);
    }
}

template <int RB, int MB, int MODE, typename TO, int CHUNK>
__global__ __launch_bounds__(kLdsWaves * kWave) void gemm_skinny_lds_kernel(
        TO* __restrict__ out, ActSource src, const bf16_t* __restrict__ w, const float* __restrict__ bias,
        int M, int N, int K, int ldo, size_t part_stride, int k_per_block, int parts) {
    constexpr int kRows = MB * 16;
    constexpr int kRowLen = CHUNK + kRowPad;
    constexpr int kPieces = kRows * (CHUNK / 8);                    // 16-byte pieces of a chunk
    constexpr int kPiecesPerThread = (kPieces + kLdsWaves * kWave - 1) / (kLdsWaves * kWave);
    __shared__ __attribute__((aligned(16))) bf16_t lds[2][kRows][kRowLen];

    const int lane = threadIdx.x & (kWave - 1), wave = threadIdx.x / kWave;
    const int r = lane & 15, g = lane >> 4;
    // Blocks go to the 8 XCDs in turn, each with an L2 of its own: a block's part of k is its
    // index modulo the parts, so that an XCD sees few parts and its L2 keeps their activations
    // (with 8 parts one each) while the weights stream through.
    const int split = blockIdx.x % parts, n_block = blockIdx.x / parts;
    const int n0 = (n_block * kLdsWaves + wave) * (16 * RB);
    const int k_begin = split * k_per_block;
    const int k_end = min(K, k_begin + k_per_block);
    const int n_chunks = (k_end - k_begin + CHUNK - 1) / CHUNK;

    const bf16_t* wrow[RB];
#pragma unroll
    for (int rb = 0; rb < RB; ++rb)                                   // rows past N read a valid row, never stored
        wrow[rb] = w + (size_t)min(n0 + rb * 16 + r, N - 1) * K + g * 8;

    f32x4 acc[RB][MB];
#pragma unroll
    for (int rb = 0; rb < RB; ++rb)
#pragma unroll
        for (int mb = 0; mb < MB; ++mb) acc[rb][mb] = f32x4{0.f, 0.f, 0.f, 0.f};

    uint4 stage[kPiecesPerThread];
    auto fetch_acts = [&](int k0) {                                   // global -> registers
#pragma unroll
        for (int i = 0; i < kPiecesPerThread; ++i) {
            const int piece = i * (kLdsWaves * kWave) + threadIdx.x;
            const int m = piece / (CHUNK / 8), kk = k0 + (piece % (CHUNK / 8)) * 8;
            stage[i] = make_uint4(0, 0, 0, 0);
            if (piece < kPieces && m < M && kk < k_end) stage[i] = produce8<MODE>(src, m, kk, K);
        }
    };
    auto store_acts = [&](int buf) {                                  // registers -> LDS
#pragma unroll
        for (int i = 0; i < kPiecesPerThread; ++i) {
            const int piece = i * (kLdsWaves * kWave) + threadIdx.x;
            if (piece < kPieces)
                *reinterpret_cast<uint4*>(&lds[buf][piece / (CHUNK / 8)][(piece % (CHUNK / 8)) * 8]) = stage[i];
        }
    };
    bf16x8 wf0[(CHUNK / 32)][RB], wf1[(CHUNK / 32)][RB];
    auto fetch_w = [&](bf16x8 (&wf)[(CHUNK / 32)][RB], int k0) {
#pragma unroll
        for (int s = 0; s < (CHUNK / 32); ++s) {
            const int kk = k0 + s * 32 + g * 8;
            const bool ok = kk < k_end;                                   // K % 8 == 0
#pragma unroll
            for (int rb = 0; rb < RB; ++rb) {
                uint4 v = make_uint4(0, 0, 0, 0);
                if (ok) v = *reinterpret_cast<const uint4*>(wrow[rb] + k0 + s * 32);
                wf[s][rb] = __builtin_bit_cast(bf16x8, v);
            }
        }
    };
    auto multiply = [&](const bf16x8 (&wf)[(CHUNK / 32)][RB], int buf) {
#pragma unroll
        for (int s = 0; s < (CHUNK / 32); ++s) {
            bf16x8 af[MB];
#pragma unroll
            for (int mb = 0; mb < MB; ++mb)
                af[mb] = __builtin_bit_cast(bf16x8, *reinterpret_cast<const uint4*>(&lds[buf][mb * 16 + r][s * 32 + g * 8]));
#pragma unroll
            for (int rb = 0; rb < RB; ++rb)
#pragma unroll
                for (int mb = 0; mb < MB; ++mb)
                    acc[rb][mb] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wf[s][rb], af[mb], acc[rb][mb], 0, 0, 0);
        }
    };

    if (n_chunks > 0) {
        fetch_acts(k_begin);
        fetch_w(wf0, k_begin);
        store_acts(0);
        __syncthreads();
    }
    for (int c = 0; c < n_chunks; c += 2) {
        const int k0 = k_begin + c * CHUNK;
        const bool has1 = c + 1 < n_chunks, has2 = c + 2 < n_chunks;
        if (has1) { fetch_acts(k0 + CHUNK); fetch_w(wf1, k0 + CHUNK); }
        multiply(wf0, 0);
        if (has1) store_acts(1);
        __syncthreads();
        if (has2) { fetch_acts(k0 + 2 * CHUNK); fetch_w(wf0, k0 + 2 * CHUNK); }
        if (has1) multiply(wf1, 1);
        if (has2) store_acts(0);
        __syncthreads();
    }

    // acc[rb][mb][i] = sum for row n0 + rb * 16 + 4 g + i of w and activation row mb * 16 + r
    TO* dst = out + (size_t)split * part_stride;
#pragma unroll
    for (int rb = 0; rb < RB; ++rb)
#pragma unroll
        for (int mb = 0; mb < MB; ++mb) {
            const int m = mb * 16 + r;
            if (m >= M) continue;
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const int n = n0 + rb * 16 + 4 * g + i;
                if (n < N) store_f32(dst + (size_t)m * ldo + n, acc[rb][mb][i] + (bias ? bias[n] : 0.f));
            }
        }
}

static int lds_k_per_block(int K, int splits) {
    return ((K + splits - 1) / splits + kChunkK - 1) / kChunkK * kChunkK;
}

LLOGOS_EXPORT int llogos_gemm_skinny_lds_parts(int K, int splits) {
    if (K <= 0 || splits <= 1) return 1;
    const int kpb = lds_k_per_block(K, splits);
    return (K + kpb - 1) / kpb;
}

template <int RB, int MB, int MODE, int CHUNK = kChunkK>
static int launch_lds(void* out, int out_dtype, const ActSource& src, const bf16_t* w, const float* bias,
                      int M, int N, int K, int ldo, size_t part_stride, int kpb, int parts, hipStream_t stream) {
    const int n_blocks = (N + 16 * RB * kLdsWaves - 1) / (16 * RB * kLdsWaves);
    if (out_dtype == DT_BF16)
        gemm_skinny_lds_kernel<RB, MB, MODE, bf16_t, CHUNK><<<n_blocks * parts, kLdsWaves * kWave, 0, stream>>>(
            (bf16_t*)out, src, w, bias, M, N, K, ldo, part_stride, kpb, parts);
    else
        gemm_skinny_lds_kernel<RB, MB, MODE, float, CHUNK><<<n_blocks * parts, kLdsWaves * kWave, 0, stream>>>(
            (float*)out, src, w, bias, M, N, K, ldo, part_stride, kpb, parts);
    return LLOGOS_LAUNCH_CHECK();
}

// act: plain bf16 activations [M][lda] (mode 0), or the fused gate/up product [act_parts][M][2 K]
// in float32 (mode 1) or bfloat16 (mode 2, act_parts = 1) from which silu(gate) * up is made on
// the way.  out: [parts][M][ldo], parts = llogos_gemm_skinny_lds_parts(K, splits); float32 and
// without bias when parts > 1.  row_blocks: 16-row blocks of w per wave (1 or 2).
LLOGOS_EXPORT int llogos_gemm_skinny_lds_bf16(void* out, int out_dtype, const void* act, int mode, int lda,
                                              int act_parts, long long act_part_stride, const void* w,
                                              const float* bias, int M, int N, int K, int ldo,
                                              long long part_stride, int splits, int row_blocks,
                                              hipStream_t stream) {
    if (M <= 0 || N <= 0 || K <= 0 || ldo < N || splits < 1 || act_parts < 1) return LLOGOS_BAD_ARGUMENT;
    if (out_dtype != DT_BF16 && out_dtype != DT_F32) return LLOGOS_BAD_ARGUMENT;
    if (mode < PRODUCE_PLAIN || mode > PRODUCE_SWIGLU_BF16) return LLOGOS_BAD_ARGUMENT;
    if (M > kLdsMaxRows || (K % 8) || (lda % 8) || ((uintptr_t)act % 16) || ((uintptr_t)w % 16) || (act_part_stride % 4))
        return LLOGOS_UNSUPPORTED;
    if (M > 64 && mode != PRODUCE_PLAIN) return LLOGOS_UNSUPPORTED;
    if (mode == PRODUCE_PLAIN ? lda < K : lda < 2 * K) return LLOGOS_BAD_ARGUMENT;
    const int parts = llogos_gemm_skinny_lds_parts(K, splits);
    if (parts > 1 && (out_dtype != DT_F32 || bias != nullptr || part_stride < (long long)M * ldo))
        return LLOGOS_BAD_ARGUMENT;
    const int kpb = lds_k_per_block(K, parts);
    ActSource src{act, lda, act_parts, (size_t)act_part_stride};
    const bf16_t* W = (const bf16_t*)w;
    const int mb = (M + 15) / 16;
#define GO(RB, MB, MODE) return launch_lds<RB, MB, MODE>(out, out_dtype, src, W, bias, M, N, K, ldo, \
                                                         (size_t)part_stride, kpb, parts, stream)
#define BY_MODE(RB, MB) do { if (mode == PRODUCE_PLAIN) GO(RB, MB, PRODUCE_PLAIN); \
                             if (mode == PRODUCE_SWIGLU_F32) GO(RB, MB, PRODUCE_SWIGLU_F32); \
                             GO(RB, MB, PRODUCE_SWIGLU_BF16); } while (0)
    // 65 to 128 rows: chunks of 128 values of k, so that two blocks' activations fit a compute unit's LDS
    if (mb > 6) { if (row_blocks >= 2) return launch_lds<2, 8, PRODUCE_PLAIN, 128>(out, out_dtype, src, W, bias, M, N, K, ldo, (size_t)part_stride, kpb, parts, stream);
                  return launch_lds<1, 8, PRODUCE_PLAIN, 128>(out, out_dtype, src, W, bias, M, N, K, ldo, (size_t)part_stride, kpb, parts, stream); }
    if (mb > 4) { if (row_blocks >= 2) return launch_lds<2, 6, PRODUCE_PLAIN, 128>(out, out_dtype, src, W, bias, M, N, K, ldo, (size_t)part_stride, kpb, parts, stream);
                  return launch_lds<1, 6, PRODUCE_PLAIN, 128>(out, out_dtype, src, W, bias, M, N, K, ldo, (size_t)part_stride, kpb, parts, stream); }
    if (mb == 1) { if (row_blocks >= 2) BY_MODE(2, 1); BY_MODE(1, 1); }
    if (mb == 2) { if (row_blocks >= 2) BY_MODE(2, 2); BY_MODE(1, 2); }
    if (row_blocks >= 2) BY_MODE(2, 4);
    BY_MODE(1, 4);
#undef BY_MODE
#undef GO
}
