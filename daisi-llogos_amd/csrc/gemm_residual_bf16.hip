// x[M, N] += a[M, K] . w[N, K]^T (+ bias) for up to 16 rows, on packed weights, in one pass:
// the product that closes a mixer or a feed-forward adds itself to the residual stream and
// leaves, beside the stream, what the norm that follows needs of it.
//
// A block owns 16 (or 32) rows of w (as many columns of x) and the whole of k: its waves take equal runs of
// k, each with one MFMA accumulator; LDS adds the waves' sums in ascending order of k, the
// block adds them to its columns of x (float32, in place) and writes for every row of x the
// sum of the squares of its new values: sums[block][16], and x * norm_w in bfloat16, the rows
// of the rmsnorm that follows without their scale.  The product that takes norm(x) as its
// activations (gemm_skinny_lds_bf16.hip, PRODUCE_UNSCALED) multiplies these rows, adds the blocks'
// sums in ascending order and applies 1 / rms to its result: no other pass over x and no kernel
// between the two products.  Nothing here depends on what else runs: the order of every addition is
// fixed by N, K and the number of waves.
//
// (With k divided over blocks instead, as the few-row product with partial sums does, a row of x
// is complete only after a kernel boundary, and the norm has to be a kernel of its own: at 8
// rows two such kernels were 9.6 of a layer's 102 us.)
//
// Weights: llogos_pack_weights' layout, [N / 64][K / 32][4 strips][64 lanes] fragments of 16
// bytes; strip s of a 64-row group is every fourth KB of the group's run.  Activations: each
// wave copies the rows of a for its own run of k (rows beyond M: zero) through its own part of
// LDS; with at most 16 rows that is at most as many bytes as the weights, and they come from
// the L2.  A block with 16 waves holds 86 to 102 KB of LDS (the waves' copies and their sums).
#include "common.h"

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef unsigned u32x4 __attribute__((ext_vector_type(4)));

constexpr int kResidualRows = 16;      // rows of a (tokens) at most
constexpr int kAhead = 4;              // MFMA steps whose operands a wave asks for together

constexpr int kActRow = kAhead * 32 + 8;   // bf16 of a wave's LDS row: 4 steps and 16 bytes of padding (rows 4 banks apart)

template <int WAVES, int RB>
__global__ __launch_bounds__(WAVES * kWave) void gemm_residual_kernel(
        float* __restrict__ x, int ldx, float* __restrict__ sums, bf16_t* __restrict__ unscaled, int ldu,
        const float* __restrict__ norm_w, const bf16_t* __restrict__ a, int lda,
        const u32x4* __restrict__ wp, const float* __restrict__ bias, int M, int N, int K) {
    __shared__ float red[WAVES][RB][4][kWave];
    __shared__ __attribute__((aligned(16))) bf16_t acts[WAVES][kResidualRows][kActRow];
    const int lane = threadIdx.x & (kWave - 1), wave = threadIdx.x / kWave;
    const int r = lane & 15, g = lane >> 4;
    const int strip0 = blockIdx.x * RB;                  // the block's RB strips of 16 rows of w follow one another
    const int steps = (K + 31) / 32;
    const int s_begin = (int)((long long)steps * wave / WAVES), s_end = (int)((long long)steps * (wave + 1) / WAVES);
    const u32x4* wsrc[RB];
#pragma unroll
    for (int rb = 0; rb < RB; ++rb) {
        const int strip = strip0 + rb;
        wsrc[rb] = wp + ((size_t)(strip >> 2) * steps * 4 + (strip & 3)) * kWave + lane;
    }
    const bool strip_ok[2] = {true, RB == 2 && (strip0 + 1) * 16 < N};
    // Activations: a wave copies the 4 steps' 128 values of k of four rows with one load (16 lanes a row,
    // whole cache lines), through registers into its own rows of LDS, and reads its MFMA operands from
    // there.  (Loading the operands themselves, 16 rows x 64 bytes a step, asked for twice the lines: the
    // 8B down projection took 23.0 us at 8 rows, 20.6 without its activations, 20.9 with this copy.)
    const int quads = (M + 3) / 4;                       // loads of four rows
    const bf16_t* asrc = a + (size_t)g * lda + r * 8;
    const int k_end = min(K, s_end * 32);

    f32x4 acc[RB];
#pragma unroll
    for (int rb = 0; rb < RB; ++rb) acc[rb] = f32x4{0.f, 0.f, 0.f, 0.f};
    u32x4 wf[2][kAhead][RB];
    uint4 af[2][kResidualRows / 4];
    auto fetch = [&](int buf, int s0) {
#pragma unroll
        for (int j = 0; j < kAhead; ++j)
#pragma unroll
            for (int rb = 0; rb < RB; ++rb) {
                u32x4 v = {0, 0, 0, 0};
                if (s0 + j < s_end && strip_ok[rb]) v = __builtin_nontemporal_load(wsrc[rb] + (size_t)(s0 + j) * (4 * kWave));
                wf[buf][j][rb] = v;
            }
#pragma unroll
        for (int q = 0; q < kResidualRows / 4; ++q) {
            uint4 t = make_uint4(0, 0, 0, 0);
            if (q < quads && 4 * q + g < M && s0 * 32 + r * 8 < k_end)
                t = *reinterpret_cast<const uint4*>(asrc + (size_t)(4 * q) * lda + s0 * 32);
            af[buf][q] = t;
        }
    };
    auto multiply = [&](int buf) {
#pragma unroll
        for (int q = 0; q < kResidualRows / 4; ++q)
            *reinterpret_cast<uint4*>(&acts[wave][4 * q + g][r * 8]) = af[buf][q];
        // the rows are this wave's own: its lanes exchange them through LDS in program order
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
#pragma unroll
        for (int j = 0; j < kAhead; ++j) {
            const uint4 t = *reinterpret_cast<const uint4*>(&acts[wave][r][j * 32 + g * 8]);
#pragma unroll
            for (int rb = 0; rb < RB; ++rb)
                acc[rb] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, wf[buf][j][rb]),
                                                                  __builtin_bit_cast(bf16x8, t), acc[rb], 0, 0, 0);
        }
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
    };
    if (s_begin < s_end) fetch(0, s_begin);
    for (int s = s_begin; s < s_end; s += 2 * kAhead) {
        if (s + kAhead < s_end) fetch(1, s + kAhead);
        multiply(0);
        if (s + 2 * kAhead < s_end) fetch(0, s + 2 * kAhead);
        if (s + kAhead < s_end) multiply(1);
    }

    // acc[rb][i]: column 16 (strip0 + rb) + 4 g + i of x, row r
#pragma unroll
    for (int rb = 0; rb < RB; ++rb)
#pragma unroll
        for (int i = 0; i < 4; ++i) red[wave][rb][i][lane] = acc[rb][i];
    __syncthreads();
    if (threadIdx.x >= 256) return;
    const int m = threadIdx.x >> 4, c = threadIdx.x & 15;
    const int src_lane = (c >> 2) * 16 + m, i = c & 3;
    float sq = 0.f;                                      // of this thread's row over the block's columns
#pragma unroll
    for (int rb = 0; rb < RB; ++rb) {
        if (!strip_ok[rb]) continue;
        float v = 0.f;
#pragma unroll
        for (int w = 0; w < WAVES; ++w) v += red[w][rb][i][src_lane];
        const int n = (strip0 + rb) * 16 + c;
        if (m < M && n < N) {
            float* xp = x + (size_t)m * ldx + n;
            const float y = *xp + (v + (bias ? bias[n] : 0.f));
            *xp = y;
            sq += y * y;
            if (unscaled) unscaled[(size_t)m * ldu + n] = f32_to_bf16(y * norm_w[n]);
        }
    }
    // the 16 lanes of a row are neighbours: a fixed tree of additions
#pragma unroll
    for (int o = 8; o > 0; o >>= 1) sq += __shfl_xor(sq, o, kWave);
    if (c == 0) sums[(size_t)blockIdx.x * kResidualRows + m] = sq;
}

// strips_per_block: 1 or 2 strips of 16 rows of w a block (two share a wave's copy of the activations and halve
// the number of blocks).  sums: float32 [blocks][16], blocks = ceil(ceil(N / 16) / strips_per_block), written
// whole (rows from M on hold 0): a block's sum of squares of each row of x over its 16 or 32 columns.  unscaled (optional, with norm_w
// [N]): bfloat16 [M][ldu] = x * norm_w of the new x, the rows of an rmsnorm that still lack their scale.
LLOGOS_EXPORT int llogos_gemm_residual_bf16(float* x, int ldx, float* sums, void* unscaled, int ldu, const float* norm_w,
                                            const void* act, int lda, const void* packed_w, const float* bias,
                                            int M, int N, int K, int waves, int strips_per_block, hipStream_t stream) {
    if (M <= 0 || N <= 0 || K <= 0 || ldx < N || lda < K || x == nullptr || sums == nullptr) return LLOGOS_BAD_ARGUMENT;
    if (unscaled != nullptr && (norm_w == nullptr || ldu < N)) return LLOGOS_BAD_ARGUMENT;
    if (M > kResidualRows || (K % 8) || (lda % 8) || ((uintptr_t)act % 16) || ((uintptr_t)packed_w % 16))
        return LLOGOS_UNSUPPORTED;
    const int strips = (N + 15) / 16;
    const u32x4* W = (const u32x4*)packed_w;
    const bf16_t* A = (const bf16_t*)act;
#define GO(WAVES, RB) gemm_residual_kernel<WAVES, RB><<<(strips + RB - 1) / RB, WAVES * kWave, 0, stream>>>( \
        x, ldx, sums, (bf16_t*)unscaled, ldu, norm_w, A, lda, W, bias, M, N, K)
    if (strips_per_block == 1 && waves == 4) GO(4, 1);
    else if (strips_per_block == 1 && waves == 8) GO(8, 1);
    else if (strips_per_block == 1 && waves == 16) GO(16, 1);
    else if (strips_per_block == 2 && waves == 4) GO(4, 2);
    else if (strips_per_block == 2 && waves == 8) GO(8, 2);
    else if (strips_per_block == 2 && waves == 16) GO(16, 2);
    else return LLOGOS_BAD_ARGUMENT;
#undef GO
    return LLOGOS_LAUNCH_CHECK();
}
