// out[M, N] = a[M, K] . w[N, K]^T for many rows (prompts) on the matrix cores, with the weights in
// their packed order (llogos_pack_weights in gemm_skinny_lds_bf16.hip: blocks of 64 rows, steps of
// 32 k, fragments of 16 rows x 32 k).
//
//  * v_mfma_f32_32x32x16_bf16: on the MI355X this shape was measured at 2.17 PFLOP/s issued back
//    to back, v_mfma_f32_16x16x32_bf16 at 1.25.  Two packed fragments (rows 0..15 and 16..31 of a
//    step) become two operands of the 32-row shape by one v_permlane16_swap per register: the
//    first then holds the k octets 0 and 2 of the step for all 32 rows, the second the octets 1
//    and 3 (the order of k within a step is free as long as both operands agree).
//  * A block is 4 waves and a tile of TM * 32 tokens x 256 rows of w; wave i owns the packed
//    block of 64 rows i of the tile and all the tile's tokens, so its weights are 4 KB of
//    consecutive memory per step, loaded straight into registers a stage (64 k) ahead, and no
//    two waves load the same weights.
//  * The activations of a stage go through LDS (two buffers), stored in the order in which the
//    waves take them as second operands (1 KB per 32 tokens, step and octet pair), so those
//    reads are consecutive and free of bank conflicts.
//  * Blocks are numbered so that an XCD (blocks i, i + 8, ...) works on few row tiles at a time
//    and walks all token tiles of a row tile before the next: its L2 then serves a row tile's
//    weights to all the token tiles.
//  * Epilogues: plain (+ bias) in bfloat16 or float32; SwiGLU for a matrix whose 16-row strips
//    alternate between gate rows and up rows (rows 16 j .. 16 j + 15 of gate, then of up): the
//    gate and the up value of one (token, column) are then in the same lane.
#include "common.h"

typedef __bf16 bf16x8_t __attribute__((ext_vector_type(8)));
typedef float f32x16_t __attribute__((ext_vector_type(16)));
typedef unsigned u32x4_t __attribute__((ext_vector_type(4)));
typedef unsigned u32x2_t __attribute__((ext_vector_type(2)));
typedef float f32x2_t __attribute__((ext_vector_type(2)));
typedef __bf16 bf16x2_t __attribute__((ext_vector_type(2)));

constexpr int kTileWaves = 4;
constexpr int kStageK = 64;                       // k per LDS stage: two packed steps
enum { EPI_PLAIN = 0, EPI_SWIGLU = 1 };

__device__ __forceinline__ uint32_t tiles_pack_bf16(float lo, float hi) {
    const f32x2_t v = {lo, hi};
    return __builtin_bit_cast(uint32_t, __builtin_convertvector(v, bf16x2_t));
}

// Two 16-row fragments of one step -> two 32-row operands (octets 0, 2 and octets 1, 3).
__device__ __forceinline__ void to_32_rows(const u32x4_t& lo, const u32x4_t& hi, bf16x8_t& even, bf16x8_t& odd) {
    u32x4_t e, o;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        const u32x2_t r = __builtin_amdgcn_permlane16_swap(lo[j], hi[j], false, false);
        e[j] = r[0];
        o[j] = r[1];
    }
    even = __builtin_bit_cast(bf16x8_t, e);
    odd = __builtin_bit_cast(bf16x8_t, o);
}

template <int TM, typename TO, int EPI>
__global__ __launch_bounds__(kTileWaves * kWave) void gemm_tiles_kernel(
        TO* __restrict__ out, const bf16_t* __restrict__ a, int lda, const u32x4_t* __restrict__ wp,
        const float* __restrict__ bias, int M, int N, int K, int ldo, int n_row_blocks, int m_tiles, int n_tiles) {
    extern __shared__ __attribute__((aligned(16))) u32x4_t lds[];          // [2][TM][2 steps][2 pairs][64]
    constexpr int kStageFrags = TM * 4 * kWave;                              // 16-byte pieces of a stage
    constexpr int kPieces = TM * 32 * 8 / (kTileWaves * kWave);            // pieces a thread copies per stage
    const int lane = threadIdx.x & (kWave - 1), wave = threadIdx.x / kWave;
    const int xcd = blockIdx.x & 7, j = blockIdx.x >> 3;
    const int m_tile = j % m_tiles, n_tile = xcd + 8 * (j / m_tiles);
    if (n_tile >= n_tiles) return;
    const int nb = n_tile * kTileWaves + wave;                               // this wave's packed block of 64 rows
    const bool has_rows = nb < n_row_blocks;
    const int steps = (K + 31) / 32, stages = (K + kStageK - 1) / kStageK;
    const u32x4_t* wbase = wp + (size_t)(has_rows ? nb : 0) * steps * (4 * kWave) + lane;
    const int m0 = m_tile * (TM * 32);

    f32x16_t acc[TM][2];
#pragma unroll
    for (int tt = 0; tt < TM; ++tt)
#pragma unroll
        for (int rt = 0; rt < 2; ++rt)
#pragma unroll
            for (int v = 0; v < 16; ++v) acc[tt][rt][v] = 0.f;

    u32x4_t stage_a[kPieces];
    auto fetch_a = [&](int stage) {                                          // global -> registers
#pragma unroll
        for (int i = 0; i < kPieces; ++i) {
            const int q = i * (kTileWaves * kWave) + threadIdx.x;
            const int token = m0 + (q >> 3), k = stage * kStageK + (q & 7) * 8;
            stage_a[i] = u32x4_t{0, 0, 0, 0};
            if (token < M && k < K) stage_a[i] = *reinterpret_cast<const u32x4_t*>(a + (size_t)token * lda + k);
        }
    };
    auto store_a = [&](int buf) {                                            // registers -> LDS, operand order
#pragma unroll
        for (int i = 0; i < kPieces; ++i) {
            const int q = i * (kTileWaves * kWave) + threadIdx.x;
            const int token = q >> 3, oct = q & 7;
            const int tt = token >> 5, c = token & 31, step = oct >> 2, pair = oct & 1, h = (oct >> 1) & 1;
            lds[buf * kStageFrags + ((tt * 2 + step) * 2 + pair) * kWave + h * 32 + c] = stage_a[i];
        }
    };
    u32x4_t w0[2][4], w1[2][4];
    auto fetch_w = [&](u32x4_t (&wf)[2][4], int stage) {
#pragma unroll
        for (int step = 0; step < 2; ++step) {
            const int ks = 2 * stage + step;
#pragma unroll
            for (int s = 0; s < 4; ++s) {
                wf[step][s] = u32x4_t{0, 0, 0, 0};
                if (has_rows && ks < steps) wf[step][s] = wbase[(size_t)(ks * 4 + s) * kWave];
            }
        }
    };
    auto multiply = [&](const u32x4_t (&wf)[2][4], int buf) {
#pragma unroll
        for (int step = 0; step < 2; ++step) {
            bf16x8_t t[2][2];                                                // [row tile][octet pair]
            to_32_rows(wf[step][0], wf[step][1], t[0][0], t[0][1]);
            to_32_rows(wf[step][2], wf[step][3], t[1][0], t[1][1]);
#pragma unroll
            for (int pair = 0; pair < 2; ++pair) {
                bf16x8_t b[TM];
#pragma unroll
                for (int tt = 0; tt < TM; ++tt)
                    b[tt] = __builtin_bit_cast(bf16x8_t, lds[buf * kStageFrags + ((tt * 2 + step) * 2 + pair) * kWave + lane]);
#pragma unroll
                for (int tt = 0; tt < TM; ++tt)
#pragma unroll
                    for (int rt = 0; rt < 2; ++rt)
                        acc[tt][rt] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(t[rt][pair], b[tt], acc[tt][rt], 0, 0, 0);
            }
        }
    };

    fetch_a(0);
    fetch_w(w0, 0);
    store_a(0);
    __syncthreads();
    for (int s = 0; s < stages; s += 2) {
        const bool has1 = s + 1 < stages, has2 = s + 2 < stages;
        if (has1) { fetch_a(s + 1); fetch_w(w1, s + 1); }
        multiply(w0, 0);
        if (has1) store_a(1);
        __syncthreads();
        if (has2) { fetch_a(s + 2); fetch_w(w0, s + 2); }
        if (has1) multiply(w1, 1);
        if (has2) store_a(0);
        __syncthreads();
    }

    // acc[tt][rt][v]: token m0 + 32 tt + (lane & 31), row 64 nb + 32 rt + 8 (v / 4) + 4 (lane >> 5) + v % 4
    if (!has_rows) return;
    const int c = lane & 31, h = lane >> 5;
#pragma unroll
    for (int tt = 0; tt < TM; ++tt) {
        const int token = m0 + 32 * tt + c;
        if (token >= M) continue;
        if (EPI == EPI_SWIGLU) {
            // strips alternate gate, up: rows 0..15 of a 32-row tile are gate rows 32 nb + 16 rt + r, rows
            // 16..31 the up rows of the same columns; out is [M][N / 2]
            TO* orow = out + (size_t)token * ldo;
#pragma unroll
            for (int rt = 0; rt < 2; ++rt)
#pragma unroll
                for (int q = 0; q < 2; ++q) {
                    const int col = 32 * nb + 16 * rt + 8 * q + 4 * h;
                    float y[4];
#pragma unroll
                    for (int e = 0; e < 4; ++e) {
                        const float g = acc[tt][rt][4 * q + e], u = acc[tt][rt][8 + 4 * q + e];
                        y[e] = g / (1.0f + __expf(-g)) * u;
                    }
#pragma unroll
                    for (int e = 0; e < 4; ++e)
                        if (col + e < N / 2) store_f32(orow + col + e, y[e]);
                }
        } else {
            TO* orow = out + (size_t)token * ldo;
#pragma unroll
            for (int rt = 0; rt < 2; ++rt)
#pragma unroll
                for (int q = 0; q < 4; ++q) {
                    const int n = 64 * nb + 32 * rt + 8 * q + 4 * h;
                    float y[4];
#pragma unroll
                    for (int e = 0; e < 4; ++e) y[e] = acc[tt][rt][4 * q + e] + ((bias && n + e < N) ? bias[n + e] : 0.f);
                    if (sizeof(TO) == 2 && n + 3 < N && ((ldo & 3) == 0) && ((reinterpret_cast<uintptr_t>(out) & 7) == 0)) {
                        uint2 pk;
                        pk.x = tiles_pack_bf16(y[0], y[1]);
                        pk.y = tiles_pack_bf16(y[2], y[3]);
                        *reinterpret_cast<uint2*>(orow + n) = pk;
                    } else if (sizeof(TO) == 4 && n + 3 < N && ((ldo & 3) == 0) && ((reinterpret_cast<uintptr_t>(out) & 15) == 0)) {
                        *reinterpret_cast<float4*>(orow + n) = make_float4(y[0], y[1], y[2], y[3]);
                    } else {
#pragma unroll
                        for (int e = 0; e < 4; ++e)
                            if (n + e < N) store_f32(orow + n + e, y[e]);
                    }
                }
        }
    }
}

template <int TM, typename TO, int EPI>
static int launch_tiles(void* out, const void* a, int lda, const void* wp, const float* bias, int M, int N, int K,
                        int ldo, hipStream_t stream) {
    const int n_row_blocks = (N + 63) / 64;
    const int m_tiles = (M + TM * 32 - 1) / (TM * 32), n_tiles = (n_row_blocks + kTileWaves - 1) / kTileWaves;
    const int blocks = m_tiles * ((n_tiles + 7) / 8) * 8;
    const size_t smem = (size_t)2 * TM * 4 * kWave * 16;
    hipError_t e = hipFuncSetAttribute((const void*)gemm_tiles_kernel<TM, TO, EPI>,
                                       hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem);
    if (e != hipSuccess) return (int)e;
    gemm_tiles_kernel<TM, TO, EPI><<<blocks, kTileWaves * kWave, smem, stream>>>(
        (TO*)out, (const bf16_t*)a, lda, (const u32x4_t*)wp, bias, M, N, K, ldo, n_row_blocks, m_tiles, n_tiles);
    return LLOGOS_LAUNCH_CHECK();
}

// a: bfloat16 [M][lda]; packed_w: llogos_pack_weights of w [N][K]; out [M][ldo] bfloat16 or float32.
// epilogue 0: out = a . w^T (+ bias [N]); 1: w's 16-row strips alternate gate and up rows, out is
// [M][N / 2] = silu(gate) * up (no bias).  token_tiles: 8 (tiles of 256 tokens) or 4 (128).
LLOGOS_EXPORT int llogos_gemm_tiles_bf16(void* out, int out_dtype, const void* a, int lda, const void* packed_w,
                                         const float* bias, int M, int N, int K, int ldo, int epilogue,
                                         int token_tiles, hipStream_t stream) {
    if (M <= 0 || N <= 0 || K <= 0 || out == nullptr || a == nullptr || packed_w == nullptr) return LLOGOS_BAD_ARGUMENT;
    if (out_dtype != DT_BF16 && out_dtype != DT_F32) return LLOGOS_BAD_ARGUMENT;
    if (epilogue != EPI_PLAIN && epilogue != EPI_SWIGLU) return LLOGOS_BAD_ARGUMENT;
    if ((K % 8) || (lda % 8) || lda < K || ((uintptr_t)a % 16) || ((uintptr_t)packed_w % 16)) return LLOGOS_UNSUPPORTED;
    if (epilogue == EPI_SWIGLU && ((N % 32) || bias != nullptr || ldo < N / 2)) return LLOGOS_BAD_ARGUMENT;
    if (epilogue == EPI_PLAIN && ldo < N) return LLOGOS_BAD_ARGUMENT;
    if (token_tiles != 4 && token_tiles != 8) return LLOGOS_BAD_ARGUMENT;
#define GO(TM, EPI) do { if (out_dtype == DT_BF16) return launch_tiles<TM, bf16_t, EPI>(out, a, lda, packed_w, bias, M, N, K, ldo, stream); \
                         return launch_tiles<TM, float, EPI>(out, a, lda, packed_w, bias, M, N, K, ldo, stream); } while (0)
    if (token_tiles == 8) { if (epilogue == EPI_SWIGLU) GO(8, EPI_SWIGLU); GO(8, EPI_PLAIN); }
    if (epilogue == EPI_SWIGLU) GO(4, EPI_SWIGLU);
    GO(4, EPI_PLAIN);
#undef GO
}
