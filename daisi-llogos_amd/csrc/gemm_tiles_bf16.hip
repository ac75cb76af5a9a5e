// out[M, N] = a[M, K] . w[N, K]^T for many rows (prompts) on the matrix cores, with the weights in
// their packed order (llogos_pack_weights in gemm_skinny_lds_bf16.hip: blocks of 64 rows, steps of
// 32 k, fragments of 16 rows x 32 k).
//
//  * v_mfma_f32_32x32x16_bf16: on the MI355X this shape was measured at 2.17 PFLOP/s issued back
//    to back, v_mfma_f32_16x16x32_bf16 at 1.25.  Two packed fragments (rows 0..15 and 16..31 of a
//    step) become two operands of the 32-row shape by one v_permlane16_swap per register: the
//    first then holds the k octets 0 and 2 of the step for all 32 rows, the second the octets 1
//    and 3 (the order of k within a step is free as long as both operands agree).
//  * A block is HALVES x 4 waves and a tile of HALVES * TM * 32 tokens x 256 rows of w; wave
//    (half, i) owns the packed block of 64 rows i of the tile and TM * 32 of its tokens, so its
//    weights are 4 KB of consecutive memory per step, loaded straight into registers two stages
//    (of 64 k) ahead.  In use: HALVES = 1, TM = 4 (128 tokens x 256 rows, one wave a SIMD).
//  * Measured on the MI355X at the 8B layer sizes and 2,048 tokens: gate/up 588 us (0.82 PFLOP/s)
//    where the library's product takes 375 (1.28), down 266 against 189, o 93 against 62, qkv 172
//    against 86.  By the counters the matrix pipe is busy a third of the time, no LDS bank
//    conflicts, little waiting for loads: with one wave a SIMD the loads, the LDS reads, the
//    lane swaps and the products of a stage run one after the other, and interleaving them at the
//    instruction level is what is missing.  So prompts keep the library's product, and this one
//    serves where the row-major copy of a matrix is not wanted.
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

constexpr int kRowWaves = 4;                      // row blocks of 64 rows a tile
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

template <int TM, int HALVES, typename TO, int EPI>
__global__ __launch_bounds__(HALVES * kRowWaves * kWave) void gemm_tiles_kernel(
        TO* __restrict__ out, const bf16_t* __restrict__ a, int lda, const u32x4_t* __restrict__ wp,
        const float* __restrict__ bias, int M, int N, int K, int ldo, int n_row_blocks, int m_tiles, int n_tiles) {
    extern __shared__ __attribute__((aligned(16))) u32x4_t lds[];          // [3][2 TM][2 steps][2 pairs][64]
    constexpr int kTileWaves = HALVES * kRowWaves;
    constexpr int kStageFrags = HALVES * TM * 4 * kWave;                     // 16-byte pieces of a stage
    constexpr int kPieces = HALVES * TM * 32 * 8 / (kTileWaves * kWave);   // pieces a thread copies per stage
    const int lane = threadIdx.x & (kWave - 1), wave = threadIdx.x / kWave;
    const int xcd = blockIdx.x & 7, j = blockIdx.x >> 3;
    const int m_tile = j % m_tiles, n_tile = xcd + 8 * (j / m_tiles);
    if (n_tile >= n_tiles) return;
    const int half = wave / kRowWaves;                                       // which TM * 32 tokens of the tile (0 when HALVES == 1)
    const int nb = n_tile * kRowWaves + (wave % kRowWaves);                  // this wave's packed block of 64 rows
    const bool has_rows = nb < n_row_blocks;
    const int steps = K / 32, stages = K / kStageK;                          // K is a multiple of 64
    const u32x4_t* wbase = wp + (size_t)(has_rows ? nb : 0) * steps * (4 * kWave) + lane;
    const int m0 = m_tile * (HALVES * TM * 32);

    f32x16_t acc[TM][2];
#pragma unroll
    for (int tt = 0; tt < TM; ++tt)
#pragma unroll
        for (int rt = 0; rt < 2; ++rt)
#pragma unroll
            for (int v = 0; v < 16; ++v) acc[tt][rt][v] = 0.f;

    // activations on their way: two register sets, asked for two iterations before they are stored
    u32x4_t stage_a0[kPieces], stage_a1[kPieces];
    auto fetch_a = [&](u32x4_t (&st)[kPieces], int stage) {                  // global -> registers
#pragma unroll
        for (int i = 0; i < kPieces; ++i) {
            const int q = i * (kTileWaves * kWave) + threadIdx.x;
            // No branch around a load (the compiler waits for every outstanding load where paths with
            // different numbers of loads meet) and nothing computed from the loaded value here (that
            // would wait for it at once).  Tokens past M read the last token's row: their results
            // are never stored.  Stages past the last read the last stage again and are not used.
            // (a wave's 64 pieces are 8 tokens x 8 octets, lanes running over the tokens first: eight
            // consecutive lanes then store 128 consecutive bytes of LDS, free of bank conflicts, and
            // the wave still reads eight whole lines)
            const int token = min(m0 + 8 * (q >> 6) + (q & 7), M - 1), k = min(stage, stages - 1) * kStageK + ((q >> 3) & 7) * 8;
            st[i] = *reinterpret_cast<const u32x4_t*>(a + (size_t)token * lda + k);
        }
    };
    auto store_a = [&](const u32x4_t (&st)[kPieces], int buf) {              // registers -> LDS, operand order
#pragma unroll
        for (int i = 0; i < kPieces; ++i) {
            const int q = i * (kTileWaves * kWave) + threadIdx.x;
            const int token = 8 * (q >> 6) + (q & 7), oct = (q >> 3) & 7;
            const int tt = token >> 5, c = token & 31, step = oct >> 2, pair = oct & 1, h = (oct >> 1) & 1;
            lds[buf * kStageFrags + ((tt * 2 + step) * 2 + pair) * kWave + h * 32 + c] = st[i];
        }
    };
    u32x4_t w0[2][4], w1[2][4], w2[2][4];                                   // weights: asked for two iterations ahead
    auto fetch_w = [&](u32x4_t (&wf)[2][4], int stage) {
#pragma unroll
        for (int step = 0; step < 2; ++step) {
            const int ks = 2 * min(stage, stages - 1) + step;                // (rows past N are zero in the packed matrix)
#pragma unroll
            for (int s = 0; s < 4; ++s) wf[step][s] = wbase[(size_t)(ks * 4 + s) * kWave];
        }
    };
    auto read_b = [&](bf16x8_t (&b)[TM], int buf, int group) {                 // group = 2 step + pair
#pragma unroll
        for (int tt = 0; tt < TM; ++tt)
            b[tt] = __builtin_bit_cast(bf16x8_t, lds[buf * kStageFrags + ((half * TM + tt) * 4 + group) * kWave + lane]);
    };
    auto multiply = [&](const u32x4_t (&wf)[2][4], int buf) {
        bf16x8_t t[2][2][2];                                                 // [step][row tile][octet pair]
#pragma unroll
        for (int step = 0; step < 2; ++step) {
            to_32_rows(wf[step][0], wf[step][1], t[step][0][0], t[step][0][1]);
            to_32_rows(wf[step][2], wf[step][3], t[step][1][0], t[step][1][1]);
        }
        if (HALVES == 1) {
            // one wave a SIMD: the second operands of the next group are asked for before the products
            // of this one, so that LDS latency is not waited for at every product
            bf16x8_t b0[TM], b1[TM];
            read_b(b0, buf, 0);
#pragma unroll
            for (int group = 0; group < 4; group += 2) {
                read_b(b1, buf, group + 1);
                __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                for (int tt = 0; tt < TM; ++tt)
#pragma unroll
                    for (int rt = 0; rt < 2; ++rt)
                        acc[tt][rt] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(t[group >> 1][rt][group & 1], b0[tt], acc[tt][rt], 0, 0, 0);
                __builtin_amdgcn_sched_barrier(0);
                if (group + 2 < 4) read_b(b0, buf, group + 2);
                __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                for (int tt = 0; tt < TM; ++tt)
#pragma unroll
                    for (int rt = 0; rt < 2; ++rt)
                        acc[tt][rt] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(t[(group + 1) >> 1][rt][(group + 1) & 1], b1[tt], acc[tt][rt], 0, 0, 0);
                __builtin_amdgcn_sched_barrier(0);
            }
            return;
        }
#pragma unroll
        for (int group = 0; group < 4; ++group) {
            bf16x8_t b[TM];
            read_b(b, buf, group);
#pragma unroll
            for (int tt = 0; tt < TM; ++tt)
#pragma unroll
                for (int rt = 0; rt < 2; ++rt)
                    acc[tt][rt] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(t[group >> 1][rt][group & 1], b[tt], acc[tt][rt], 0, 0, 0);
        }
    };

    // Stage s is multiplied from LDS buffer s % 3.  Its activations were asked for three iterations
    // earlier (into one of two register sets) and stored one iteration earlier; its weights were
    // asked for two iterations earlier (three register sets): every load has two iterations to
    // arrive, and one barrier an iteration is enough (the buffer written in iteration s was last
    // read in iteration s - 2).  Six iterations make one round of the register sets.
    fetch_a(stage_a0, 0);
    fetch_w(w0, 0);
    fetch_a(stage_a1, 1);
    fetch_w(w1, 1);
    store_a(stage_a0, 0);
    fetch_a(stage_a0, 2);
    __syncthreads();
    // iteration s: store stage s + 1 (set (s + 1) % 2), ask for stage s + 3 into that set, ask for the weights
    // of stage s + 2, multiply stage s
    auto iteration = [&](int s, const u32x4_t (&w_cur)[2][4], u32x4_t (&w_far)[2][4], u32x4_t (&a_set)[kPieces]) {
        store_a(a_set, (s + 1) % 3);
        fetch_a(a_set, s + 3);
        fetch_w(w_far, s + 2);
        __builtin_amdgcn_sched_barrier(0);          // the loads are asked for before the products, not among them
        multiply(w_cur, s % 3);
        __builtin_amdgcn_sched_barrier(0);
        __syncthreads();
    };
    int s = 0;
    for (; s + 6 <= stages; s += 6) {
        iteration(s, w0, w2, stage_a1);
        iteration(s + 1, w1, w0, stage_a0);
        iteration(s + 2, w2, w1, stage_a1);
        iteration(s + 3, w0, w2, stage_a0);
        iteration(s + 4, w1, w0, stage_a1);
        iteration(s + 5, w2, w1, stage_a0);
    }
    if (s < stages) iteration(s, w0, w2, stage_a1);
    if (s + 1 < stages) iteration(s + 1, w1, w0, stage_a0);
    if (s + 2 < stages) iteration(s + 2, w2, w1, stage_a1);
    if (s + 3 < stages) iteration(s + 3, w0, w2, stage_a0);
    if (s + 4 < stages) iteration(s + 4, w1, w0, stage_a1);

    // acc[tt][rt][v]: token m0 + 32 tt + (lane & 31), row 64 nb + 32 rt + 8 (v / 4) + 4 (lane >> 5) + v % 4
    if (!has_rows) return;
    const int c = lane & 31, h = lane >> 5;
#pragma unroll
    for (int tt = 0; tt < TM; ++tt) {
        const int token = m0 + 32 * (half * TM + tt) + c;
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

template <int TM, int HALVES, typename TO, int EPI>
static int launch_tiles(void* out, const void* a, int lda, const void* wp, const float* bias, int M, int N, int K,
                        int ldo, hipStream_t stream) {
    const int n_row_blocks = (N + 63) / 64;
    const int m_tiles = (M + HALVES * TM * 32 - 1) / (HALVES * TM * 32), n_tiles = (n_row_blocks + kRowWaves - 1) / kRowWaves;
    const int blocks = m_tiles * ((n_tiles + 7) / 8) * 8;
    const size_t smem = (size_t)3 * HALVES * TM * 4 * kWave * 16;
    hipError_t e = hipFuncSetAttribute((const void*)gemm_tiles_kernel<TM, HALVES, TO, EPI>,
                                       hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem);
    if (e != hipSuccess) return (int)e;
    gemm_tiles_kernel<TM, HALVES, TO, EPI><<<blocks, HALVES * kRowWaves * kWave, smem, stream>>>(
        (TO*)out, (const bf16_t*)a, lda, (const u32x4_t*)wp, bias, M, N, K, ldo, n_row_blocks, m_tiles, n_tiles);
    return LLOGOS_LAUNCH_CHECK();
}

// a: bfloat16 [M][lda]; packed_w: llogos_pack_weights of w [N][K]; out [M][ldo] bfloat16 or float32.
// epilogue 0: out = a . w^T (+ bias [N]); 1: w's 16-row strips alternate gate and up rows, out is
// [M][N / 2] = silu(gate) * up (no bias).  token_tiles: 32-token tiles a wave (4: blocks of 128 tokens x 256 rows,
// 4 waves; the other shapes that were tried, 8 waves with two token halves and 256-token tiles, were slower or
// spilled registers).  K must be a multiple of 64.
LLOGOS_EXPORT int llogos_gemm_tiles_bf16(void* out, int out_dtype, const void* a, int lda, const void* packed_w,
                                         const float* bias, int M, int N, int K, int ldo, int epilogue,
                                         int token_tiles, hipStream_t stream) {
    if (M <= 0 || N <= 0 || K <= 0 || out == nullptr || a == nullptr || packed_w == nullptr) return LLOGOS_BAD_ARGUMENT;
    if (out_dtype != DT_BF16 && out_dtype != DT_F32) return LLOGOS_BAD_ARGUMENT;
    if (epilogue != EPI_PLAIN && epilogue != EPI_SWIGLU) return LLOGOS_BAD_ARGUMENT;
    if ((K % kStageK) || (lda % 8) || lda < K || ((uintptr_t)a % 16) || ((uintptr_t)packed_w % 16)) return LLOGOS_UNSUPPORTED;
    if (epilogue == EPI_SWIGLU && ((N % 32) || bias != nullptr || ldo < N / 2)) return LLOGOS_BAD_ARGUMENT;
    if (epilogue == EPI_PLAIN && ldo < N) return LLOGOS_BAD_ARGUMENT;
    if (token_tiles != 4) return LLOGOS_BAD_ARGUMENT;
#define GO(TM, HV, EPI) do { if (out_dtype == DT_BF16) return launch_tiles<TM, HV, bf16_t, EPI>(out, a, lda, packed_w, bias, M, N, K, ldo, stream); \
                             return launch_tiles<TM, HV, float, EPI>(out, a, lda, packed_w, bias, M, N, K, ldo, stream); } while (0)
    if (epilogue == EPI_SWIGLU) GO(4, 1, EPI_SWIGLU);
    GO(4, 1, EPI_PLAIN);
#undef GO
}
