// out[M, N] = a[M, K] . w[N, K]^T for many rows (prompts) on the matrix cores, with the weights in
// their packed order (llogos_pack_weights in gemm_skinny_lds_bf16.hip: blocks of 64 rows, steps of
// 32 k, fragments of 16 rows x 32 k).
//
//  * v_mfma_f32_32x32x16_bf16.  The rows of w are the first operand, the tokens the second: a
//    lane's 16 sums are 4 x 4 consecutive rows of w for one token, so for a matrix whose 16-row
//    strips alternate gate and up rows the two values of one column of silu(gate) * up are in
//    the same lane, and the SwiGLU epilogue needs no exchange.
//  * A block is 8 waves, two to a SIMD, so that one wave's products cover the other's waits: 4
//    waves along the rows of w (one packed block of 64 rows each, a tile of 256 rows) times 2
//    along the tokens (TM x 32 tokens each; TM = 4: tiles of 256 tokens, TM = 2: of 128).  A
//    wave holds 128 accumulator registers, two sets of operand fragments and the 32 registers
//    of its copies in flight: 229 of the 256 registers that two waves a SIMD leave it.
//  * Stages of 64 values of k, two LDS buffers of 64 KB.  Copies go through registers
//    (global_load -> ds_write): measured on the MI355X, loads straight into LDS
//    (global_load_lds) bring at most 16 TB/s over all compute units and only with several stages
//    in flight, for which 160 KB of LDS have no room at this tile size; loads to registers
//    bring 22 TB/s.  A burst of a whole stage's loads right after the barrier came back after
//    1.5 us, longer than the stage is multiplied; so every wave copies two of its eight pieces
//    per sub-step of 16 k: it stores what it asked for one stage ago and asks for the same pieces
//    of the stage after next, and requests flow evenly (486 -> 412 us for the 8B gate/up matrix
//    at 2,048 tokens).
//  * LDS order.  Weights: a wave's load picks the 64 pieces of the packed matrix that make one
//    32-row operand (two strips, two octets of k), so the operand is stored and read as 1 KB in
//    lane order.  Activations: rows of 128 bytes, eight rows a load and a store (whole lines of
//    global memory, 1 KB in lane order into LDS); the eight 16-byte pieces of a row are swizzled
//    (piece p of row r holds octet p ^ ((r >> 1) & 7)), which spreads the 32 rows that an operand
//    read touches over all banks (no bank conflicts by the counter).
//  * Within a sub-step the products, the LDS reads of the next sub-step's fragments and the
//    copies are written in the order in which they are to issue, and scheduling barriers keep the
//    compiler from moving them (left alone it waits for every fragment right before its use).
//    The last stage is peeled off, so that no product sits on a branch: an accumulator written on
//    two paths costs register copies and spills.
//  * One barrier a stage, in the middle of the last sub-step: before it the stores of the next
//    stage, after it the first reads of that stage, beside the sub-step's remaining products.
//  * Blocks are numbered so that an XCD (blocks i, i + 8, ...) works on few row tiles at a time
//    and walks all token tiles of a row tile before the next: its L2 then serves a row tile's
//    weights to all the token tiles (hit rate 80 % with 8 x 4 tiles in flight on an XCD).
//  * When the tiles of 256 tokens leave less than half of a last round of blocks, the row tiles
//    of that round are taken in tiles of 128 tokens, which fill the round at half its length.
//  * Parts of k (blocks along k, float32 partial sums [parts][M][N] that the consumer adds) for
//    matrices with few rows, whose tiles do not fill the compute units.
//  * Epilogues: plain (+ bias) in bfloat16 or float32; SwiGLU for a matrix packed with gate_rows.
//  * Measured, 2,048 tokens of the 8B layer sizes: gate/up with SwiGLU 395 to 412 us against the
//    library's 392 + 31 for a SwiGLU pass; down 214 (two parts of k) against 189; qkv 100 against
//    87; o 80 against 61.  By the counters the matrix pipe is busy 76 % of a tile's time (86 %
//    with the copies left out, barriers 9 %); the rest of the distance to the library's kernels
//    on the short matrices is the round of blocks that their tiles do not fill.
#include "common.h"

typedef __bf16 bf16x8_t __attribute__((ext_vector_type(8)));
typedef float f32x16_t __attribute__((ext_vector_type(16)));
typedef unsigned u32x4_t __attribute__((ext_vector_type(4)));
typedef float f32x2_t __attribute__((ext_vector_type(2)));
typedef __bf16 bf16x2_t __attribute__((ext_vector_type(2)));

constexpr int kWavesN = 4, kWavesM = 2, kTileWaves = 8;
constexpr int kStageK = 64;
constexpr int kStageW = kWavesN * 64 * kStageK * 2;   // 32 KB
enum { EPI_PLAIN = 0, EPI_SWIGLU = 1 };

__device__ __forceinline__ uint32_t tiles_pack_bf16(float lo, float hi) {
    const f32x2_t v = {lo, hi};
    return __builtin_bit_cast(uint32_t, __builtin_convertvector(v, bf16x2_t));
}
#define SB() __builtin_amdgcn_sched_barrier(0)

template <int N> __device__ __forceinline__ void tiles_wait_loads() {
    static_assert(N == 4 || N == 5 || N == 6, "loads of the other sub-steps of a stage");
    if (N == 4) asm volatile("s_waitcnt vmcnt(4)" ::: "memory");
    if (N == 5) asm volatile("s_waitcnt vmcnt(5)" ::: "memory");
    if (N == 6) asm volatile("s_waitcnt vmcnt(6)" ::: "memory");
}

// One tile: TM x 64 tokens by 256 rows of w, stages [stage_begin, stage_end) of k.
template <int TM, typename TO, int EPI>
__device__ __forceinline__ void tile_body(
        unsigned char* tiles_lds, TO* __restrict__ out, const bf16_t* __restrict__ a, int lda,
        const unsigned char* __restrict__ wp, const float* __restrict__ bias, int M, int N, int K, int ldo,
        int n_row_blocks, int m_tile, int n_tile, int stage_begin, int stage_end) {
    constexpr int BM = kWavesM * TM * 32;
    constexpr int kStageBytes = kStageW + BM * kStageK * 2;
    constexpr int kPieces = 4 + TM;                                          // copies per wave and stage: 4 of w, TM of the activations
    const int lane = threadIdx.x & (kWave - 1);
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / kWave);
    const int wn = wave & (kWavesN - 1), wm = wave / kWavesN;
    const int steps = K / 32, stages = stage_end - stage_begin;
    const int m0 = m_tile * BM;
    const int nb = n_tile * kWavesN + wn;
    const bool has_rows = nb < n_row_blocks;
    const int r32 = lane & 31, h = lane >> 5;

    const int w_block = min(n_tile * kWavesN + (wave & 3), n_row_blocks - 1);
    const unsigned char* w_src = wp + ((size_t)w_block * steps + 2 * stage_begin + (wave >> 2)) * 4096 + (size_t)(r32 >> 4) * 1024 +
                                 (size_t)((r32 & 15) + 16 * h) * 16;
    const int w_dst = ((wave & 3) * 2 + (wave >> 2)) * 4096 + lane * 16;
    const bf16_t* a_src[TM];
    int a_dst[TM];
#pragma unroll
    for (int i = 0; i < TM; ++i) {
        const int row = 8 * (wave * TM + i) + (lane >> 3), oct = (lane & 7) ^ ((row >> 1) & 7);
        a_src[i] = a + (size_t)min(m0 + row, M - 1) * lda + (size_t)stage_begin * kStageK + 8 * oct;
        a_dst[i] = kStageW + (wave * TM + i) * 1024 + lane * 16;
    }
    u32x4_t g[kPieces];
    auto fetch_one = [&](int c, int stage) {
        if (c < 4) g[c] = *reinterpret_cast<const u32x4_t*>(w_src + (size_t)stage * 2 * 4096 + (c >> 1) * 2048 + (c & 1) * 512);
        else g[c] = *reinterpret_cast<const u32x4_t*>(a_src[c - 4] + (size_t)stage * kStageK);
    };
    auto store_one = [&](int buf, int c) {
        unsigned char* base = tiles_lds + buf * kStageBytes;
        if (c < 4) *reinterpret_cast<u32x4_t*>(base + w_dst + c * 1024) = g[c];
        else *reinterpret_cast<u32x4_t*>(base + a_dst[c - 4]) = g[c];
    };

    f32x16_t acc[TM][2];
#pragma unroll
    for (int tt = 0; tt < TM; ++tt)
#pragma unroll
        for (int rt = 0; rt < 2; ++rt)
#pragma unroll
            for (int v = 0; v < 16; ++v) acc[tt][rt][v] = 0.f;

    const int w_read = wn * 2 * 4096 + lane * 16;
    int a_read[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) a_read[j] = kStageW + (wm * TM * 32 + r32) * 128 + (((2 * j + h) ^ ((r32 >> 1) & 7)) * 16);
    struct Frags { bf16x8_t w[2]; bf16x8_t a[TM]; };
    auto read_w = [&](Frags& f, int buf, int j, int rt) {
        f.w[rt] = __builtin_bit_cast(bf16x8_t, *reinterpret_cast<const u32x4_t*>(
            tiles_lds + buf * kStageBytes + w_read + (j >> 1) * 4096 + (2 * rt + (j & 1)) * 1024));
    };
    auto read_a = [&](Frags& f, int buf, int j, int tt) {
        f.a[tt] = __builtin_bit_cast(bf16x8_t, *reinterpret_cast<const u32x4_t*>(
            tiles_lds + buf * kStageBytes + a_read[j] + tt * 4096));
    };
    auto mfma = [&](const Frags& f, int tt, int rt) {
        acc[tt][rt] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(f.w[rt], f.a[tt], acc[tt][rt], 0, 0, 0);
    };
    // Sub-step j of a stage: piece j of w and, for j < TM, piece 4 + j of the activations are copied: stored for the
    // next stage (asked for one stage ago; all but the loads of the other sub-steps since have arrived), then asked
    // for again for the stage after next.
    auto wait_pieces = [&](int j) {
        if (TM == 4) tiles_wait_loads<6>();
        else if (j < TM) tiles_wait_loads<4>();
        else tiles_wait_loads<5>();
    };
    // sub-step j < 3: its 2 TM products with the reads of sub-step j + 1 and the copies between them
    auto sub = [&](const Frags& cur, Frags& nxt, int buf, int j, int far) {
        read_w(nxt, buf, j + 1, 0); read_w(nxt, buf, j + 1, 1); read_a(nxt, buf, j + 1, 0); SB();
        mfma(cur, 0, 0); SB();
        wait_pieces(j); store_one(buf ^ 1, j); SB();
        mfma(cur, 0, 1); SB();
        read_a(nxt, buf, j + 1, 1); SB();
        mfma(cur, 1, 0); SB();
        if (j < TM) { store_one(buf ^ 1, 4 + j); SB(); }
        mfma(cur, 1, 1); SB();
        if (TM == 4) {
            read_a(nxt, buf, j + 1, 2); SB();
            mfma(cur, 2, 0); SB();
            fetch_one(j, far); SB();
            mfma(cur, 2, 1); SB();
            read_a(nxt, buf, j + 1, 3); SB();
            mfma(cur, 3, 0); SB();
            fetch_one(4 + j, far); SB();
            mfma(cur, 3, 1); SB();
        } else {
            fetch_one(j, far); SB();
            if (j < TM) { fetch_one(4 + j, far); SB(); }
        }
    };

    Frags f0, f1;
    // prologue: the first stage into buffer 0; the pieces of the second asked for in the order in which they are stored
#pragma unroll
    for (int c = 0; c < kPieces; ++c) fetch_one(c, 0);
#pragma unroll
    for (int c = 0; c < kPieces; ++c) store_one(0, c);
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        fetch_one(j, min(1, stages - 1));
        if (j < TM) fetch_one(4 + j, min(1, stages - 1));
    }
    __syncthreads();
    read_w(f0, 0, 0, 0); read_w(f0, 0, 0, 1);
#pragma unroll
    for (int tt = 0; tt < TM; ++tt) read_a(f0, 0, 0, tt);
    SB();
    for (int s = 0; s + 1 < stages; ++s) {
        const int buf = s & 1, far = min(s + 2, stages - 1);                 // (past the end: the last stage again, never stored)
        sub(f0, f1, buf, 0, far);
        sub(f1, f0, buf, 1, far);
        sub(f0, f1, buf, 2, far);
        // sub-step 3: the last copies and half of the products, the barrier, then the first reads of the next stage
        mfma(f1, 0, 0); SB();
        wait_pieces(3); store_one(buf ^ 1, 3); SB();
        mfma(f1, 1, 0); SB();
        if (TM == 4) { store_one(buf ^ 1, 7); SB(); mfma(f1, 2, 0); SB(); }
        fetch_one(3, far); SB();
        if (TM == 4) { mfma(f1, 3, 0); SB(); fetch_one(7, far); SB(); }
        __syncthreads();
        SB();
        read_w(f0, buf ^ 1, 0, 0); read_w(f0, buf ^ 1, 0, 1);
#pragma unroll
        for (int tt = 0; tt < TM; ++tt) read_a(f0, buf ^ 1, 0, tt);
        SB();
#pragma unroll
        for (int tt = 0; tt < TM; ++tt) { mfma(f1, tt, 1); SB(); }
    }
    {
        const int buf = (stages - 1) & 1;
        auto last = [&](const Frags& cur, Frags& nxt, int j) {
            read_w(nxt, buf, j + 1, 0); read_w(nxt, buf, j + 1, 1);
#pragma unroll
            for (int tt = 0; tt < TM; ++tt) read_a(nxt, buf, j + 1, tt);
            SB();
#pragma unroll
            for (int tt = 0; tt < TM; ++tt) { mfma(cur, tt, 0); SB(); mfma(cur, tt, 1); SB(); }
        };
        last(f0, f1, 0); last(f1, f0, 1); last(f0, f1, 2);
#pragma unroll
        for (int tt = 0; tt < TM; ++tt) { mfma(f1, tt, 0); SB(); mfma(f1, tt, 1); SB(); }
    }

    if (!has_rows) return;
#pragma unroll
    for (int tt = 0; tt < TM; ++tt) {
        const int token = m0 + 32 * (wm * TM + tt) + r32;
        if (token >= M) continue;
        TO* orow = out + (size_t)token * ldo;
        if (EPI == EPI_SWIGLU) {
#pragma unroll
            for (int rt = 0; rt < 2; ++rt)
#pragma unroll
                for (int q = 0; q < 2; ++q) {
                    const int col = 32 * nb + 16 * rt + 8 * q + 4 * h;
                    float y[4];
#pragma unroll
                    for (int e = 0; e < 4; ++e) {
                        const float gt = acc[tt][rt][4 * q + e], u = acc[tt][rt][8 + 4 * q + e];
                        y[e] = gt / (1.0f + __expf(-gt)) * u;
                    }
                    if (sizeof(TO) == 2 && col + 3 < N / 2 && ((ldo & 3) == 0) && ((reinterpret_cast<uintptr_t>(out) & 7) == 0)) {
                        uint2 pk;
                        pk.x = tiles_pack_bf16(y[0], y[1]);
                        pk.y = tiles_pack_bf16(y[2], y[3]);
                        *reinterpret_cast<uint2*>(orow + col) = pk;
                    } else if (sizeof(TO) == 4 && col + 3 < N / 2 && ((ldo & 3) == 0) && ((reinterpret_cast<uintptr_t>(out) & 15) == 0)) {
                        *reinterpret_cast<float4*>(orow + col) = make_float4(y[0], y[1], y[2], y[3]);
                    } else {
#pragma unroll
                        for (int e = 0; e < 4; ++e)
                            if (col + e < N / 2) store_f32(orow + col + e, y[e]);
                    }
                }
        } else {
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

// Blocks 0 .. blocks4 - 1 take tiles of 256 tokens over the first n_full row tiles, the blocks after them tiles of
// 128 tokens over the remaining row tiles.  A row tile and a part of k together are one index u = row tile *
// parts + part, and XCD x takes the u that are x modulo 8, walking all token tiles of one before the next: blocks
// that run together on an XCD then share their weights (same u) and their activations (same part of k).
template <typename TO, int EPI>
__global__ __launch_bounds__(kTileWaves * kWave) void gemm_tiles_kernel(
        TO* __restrict__ out, const bf16_t* __restrict__ a, int lda, const unsigned char* __restrict__ wp,
        const float* __restrict__ bias, int M, int N, int K, int ldo, size_t part_stride, int n_row_blocks,
        int m_tiles4, int m_tiles2, int n_full, int n_tiles, int blocks4, int parts) {
    extern __shared__ __attribute__((aligned(1024))) unsigned char tiles_lds[];
    const int stages = K / kStageK;
    const bool big = (int)blockIdx.x < blocks4;
    const int b = big ? blockIdx.x : blockIdx.x - blocks4;
    const int m_tiles = big ? m_tiles4 : m_tiles2;
    const int xcd = b & 7, jb = b >> 3;
    const int m_tile = jb % m_tiles, u = xcd + 8 * (jb / m_tiles);
    const int part = u % parts, n_tile = (big ? 0 : n_full) + u / parts;
    if (n_tile >= (big ? n_full : n_tiles)) return;
    // the parts divide the stages evenly: part p takes [stages p / parts, stages (p + 1) / parts), none is empty
    // when there are at least as many stages as parts
    const int s0 = (int)((long long)stages * part / parts), s1 = (int)((long long)stages * (part + 1) / parts);
    TO* dst = out + (size_t)part * part_stride;
    if (big) tile_body<4, TO, EPI>(tiles_lds, dst, a, lda, wp, bias, M, N, K, ldo, n_row_blocks, m_tile, n_tile, s0, s1);
    else tile_body<2, TO, EPI>(tiles_lds, dst, a, lda, wp, bias, M, N, K, ldo, n_row_blocks, m_tile, n_tile, s0, s1);
}

// How the tiles are cut: row tiles 0 .. n_full - 1 in tiles of 256 tokens, the rest in tiles of 128 tokens.
// token_tiles 4: all of 256, 2: all of 128, 0: the last round of blocks in tiles of 128 tokens when the tiles of 256
// would fill less than half of it.
static int tiles_n_full(int n_tiles, int m_tiles4, int parts, int token_tiles, int compute_units) {
    if (token_tiles == 4) return n_tiles;
    if (token_tiles == 2) return 0;
    const int per_row_tile = m_tiles4 * parts;
    const int rest = (n_tiles * per_row_tile) % compute_units;
    if (rest == 0 || rest > compute_units / 2 || n_tiles * per_row_tile < compute_units) return n_tiles;
    return n_tiles - (rest + per_row_tile - 1) / per_row_tile;
}

template <typename TO, int EPI>
static int launch_tiles(void* out, const void* a, int lda, const void* wp, const float* bias, int M, int N, int K,
                        int ldo, long long part_stride, int parts, int token_tiles, int compute_units, hipStream_t stream) {
    const int n_row_blocks = (N + 63) / 64, n_tiles = (n_row_blocks + kWavesN - 1) / kWavesN;
    const int m4 = (M + 255) / 256, m2 = (M + 127) / 128;
    const int n_full = tiles_n_full(n_tiles, m4, parts, token_tiles, compute_units);
    const int u4 = n_full * parts, u2 = (n_tiles - n_full) * parts;
    const int blocks4 = m4 * ((u4 + 7) / 8) * 8, blocks2 = m2 * ((u2 + 7) / 8) * 8;
    constexpr size_t smem = (size_t)2 * (kStageW + 256 * kStageK * 2);
    // (the attribute is set once per instance: not per launch, which may be recorded into a graph)
    static bool ready = false;
    if (!ready) {
        hipError_t e = hipFuncSetAttribute((const void*)gemm_tiles_kernel<TO, EPI>,
                                           hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem);
        if (e != hipSuccess) return (int)e;
        ready = true;
    }
    gemm_tiles_kernel<TO, EPI><<<blocks4 + blocks2, kTileWaves * kWave, smem, stream>>>(
        (TO*)out, (const bf16_t*)a, lda, (const unsigned char*)wp, bias, M, N, K, ldo, (size_t)part_stride, n_row_blocks,
        m4, m2, n_full, n_tiles, blocks4, parts);
    return LLOGOS_LAUNCH_CHECK();
}

// a: bfloat16 [M][lda]; packed_w: llogos_pack_weights of w [N][K]; out [parts][M][ldo] bfloat16 or float32.
// epilogue 0: out = a . w^T (+ bias [N]); 1: w's 16-row strips alternate gate and up rows, out is
// [M][N / 2] = silu(gate) * up (no bias, one part).  parts > 1: float32 partial sums over ranges of k, part_stride
// elements apart, no bias.  token_tiles: see tiles_n_full.  compute_units: of the GPU, for that choice.
// K must be a multiple of 64 and every part must hold at least two stages of 64.
LLOGOS_EXPORT int llogos_gemm_tiles_bf16(void* out, int out_dtype, const void* a, int lda, const void* packed_w,
                                         const float* bias, int M, int N, int K, int ldo, long long part_stride,
                                         int epilogue, int parts, int token_tiles, int compute_units, hipStream_t stream) {
    if (M <= 0 || N <= 0 || K <= 0 || out == nullptr || a == nullptr || packed_w == nullptr) return LLOGOS_BAD_ARGUMENT;
    if (out_dtype != DT_BF16 && out_dtype != DT_F32) return LLOGOS_BAD_ARGUMENT;
    if (epilogue != EPI_PLAIN && epilogue != EPI_SWIGLU) return LLOGOS_BAD_ARGUMENT;
    if ((K % kStageK) || (lda % 8) || lda < K || ((uintptr_t)a % 16) || ((uintptr_t)packed_w % 16)) return LLOGOS_UNSUPPORTED;
    if (epilogue == EPI_SWIGLU && ((N % 32) || bias != nullptr || ldo < N / 2 || parts != 1)) return LLOGOS_BAD_ARGUMENT;
    if (epilogue == EPI_PLAIN && ldo < N) return LLOGOS_BAD_ARGUMENT;
    if (token_tiles != 4 && token_tiles != 2 && token_tiles != 0) return LLOGOS_BAD_ARGUMENT;
    if (parts < 1 || compute_units < 1) return LLOGOS_BAD_ARGUMENT;
    if (parts > 1 && (out_dtype != DT_F32 || bias != nullptr || part_stride < (long long)M * ldo)) return LLOGOS_BAD_ARGUMENT;
    if (parts > 1 && (K / kStageK) / parts < 2) return LLOGOS_UNSUPPORTED;          // every part holds two stages or more
#define GO(EPI) do { if (out_dtype == DT_BF16) return launch_tiles<bf16_t, EPI>(out, a, lda, packed_w, bias, M, N, K, ldo, part_stride, parts, token_tiles, compute_units, stream); \
                     return launch_tiles<float, EPI>(out, a, lda, packed_w, bias, M, N, K, ldo, part_stride, parts, token_tiles, compute_units, stream); } while (0)
    if (epilogue == EPI_SWIGLU) GO(EPI_SWIGLU);
    GO(EPI_PLAIN);
#undef GO
}
