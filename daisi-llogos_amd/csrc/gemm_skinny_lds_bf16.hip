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
//
// PACKED: the weights are a copy of w in the order the waves take them (llogos_pack_weights):
// a wave's fragment of 16 rows x 32 k is 1 KB of consecutive memory, a block's four fragments of a
// step 4 KB, its steps follow one another.  Every load then asks for whole cache lines (the
// row-major form asks for 16 half lines), and the loads are non-temporal: the weights are read
// once.  llogos_gemm_packed_bf16 at the end of the file.
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

enum { PRODUCE_PLAIN = 0, PRODUCE_SWIGLU_F32 = 1, PRODUCE_SWIGLU_BF16 = 2, PRODUCE_UNSCALED = 3 };
constexpr int kNormRows = 16;        // rows at most when the activations are rows of a norm without their scale

struct ActSource {
    const void* ptr;        // plain, unscaled: bf16 [M][lda]; swiglu: [parts][M][2 K] float32 or bf16
    int lda;                // plain, unscaled: row stride in elements; swiglu: 2 K
    int parts;              // swiglu: partial products to add
    size_t part_stride;     // elements between parts
    // unscaled: the activations are x * w of an rmsnorm over rows x of `width` values whose sums of squares
    // lie in sums [n_sums][kNormRows] by parts (llogos_gemm_residual_bf16); the product of row m is
    // multiplied by 1 / sqrt(sum_m / width + eps) in the epilogue
    const float* sums;
    int n_sums;
    int width;
    float eps;
};

// eight consecutive activations (k .. k + 7 of row m) as bf16
template <int MODE>
__device__ __forceinline__ uint4 produce8(const ActSource& src, int m, int k, int K) {
    if (MODE == PRODUCE_PLAIN || MODE == PRODUCE_UNSCALED) {
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

typedef unsigned u32x4 __attribute__((ext_vector_type(4)));

template <int RB, int MB, int MODE, typename TO, int CHUNK, int WAVES = kLdsWaves, bool PACKED = false, bool GATED = false>
__global__ __launch_bounds__(WAVES * kWave) void gemm_skinny_lds_kernel(
        TO* __restrict__ out, ActSource src, const bf16_t* __restrict__ w, const float* __restrict__ bias,
        int M, int N, int K, int ldo, size_t part_stride, int k_per_block, int parts) {
    constexpr int kRows = MB * 16;
    constexpr int kRowLen = CHUNK + kRowPad;
    constexpr int kPieces = kRows * (CHUNK / 8);                    // 16-byte pieces of a chunk
    constexpr int kPiecesPerThread = (kPieces + WAVES * kWave - 1) / (WAVES * kWave);
    __shared__ __attribute__((aligned(16))) bf16_t lds[2][kRows][kRowLen];
    __shared__ float inv_rms[kNormRows], squares_by_part[16 * kNormRows];

    const int lane = threadIdx.x & (kWave - 1), wave = threadIdx.x / kWave;
    const int r = lane & 15, g = lane >> 4;
    // Blocks go to the 8 XCDs in turn, each with an L2 of its own: a block's part of k is its
    // index modulo the parts, so that an XCD sees few parts and its L2 keeps their activations
    // (with 8 parts one each) while the weights stream through.
    const int split = blockIdx.x % parts, n_block = blockIdx.x / parts;
    const int n0 = (n_block * WAVES + wave) * (16 * RB);
    const int k_begin = split * k_per_block;
    const int k_end = min(K, k_begin + k_per_block);
    const int n_chunks = (k_end - k_begin + CHUNK - 1) / CHUNK;

    const bf16_t* wrow[RB];
#pragma unroll
    for (int rb = 0; rb < RB; ++rb)                                   // rows past N read a valid row, never stored
        wrow[rb] = w + (size_t)min(n0 + rb * 16 + r, N - 1) * K + g * 8;

    // PACKED: w is [blocks of 16 * WAVES rows][steps of 32 k][wave][lane] 16-byte fragments, zero-padded
    // (packed blocks are 64 rows: a block of 8 waves takes two of them)
    const u32x4* wpk = reinterpret_cast<const u32x4*>(w) +
                       ((size_t)(n_block * (WAVES / 4) + wave / 4) * ((K + 31) / 32) * 4 + (wave & 3)) * kWave + lane;

    f32x4 acc[RB][MB];
#pragma unroll
    for (int rb = 0; rb < RB; ++rb)
#pragma unroll
        for (int mb = 0; mb < MB; ++mb) acc[rb][mb] = f32x4{0.f, 0.f, 0.f, 0.f};

    uint4 stage[kPiecesPerThread];
    auto fetch_acts = [&](int k0) {                                   // global -> registers
#pragma unroll
        for (int i = 0; i < kPiecesPerThread; ++i) {
            const int piece = i * (WAVES * kWave) + threadIdx.x;
            const int m = piece / (CHUNK / 8), kk = k0 + (piece % (CHUNK / 8)) * 8;
            stage[i] = make_uint4(0, 0, 0, 0);
            if (piece < kPieces && m < M && kk < k_end) stage[i] = produce8<MODE>(src, m, kk, K);
        }
    };
    auto store_acts = [&](int buf) {                                  // registers -> LDS
#pragma unroll
        for (int i = 0; i < kPiecesPerThread; ++i) {
            const int piece = i * (WAVES * kWave) + threadIdx.x;
            if (piece < kPieces)
                *reinterpret_cast<uint4*>(&lds[buf][piece / (CHUNK / 8)][(piece % (CHUNK / 8)) * 8]) = stage[i];
        }
    };
    bf16x8 wf0[(CHUNK / 32)][RB], wf1[(CHUNK / 32)][RB];
    auto fetch_w = [&](bf16x8 (&wf)[(CHUNK / 32)][RB], int k0) {
#pragma unroll
        for (int s = 0; s < (CHUNK / 32); ++s) {
            if (PACKED) {
                u32x4 v = {0, 0, 0, 0};
                if (k0 + s * 32 < k_end) v = __builtin_nontemporal_load(wpk + (size_t)((k0 >> 5) + s) * (4 * kWave));
                wf[s][0] = __builtin_bit_cast(bf16x8, v);
                continue;
            }
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

    // PRODUCE_UNSCALED: thread (j, m) adds parts j, j + 16, ... of row m's sum of squares; its loads go out
    // first, so that they have arrived with the first activations and cost no wait of their own; thread m adds
    // the 16 sums in ascending j at the end: the same additions in every block
    float row_squares = 0.f, early[16];
    if (MODE == PRODUCE_UNSCALED && threadIdx.x < 16 * kNormRows) {
#pragma unroll
        for (int i = 0; i < 16; ++i) {
            const int p = threadIdx.x / kNormRows + 16 * i;
            early[i] = p < src.n_sums ? src.sums[(size_t)p * kNormRows + (threadIdx.x & (kNormRows - 1))] : 0.f;
        }
    }
    auto add_row_squares = [&]() {
        if (MODE == PRODUCE_UNSCALED && threadIdx.x < 16 * kNormRows) {
            const int m = threadIdx.x & (kNormRows - 1), j = threadIdx.x / kNormRows;
#pragma unroll
            for (int i = 0; i < 16; ++i) row_squares += early[i];
            for (int p = j + 256; p < src.n_sums; p += 16) row_squares += src.sums[(size_t)p * kNormRows + m];
            squares_by_part[threadIdx.x] = row_squares;
        }
    };
    if (n_chunks > 0) {
        fetch_acts(k_begin);
        fetch_w(wf0, k_begin);
        store_acts(0);
        add_row_squares();
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

    if (MODE == PRODUCE_UNSCALED) {
        if (n_chunks <= 0) { add_row_squares(); __syncthreads(); }
        if (threadIdx.x < kNormRows) {
            float t = 0.f;
#pragma unroll
            for (int j = 0; j < 16; ++j) t += squares_by_part[j * kNormRows + threadIdx.x];
            inv_rms[threadIdx.x] = 1.0f / sqrtf(t / (float)src.width + src.eps);
        }
        __syncthreads();
    }
    if (GATED) {
        // The packed strips alternate between 16 gate rows and the 16 up rows of the same columns
        // (llogos_pack_weights with gate_rows): waves 0 and 2 hold gate values, waves 1 and 3 the up
        // values of the same (column, token) in the same lane and register.  The up waves hand
        // theirs over through LDS, and out [M][N / 2] gets silu(gate) * up: the gate/up product
        // never goes to memory.  One part only.
        float* xch = reinterpret_cast<float*>(&lds[0][0][0]);
        __syncthreads();                                             // the last chunk has been read
        if (wave & 1) {
#pragma unroll
            for (int mb = 0; mb < MB; ++mb)
#pragma unroll
                for (int i = 0; i < 4; ++i) xch[(((wave >> 1) * MB + mb) * 4 + i) * kWave + lane] = acc[0][mb][i];
        }
        __syncthreads();
        if (wave & 1) return;
        const int col0 = (n_block * 2 + (wave >> 1)) * 16 + 4 * g;   // column of silu(gate) * up
#pragma unroll
        for (int mb = 0; mb < MB; ++mb) {
            const int m = mb * 16 + r;
            if (m >= M) continue;
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const float row_scale = MODE == PRODUCE_UNSCALED ? inv_rms[m] : 1.0f;
                const float gate = acc[0][mb][i] * row_scale, up = xch[(((wave >> 1) * MB + mb) * 4 + i) * kWave + lane] * row_scale;
                const float y = gate * __builtin_amdgcn_rcpf(1.0f + __builtin_amdgcn_exp2f(-1.4426950408889634f * gate)) * up;
                if (col0 + i < N / 2) store_f32(out + (size_t)m * ldo + col0 + i, y);
            }
        }
        return;
    }
    // acc[rb][mb][i] = sum for row n0 + rb * 16 + 4 g + i of w and activation row mb * 16 + r
    TO* dst = out + (size_t)split * part_stride;
#pragma unroll
    for (int rb = 0; rb < RB; ++rb)
#pragma unroll
        for (int mb = 0; mb < MB; ++mb) {
            const int m = mb * 16 + r;
            if (m >= M) continue;
            const float row_scale = MODE == PRODUCE_UNSCALED ? inv_rms[m] : 1.0f;
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const int n = n0 + rb * 16 + 4 * g + i;
                if (n < N) store_f32(dst + (size_t)m * ldo + n, acc[rb][mb][i] * row_scale + (bias ? bias[n] : 0.f));
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

template <int RB, int MB, int MODE, int CHUNK = kChunkK, int WAVES = kLdsWaves, bool PACKED = false, bool GATED = false>
static int launch_lds(void* out, int out_dtype, const ActSource& src, const bf16_t* w, const float* bias,
                      int M, int N, int K, int ldo, size_t part_stride, int kpb, int parts, hipStream_t stream) {
    const int n_blocks = (N + 16 * RB * WAVES - 1) / (16 * RB * WAVES);
    if (out_dtype == DT_BF16)
        gemm_skinny_lds_kernel<RB, MB, MODE, bf16_t, CHUNK, WAVES, PACKED, GATED><<<n_blocks * parts, WAVES * kWave, 0, stream>>>(
            (bf16_t*)out, src, w, bias, M, N, K, ldo, part_stride, kpb, parts);
    else
        gemm_skinny_lds_kernel<RB, MB, MODE, float, CHUNK, WAVES, PACKED, GATED><<<n_blocks * parts, WAVES * kWave, 0, stream>>>(
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


// w [N][K] bf16 row-major -> packed [ceil(N / 64)][ceil(K / 32)][4][64] fragments of 8 bf16, zero-padded:
// fragment (block, step, wave, lane) holds row 64 block + 16 wave + (lane & 15), k = 32 step + 8 (lane >> 4) .. + 7
// gate_rows > 0: w is [gate (gate_rows rows); up (gate_rows rows)], gate_rows a multiple of 16, and the packed
// strips alternate: strip 2 j holds gate rows 16 j .., strip 2 j + 1 the up rows 16 j .. (for the products
// that make silu(gate) * up in their epilogue).
__global__ void pack_weights_kernel(uint4* __restrict__ dst, const bf16_t* __restrict__ src, int N, int K, long long pieces,
                                    int gate_rows) {
    const long long i = (long long)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= pieces) return;
    const int lane = (int)(i & 63), wave = (int)((i >> 6) & 3);
    const long long bs = i >> 8;
    const int steps = (K + 31) / 32;
    const int step = (int)(bs % steps), block = (int)(bs / steps);
    int n = block * 64 + wave * 16 + (lane & 15);
    const int k = step * 32 + (lane >> 4) * 8;
    if (gate_rows > 0) {
        const int strip = n >> 4;
        n = ((strip & 1) ? gate_rows : 0) + (strip >> 1) * 16 + (n & 15);
    }
    bf16_t v[8];
#pragma unroll
    for (int e = 0; e < 8; ++e) v[e] = (n < N && k + e < K) ? src[(size_t)n * K + k + e] : (bf16_t)0;
    dst[i] = *reinterpret_cast<const uint4*>(v);
}

LLOGOS_EXPORT long long llogos_packed_weight_bytes(int N, int K) {
    return (long long)((N + 63) / 64) * ((K + 31) / 32) * 4096;
}

LLOGOS_EXPORT int llogos_pack_weights(void* dst, const void* src, int N, int K, int gate_rows, hipStream_t stream) {
    if (N <= 0 || K <= 0 || dst == nullptr || src == nullptr) return LLOGOS_BAD_ARGUMENT;
    if (gate_rows < 0 || (gate_rows > 0 && (gate_rows % 16 || N != 2 * gate_rows))) return LLOGOS_BAD_ARGUMENT;
    const long long pieces = llogos_packed_weight_bytes(N, K) / 16;
    pack_weights_kernel<<<(unsigned)((pieces + 255) / 256), 256, 0, stream>>>((uint4*)dst, (const bf16_t*)src, N, K, pieces, gate_rows);
    return LLOGOS_LAUNCH_CHECK();
}

// The few-row product on packed weights (llogos_pack_weights): the same kernel, whose waves then
// read their weights as whole 1 KB fragments, a block 4 KB at a time and its whole share of a
// matrix as one contiguous run, with loads that do not stay in the caches.  Measured on the
// MI355X against the row-major form (16 rows x 64 bytes per load): 8B gate/up at 8 rows 35.8 us
// against 46.3 (6.6 TB/s against 5.1), o 7.8 against 13.6, the head 156 against 185.
// Arguments as llogos_gemm_skinny_lds_bf16; `chunk` (128 or 256) is the k an LDS buffer holds and
// the unit of the parts: parts = llogos_gemm_packed_parts(K, splits, chunk).
static int packed_k_per_block(int K, int splits, int chunk) {
    return ((K + splits - 1) / splits + chunk - 1) / chunk * chunk;
}

LLOGOS_EXPORT int llogos_gemm_packed_parts(int K, int splits, int chunk) {
    if (K <= 0 || (chunk != 128 && chunk != 256)) return 0;
    if (splits <= 1) return 1;
    const int kpb = packed_k_per_block(K, splits, chunk);
    return (K + kpb - 1) / kpb;
}

LLOGOS_EXPORT int llogos_gemm_packed_bf16(void* out, int out_dtype, const void* act, int mode, int lda,
                                          int act_parts, long long act_part_stride, const void* packed_w,
                                          const float* bias, int M, int N, int K, int ldo,
                                          long long part_stride, int splits, int chunk, hipStream_t stream) {
    if (M <= 0 || N <= 0 || K <= 0 || ldo < N || splits < 1 || act_parts < 1) return LLOGOS_BAD_ARGUMENT;
    if (out_dtype != DT_BF16 && out_dtype != DT_F32) return LLOGOS_BAD_ARGUMENT;
    if (mode < PRODUCE_PLAIN || mode > PRODUCE_SWIGLU_BF16 || (chunk != 128 && chunk != 256)) return LLOGOS_BAD_ARGUMENT;
    if (M > 64 || (K % 8) || (lda % 8) || ((uintptr_t)act % 16) || ((uintptr_t)packed_w % 16) || (act_part_stride % 4))
        return LLOGOS_UNSUPPORTED;
    if (mode == PRODUCE_PLAIN ? lda < K : lda < 2 * K) return LLOGOS_BAD_ARGUMENT;
    const int parts = llogos_gemm_packed_parts(K, splits, chunk);
    if (parts > 1 && (out_dtype != DT_F32 || bias != nullptr || part_stride < (long long)M * ldo))
        return LLOGOS_BAD_ARGUMENT;
    const int kpb = packed_k_per_block(K, parts, chunk);
    ActSource src{act, lda, act_parts, (size_t)act_part_stride};
    const bf16_t* W = (const bf16_t*)packed_w;
    const int mb = (M + 15) / 16;
#define GO(MB, MODE, CH) return launch_lds<1, MB, MODE, CH, kLdsWaves, true>(out, out_dtype, src, W, bias, M, N, K, ldo, \
                                                                            (size_t)part_stride, kpb, parts, stream)
#define BY_MODE(MB, CH) do { if (mode == PRODUCE_PLAIN) GO(MB, PRODUCE_PLAIN, CH); \
                             if (mode == PRODUCE_SWIGLU_F32) GO(MB, PRODUCE_SWIGLU_F32, CH); \
                             GO(MB, PRODUCE_SWIGLU_BF16, CH); } while (0)
#define BY_ROWS(CH) do { if (mb == 1) BY_MODE(1, CH); if (mb == 2) BY_MODE(2, CH); if (mb == 3) BY_MODE(3, CH); BY_MODE(4, CH); } while (0)
    if (chunk == 128) BY_ROWS(128);
    BY_ROWS(256);
#undef BY_ROWS
#undef BY_MODE
#undef GO
}

// The same on a matrix packed with gate_rows (strips of gate and up rows in turn): out [M][ldo]
// (ldo >= N / 2) = silu(a . gate^T) * (a . up^T) in bfloat16 or float32; plain activations, one
// part, no bias.
LLOGOS_EXPORT int llogos_gemm_packed_gated_bf16(void* out, int out_dtype, const void* act, int lda, const void* packed_w,
                                                int M, int N, int K, int ldo, int chunk, hipStream_t stream) {
    if (M <= 0 || N <= 0 || K <= 0 || (N % 32) || ldo < N / 2) return LLOGOS_BAD_ARGUMENT;
    if (out_dtype != DT_BF16 && out_dtype != DT_F32) return LLOGOS_BAD_ARGUMENT;
    if (chunk != 128 && chunk != 256) return LLOGOS_BAD_ARGUMENT;
    if (M > 64 || (K % 8) || (lda % 8) || lda < K || ((uintptr_t)act % 16) || ((uintptr_t)packed_w % 16)) return LLOGOS_UNSUPPORTED;
    const int kpb = packed_k_per_block(K, 1, chunk);
    ActSource src{act, lda, 1, 0};
    const bf16_t* W = (const bf16_t*)packed_w;
    const int mb = (M + 15) / 16;
#define GO(MB, CH) return launch_lds<1, MB, PRODUCE_PLAIN, CH, kLdsWaves, true, true>(out, out_dtype, src, W, nullptr, M, N, K, ldo, \
                                                                                     0, kpb, 1, stream)
#define BY_ROWS(CH) do { if (mb == 1) GO(1, CH); if (mb == 2) GO(2, CH); if (mb == 3) GO(3, CH); GO(4, CH); } while (0)
    if (chunk == 128) BY_ROWS(128);
    BY_ROWS(256);
#undef BY_ROWS
#undef GO
}

// The same two products on the rows of an rmsnorm that still lack their scale: act [M][lda] = x * norm_w in
// bfloat16, for up to 16 rows, and sums [n_sums][16] the partial sums of squares of the rows of x over
// `width` values, both left by the product that completed x (llogos_gemm_residual_bf16).  The scale
// 1 / sqrt(sum / width + eps) is a factor of the whole row, so it is applied to the product in the
// epilogue, in float32: no kernel between the product that completes x and this one.  gated = 0: out
// [parts][M][ldo] as llogos_gemm_packed_bf16 (a bias is added after the scale); gated = 1: out [M][ldo] =
// silu(gate) * up as llogos_gemm_packed_gated_bf16.
LLOGOS_EXPORT int llogos_gemm_packed_unscaled_bf16(void* out, int out_dtype, const void* act, int lda, const float* sums,
                                                   int n_sums, int width, float eps, const void* packed_w,
                                                   const float* bias, int M, int N, int K, int ldo,
                                                   long long part_stride, int splits, int chunk, int gated,
                                                   hipStream_t stream) {
    if (M <= 0 || N <= 0 || K <= 0 || splits < 1 || n_sums < 1 || width < 1 || act == nullptr || sums == nullptr)
        return LLOGOS_BAD_ARGUMENT;
    if (out_dtype != DT_BF16 && out_dtype != DT_F32) return LLOGOS_BAD_ARGUMENT;
    if (chunk != 128 && chunk != 256) return LLOGOS_BAD_ARGUMENT;
    if (gated ? ((N % 32) || ldo < N / 2 || bias != nullptr) : ldo < N) return LLOGOS_BAD_ARGUMENT;
    if (M > kNormRows || (K % 8) || (lda % 8) || lda < K || ((uintptr_t)act % 16) || ((uintptr_t)packed_w % 16))
        return LLOGOS_UNSUPPORTED;
    const int parts = gated ? 1 : llogos_gemm_packed_parts(K, splits, chunk);
    if (parts > 1 && (out_dtype != DT_F32 || bias != nullptr || part_stride < (long long)M * ldo))
        return LLOGOS_BAD_ARGUMENT;
    const int kpb = packed_k_per_block(K, parts, chunk);
    ActSource src{act, lda, 1, 0, sums, n_sums, width, eps};
    const bf16_t* W = (const bf16_t*)packed_w;
#define GO(CH, GATED) return launch_lds<1, 1, PRODUCE_UNSCALED, CH, kLdsWaves, true, GATED>(out, out_dtype, src, W, bias, M, N, K, ldo, \
                                                                                            (size_t)part_stride, kpb, parts, stream)
    if (gated) { if (chunk == 128) GO(128, true); GO(256, true); }
    if (chunk == 128) GO(128, false);
    GO(256, false);
#undef GO
}
