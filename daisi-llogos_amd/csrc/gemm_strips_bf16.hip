// out[M, N] = a[M, K] . w[N, K]^T for up to 128 rows, third form: both operands go from global
// memory straight into LDS (16 bytes a lane, no registers in between), two to four stages of 64
// values of k ahead of the one that is multiplied, and a block takes 2 to 9 strips of 16 rows of
// w, so that the blocks of a tall matrix come out even over the compute units and the
// activations are read once per 112 or 144 rows of w instead of once per 64.
//
// It is faster than the second form (gemm_skinny_lds_bf16.hip) where all its blocks are resident
// at once, two to a compute unit, and the matrix is tall: gate/up of the Qwen3-14B sizes at 32
// and 64 rows (75 and 85 us against 94 and 108; 9 strips, 2 parts of k, 484 blocks), of the
// Llama-3.1-70B sizes (186 and 200 us against 205 and 227; 7 strips, 512 blocks).  On smaller
// matrices and with more blocks than places it is level or slower, and which height is best is
// erratic; the dispatch uses it only in the first case.
// As many stages are taken as leave LDS for two blocks a unit: one block of 4 waves a unit
// covers too little latency (measured: up to 40 % slower).
// A copy into LDS cannot pad rows, so the 16-byte pieces of a 128-byte row are swizzled: piece p
// of row r lies at p ^ 2 ((r >> 1) & 3), which spreads the 8 rows that a group of lanes reads
// together (two rows share a line of 64 banks) over all banks.
// Outputs are [parts][M][N] like the second form's, summed in the same order (k ascending, the
// same MFMA, the same slots), so the two forms agree bit for bit for equal parts of k.
#include "common.h"

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float f32x4 __attribute__((ext_vector_type(4)));

constexpr int kStripWaves = 4;
constexpr int kStageK = 64;                   // values of k per stage: rows of 128 bytes
constexpr int kMaxStrips = 9;                 // strips of 16 rows of w per block
constexpr int kMaxWaveStrips = (kMaxStrips + kStripWaves - 1) / kStripWaves;

__device__ __forceinline__ int strips_swizzle(int row) { return 2 * ((row >> 1) & 3); }

// waits until at most n of this wave's loads are outstanding (the count must be an immediate)
__device__ __forceinline__ void wait_loads(int n) {
#define LLOGOS_W(N) case N: asm volatile("s_waitcnt vmcnt(" #N ")" ::: "memory"); break;
    switch (n) {
        LLOGOS_W(0) LLOGOS_W(1) LLOGOS_W(2) LLOGOS_W(3) LLOGOS_W(4) LLOGOS_W(5) LLOGOS_W(6) LLOGOS_W(7)
        LLOGOS_W(8) LLOGOS_W(9) LLOGOS_W(10) LLOGOS_W(11) LLOGOS_W(12) LLOGOS_W(13) LLOGOS_W(14) LLOGOS_W(15)
        LLOGOS_W(16) LLOGOS_W(17) LLOGOS_W(18) LLOGOS_W(19) LLOGOS_W(20) LLOGOS_W(21) LLOGOS_W(22) LLOGOS_W(23)
        LLOGOS_W(24) LLOGOS_W(25) LLOGOS_W(26) LLOGOS_W(27) LLOGOS_W(28) LLOGOS_W(29) LLOGOS_W(30) LLOGOS_W(31)
        LLOGOS_W(32) LLOGOS_W(33) LLOGOS_W(34) LLOGOS_W(35) LLOGOS_W(36)
        default: asm volatile("s_waitcnt vmcnt(0)" ::: "memory"); break;
    }
#undef LLOGOS_W
}

// LDS: STAGES x (strips x 16 rows of w, then MB x 16 rows of activations), rows of 128 bytes.
template <int MB, int STAGES, typename TO>
__global__ __launch_bounds__(kStripWaves * kWave) void gemm_strips_kernel(
        TO* __restrict__ out, const bf16_t* __restrict__ a, int lda, const bf16_t* __restrict__ w,
        const float* __restrict__ bias, int M, int N, int K, int ldo, size_t part_stride,
        int strips, int k_per_block, int parts) {
    extern __shared__ __attribute__((aligned(16))) unsigned char strips_raw[];
    const int lane = threadIdx.x & (kWave - 1);
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / kWave);
    const int r = lane & 15, g = lane >> 4;
    const int split = blockIdx.x % parts, tile = blockIdx.x / parts;
    const int n0 = tile * strips * 16;
    const int k_begin = split * k_per_block;
    const int n_stages = (min(K, k_begin + k_per_block) - k_begin) / kStageK;      // K % 64 == 0
    const int w_rows = strips * 16, stage_bytes = (w_rows + MB * 16) * (kStageK * 2);
    // The copy of a stage: instructions of 1 KB = 8 rows; instruction q < 2 strips brings rows of w,
    // the 2 MB after them rows of the activations; they go to the waves in turn.
    const int n_instr = 2 * strips + 2 * MB;
    const int my_instr = (n_instr - wave + kStripWaves - 1) / kStripWaves;           // loads of this wave per stage
    auto copy_stage = [&](int stage, int slot) {
        unsigned char* base = strips_raw + (size_t)slot * stage_bytes;
        const int k0 = k_begin + stage * kStageK;
        for (int q = wave; q < n_instr; q += kStripWaves) {
            const int row = 8 * q + (lane >> 3);                                      // row of the stage's LDS image
            const int piece = (lane & 7) ^ strips_swizzle(row);
            const bf16_t* src;
            if (q < 2 * strips) src = w + (size_t)min(n0 + row, N - 1) * K + k0 + 8 * piece;
            else src = a + (size_t)min(row - w_rows, M - 1) * lda + k0 + 8 * piece;
            __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)src,
                                             (__attribute__((address_space(3))) void*)(base + (size_t)q * 1024), 16, 0, 0);
        }
    };
    f32x4 acc[kMaxWaveStrips][MB];
#pragma unroll
    for (int i = 0; i < kMaxWaveStrips; ++i)
#pragma unroll
        for (int mb = 0; mb < MB; ++mb) acc[i][mb] = f32x4{0.f, 0.f, 0.f, 0.f};

    for (int s = 0; s < STAGES - 1 && s < n_stages; ++s) copy_stage(s, s);
    for (int s = 0; s < n_stages; ++s) {
        // stage s has arrived when only the stages asked for after it are outstanding
        wait_loads(min(STAGES - 2, n_stages - 1 - s) * my_instr);
        __syncthreads();                                   // ... for every wave; and stage s - 1 has been read by all
        if (s + STAGES - 1 < n_stages) copy_stage(s + STAGES - 1, (s + STAGES - 1) % STAGES);
        const unsigned char* base = strips_raw + (size_t)(s % STAGES) * stage_bytes;
#pragma unroll
        for (int ks = 0; ks < kStageK / 32; ++ks) {
            bf16x8 af[MB];
#pragma unroll
            for (int mb = 0; mb < MB; ++mb) {
                const int row = w_rows + mb * 16 + r;
                af[mb] = __builtin_bit_cast(bf16x8, *reinterpret_cast<const uint4*>(
                    base + (size_t)row * 128 + 16 * ((4 * ks + g) ^ strips_swizzle(row))));
            }
#pragma unroll
            for (int i = 0; i < kMaxWaveStrips; ++i) {
                const int st = wave + i * kStripWaves;
                if (st < strips) {
                    const int row = st * 16 + r;
                    const bf16x8 wf = __builtin_bit_cast(bf16x8, *reinterpret_cast<const uint4*>(
                        base + (size_t)row * 128 + 16 * ((4 * ks + g) ^ strips_swizzle(row))));
#pragma unroll
                    for (int mb = 0; mb < MB; ++mb)
                        acc[i][mb] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wf, af[mb], acc[i][mb], 0, 0, 0);
                }
            }
        }
    }
    // acc[i][mb][j] = sum for row n0 + 16 (wave + 4 i) + 4 g + j of w and activation row 16 mb + r
    TO* dst = out + (size_t)split * part_stride;
#pragma unroll
    for (int i = 0; i < kMaxWaveStrips; ++i) {
        const int st = wave + i * kStripWaves;
        if (st >= strips) continue;
#pragma unroll
        for (int mb = 0; mb < MB; ++mb) {
            const int m = mb * 16 + r;
            if (m >= M) continue;
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const int n = n0 + st * 16 + 4 * g + j;
                if (n < N) store_f32(dst + (size_t)m * ldo + n, acc[i][mb][j] + (bias ? bias[n] : 0.f));
            }
        }
    }
}

static int strips_k_per_block(int K, int splits) {            // the same parts of k as the second form takes
    return ((K + splits - 1) / splits + 255) / 256 * 256;
}

// out: [parts][M][ldo] with parts as llogos_gemm_skinny_lds_parts(K, splits) gives them; float32
// and without bias when parts > 1.  strips: 16-row strips of w per block, 2 to 9.  Unsupported
// (-2): K not a multiple of 64, more than 128 rows.
LLOGOS_EXPORT int llogos_gemm_strips_bf16(void* out, int out_dtype, const void* act, int lda, const void* w,
                                          const float* bias, int M, int N, int K, int ldo, long long part_stride,
                                          int splits, int strips, hipStream_t stream) {
    if (M <= 0 || N <= 0 || K <= 0 || ldo < N || splits < 1 || lda < K) return LLOGOS_BAD_ARGUMENT;
    if (strips < 2 || strips > kMaxStrips) return LLOGOS_BAD_ARGUMENT;
    if (out_dtype != DT_BF16 && out_dtype != DT_F32) return LLOGOS_BAD_ARGUMENT;
    if (M > 128 || (K % kStageK) || (lda % 8) || ((uintptr_t)act % 16) || ((uintptr_t)w % 16)) return LLOGOS_UNSUPPORTED;
    int kpb = K, parts = 1;
    if (splits > 1) {
        kpb = strips_k_per_block(K, splits);
        parts = (K + kpb - 1) / kpb;
    }
    if (parts > 1 && (out_dtype != DT_F32 || bias != nullptr || part_stride < (long long)M * ldo))
        return LLOGOS_BAD_ARGUMENT;
    const int mb = (M + 15) / 16, mbt = mb <= 2 ? 2 : (mb <= 4 ? 4 : (mb <= 6 ? 6 : 8));
    // as many stages as leave LDS for two blocks a compute unit (4 waves a unit cover too little latency)
    int stages = 4;
    while (stages > 2 && (size_t)stages * (strips * 16 + mbt * 16) * (kStageK * 2) > 80 * 1024) --stages;
    const size_t smem = (size_t)stages * (strips * 16 + mbt * 16) * (kStageK * 2);
    if (smem > 160 * 1024) return LLOGOS_UNSUPPORTED;
    const int tiles = (N + strips * 16 - 1) / (strips * 16);
    // (the attribute is set once per instance, with the most any call can ask for: not per launch,
    // which may be recorded into a graph)
#define GOS(MB, ST, TO) do { \
        static bool ready = false; \
        if (!ready) { \
            hipError_t e = hipFuncSetAttribute((const void*)gemm_strips_kernel<MB, ST, TO>, \
                                               hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024); \
            if (e != hipSuccess) return (int)e; \
            ready = true; \
        } \
        gemm_strips_kernel<MB, ST, TO><<<tiles * parts, kStripWaves * kWave, smem, stream>>>( \
            (TO*)out, (const bf16_t*)act, lda, (const bf16_t*)w, bias, M, N, K, ldo, (size_t)part_stride, strips, kpb, parts); \
        return LLOGOS_LAUNCH_CHECK(); } while (0)
#define BY_TYPE(MB, ST) do { if (out_dtype == DT_BF16) GOS(MB, ST, bf16_t); else GOS(MB, ST, float); } while (0)
#define BY_STAGES(MB) do { if (stages == 4) BY_TYPE(MB, 4); if (stages == 3) BY_TYPE(MB, 3); BY_TYPE(MB, 2); } while (0)
    if (mbt == 2) BY_STAGES(2);
    if (mbt == 4) BY_STAGES(4);
    if (mbt == 6) BY_STAGES(6);
    BY_STAGES(8);
#undef BY_STAGES
#undef BY_TYPE
#undef GOS
}
