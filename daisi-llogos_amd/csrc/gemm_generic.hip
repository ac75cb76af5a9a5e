// out[M, N] = a[M, K] . w[N, K]^T (+ bias[N]) with every product and sum in 32-bit
// floats (plain FMA, no matrix-core input rounding).  It is the matrix product of the
// float32 engine and the fallback of the bfloat16 engine for shapes its fast kernels
// refuse.  Each output element is summed in the same order whatever M is, so a row's result
// does not depend on the other rows of the batch.  The order is blocked: 16 products into a
// partial sum, 16 of those into a second, those into the total, so that the rounding error
// of a sum over thousands of k grows with the sum's blocks (about 16 + 16 + K / 256 additions
// deep) and not with K.  On 32 layers of k = 4096 and 14336 the logits' largest distance from
// float64 arithmetic was 1.7e-4 with one running sum and is 3.4e-5 with this order.
// (reference: y = x . W^T with W [out, in], Daisi.Llogos.Cuda/kernels/dequant_matmul.cu:216-253.)
#include "common.h"

constexpr int TM = 64, TN = 64, TK = 16;

template <typename TA, typename TW, typename TO>
__global__ __launch_bounds__(256) void gemm_generic_kernel(
        TO* __restrict__ out, const TA* __restrict__ a, const TW* __restrict__ w,
        const float* __restrict__ bias, int M, int N, int K, int lda, int ldo) {
    __shared__ float As[TK][TM + 4];
    __shared__ float Ws[TK][TN + 4];
    const int tid = threadIdx.x;
    const int m0 = blockIdx.y * TM, n0 = blockIdx.x * TN;
    const int ty = tid / 16, tx = tid % 16;
    const int lr = tid / 4, lk = (tid % 4) * 4;   // this thread stages row lr, k lk..lk+3
    float acc[4][4] = {}, mid[4][4] = {};
    for (int k0 = 0; k0 < K; k0 += TK) {
        float part[4][4] = {};
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int k = k0 + lk + j;
            const int am = m0 + lr, wn = n0 + lr;
            As[lk + j][lr] = (am < M && k < K) ? load_f32(a + (size_t)am * lda + k) : 0.f;
            Ws[lk + j][lr] = (wn < N && k < K) ? load_f32(w + (size_t)wn * K + k) : 0.f;
        }
        __syncthreads();
#pragma unroll
        for (int k = 0; k < TK; ++k) {
            float av[4], wv[4];
#pragma unroll
            for (int i = 0; i < 4; ++i) { av[i] = As[k][ty * 4 + i]; wv[i] = Ws[k][tx * 4 + i]; }
#pragma unroll
            for (int i = 0; i < 4; ++i)
#pragma unroll
                for (int j = 0; j < 4; ++j) part[i][j] = fmaf(av[i], wv[j], part[i][j]);
        }
        const bool fold = ((k0 / TK) & 15) == 15;
#pragma unroll
        for (int i = 0; i < 4; ++i)
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                mid[i][j] += part[i][j];
                if (fold) { acc[i][j] += mid[i][j]; mid[i][j] = 0.f; }
            }
        __syncthreads();
    }
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[i][j] += mid[i][j];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const int m = m0 + ty * 4 + i;
        if (m >= M) continue;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int n = n0 + tx * 4 + j;
            if (n >= N) continue;
            float v = acc[i][j];
            if (bias) v += bias[n];
            store_f32(out + (size_t)m * ldo + n, v);
        }
    }
}

// Few rows in float32 (the float32 engine's single-token steps): the tiled kernel above has one
// block for 64 columns whatever M is, 32 blocks for a matrix of 2,048 rows, and ran such steps at
// 127 GB/s.  Here a wave takes COLS columns and all (up to MR) rows of a: a lane holds 16
// consecutive k of every row and chains their products in ascending k, which is a `part` of the
// tiled kernel; the 16 parts of 256 consecutive k lie in 16 neighbouring lanes and are added in
// ascending order into a `mid`, the mids in ascending order into the total: every sum in the
// order of the tiled kernel, so that the two give the same bits and a row's result does not
// depend on which of them a step's row count selects.
template <int MR, int COLS>
__global__ __launch_bounds__(256) void gemm_few_rows_f32_kernel(
        float* __restrict__ out, const float* __restrict__ a, const float* __restrict__ w,
        const float* __restrict__ bias, int M, int N, int K, int lda, int ldo) {
    const int lane = threadIdx.x & (kWave - 1), wave = threadIdx.x / kWave;
    const int n0 = (blockIdx.x * 4 + wave) * COLS;
    if (n0 >= N) return;
    const int m0 = blockIdx.y * MR;
    float acc[MR];                                              // lane c: the totals of column n0 + c
#pragma unroll
    for (int m = 0; m < MR; ++m) acc[m] = 0.f;
    for (int k0 = 0; k0 < K; k0 += 16 * kWave) {
        const int k = k0 + 16 * lane;                           // this lane's 16 values of k
        float av[MR][16];
#pragma unroll
        for (int m = 0; m < MR; ++m) {
            const float* row = a + (size_t)min(m0 + m, M - 1) * lda;
#pragma unroll
            for (int j = 0; j < 16; j += 4) {
                if (k + j + 3 < K && (lda & 3) == 0 && ((uintptr_t)a & 15) == 0) {
                    const float4 v = *reinterpret_cast<const float4*>(row + k + j);
                    av[m][j] = v.x; av[m][j + 1] = v.y; av[m][j + 2] = v.z; av[m][j + 3] = v.w;
                } else {
#pragma unroll
                    for (int e = 0; e < 4; ++e) av[m][j + e] = k + j + e < K ? row[k + j + e] : 0.f;
                }
            }
        }
#pragma unroll 1
        for (int c = 0; c < COLS; ++c) {
            const float* wrow = w + (size_t)min(n0 + c, N - 1) * K;
            float wv[16];
#pragma unroll
            for (int j = 0; j < 16; j += 4) {
                if (k + j + 3 < K && (K & 3) == 0 && ((uintptr_t)w & 15) == 0) {
                    const float4 v = *reinterpret_cast<const float4*>(wrow + k + j);
                    wv[j] = v.x; wv[j + 1] = v.y; wv[j + 2] = v.z; wv[j + 3] = v.w;
                } else {
#pragma unroll
                    for (int e = 0; e < 4; ++e) wv[j + e] = k + j + e < K ? wrow[k + j + e] : 0.f;
                }
            }
#pragma unroll
            for (int m = 0; m < MR; ++m) {
                float part = 0.f;
#pragma unroll
                for (int j = 0; j < 16; ++j) part = fmaf(av[m][j], wv[j], part);
                // the 16 parts of this lane's group of 16 lanes, added in ascending order
                float mid = 0.f;
#pragma unroll
                for (int j = 0; j < 16; ++j) mid += __shfl(part, (lane & 48) + j, kWave);
                // the four mids of these 1,024 k, in ascending order (groups past K hold zeros)
                float total = acc[m];
#pragma unroll
                for (int g = 0; g < 4; ++g) {
                    const float mg = __shfl(mid, 16 * g, kWave);
                    if (k0 + 256 * g < K) total += mg;
                }
                acc[m] = lane == c ? total : acc[m];
            }
        }
    }
    if (lane < COLS && n0 + lane < N) {
#pragma unroll
        for (int m = 0; m < MR; ++m)
            if (m0 + m < M) out[(size_t)(m0 + m) * ldo + n0 + lane] = acc[m] + (bias ? bias[n0 + lane] : 0.f);
    }
}

LLOGOS_EXPORT int llogos_gemm_generic(void* out, int out_dtype, const void* a, int a_dtype,
                                      const void* w, int w_dtype, const float* bias,
                                      int M, int N, int K, int lda, int ldo, hipStream_t stream) {
    if (M <= 0 || N <= 0 || K <= 0 || lda < K || ldo < N) return LLOGOS_BAD_ARGUMENT;
    if (a_dtype == DT_F32 && w_dtype == DT_F32 && out_dtype == DT_F32 && M <= 32) {
        // enough waves to fill the GPU, then as many columns a wave as that leaves (its rows of a are
        // read once for all of them)
        const int cols = N >= 16 * 4096 ? 16 : (N >= 8 * 4096 ? 8 : (N >= 4 * 4096 ? 4 : 2));
        const int rows = M <= 1 ? 1 : (M <= 2 ? 2 : (M <= 4 ? 4 : 8));
        dim3 fgrid((N + 4 * cols - 1) / (4 * cols), (M + rows - 1) / rows);
#define FEW(MR, COLS) gemm_few_rows_f32_kernel<MR, COLS><<<fgrid, 256, 0, stream>>>( \
        (float*)out, (const float*)a, (const float*)w, bias, M, N, K, lda, ldo)
#define BY_COLS(MR) do { if (cols == 16) FEW(MR, 16); else if (cols == 8) FEW(MR, 8); else if (cols == 4) FEW(MR, 4); \
                         else FEW(MR, 2); } while (0)
        if (rows == 1) BY_COLS(1); else if (rows == 2) BY_COLS(2); else if (rows == 4) BY_COLS(4); else BY_COLS(8);
#undef BY_COLS
#undef FEW
        return LLOGOS_LAUNCH_CHECK();
    }
    dim3 grid((N + TN - 1) / TN, (M + TM - 1) / TM);
#define LAUNCH(TA, TW, TO) gemm_generic_kernel<TA, TW, TO><<<grid, 256, 0, stream>>>( \
        (TO*)out, (const TA*)a, (const TW*)w, bias, M, N, K, lda, ldo)
    const int key = a_dtype * 4 + w_dtype * 2 + out_dtype;
    switch (key) {
        case 0: LAUNCH(float, float, float); break;
        case 1: LAUNCH(float, float, bf16_t); break;
        case 2: LAUNCH(float, bf16_t, float); break;
        case 3: LAUNCH(float, bf16_t, bf16_t); break;
        case 4: LAUNCH(bf16_t, float, float); break;
        case 5: LAUNCH(bf16_t, float, bf16_t); break;
        case 6: LAUNCH(bf16_t, bf16_t, float); break;
        case 7: LAUNCH(bf16_t, bf16_t, bf16_t); break;
        default: return LLOGOS_BAD_ARGUMENT;
    }
#undef LAUNCH
    return LLOGOS_LAUNCH_CHECK();
}
