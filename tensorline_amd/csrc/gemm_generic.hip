// C[M, N] = A[M, K] * W[N, K]^T (+ bias[N]):  the plain tiled matrix product.
//
// This is the true 32-bit path (float inputs, float FMA, float accumulation in a fixed order over
// k, no reduced-precision matrix mode) and the any-shape fallback for bfloat16 inputs.  The order
// of accumulation of one output element does not depend on M, so cutting a batch differently does
// not change a result.
#include "common.h"

#define GT_BM 64
#define GT_BN 64
#define GT_BK 16

template <typename TA, typename TW, typename TO>
__global__ __launch_bounds__(256) void gemm_generic_kernel(const TA* __restrict__ A, const TW* __restrict__ W,
                                                          const float* __restrict__ bias, TO* __restrict__ C, int M,
                                                          int N, int K, int lda, int ldc) {
    __shared__ float As[GT_BK][GT_BM + 4];
    __shared__ float Ws[GT_BK][GT_BN + 4];
    const int tid = threadIdx.x;
    const int m0 = blockIdx.y * GT_BM, n0 = blockIdx.x * GT_BN;
    const int tx = tid & 15, ty = tid >> 4;  // 16 x 16 threads, 4 x 4 outputs each
    const int lr = tid >> 2, lk = (tid & 3) * 4;  // loader: row lr of the tile, k offset lk..lk+3

    float acc[4][4];
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[i][j] = 0.f;

    for (int k0 = 0; k0 < K; k0 += GT_BK) {
        const int am = m0 + lr, wn = n0 + lr;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int k = k0 + lk + j;
            As[lk + j][lr] = (am < M && k < K) ? tl_to_float(A[(size_t)am * lda + k]) : 0.f;
            Ws[lk + j][lr] = (wn < N && k < K) ? tl_to_float(W[(size_t)wn * K + k]) : 0.f;
        }
        __syncthreads();
#pragma unroll
        for (int k = 0; k < GT_BK; ++k) {
            float a[4], w[4];
#pragma unroll
            for (int i = 0; i < 4; ++i) a[i] = As[k][ty * 4 + i];
#pragma unroll
            for (int j = 0; j < 4; ++j) w[j] = Ws[k][tx * 4 + j];
#pragma unroll
            for (int i = 0; i < 4; ++i)
#pragma unroll
                for (int j = 0; j < 4; ++j) acc[i][j] = fmaf(a[i], w[j], acc[i][j]);
        }
        __syncthreads();
    }
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const int m = m0 + ty * 4 + i;
        if (m >= M) continue;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int n = n0 + tx * 4 + j;
            if (n >= N) continue;
            const float v = acc[i][j] + (bias ? bias[n] : 0.f);
            C[(size_t)m * ldc + n] = tl_from_float<TO>(v);
        }
    }
}

// A: [M, K] with row stride lda; W: [N, K] contiguous; C: [M, N] with row stride ldc.
extern "C" int tl_gemm_generic(const void* A, int a_dtype, const void* W, int w_dtype, const float* bias, void* C,
                               int c_dtype, int M, int N, int K, int lda, int ldc, hipStream_t stream) {
    TL_CHECK_ARG(M >= 0 && N > 0 && K > 0, "tl_gemm_generic: bad sizes M=%d N=%d K=%d", M, N, K);
    TL_CHECK_ARG(lda >= K && ldc >= N, "tl_gemm_generic: row strides lda=%d ldc=%d too small for K=%d N=%d", lda, ldc, K, N);
    if (M == 0) return 0;
    for (int m0 = 0; m0 < M; m0 += 65535 * GT_BM) {  // grid.y limit
        const int mm = (M - m0 < 65535 * GT_BM) ? M - m0 : 65535 * GT_BM;
        dim3 grid(tl_ceil_div(N, GT_BN), tl_ceil_div(mm, GT_BM)), block(256);
#define TL_GEMM_CASE(AD, AT, WD, WT, CD, CT)                                                                     \
    if (a_dtype == AD && w_dtype == WD && c_dtype == CD) {                                                       \
        hipLaunchKernelGGL((gemm_generic_kernel<AT, WT, CT>), grid, block, 0, stream,                            \
                           (const AT*)A + (size_t)m0 * lda, (const WT*)W, bias, (CT*)C + (size_t)m0 * ldc, mm, N, K, \
                           lda, ldc);                                                                            \
        continue;                                                                                                \
    }
        TL_GEMM_CASE(TL_F32, float, TL_F32, float, TL_F32, float)
        TL_GEMM_CASE(TL_BF16, bf16_t, TL_BF16, bf16_t, TL_BF16, bf16_t)
        TL_GEMM_CASE(TL_BF16, bf16_t, TL_BF16, bf16_t, TL_F32, float)
        TL_GEMM_CASE(TL_F32, float, TL_BF16, bf16_t, TL_F32, float)
#undef TL_GEMM_CASE
        return tl_fail("tl_gemm_generic: unsupported dtypes a=%d w=%d c=%d", a_dtype, w_dtype, c_dtype);
    }
    TL_CHECK_LAUNCH("tl_gemm_generic");
    return 0;
}
