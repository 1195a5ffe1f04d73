// C[M, N] = A[M, K] * W[N, K]^T (+ bias) for few rows (M <= 64), bfloat16 inputs: the matrix
// products of a decode step.  The work is streaming W once from HBM; every byte of W is loaded by
// exactly one lane, with 16-byte loads that cover whole 128-byte lines per row.
//
// Mapping (wave64, gfx950 MFMA 16x16x32 bf16).  A work-group owns 16 rows of W (16 output
// columns) and all M rows of A; its waves split K among themselves and add their partial sums
// through LDS in a fixed order, so a result never depends on timing.  In a wave, lane l holds row
// r = l % 16 of the W tile and the 16 consecutive k values starting at chunk*64 + (l / 16)*16,
// feeding two MFMAs (8 values each); the A fragment of lane l is row m = l % 16 of A at the same k
// values.  The matrix core pairs element j of lane l's W fragment with element j of the A fragment
// of the lanes with the same l / 16, so any assignment of k values to (l / 16, j) gives the same
// dot product as long as both operands use it.  W is the first operand (rows n), A the second
// (columns m): the accumulator of lane l, register i, is C[m = l % 16][n = 4*(l / 16) + i].
//
// DUAL: the work-group owns rows [n0, n0+16) and [n_second + n0, n_second + n0 + 16) of W and
// writes silu(first) * second, the SwiGLU gate, for a fused [2I, K] gate/up matrix.
#include "common.h"

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float f32x4 __attribute__((ext_vector_type(4)));

#define SKG_CHUNK 64

__device__ __forceinline__ bf16x8 as_frag(uint4 v) { return __builtin_bit_cast(bf16x8, v); }

template <int MT, bool DUAL, typename TO>
__global__ __launch_bounds__(DUAL ? 256 : 1024) void gemm_skinny_kernel(const bf16_t* __restrict__ A, const bf16_t* __restrict__ W,
                                                           const float* __restrict__ bias, TO* __restrict__ C, int M,
                                                           int N, int K, int lda, int ldc, int n_second) {
    extern __shared__ float red[];   // [nwaves][NACC*4][64]
    constexpr int NACC = MT * (DUAL ? 2 : 1);
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, nwaves = blockDim.x >> 6;
    const int r = lane & 15, g = lane >> 4;
    const int n0 = blockIdx.x * 16;
    const int n_out = DUAL ? n_second : N;          // number of output columns
    int nrow = n0 + r;
    if (nrow > n_out - 1) nrow = n_out - 1;         // rows past the end repeat the last one; never written
    const bf16_t* w1p = W + (size_t)nrow * K + g * 16;
    const bf16_t* w2p = DUAL ? W + (size_t)(n_second + nrow) * K + g * 16 : nullptr;
    const bf16_t* ap[MT];
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) {
        const int m = mt * 16 + r;
        ap[mt] = A + (size_t)(m < M ? m : 0) * lda + g * 16;
    }

    f32x4 acc[NACC];
#pragma unroll
    for (int i = 0; i < NACC; ++i) acc[i] = f32x4{0.f, 0.f, 0.f, 0.f};

    const int nchunks = (K + SKG_CHUNK - 1) / SKG_CHUNK;
    const int full = K / SKG_CHUNK;                 // chunks that need no bounds check
    const int per = (nchunks + nwaves - 1) / nwaves;
    const int c0 = wave * per;
    const int c1 = (c0 + per < nchunks) ? c0 + per : nchunks;
    const int c_full = (c1 < full) ? c1 : full;
    const uint4 zero = make_uint4(0, 0, 0, 0);

#pragma unroll 4
    for (int c = c0; c < c_full; ++c) {
        const int k = c * SKG_CHUNK;
        const uint4 wa = *reinterpret_cast<const uint4*>(w1p + k);
        const uint4 wb = *reinterpret_cast<const uint4*>(w1p + k + 8);
        uint4 ua = zero, ub = zero;
        if (DUAL) {
            ua = *reinterpret_cast<const uint4*>(w2p + k);
            ub = *reinterpret_cast<const uint4*>(w2p + k + 8);
        }
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) {
            // rows of A past M read row 0: they only feed output columns that are never written
            const uint4 xa = *reinterpret_cast<const uint4*>(ap[mt] + k);
            const uint4 xb = *reinterpret_cast<const uint4*>(ap[mt] + k + 8);
            acc[mt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(as_frag(wa), as_frag(xa), acc[mt], 0, 0, 0);
            acc[mt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(as_frag(wb), as_frag(xb), acc[mt], 0, 0, 0);
            if (DUAL) {
                acc[MT + mt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(as_frag(ua), as_frag(xa), acc[MT + mt], 0, 0, 0);
                acc[MT + mt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(as_frag(ub), as_frag(xb), acc[MT + mt], 0, 0, 0);
            }
        }
    }
    // the last, partial chunk (K is a multiple of 8, so a group of 8 values is all in or all out)
    for (int c = (c_full > c0 ? c_full : c0); c < c1; ++c) {
        const int k = c * SKG_CHUNK;
        const int kk = k + g * 16;
        const bool in_a = kk < K, in_b = kk + 8 < K;
        const uint4 wa = in_a ? *reinterpret_cast<const uint4*>(w1p + k) : zero;
        const uint4 wb = in_b ? *reinterpret_cast<const uint4*>(w1p + k + 8) : zero;
        uint4 ua = zero, ub = zero;
        if (DUAL) {
            ua = in_a ? *reinterpret_cast<const uint4*>(w2p + k) : zero;
            ub = in_b ? *reinterpret_cast<const uint4*>(w2p + k + 8) : zero;
        }
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) {
            const uint4 xa = in_a ? *reinterpret_cast<const uint4*>(ap[mt] + k) : zero;
            const uint4 xb = in_b ? *reinterpret_cast<const uint4*>(ap[mt] + k + 8) : zero;
            acc[mt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(as_frag(wa), as_frag(xa), acc[mt], 0, 0, 0);
            acc[mt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(as_frag(wb), as_frag(xb), acc[mt], 0, 0, 0);
            if (DUAL) {
                acc[MT + mt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(as_frag(ua), as_frag(xa), acc[MT + mt], 0, 0, 0);
                acc[MT + mt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(as_frag(ub), as_frag(xb), acc[MT + mt], 0, 0, 0);
            }
        }
    }

    // partial sums of the waves -> LDS, then a fixed-order sum
#pragma unroll
    for (int a = 0; a < NACC; ++a)
#pragma unroll
        for (int i = 0; i < 4; ++i) red[((size_t)wave * NACC * 4 + a * 4 + i) * 64 + lane] = acc[a][i];
    __syncthreads();
    // element e = (mt, i, l): C[m = mt*16 + l % 16][n = n0 + 4*(l / 16) + i]
    for (int e = threadIdx.x; e < MT * 4 * 64; e += blockDim.x) {
        const int l = e & 63, i = (e >> 6) & 3, mt = e >> 8;
        const int m = mt * 16 + (l & 15), n = n0 + 4 * (l >> 4) + i;
        if (m >= M || n >= n_out) continue;
        float v = 0.f, u = 0.f;
        for (int w = 0; w < nwaves; ++w) {
            v += red[((size_t)w * NACC * 4 + mt * 4 + i) * 64 + l];
            if (DUAL) u += red[((size_t)w * NACC * 4 + (MT + mt) * 4 + i) * 64 + l];
        }
        if (DUAL) {
            v = v / (1.0f + expf(-v)) * u;
        } else if (bias) {
            v += bias[n];
        }
        C[(size_t)m * ldc + n] = tl_from_float<TO>(v);
    }
}

static int pick_waves(int tiles, int nchunks, int nacc, int max_waves) {
    // enough waves in flight to cover HBM latency on 256 CUs; K is split among the waves of a group
    int w = 1;
    while (w < max_waves && tiles * w < 4096 && nchunks >= 4 * w) w <<= 1;
    while (w > 1 && (size_t)w * nacc * 4 * 64 * sizeof(float) > 64 * 1024) w >>= 1;
    return w;
}

template <int MT, bool DUAL, typename TO>
static void launch_skinny(const bf16_t* A, const bf16_t* W, const float* bias, TO* C, int M, int N, int K, int lda,
                          int ldc, int n_second, hipStream_t stream) {
    const int n_out = DUAL ? n_second : N;
    const int tiles = tl_ceil_div(n_out, 16);
    const int nacc = MT * (DUAL ? 2 : 1);
    const int nwaves = pick_waves(tiles, tl_ceil_div(K, SKG_CHUNK), nacc, DUAL ? 4 : 16);
    const size_t smem = (size_t)nwaves * nacc * 4 * 64 * sizeof(float);
    hipLaunchKernelGGL((gemm_skinny_kernel<MT, DUAL, TO>), dim3(tiles), dim3(nwaves * 64), smem, stream, A, W, bias, C,
                       M, N, K, lda, ldc, n_second);
}

template <bool DUAL, typename TO>
static int dispatch_skinny(const bf16_t* A, const bf16_t* W, const float* bias, TO* C, int M, int N, int K, int lda,
                           int ldc, int n_second, hipStream_t stream) {
    if (M <= 16) launch_skinny<1, DUAL, TO>(A, W, bias, C, M, N, K, lda, ldc, n_second, stream);
    else if (M <= 32) launch_skinny<2, DUAL, TO>(A, W, bias, C, M, N, K, lda, ldc, n_second, stream);
    else if (M <= 48) launch_skinny<3, DUAL, TO>(A, W, bias, C, M, N, K, lda, ldc, n_second, stream);
    else launch_skinny<4, DUAL, TO>(A, W, bias, C, M, N, K, lda, ldc, n_second, stream);
    TL_CHECK_LAUNCH("tl_gemm_skinny");
    return 0;
}

static int check_skinny(const void* A, const void* W, const void* C, int M, int N, int K, int lda, int ldc) {
    TL_CHECK_ARG(M >= 0 && M <= 64, "tl_gemm_skinny: M=%d is outside [0, 64]", M);
    TL_CHECK_ARG(N > 0 && K > 0, "tl_gemm_skinny: bad sizes N=%d K=%d", N, K);
    TL_CHECK_ARG(K % 8 == 0 && lda % 8 == 0, "tl_gemm_skinny: K=%d and the row stride %d must be multiples of 8", K, lda);
    TL_CHECK_ARG(((uintptr_t)A % 16) == 0 && ((uintptr_t)W % 16) == 0, "tl_gemm_skinny: operands must be 16-byte aligned");
    TL_CHECK_ARG(lda >= K && ldc > 0 && C != nullptr, "tl_gemm_skinny: bad strides");
    return 0;
}

// bfloat16 A [M, K] (row stride lda), W [N, K]; C [M, N] float or bfloat16 (row stride ldc).
extern "C" int tl_gemm_skinny(const void* A, const void* W, const float* bias, void* C, int c_dtype, int M, int N, int K,
                              int lda, int ldc, hipStream_t stream) {
    if (int rc = check_skinny(A, W, C, M, N, K, lda, ldc)) return rc;
    TL_CHECK_ARG(ldc >= N, "tl_gemm_skinny: output row stride %d < N=%d", ldc, N);
    if (M == 0) return 0;
    if (c_dtype == TL_F32)
        return dispatch_skinny<false, float>((const bf16_t*)A, (const bf16_t*)W, bias, (float*)C, M, N, K, lda, ldc, 0, stream);
    if (c_dtype == TL_BF16)
        return dispatch_skinny<false, bf16_t>((const bf16_t*)A, (const bf16_t*)W, bias, (bf16_t*)C, M, N, K, lda, ldc, 0, stream);
    return tl_fail("tl_gemm_skinny: unknown output dtype %d", c_dtype);
}

// W is [2I, K]: rows [0, I) the gate, rows [I, 2I) the up projection.  C [M, I] = silu(A Wg^T) * (A Wu^T).
extern "C" int tl_gemm_skinny_swiglu(const void* A, const void* W, void* C, int M, int I, int K, int lda, int ldc,
                                     hipStream_t stream) {
    if (int rc = check_skinny(A, W, C, M, 2 * I, K, lda, ldc)) return rc;
    TL_CHECK_ARG(ldc >= I, "tl_gemm_skinny_swiglu: output row stride %d < I=%d", ldc, I);
    if (M == 0) return 0;
    return dispatch_skinny<true, bf16_t>((const bf16_t*)A, (const bf16_t*)W, nullptr, (bf16_t*)C, M, 2 * I, K, lda, ldc, I, stream);
}
