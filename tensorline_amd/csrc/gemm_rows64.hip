// C[M, N] = A[M, K] * W[N, K]^T (+ bias) for 17 to 64 rows, bfloat16: decode steps of large
// batches and short prompt portions.  Same matrix-core ordered weight copy as the few-row kernel
// (gemm_skinny.hip); what differs is how the work is cut, because with up to 64 rows the rows of A
// weigh as much as a 128-column slab of W and must not be re-read per 16 columns.
//
// A work-group of eight waves owns 128 output columns (one 16-column tile per wave) and one share
// of K.  Per step of 128 k the group brings A[0:64, k:k+128] into LDS once, with row-contiguous
// loads by all 512 threads, and every wave multiplies it with its own W fragments, which it loads
// straight into registers one step ahead.  LDS is double-buffered: one barrier per step.
//
// K is split over the grid so that small matrices still fill 256 CUs.  With one share the result
// is written at once; otherwise every share writes a float partial [share, M, N] and a second
// kernel adds the shares in ascending order (and applies bias, or SiLU(gate) * up for a fused
// gate/up matrix), so the result does not depend on timing.
#include "common.h"

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float f32x4 __attribute__((ext_vector_type(4)));

#define R64_WAVES 8
#define R64_SC 128
#define R64_UNITS (R64_SC / 8)
#define R64_ROWPAD 17
#define R64_MT 4

__device__ __forceinline__ bf16x8 r64_frag(uint4 v) { return __builtin_bit_cast(bf16x8, v); }

template <typename TO>
__global__ __launch_bounds__(R64_WAVES * 64) void gemm_rows64_kernel(
    const bf16_t* __restrict__ A, const uint4* __restrict__ Ws, const float* __restrict__ bias, TO* __restrict__ C,
    float* __restrict__ partial, int M, int N, int K, int K32, int lda, int ldc, int steps_per_share, int ntiles) {
    __shared__ uint4 xs[2][R64_MT * R64_UNITS * R64_ROWPAD];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int r = lane & 15, g = lane >> 4;
    const int nsc = (K32 + 3) / 4;
    const int s0 = blockIdx.y * steps_per_share;
    const int s1 = (s0 + steps_per_share < nsc) ? s0 + steps_per_share : nsc;
    int tile = blockIdx.x * R64_WAVES + wave;
    const bool tile_live = tile < ntiles;
    if (!tile_live) tile = ntiles - 1;                       // loads stay in bounds; nothing is written
    const uint4* w1 = Ws + (size_t)tile * K32 * 64 + lane;
    const uint4 zero = make_uint4(0, 0, 0, 0);
    const int last_c = K32 - 1;

    f32x4 acc[R64_MT];
#pragma unroll
    for (int i = 0; i < R64_MT; ++i) acc[i] = f32x4{0.f, 0.f, 0.f, 0.f};

    // loader of A: 64 rows x 16 units = 1024 16-byte pieces, two per thread
    const bf16_t* xp[2];
    int xslot[2];
#pragma unroll
    for (int i = 0; i < 2; ++i) {
        const int idx = tid + 512 * i;
        const int row = idx >> 4, unit = idx & 15;
        xp[i] = A + (size_t)(row < M ? row : 0) * lda + unit * 8;
        xslot[i] = ((row >> 4) * R64_UNITS + unit) * R64_ROWPAD + (row & 15);
    }
    const int xunit = tid & 15;
    uint4 xr[2], wf[4], wn[4];
    {
        const int kx = s0 * R64_SC + xunit * 8;
        const int kbase = (kx < K) ? s0 * R64_SC : 0;
#pragma unroll
        for (int i = 0; i < 2; ++i) xr[i] = *reinterpret_cast<const uint4*>(xp[i] + kbase);
        if (kx >= K) xr[0] = xr[1] = zero;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            int c = s0 * 4 + i;
            if (c > last_c) c = last_c;
            wf[i] = w1[(size_t)c * 64];
        }
    }
    int cur = 0;
    for (int sc = s0; sc < s1; ++sc) {
        xs[cur][xslot[0]] = xr[0];
        xs[cur][xslot[1]] = xr[1];
        __syncthreads();
        const int sn = (sc + 1 < s1) ? sc + 1 : sc;          // past the end: the same step again, unused
        const int kxn = sn * R64_SC + xunit * 8;
        const int kbn = (kxn < K) ? sn * R64_SC : 0;
#pragma unroll
        for (int i = 0; i < 2; ++i) xr[i] = *reinterpret_cast<const uint4*>(xp[i] + kbn);
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            int c = sn * 4 + i;
            if (c > last_c) c = last_c;
            wn[i] = w1[(size_t)c * 64];
        }
        const int cbase = sc * 4;
#pragma unroll
        for (int cc = 0; cc < 4; ++cc) {
            const bool live = cbase + cc <= last_c;          // chunks past K32 read a clamped chunk
#pragma unroll
            for (int mt = 0; mt < R64_MT; ++mt) {
                uint4 xf = xs[cur][(mt * R64_UNITS + cc * 4 + g) * R64_ROWPAD + r];
                if (!live) xf = zero;
                acc[mt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(r64_frag(wf[cc]), r64_frag(xf), acc[mt], 0, 0, 0);
            }
        }
        if (kxn >= K) xr[0] = xr[1] = zero;
#pragma unroll
        for (int i = 0; i < 4; ++i) wf[i] = wn[i];
        cur ^= 1;
    }
    if (!tile_live) return;
    // accumulator register i of lane l: C[m = mt*16 + l % 16][n = tile*16 + 4*(l / 16) + i]
    const int n0 = tile * 16 + 4 * g;
#pragma unroll
    for (int mt = 0; mt < R64_MT; ++mt) {
        const int m = mt * 16 + r;
        if (m >= M) continue;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const int n = n0 + i;
            if (n >= N) continue;
            if (partial) {
                partial[((size_t)blockIdx.y * M + m) * N + n] = acc[mt][i];
            } else {
                C[(size_t)m * ldc + n] = tl_from_float<TO>(acc[mt][i] + (bias ? bias[n] : 0.f));
            }
        }
    }
}

// out[m, n] = sum over shares of partial[share, m, n] (+ bias[n]); with swiglu: n < I and
// out[m, n] = silu(sum gate) * (sum up), gate at column n and up at column I + n of the partials.
template <typename TO>
__global__ void gemm_rows64_reduce_kernel(const float* __restrict__ partial, const float* __restrict__ bias,
                                          TO* __restrict__ C, int M, int N, int n_out, int ldc, int shares, int swiglu) {
    const int n = blockIdx.x * blockDim.x + threadIdx.x;
    const int m = blockIdx.y;
    if (n >= n_out) return;
    float v = 0.f, u = 0.f;
    for (int s = 0; s < shares; ++s) {
        const float* p = partial + ((size_t)s * M + m) * N;
        v += p[n];
        if (swiglu) u += p[n_out + n];
    }
    if (swiglu) v = v / (1.0f + expf(-v)) * u;
    else if (bias) v += bias[n];
    C[(size_t)m * ldc + n] = tl_from_float<TO>(v);
}

// Number of shares K is cut into for a [N, K] matrix and M rows: enough work-groups to fill the
// GPU, partial sums that stay well below the weight bytes, at least two steps per share.
extern "C" int tl_gemm_rows64_shares(int M, int N, int K) {
    const int groups = tl_ceil_div(tl_ceil_div(N, 16), R64_WAVES);
    const int nsc = tl_ceil_div(tl_ceil_div(K, 32), 4);
    if (groups >= 256) return 1;                 // wide matrices fill the GPU without a split
    int ks = tl_ceil_div(512, groups);
    const int by_traffic = K / (8 * (M > 0 ? M : 1));
    if (ks > by_traffic) ks = by_traffic;
    if (ks > nsc / 2) ks = nsc / 2;
    if (ks < 1) ks = 1;
    const int steps = tl_ceil_div(nsc, ks);
    return tl_ceil_div(nsc, steps);
}

// A: bfloat16 [M, K], 16 < M <= 64 is what it is for (any M from 1 to 64 works); Ws: shuffled copy of
// W [N, K]; C [M, n_out] bfloat16 or float.  shares = tl_gemm_rows64_shares(M, N, K); with shares > 1
// `partial` holds shares*M*N floats.  swiglu: W is a fused [2I, K] gate/up matrix (N = 2I), C is
// [M, I] = silu(gate) * up and bias is not used.
extern "C" int tl_gemm_rows64(const void* A, const void* Ws, const float* bias, void* C, int c_dtype, float* partial,
                              int M, int N, int K, int lda, int ldc, int shares, int swiglu, hipStream_t stream) {
    TL_CHECK_ARG(M >= 0 && M <= 64 && N > 0 && K > 0, "tl_gemm_rows64: bad sizes M=%d N=%d K=%d", M, N, K);
    TL_CHECK_ARG(K % 8 == 0 && lda % 8 == 0 && lda >= K, "tl_gemm_rows64: K=%d and the row stride %d must be multiples of 8", K, lda);
    TL_CHECK_ARG(((uintptr_t)A % 16) == 0 && ((uintptr_t)Ws % 16) == 0, "tl_gemm_rows64: operands must be 16-byte aligned");
    TL_CHECK_ARG(shares == tl_gemm_rows64_shares(M, N, K), "tl_gemm_rows64: %d shares do not fit this shape", shares);
    TL_CHECK_ARG(shares == 1 || partial, "tl_gemm_rows64: shares need a workspace");
    TL_CHECK_ARG(!swiglu || (N % 2 == 0 && shares > 1), "tl_gemm_rows64: the SwiGLU form needs N even and split K");
    const int n_out = swiglu ? N / 2 : N;
    TL_CHECK_ARG(ldc >= n_out && C, "tl_gemm_rows64: bad output");
    if (M == 0) return 0;
    const int K32 = tl_ceil_div(K, 32), nsc = tl_ceil_div(K32, 4), ntiles = tl_ceil_div(N, 16);
    const int steps = tl_ceil_div(nsc, shares);
    dim3 grid(tl_ceil_div(ntiles, R64_WAVES), shares), block(R64_WAVES * 64);
    float* part = shares > 1 ? partial : nullptr;
    if (c_dtype == TL_F32)
        hipLaunchKernelGGL(gemm_rows64_kernel<float>, grid, block, 0, stream, (const bf16_t*)A, (const uint4*)Ws, bias,
                           (float*)C, part, M, N, K, K32, lda, ldc, steps, ntiles);
    else if (c_dtype == TL_BF16)
        hipLaunchKernelGGL(gemm_rows64_kernel<bf16_t>, grid, block, 0, stream, (const bf16_t*)A, (const uint4*)Ws, bias,
                           (bf16_t*)C, part, M, N, K, K32, lda, ldc, steps, ntiles);
    else
        return tl_fail("tl_gemm_rows64: unknown output dtype %d", c_dtype);
    TL_CHECK_LAUNCH("tl_gemm_rows64");
    if (shares > 1) {
        dim3 rgrid(tl_ceil_div(n_out, 256), M), rblock(256);
        if (c_dtype == TL_F32)
            hipLaunchKernelGGL(gemm_rows64_reduce_kernel<float>, rgrid, rblock, 0, stream, partial, bias, (float*)C, M, N,
                               n_out, ldc, shares, swiglu);
        else
            hipLaunchKernelGGL(gemm_rows64_reduce_kernel<bf16_t>, rgrid, rblock, 0, stream, partial, bias, (bf16_t*)C, M, N,
                               n_out, ldc, shares, swiglu);
        TL_CHECK_LAUNCH("tl_gemm_rows64 reduce");
    }
    return 0;
}
