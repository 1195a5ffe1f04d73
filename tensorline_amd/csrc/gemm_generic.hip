// C[M, N] = A[M, K] * W[N, K]^T (+ bias[N]):  the any-shape matrix product.
//
// This is the product of the true 32-bit path (float inputs, float products and sums on the matrix
// cores' float instruction v_mfma_f32_16x16x4_f32, no reduced precision anywhere) and the any-shape
// fallback for bfloat16 inputs (converted to float on the way into LDS, which is exact).  Any M, N
// and K, any row strides.
//
// One output element is summed over k in one fixed order: steps of 16 from k = 0 upwards, four
// products per step, the lanes' k within a step fixed by the operand layout.  The order does not
// depend on M or on which tile shape the launch picked, so cutting a batch differently does not
// change a bit of a result, and neither does the number of rows that come along (from 17 rows on;
// up to 16 rows have an order of their own, see gemm_fewrows_kernel).
//
// Tiles: four waves compute BM x BN outputs, a wave MB x NB blocks of 16 x 16; 128 x 128 for many
// rows, 64 x 128 and 32 x 64 for few (more work-groups stream the weights then); at most 16 rows
// have a kernel of their own (gemm_fewrows_kernel), which sums K in segments.  A k-step's rows
// of A and W go from memory into registers while the step before is computed, then as float into
// LDS [row][16 + 4] (the padding keeps the 16-byte operand reads off each other's banks).
//
// Operand layout of the 16x16x4 product D = A B + C: lane l gives A[l % 16][l / 16] and
// B[l / 16][l % 16]; it holds D[4 (l / 16) + v][l % 16] in register v.  Lane group g = l / 16 feeds
// k = 4 g + v of the step to the v-th of its four products, for A and B alike, so a lane's four
// operands are one 16-byte read.
#include "common.h"

#define GG_THREADS 256
#define GG_KS 16              // k per step
#define GG_LD (GG_KS + 4)     // LDS row stride in floats

typedef float gg_f32x4 __attribute__((ext_vector_type(4)));

// Four consecutive k of one row as floats; zero where the row or k is outside the matrix.
template <typename T>
__device__ __forceinline__ float4 gg_load4(const T* __restrict__ base, bool row_ok, int k, int K, bool vec_ok);

template <>
__device__ __forceinline__ float4 gg_load4<float>(const float* __restrict__ base, bool row_ok, int k, int K, bool vec_ok) {
    if (!row_ok || k >= K) return make_float4(0.f, 0.f, 0.f, 0.f);
    if (vec_ok && k + 3 < K) return *reinterpret_cast<const float4*>(base + k);
    float4 r;
    r.x = base[k];
    r.y = (k + 1 < K) ? base[k + 1] : 0.f;
    r.z = (k + 2 < K) ? base[k + 2] : 0.f;
    r.w = (k + 3 < K) ? base[k + 3] : 0.f;
    return r;
}

template <>
__device__ __forceinline__ float4 gg_load4<bf16_t>(const bf16_t* __restrict__ base, bool row_ok, int k, int K, bool vec_ok) {
    if (!row_ok || k >= K) return make_float4(0.f, 0.f, 0.f, 0.f);
    if (vec_ok && k + 3 < K) {
        const uint2 raw = *reinterpret_cast<const uint2*>(base + k);
        return make_float4(__uint_as_float(raw.x << 16), __uint_as_float(raw.x & 0xffff0000u),
                           __uint_as_float(raw.y << 16), __uint_as_float(raw.y & 0xffff0000u));
    }
    float4 r;
    r.x = tl_to_float(base[k]);
    r.y = (k + 1 < K) ? tl_to_float(base[k + 1]) : 0.f;
    r.z = (k + 2 < K) ? tl_to_float(base[k + 2]) : 0.f;
    r.w = (k + 3 < K) ? tl_to_float(base[k + 3]) : 0.f;
    return r;
}

// The same four k with nothing to check: the caller knows that the row exists, that all four k do
// and that the piece is aligned.
template <typename T>
__device__ __forceinline__ float4 gg_load4_whole(const T* __restrict__ p);
template <>
__device__ __forceinline__ float4 gg_load4_whole<float>(const float* __restrict__ p) {
    return *reinterpret_cast<const float4*>(p);
}
template <>
__device__ __forceinline__ float4 gg_load4_whole<bf16_t>(const bf16_t* __restrict__ p) {
    const uint2 raw = *reinterpret_cast<const uint2*>(p);
    return make_float4(__uint_as_float(raw.x << 16), __uint_as_float(raw.x & 0xffff0000u), __uint_as_float(raw.y << 16),
                       __uint_as_float(raw.y & 0xffff0000u));
}

// WM x WN waves (WM * WN == 4), each MB x NB blocks of 16 x 16.
template <typename TA, typename TW, typename TO, int WM, int WN, int MB, int NB>
__global__ __launch_bounds__(GG_THREADS) void gemm_generic_kernel(const TA* __restrict__ A, const TW* __restrict__ W,
                                                                 const float* __restrict__ bias, TO* __restrict__ C,
                                                                 int M, int N, int K, int lda, int ldc, int a_vec,
                                                                 int w_vec) {
    constexpr int BM = WM * MB * 16, BN = WN * NB * 16;
    constexpr int A_PIECES = BM * 4, W_PIECES = BN * 4;                 // 16-byte (four k) pieces per step
    constexpr int A_PER = (A_PIECES + GG_THREADS - 1) / GG_THREADS, W_PER = (W_PIECES + GG_THREADS - 1) / GG_THREADS;
    __shared__ float As[2][BM * GG_LD];
    __shared__ float Ws[2][BN * GG_LD];

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int li = lane & 15, lg = lane >> 4;
    const int wm = wave / WN, wn = wave - wm * WN;
    const int m0 = blockIdx.y * BM, n0 = blockIdx.x * BN;

    gg_f32x4 acc[MB][NB];
#pragma unroll
    for (int i = 0; i < MB; ++i)
#pragma unroll
        for (int j = 0; j < NB; ++j) acc[i][j] = (gg_f32x4){0.f, 0.f, 0.f, 0.f};

    float4 areg[A_PER], wreg[W_PER];
    auto fetch = [&](int k0) {
#pragma unroll
        for (int it = 0; it < A_PER; ++it) {
            const int p = tid + it * GG_THREADS;
            const int r = p >> 2, c4 = p & 3;
            areg[it] = gg_load4<TA>(A + (size_t)(m0 + r) * lda, p < A_PIECES && m0 + r < M, k0 + 4 * c4, K, a_vec != 0);
        }
#pragma unroll
        for (int it = 0; it < W_PER; ++it) {
            const int p = tid + it * GG_THREADS;
            const int r = p >> 2, c4 = p & 3;
            wreg[it] = gg_load4<TW>(W + (size_t)(n0 + r) * K, p < W_PIECES && n0 + r < N, k0 + 4 * c4, K, w_vec != 0);
        }
    };
    auto to_lds = [&](int buf) {
#pragma unroll
        for (int it = 0; it < A_PER; ++it) {
            const int p = tid + it * GG_THREADS;
            if (p < A_PIECES) *reinterpret_cast<float4*>(&As[buf][(p >> 2) * GG_LD + 4 * (p & 3)]) = areg[it];
        }
#pragma unroll
        for (int it = 0; it < W_PER; ++it) {
            const int p = tid + it * GG_THREADS;
            if (p < W_PIECES) *reinterpret_cast<float4*>(&Ws[buf][(p >> 2) * GG_LD + 4 * (p & 3)]) = wreg[it];
        }
    };

    fetch(0);
    to_lds(0);
    __syncthreads();
    int buf = 0;
    for (int k0 = 0; k0 < K; k0 += GG_KS) {
        const bool more = k0 + GG_KS < K;
        if (more) fetch(k0 + GG_KS);
        float4 af[MB], wf[NB];
#pragma unroll
        for (int i = 0; i < MB; ++i)
            af[i] = *reinterpret_cast<const float4*>(&As[buf][((wm * MB + i) * 16 + li) * GG_LD + 4 * lg]);
#pragma unroll
        for (int j = 0; j < NB; ++j)
            wf[j] = *reinterpret_cast<const float4*>(&Ws[buf][((wn * NB + j) * 16 + li) * GG_LD + 4 * lg]);
#pragma unroll
        for (int i = 0; i < MB; ++i)
#pragma unroll
            for (int j = 0; j < NB; ++j) {
                acc[i][j] = __builtin_amdgcn_mfma_f32_16x16x4f32(af[i].x, wf[j].x, acc[i][j], 0, 0, 0);
                acc[i][j] = __builtin_amdgcn_mfma_f32_16x16x4f32(af[i].y, wf[j].y, acc[i][j], 0, 0, 0);
                acc[i][j] = __builtin_amdgcn_mfma_f32_16x16x4f32(af[i].z, wf[j].z, acc[i][j], 0, 0, 0);
                acc[i][j] = __builtin_amdgcn_mfma_f32_16x16x4f32(af[i].w, wf[j].w, acc[i][j], 0, 0, 0);
            }
        if (more) {
            to_lds(buf ^ 1);          // the other buffer: nobody reads it during this step
            __syncthreads();
            buf ^= 1;
        }
    }

    // this lane holds rows 4 lg + v and column li of each block
#pragma unroll
    for (int j = 0; j < NB; ++j) {
        const int n = n0 + (wn * NB + j) * 16 + li;
        if (n >= N) continue;
        const float b = bias ? bias[n] : 0.f;
#pragma unroll
        for (int i = 0; i < MB; ++i)
#pragma unroll
            for (int v = 0; v < 4; ++v) {
                const int m = m0 + (wm * MB + i) * 16 + 4 * lg + v;
                if (m < M) C[(size_t)m * ldc + n] = tl_from_float<TO>(acc[i][j][v] + b);
            }
    }
}

// At most 16 rows (a decode step of few sequences): the work is streaming W once, and a tile of the
// kernel above would leave most of the GPU without work (56 work-groups for 3,584 columns) with one
// k-step in flight each.  Here a work-group owns 16 columns and its waves share K: K is cut into
// segments of GF_SEG at absolute k, wave w sums segments w, w + waves, ... each in the order above
// (steps of 16 upwards, four products per step), with the next GF_RING - 1 steps' operands on their
// way in a ring of registers, and the segments' sums are added in ascending order at the end.  So
// one output element is again summed in one fixed order that depends on K alone, not on M (1 to 16),
// on the number of waves or on timing; it is not the order of the kernel above, whose results differ
// from this one's by rounding.
// Sixteen waves and segments of 256: a product with fewer tiles than the GPU has CUs (the down projection
// of a 7B model: 224) has one work-group per CU, and what streams its weights is the loads that
// group keeps in flight (eight waves: 2.5 TB/s for the float down projection, sixteen: 3.4), and how
// evenly the segments deal out over the waves (74 segments of 256 over 16 waves: 5 at most, 4.6 on
// average; 37 of 512: 3 against 2.3).  A deeper ring gains nothing (8 steps ahead: slower).
#define GF_SEG 256
#define GF_RING 4
#define GF_WAVES 16
#define GF_MAX_SEGMENTS 128   // 128 KB of LDS for the segments' sums: K up to 32,768 (beyond: the kernel above)

// The waves of a work-group: all sixteen where the tiles are about as many as the CUs, eight where
// every CU holds several work-groups anyway (their loads in flight add up, and a wave with more steps
// fills its ring less often: gate/up of a 7B model 120 against 125 us).  The result does not depend on it.
static inline int gf_waves(int nseg, int tiles) {
    const int most = tiles >= 512 ? GF_WAVES / 2 : GF_WAVES;
    return nseg < most ? nseg : most;
}

// SHUF: W is the matrix-core ordered copy of a float matrix, [ceil(N/16) tiles][ceil(K/16) steps][64
// lanes][4 values], lane 16 lg + li holding row li of the tile at k = 16 step + 4 lg .. + 4, zero
// where it pads: a step's load of a wave is 1 KB of consecutive memory (from the row-major matrix it
// is 16 pieces of 64 bytes, which streams at about two thirds of the rate), and needs no check.
template <typename TA, typename TW, typename TO, bool SHUF>
__global__ __launch_bounds__(GF_WAVES * 64) void gemm_fewrows_kernel(const TA* __restrict__ A, const TW* __restrict__ W,
                                                           const float* __restrict__ bias, TO* __restrict__ C, int M,
                                                           int N, int K, int lda, int ldc, int a_vec, int w_vec) {
    extern __shared__ float gf_part[];                       // [segment][register v][lane]
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, nwaves = blockDim.x >> 6;
    const int li = lane & 15, lg = lane >> 4;
    const int n0 = blockIdx.x * 16;
    const int nseg = (K + GF_SEG - 1) / GF_SEG;
    constexpr int SPS = GF_SEG / GG_KS;                      // steps per segment
    const TW* wrow = W + (size_t)(n0 + li) * K;
    const TA* arow = A + (size_t)li * lda;
    const bool w_ok = n0 + li < N, a_ok = li < M;
    // Whole steps (all 16 k inside K, aligned pieces) load without a condition, so that the loads of
    // the steps ahead stay in flight: a row that does not exist is read from one that does (what it
    // brings only reaches outputs that are not written).
    const TW* wrow_any = W + (size_t)(w_ok ? n0 + li : N - 1) * K;
    const TA* arow_any = A + (size_t)(a_ok ? li : 0) * lda;
    const bool pieces_whole = a_vec != 0 && w_vec != 0;
    const float4* wtile = reinterpret_cast<const float4*>(W) + (size_t)blockIdx.x * ((K + GG_KS - 1) / GG_KS) * 64 + lane;
    auto load_step = [&](int k0, float4& wv, float4& av) {
        if (SHUF) {
            if (k0 >= K) {                                      // past the last segment's end: the copy ends with K
                wv = av = make_float4(0.f, 0.f, 0.f, 0.f);
            } else {
                wv = __builtin_bit_cast(float4, tl_load_stream(reinterpret_cast<const uint4*>(wtile + (size_t)(k0 / GG_KS) * 64)));
                if (a_vec != 0 && k0 + GG_KS <= K) av = gg_load4_whole<TA>(arow_any + k0 + 4 * lg);
                else av = gg_load4<TA>(arow, a_ok, k0 + 4 * lg, K, a_vec != 0);
            }
        } else if (pieces_whole && k0 + GG_KS <= K) {           // the same for the whole wave
            wv = gg_load4_whole<TW>(wrow_any + k0 + 4 * lg);
            av = gg_load4_whole<TA>(arow_any + k0 + 4 * lg);
        } else {                                              // past K (the last segment's end): zeros
            wv = gg_load4<TW>(wrow, w_ok, k0 + 4 * lg, K, w_vec != 0);
            av = gg_load4<TA>(arow, a_ok, k0 + 4 * lg, K, a_vec != 0);
        }
    };
    // this wave's steps, numbered through its segments: step j is step j % SPS of segment wave + (j / SPS) * nwaves
    const int my_segs = (nseg - wave + nwaves - 1) / nwaves;   // 0 for a wave beyond the segments
    const int nsteps = my_segs * SPS;
    auto k_of = [&](int j) { return (wave + (j / SPS) * nwaves) * GF_SEG + (j % SPS) * GG_KS; };
    float4 wreg[GF_RING], areg[GF_RING];
#pragma unroll
    for (int r = 0; r < GF_RING - 1; ++r) {
        if (r < nsteps) load_step(k_of(r), wreg[r], areg[r]);
    }
    gg_f32x4 acc = (gg_f32x4){0.f, 0.f, 0.f, 0.f};
    for (int jb = 0; jb < nsteps; jb += GF_RING) {
#pragma unroll
        for (int r = 0; r < GF_RING; ++r) {
            const int j = jb + r;
            if (j < nsteps) {                                 // the same for the whole wave
                const int ahead = j + GF_RING - 1;
                if (ahead < nsteps) load_step(k_of(ahead), wreg[(r + GF_RING - 1) % GF_RING], areg[(r + GF_RING - 1) % GF_RING]);
                // as in the kernel above: the lane gives row li of A and row li of the W tile at k = k0 + 4 lg + v
                // to the v-th product and holds C[4 lg + v][n0 + li]
                acc = __builtin_amdgcn_mfma_f32_16x16x4f32(areg[r].x, wreg[r].x, acc, 0, 0, 0);
                acc = __builtin_amdgcn_mfma_f32_16x16x4f32(areg[r].y, wreg[r].y, acc, 0, 0, 0);
                acc = __builtin_amdgcn_mfma_f32_16x16x4f32(areg[r].z, wreg[r].z, acc, 0, 0, 0);
                acc = __builtin_amdgcn_mfma_f32_16x16x4f32(areg[r].w, wreg[r].w, acc, 0, 0, 0);
                if (j % SPS == SPS - 1) {                     // the segment is complete
                    const int seg = wave + (j / SPS) * nwaves;
#pragma unroll
                    for (int v = 0; v < 4; ++v) gf_part[(seg * 4 + v) * 64 + lane] = acc[v];
                    acc = (gg_f32x4){0.f, 0.f, 0.f, 0.f};
                }
            }
        }
    }
    __syncthreads();
    // element (v, lane): row m = 4 lg + v, column n0 + li; segments in ascending order
    for (int e = tid; e < 256; e += blockDim.x) {
        const int l = e & 63, v = e >> 6;
        const int m = 4 * (l >> 4) + v, n = n0 + (l & 15);
        if (m >= M || n >= N) continue;
        float sum = 0.f;
        for (int seg = 0; seg < nseg; ++seg) sum += gf_part[(seg * 4 + v) * 64 + l];
        C[(size_t)m * ldc + n] = tl_from_float<TO>(sum + (bias ? bias[n] : 0.f));
    }
}

template <typename TA, typename TW, typename TO>
static int gg_launch(const void* A, const void* W, const float* bias, void* C, int M, int N, int K, int lda, int ldc,
                     hipStream_t stream) {
    // whole 16-byte (8-byte for bfloat16) pieces can be read where rows start aligned
    const int a_vec = ((uintptr_t)A % (4 * sizeof(TA)) == 0 && lda % 4 == 0) ? 1 : 0;
    const int w_vec = ((uintptr_t)W % (4 * sizeof(TW)) == 0 && K % 4 == 0) ? 1 : 0;
#define GG_GO(WM, WN, MB, NB)                                                                                    \
    do {                                                                                                         \
        constexpr int BM = WM * MB * 16, BN = WN * NB * 16;                                                      \
        const long long gy = tl_ceil_div(M, BM);                                                                 \
        if (gy > 65535) return tl_fail("tl_gemm_generic: %d rows are too many for one launch", M);               \
        dim3 grid(tl_ceil_div(N, BN), (unsigned)gy), block(GG_THREADS);                                          \
        hipLaunchKernelGGL((gemm_generic_kernel<TA, TW, TO, WM, WN, MB, NB>), grid, block, 0, stream,            \
                           (const TA*)A, (const TW*)W, bias, (TO*)C, M, N, K, lda, ldc, a_vec, w_vec);           \
    } while (0)
    const int nseg = tl_ceil_div(K, GF_SEG);
    if (M <= 16 && nseg <= GF_MAX_SEGMENTS) {
        const int waves = gf_waves(nseg, tl_ceil_div(N, 16));
        const size_t lds = (size_t)nseg * 4 * 64 * sizeof(float);
        hipLaunchKernelGGL((gemm_fewrows_kernel<TA, TW, TO, false>), dim3(tl_ceil_div(N, 16)), dim3(64 * waves), lds, stream,
                           (const TA*)A, (const TW*)W, bias, (TO*)C, M, N, K, lda, ldc, a_vec, w_vec);
    } else if (M <= 32)
        GG_GO(1, 4, 2, 1);        // 32 x 64
    else if (M <= 64)
        GG_GO(1, 4, 4, 2);        // 64 x 128
    else
        GG_GO(2, 2, 4, 4);        // 128 x 128
#undef GG_GO
    return 0;
}

// Whether the few-row kernel takes a product of this K (the segments' sums must fit its LDS).
extern "C" int tl_gemm_fewrows_takes(int K) { return K > 0 && tl_ceil_div(K, GF_SEG) <= GF_MAX_SEGMENTS ? 1 : 0; }

// The float product for at most 16 rows from the matrix-core ordered copy of W (see gemm_fewrows_kernel,
// SHUF): A float [M, K] with row stride lda, Ws float [ceil(N/16), ceil(K/16), 64, 4], C float [M, N].
// The same sums in the same order as tl_gemm_generic gives for these rows.
extern "C" int tl_gemm_fewrows_shuffled(const float* A, const float* Ws, const float* bias, float* C, int M, int N, int K,
                                        int lda, int ldc, hipStream_t stream) {
    TL_CHECK_ARG(M >= 0 && M <= 16 && N > 0 && K > 0, "tl_gemm_fewrows_shuffled: bad sizes M=%d N=%d K=%d", M, N, K);
    TL_CHECK_ARG(lda >= K && ldc >= N, "tl_gemm_fewrows_shuffled: row strides lda=%d ldc=%d too small for K=%d N=%d", lda, ldc, K, N);
    TL_CHECK_ARG(tl_gemm_fewrows_takes(K), "tl_gemm_fewrows_shuffled: K=%d is too long for the segments' sums", K);
    TL_CHECK_ARG(((uintptr_t)Ws % 16) == 0, "tl_gemm_fewrows_shuffled: the weight copy must be 16-byte aligned");
    if (M == 0) return 0;
    const int a_vec = ((uintptr_t)A % 16 == 0 && lda % 4 == 0) ? 1 : 0;
    const int nseg = tl_ceil_div(K, GF_SEG);
    const int waves = gf_waves(nseg, tl_ceil_div(N, 16));
    const size_t lds = (size_t)nseg * 4 * 64 * sizeof(float);
    hipLaunchKernelGGL((gemm_fewrows_kernel<float, float, float, true>), dim3(tl_ceil_div(N, 16)), dim3(64 * waves), lds, stream,
                       A, Ws, bias, C, M, N, K, lda, ldc, a_vec, 1);
    TL_CHECK_LAUNCH("tl_gemm_fewrows_shuffled");
    return 0;
}

// A: [M, K] with row stride lda; W: [N, K] contiguous; C: [M, N] with row stride ldc.
extern "C" int tl_gemm_generic(const void* A, int a_dtype, const void* W, int w_dtype, const float* bias, void* C,
                               int c_dtype, int M, int N, int K, int lda, int ldc, hipStream_t stream) {
    TL_CHECK_ARG(M >= 0 && N > 0 && K > 0, "tl_gemm_generic: bad sizes M=%d N=%d K=%d", M, N, K);
    TL_CHECK_ARG(lda >= K && ldc >= N, "tl_gemm_generic: row strides lda=%d ldc=%d too small for K=%d N=%d", lda, ldc, K, N);
    if (M == 0) return 0;
    int rc;
    if (a_dtype == TL_F32 && w_dtype == TL_F32 && c_dtype == TL_F32)
        rc = gg_launch<float, float, float>(A, W, bias, C, M, N, K, lda, ldc, stream);
    else if (a_dtype == TL_BF16 && w_dtype == TL_BF16 && c_dtype == TL_BF16)
        rc = gg_launch<bf16_t, bf16_t, bf16_t>(A, W, bias, C, M, N, K, lda, ldc, stream);
    else if (a_dtype == TL_BF16 && w_dtype == TL_BF16 && c_dtype == TL_F32)
        rc = gg_launch<bf16_t, bf16_t, float>(A, W, bias, C, M, N, K, lda, ldc, stream);
    else if (a_dtype == TL_F32 && w_dtype == TL_BF16 && c_dtype == TL_F32)
        rc = gg_launch<float, bf16_t, float>(A, W, bias, C, M, N, K, lda, ldc, stream);
    else
        return tl_fail("tl_gemm_generic: unsupported dtypes a=%d w=%d c=%d", a_dtype, w_dtype, c_dtype);
    if (rc) return rc;
    TL_CHECK_LAUNCH("tl_gemm_generic");
    return 0;
}
