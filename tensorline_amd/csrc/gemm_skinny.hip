// C[M, N] = A[M, K] * W[N, K]^T (+ bias) for few rows (M <= 16), bfloat16 inputs: the matrix
// products of a decode step.  The work is streaming W once from HBM.
//
// W is read from a copy laid out for the matrix cores ("shuffled", made once when the weights are
// loaded): [N/16 tiles][K/32 chunks][64 lanes][8 values], where lane l = 16*g + r holds row r of
// the tile and the 8 consecutive k values starting at 32*chunk + 8*g.  That is exactly the first
// operand of v_mfma_f32_16x16x32_bf16, so one load instruction of a wave reads 1 KB of contiguous
// memory and a wave walks straight through memory along K.  (Loading the same fragments from a
// row-major W touches 16 rows x 64 bytes per instruction: 64 cache-line lookups per KB instead of
// 8, which limits the rate well below HBM's.)
//
// A work-group owns one tile of 16 output columns and all M rows of A; its waves split K among
// themselves and add their partial sums through LDS in a fixed order, so a result never depends
// on timing.  Each wave brings its slice of A in with row-contiguous loads, 128 k at a time, into
// a private LDS region laid out [8-k unit][row] (+1 row of padding per unit, conflict-free both
// ways) and reads the second MFMA operand from there: lane l = 16*g + r reads row m = r of A at
// the k values of unit 4*chunk + g.  No barrier is needed for that: a wave's LDS operations
// complete in order.  The accumulator of lane l, register i, is C[m = l % 16][n = 4*(l / 16) + i].
//
// Two tiles per work-group (MODE_SWIGLU, MODE_QKV), sharing the A fragments:
//  * MODE_SWIGLU owns tile t of the first I/16 tiles and tile t of the next I/16 of a fused
//    [2I, K] gate/up matrix and writes silu(first) * second.
//  * MODE_QKV owns, in head h of a fused q/k/v projection, tiles j and j + d/32: the two halves
//    that rotate-half RoPE pairs.  Its epilogue adds the bias, rotates query and key heads by the
//    token's position (angle pos * inv_freq[i] in float, as tl_rope_store does), writes queries to
//    a [M, nq*d] matrix and keys and values straight into the paged cache at the token's slot:
//    the projection, the position encoding and the cache write of a decode step in one kernel.
//
// RMS normalisation around the products (NormArgs), so that a decode step needs no kernel of its
// own for a norm.  y = W (h * g / rms(h)) equals (W (h * g)) / rms(h): a product may take rows
// A = h * g whose division is still owed, with partial sums of h^2 per row, and scale its results
// by 1/sqrt(sum / dim + eps) in float.  And a plain product that ends a residual branch may do
// the add and prepare the next norm: resid += result (float), a_out = resid * next_weight, and
// the sum of resid^2 over the tile's 16 columns as one partial per row.  Sums of squares are
// added in a fixed order that depends on the shapes only.
#include "common.h"

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float f32x4 __attribute__((ext_vector_type(4)));

#define MODE_PLAIN 0
#define MODE_SWIGLU 1
#define MODE_QKV 2

// what MODE_QKV needs beyond the product
struct QkvArgs {
    const int32_t* pos;        // [M] positions
    const float* inv_freq;     // [d/2]
    const int32_t* slots;      // [M] cache rows (negative: do not store)
    bf16_t* q_out;             // [M, nq*d]
    bf16_t* k_cache;           // [pages, page, nkv, d]
    bf16_t* v_cache;           // [pages, nkv, d, page]
    int nq, nkv, d, bs;
};


#define SK_MAX_LDS (80 * 1024)          // LDS of a work-group; a CU has 160 KB
#define SK_SC 128                    // k values staged per step (4 chunks of 32)
#define SK_UNITS (SK_SC / 8)         // 16-byte units per row of a step
#define SK_ROWPAD 17                 // rows per unit in LDS: 16 + 1 of padding

__device__ __forceinline__ bf16x8 as_frag(uint4 v) { return __builtin_bit_cast(bf16x8, v); }

// Keeps the compiler from moving a wave's LDS reads above its earlier LDS writes (and the other
// way round) without waiting for anything: the hardware completes a wave's LDS operations in
// order, and the global loads in flight (the next step's W fragments) must stay in flight.
__device__ __forceinline__ void wave_lds_order() {
    __builtin_amdgcn_wave_barrier();
    asm volatile("" ::: "memory");
}

template <int MT, int MODE, typename TO>
__global__ __launch_bounds__(MODE == MODE_SWIGLU ? 256 : 512) void gemm_skinny_kernel(
    const bf16_t* __restrict__ A, const uint4* __restrict__ Ws, const float* __restrict__ bias, TO* __restrict__ C,
    int M, int n_out, int K, int K32, int lda, int ldc, int second_tile, QkvArgs qa, TlNormArgs na) {
    extern __shared__ uint4 smem[];
    __shared__ float sh_part[64 * 16];               // [part][row] partial sums of squares
    __shared__ float sh_rstd[16];
    __shared__ float sh_sq[16 * 17];                 // [row][column of the tile] squares of the new residual
    constexpr bool DUAL = MODE != MODE_PLAIN;
    constexpr int NACC = MT * (DUAL ? 2 : 1);
    constexpr int XS_PER_WAVE = MT * SK_UNITS * SK_ROWPAD;     // in uint4
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, nwaves = blockDim.x >> 6;
    const int r = lane & 15, g = lane >> 4;
    int tile = blockIdx.x, tile2 = second_tile + blockIdx.x;
    if (MODE == MODE_QKV) {
        const int pph = qa.d / 32;                   // tile pairs per head
        const int head = blockIdx.x / pph, j = blockIdx.x - head * pph;
        tile = head * (qa.d / 16) + j;
        tile2 = tile + pph;
    }
    const uint4* w1 = Ws + (size_t)tile * K32 * 64 + lane;
    const uint4* w2 = DUAL ? Ws + (size_t)tile2 * K32 * 64 + lane : nullptr;
    uint4* xs = smem + (size_t)wave * XS_PER_WAVE;
    const uint4 zero = make_uint4(0, 0, 0, 0);

    f32x4 acc[NACC];
#pragma unroll
    for (int i = 0; i < NACC; ++i) acc[i] = f32x4{0.f, 0.f, 0.f, 0.f};

    // What the epilogue needs from memory is asked for now, so that it has arrived when the sums
    // are done: this thread's partial sums of squares (thread (row, part) owns every nparts-th
    // partial of its row; the first SS_PRE of them are fetched here) and, with a residual sink,
    // the residual, norm weight and bias of the thread's first output element.  Addresses are
    // clamped; what a clamped load brings is not used.
    const bool owed = na.ss_in != nullptr;
    const bool sink = MODE == MODE_PLAIN && na.resid != nullptr;
    const int ss_row = threadIdx.x & 15, ss_part = threadIdx.x >> 4, ss_nparts = blockDim.x >> 4;
    // groups of few waves (gate/up) have many partials per thread, wide groups have few
    constexpr int SS_PRE = (MODE == MODE_SWIGLU) ? 16 : 4;
    float ssv[SS_PRE];
    if (owed) {
        const float* sp = na.ss_in + (ss_row < M ? ss_row : 0);
#pragma unroll
        for (int k = 0; k < SS_PRE; ++k) {
            const int t = ss_part + k * ss_nparts;
            ssv[k] = sp[(size_t)(t < na.ss_n ? t : 0) * na.ss_ld];
        }
    }
    float pre_resid = 0.f, pre_weight = 0.f, pre_bias = 0.f;
    if (sink && threadIdx.x < 256) {
        const int l = threadIdx.x & 63, i = (threadIdx.x >> 6) & 3;
        const int m = l & 15, n = tile * 16 + 4 * (l >> 4) + i;
        const int mc = m < M ? m : 0, nc = n < n_out ? n : 0;
        pre_resid = na.resid[(size_t)mc * na.resid_ld + nc];
        pre_weight = na.next_weight[nc];
        if (bias) pre_bias = bias[nc];
    }

    const int nsc = (K32 + 3) / 4;                   // steps of 128 k
    const int per = (nsc + nwaves - 1) / nwaves;
    const int s0 = wave * per;
    const int s1 = (s0 + per < nsc) ? s0 + per : nsc;

    // Software pipeline, one step (128 k) deep: while a step is multiplied, the A rows and the W
    // fragments of the next one are in flight.  Loads retire in issue order, so within a step the
    // A rows (needed first, for the LDS write) are requested before the W fragments.  Every load is
    // unconditional: an address past the end is clamped to a valid one, and what it brings is
    // either never used (rows of A past M feed output rows that are not written; the step after
    // the last is not multiplied) or replaced by zero (k past K).
    uint4 wf[4], uf[4], wn[4], un[4], xr[MT * 4];
    const int xrow0 = lane >> 4, xunit = lane & 15;
    const bf16_t* xp[MT * 4];
#pragma unroll
    for (int i = 0; i < MT * 4; ++i) {
        const int row = xrow0 + 4 * i;
        xp[i] = A + (size_t)(row < M ? row : 0) * lda;       // the row's start: the unit is part of the k offset
    }
    const int last_c = K32 - 1;
    {
        const int sc = (s0 < s1) ? s0 : 0;
        const int kx = sc * SK_SC + xunit * 8;
        const int kxc = (kx < K) ? kx : 0;               // past K: the row's first unit, inside the row whatever K is
#pragma unroll
        for (int i = 0; i < MT * 4; ++i) xr[i] = *reinterpret_cast<const uint4*>(xp[i] + kxc);
        if (kx >= K) {
#pragma unroll
            for (int i = 0; i < MT * 4; ++i) xr[i] = zero;
        }
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            int c = sc * 4 + i;
            if (c > last_c) c = last_c;
            wf[i] = tl_load_stream(w1 + (size_t)c * 64);
            if (DUAL) uf[i] = tl_load_stream(w2 + (size_t)c * 64);
        }
    }
    for (int sc = s0; sc < s1; ++sc) {
        // A rows of this step: registers -> LDS, lane (row = lane/16 + 4i, unit = lane%16)
#pragma unroll
        for (int i = 0; i < MT * 4; ++i) {
            const int row = xrow0 + 4 * i;
            xs[((row >> 4) * SK_UNITS + xunit) * SK_ROWPAD + (row & 15)] = xr[i];
        }
        wave_lds_order();
        // request the next step (clamped to the last one when there is none)
        const int sn = (sc + 1 < s1) ? sc + 1 : sc;
        const int kxn = sn * SK_SC + xunit * 8;
        const int kxnc = (kxn < K) ? kxn : 0;
#pragma unroll
        for (int i = 0; i < MT * 4; ++i) xr[i] = *reinterpret_cast<const uint4*>(xp[i] + kxnc);
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            int c = sn * 4 + i;
            if (c > last_c) c = last_c;
            wn[i] = tl_load_stream(w1 + (size_t)c * 64);
            if (DUAL) un[i] = tl_load_stream(w2 + (size_t)c * 64);
        }
        // chunks past K32 of the last step read a clamped chunk: they must count as zero
        const int cbase = sc * 4;
#pragma unroll
        for (int cc = 0; cc < 4; ++cc) {
            const bool live = cbase + cc <= last_c;
#pragma unroll
            for (int mt = 0; mt < MT; ++mt) {
                uint4 xf = xs[(mt * SK_UNITS + cc * 4 + g) * SK_ROWPAD + r];
                if (!live) xf = zero;
                acc[mt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(as_frag(wf[cc]), as_frag(xf), acc[mt], 0, 0, 0);
                if (DUAL)
                    acc[MT + mt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(as_frag(uf[cc]), as_frag(xf), acc[MT + mt], 0, 0, 0);
            }
        }
        wave_lds_order();
        if (kxn >= K) {
#pragma unroll
            for (int i = 0; i < MT * 4; ++i) xr[i] = zero;
        }
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            wf[i] = wn[i];
            if (DUAL) uf[i] = un[i];
        }
    }

    // Owed normalisation: thread (row, part) adds its partials in ascending order, then one thread
    // per row adds the parts in order.  (MT is 1 wherever this is used: rows 0..15.)
    if (owed) {
        float ssum = 0.f;
        if (ss_row < M) {
#pragma unroll
            for (int k = 0; k < SS_PRE; ++k)
                if (ss_part + k * ss_nparts < na.ss_n) ssum += ssv[k];
            // the rest, eight loads at a time so that they overlap
            for (int t0 = ss_part + SS_PRE * ss_nparts; t0 < na.ss_n; t0 += 8 * ss_nparts) {
                float more[8];
#pragma unroll
                for (int k = 0; k < 8; ++k) {
                    const int t = t0 + k * ss_nparts;
                    more[k] = na.ss_in[(size_t)(t < na.ss_n ? t : 0) * na.ss_ld + ss_row];
                }
#pragma unroll
                for (int k = 0; k < 8; ++k)
                    if (t0 + k * ss_nparts < na.ss_n) ssum += more[k];
            }
        }
        sh_part[ss_part * 16 + ss_row] = ssum;
    }
    if (sink)
        for (int e = threadIdx.x; e < 16 * 17; e += blockDim.x) sh_sq[e] = 0.f;
    // partial sums of the waves -> LDS (the staging regions are done with), then a fixed-order sum
    __syncthreads();
    float* red = reinterpret_cast<float*>(smem);     // [nwaves][NACC*4][64]
#pragma unroll
    for (int a = 0; a < NACC; ++a)
#pragma unroll
        for (int i = 0; i < 4; ++i) red[((size_t)wave * NACC * 4 + a * 4 + i) * 64 + lane] = acc[a][i];
    if (owed && threadIdx.x < 16) {
        const int nparts = blockDim.x >> 4;
        float ssum = 0.f;
        for (int p2 = 0; p2 < nparts; ++p2) ssum += sh_part[p2 * 16 + threadIdx.x];
        sh_rstd[threadIdx.x] = 1.0f / sqrtf(ssum / na.dim + na.eps);
    }
    __syncthreads();
    const int n0 = tile * 16;
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
        if (owed) {
            const float rs = sh_rstd[m & 15];
            v *= rs;
            if (DUAL) u *= rs;
        }
        if (MODE == MODE_QKV) {
            // v, u: dims idx and idx + d/2 of head `head` for token m
            const int d = qa.d, half = d / 2;
            const int head = n / d, idx = n - head * d;
            if (bias) {
                v += bias[n];
                u += bias[n + half];
            }
            const int slot = qa.slots[m];
            if (head < qa.nq + qa.nkv) {
                float sn, cs;
                sincosf((float)qa.pos[m] * qa.inv_freq[idx], &sn, &cs);
                const float o1 = v * cs - u * sn, o2 = u * cs + v * sn;
                if (head < qa.nq) {
                    bf16_t* qp = qa.q_out + (size_t)m * qa.nq * d + (size_t)head * d + idx;
                    qp[0] = tl_from_float<bf16_t>(o1);
                    qp[half] = tl_from_float<bf16_t>(o2);
                } else if (slot >= 0) {
                    bf16_t* kp = qa.k_cache + ((size_t)slot * qa.nkv + (head - qa.nq)) * d + idx;
                    kp[0] = tl_from_float<bf16_t>(o1);
                    kp[half] = tl_from_float<bf16_t>(o2);
                }
            } else if (slot >= 0) {
                const int page = slot / qa.bs, off = slot - page * qa.bs;
                bf16_t* vp = qa.v_cache + (((size_t)page * qa.nkv + (head - qa.nq - qa.nkv)) * d + idx) * qa.bs + off;
                vp[0] = tl_from_float<bf16_t>(v);
                vp[(size_t)half * qa.bs] = tl_from_float<bf16_t>(u);
            }
            continue;
        }
        if (sink) {
            const bool first = e < (int)blockDim.x;      // the element whose operands were fetched at the start
            if (bias) v += first ? pre_bias : bias[n];
            float* rp = na.resid + (size_t)m * na.resid_ld + n;
            const float h = (first ? pre_resid : *rp) + v;
            *rp = h;
            na.a_out[(size_t)m * na.a_ld + n] = tl_from_float<bf16_t>(h * (first ? pre_weight : na.next_weight[n]));
            sh_sq[(m & 15) * 17 + (n - n0)] = h * h;
            continue;
        }
        if (MODE == MODE_SWIGLU) {
            v = v / (1.0f + expf(-v)) * u;
        } else if (bias) {
            v += bias[n];
        }
        C[(size_t)m * ldc + n] = tl_from_float<TO>(v);
    }
    if (sink) {
        __syncthreads();
        if ((int)threadIdx.x < M && threadIdx.x < 16) {
            float ssum = 0.f;
            for (int c = 0; c < 16; ++c) ssum += sh_sq[threadIdx.x * 17 + c];
            na.ss_out[(size_t)tile * na.ss_out_ld + threadIdx.x] = ssum;
        }
    }
}

static size_t lds_per_wave(int MT, int nacc) {
    const size_t stage = (size_t)MT * SK_UNITS * SK_ROWPAD * sizeof(uint4);
    const size_t red = (size_t)nacc * 4 * 64 * sizeof(float);
    return stage > red ? stage : red;
}

static int pick_waves(int tiles, int nsc, int MT, int nacc, int max_waves) {
    // enough waves in flight to cover HBM latency on 256 CUs; K is split among the waves of a group
    int w = 1;
    while (w < max_waves && tiles * w < 4096 && nsc >= 2 * w) w <<= 1;
    while (w > 1 && (size_t)w * lds_per_wave(MT, nacc) > SK_MAX_LDS) w >>= 1;
    return w;
}

template <int MT, int MODE, typename TO>
static void launch_skinny(const bf16_t* A, const uint4* Ws, const float* bias, TO* C, int M, int n_out, int K, int K32,
                          int lda, int ldc, int second_tile, hipStream_t stream, const TlNormArgs& na,
                          QkvArgs qa = QkvArgs()) {
    // the grid: one group per tile, or per pair of tiles in the two-tile modes
    const int groups = (MODE == MODE_QKV) ? tl_ceil_div(n_out, 32) : tl_ceil_div(n_out, 16);
    const int nacc = MT * (MODE != MODE_PLAIN ? 2 : 1);
    // at most 8 waves to a group (4 in the gate/up form): measured at the 7B shapes, 16 waves stream
    // the down projection in 30.9 us and 8 in 28.0, the fused q/k/v projection in 12.1 and 11.3
    const int nwaves = pick_waves(groups, (K32 + 3) / 4, MT, nacc, MODE == MODE_SWIGLU ? 4 : 8);
    const size_t smem = (size_t)nwaves * lds_per_wave(MT, nacc);
    hipLaunchKernelGGL((gemm_skinny_kernel<MT, MODE, TO>), dim3(groups), dim3(nwaves * 64), smem, stream, A, Ws, bias, C,
                       M, n_out, K, K32, lda, ldc, second_tile, qa, na);
}

template <int DUAL, typename TO>
static int dispatch_skinny(const bf16_t* A, const uint4* Ws, const float* bias, TO* C, int M, int n_out, int K, int K32,
                           int lda, int ldc, int second_tile, hipStream_t stream, const TlNormArgs& na) {
    // one 16-row MFMA tile of A; more rows go to gemm_rows64.hip
    launch_skinny<1, DUAL, TO>(A, Ws, bias, C, M, n_out, K, K32, lda, ldc, second_tile, stream, na);
    TL_CHECK_LAUNCH("tl_gemm_skinny");
    return 0;
}

// `norm` as the entry points take it: null for none.  A sink needs MODE_PLAIN (checked by the caller).
static int check_norm(const TlNormArgs* norm, TlNormArgs* na, int M, int N, bool sink_allowed) {
    *na = TlNormArgs();
    if (!norm) return 0;
    *na = *norm;
    if (na->ss_in)
        TL_CHECK_ARG(na->ss_n > 0 && na->ss_ld >= M && na->dim > 0.f && na->eps >= 0.f,
                     "tl_gemm_skinny: bad owed-norm arguments (partials %d, stride %d)", na->ss_n, na->ss_ld);
    if (na->resid) {
        TL_CHECK_ARG(sink_allowed, "tl_gemm_skinny: only a plain product can add into the residual");
        TL_CHECK_ARG(na->next_weight && na->a_out && na->ss_out && na->resid_ld >= N && na->a_ld >= N &&
                         na->ss_out_ld >= M && M <= 16,
                     "tl_gemm_skinny: bad residual-sink arguments for M=%d N=%d", M, N);
    }
    return 0;
}

static int check_skinny(const void* A, const void* Ws, const void* C, int M, int N, int K, int lda, int ldc) {
    TL_CHECK_ARG(M >= 0 && M <= 16, "tl_gemm_skinny: M=%d is outside [0, 16]", M);
    TL_CHECK_ARG(N > 0 && K > 0, "tl_gemm_skinny: bad sizes N=%d K=%d", N, K);
    TL_CHECK_ARG(K % 8 == 0 && lda % 8 == 0, "tl_gemm_skinny: K=%d and the row stride %d must be multiples of 8", K, lda);
    TL_CHECK_ARG(((uintptr_t)A % 16) == 0 && ((uintptr_t)Ws % 16) == 0, "tl_gemm_skinny: operands must be 16-byte aligned");
    TL_CHECK_ARG(lda >= K && ldc > 0, "tl_gemm_skinny: bad strides");
    return 0;
}

// bfloat16 A [M, K] (row stride lda); Ws: the shuffled copy of W [N, K], ceil(N/16) * ceil(K/32) * 512
// values, zero where it pads; C [M, N] float or bfloat16 (row stride ldc).
// norm: null, or what the product does for the norms around it (TlNormArgs); with a residual sink
// C is not written and may be null.
extern "C" int tl_gemm_skinny(const void* A, const void* Ws, const float* bias, void* C, int c_dtype, int M, int N, int K,
                              int lda, int ldc, const TlNormArgs* norm, hipStream_t stream) {
    if (int rc = check_skinny(A, Ws, C, M, N, K, lda, ldc)) return rc;
    TlNormArgs na;
    if (int rc = check_norm(norm, &na, M, N, true)) return rc;
    TL_CHECK_ARG(na.resid || (C && ldc >= N), "tl_gemm_skinny: output row stride %d < N=%d, or no output", ldc, N);
    if (M == 0) return 0;
    const int K32 = tl_ceil_div(K, 32);
    if (c_dtype == TL_F32)
        return dispatch_skinny<MODE_PLAIN, float>((const bf16_t*)A, (const uint4*)Ws, bias, (float*)C, M, N, K, K32, lda, ldc, 0, stream, na);
    if (c_dtype == TL_BF16)
        return dispatch_skinny<MODE_PLAIN, bf16_t>((const bf16_t*)A, (const uint4*)Ws, bias, (bf16_t*)C, M, N, K, K32, lda, ldc, 0, stream, na);
    return tl_fail("tl_gemm_skinny: unknown output dtype %d", c_dtype);
}

// Ws: the shuffled copy of a [2I, K] matrix, rows [0, I) the gate and rows [I, 2I) the up projection;
// I is a multiple of 16.  C [M, I] = silu(A Wg^T) * (A Wu^T), bfloat16.
extern "C" int tl_gemm_skinny_swiglu(const void* A, const void* Ws, void* C, int M, int I, int K, int lda, int ldc,
                                     const TlNormArgs* norm, hipStream_t stream) {
    if (int rc = check_skinny(A, Ws, C, M, 2 * I, K, lda, ldc)) return rc;
    TlNormArgs na;
    if (int rc = check_norm(norm, &na, M, 2 * I, false)) return rc;
    TL_CHECK_ARG(I % 16 == 0, "tl_gemm_skinny_swiglu: I=%d must be a multiple of 16", I);
    TL_CHECK_ARG(C && ldc >= I, "tl_gemm_skinny_swiglu: output row stride %d < I=%d", ldc, I);
    if (M == 0) return 0;
    return dispatch_skinny<MODE_SWIGLU, bf16_t>((const bf16_t*)A, (const uint4*)Ws, nullptr, (bf16_t*)C, M, I, K,
                                         tl_ceil_div(K, 32), lda, ldc, I / 16, stream, na);
}

// The fused q/k/v projection of a decode step: Ws is the shuffled copy of the [(nq + 2 nkv) d, K]
// matrix, bias float [(nq + 2 nkv) d] or null.  Writes rotated queries to q_out [M, nq*d] and rotated
// keys and the values into the cache at slots[m] (k_cache [pages, page, nkv, d], v_cache
// [pages, nkv, d, page]).  Full-width rotate-half RoPE only: inv_freq holds d/2 values.
extern "C" int tl_gemm_skinny_qkv_rope(const void* A, const void* Ws, const float* bias, const int32_t* pos,
                                       const float* inv_freq, const int32_t* slots, void* q_out, void* k_cache,
                                       void* v_cache, int M, int K, int lda, int nq, int nkv, int d, int bs,
                                       const TlNormArgs* norm, hipStream_t stream) {
    const int N = (nq + 2 * nkv) * d;
    if (int rc = check_skinny(A, Ws, q_out, M, N, K, lda, 1)) return rc;
    TlNormArgs na;
    if (int rc = check_norm(norm, &na, M, N, false)) return rc;
    TL_CHECK_ARG(M <= 16, "tl_gemm_skinny_qkv_rope: M=%d is above 16", M);
    TL_CHECK_ARG(d % 32 == 0 && d > 0 && nq > 0 && nkv > 0 && bs > 0, "tl_gemm_skinny_qkv_rope: bad sizes d=%d nq=%d nkv=%d page=%d", d, nq, nkv, bs);
    TL_CHECK_ARG(pos && inv_freq && slots && q_out && k_cache && v_cache, "tl_gemm_skinny_qkv_rope: missing argument");
    if (M == 0) return 0;
    QkvArgs qa;
    qa.pos = pos;
    qa.inv_freq = inv_freq;
    qa.slots = slots;
    qa.q_out = (bf16_t*)q_out;
    qa.k_cache = (bf16_t*)k_cache;
    qa.v_cache = (bf16_t*)v_cache;
    qa.nq = nq;
    qa.nkv = nkv;
    qa.d = d;
    qa.bs = bs;
    launch_skinny<1, MODE_QKV, bf16_t>((const bf16_t*)A, (const uint4*)Ws, bias, (bf16_t*)nullptr, M, N, K,
                                       tl_ceil_div(K, 32), lda, N, 0, stream, na, qa);
    TL_CHECK_LAUNCH("tl_gemm_skinny_qkv_rope");
    return 0;
}
