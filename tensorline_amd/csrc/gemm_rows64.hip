// C[M, N] = A[M, K] * W[N, K]^T (+ bias) for 17 to 64 rows, bfloat16: decode steps of large
// batches and short prompt portions.  Same matrix-core ordered weight copy as the few-row kernel
// (gemm_skinny.hip); what differs is how the work is cut, because with up to 64 rows the rows of A
// weigh as much as several 16-column tiles of W and must not be read again for every tile.
//
// A work-group of `waves` waves owns one 16-column tile per wave and one share of K.  Per step of
// 128 k the group brings A[0:64, k:k+128] into LDS once, with row-contiguous loads by all its
// threads, and every wave multiplies it with its own W fragments, which it loads straight into
// registers.  Loads of A and W run two steps ahead in a ring of registers (one step ahead leaves
// every step waiting a full memory latency: 77 us against 61 for the 7B gate/up product; three and
// four gain nothing more); LDS is double-buffered: one barrier per step.
//
// How the work is cut decides the speed.  A CU streams weights at a bounded rate however many
// loads its waves have in flight, so the product is as fast as the busiest CU: the cut (waves per
// group, shares of K) is chosen so that the groups fill the 256 CUs in whole rounds with as little
// left over as possible (r64_plan).  With one share the result is written at once; otherwise every
// share writes a float partial [share, M, N] and a second kernel adds the shares in ascending
// order, so the result does not depend on timing.  Whichever kernel completes the sums also does
// what follows them: bias; an owed RMS normalisation and the residual add with the next norm's
// input (TlNormArgs); SiLU(gate) * up for a fused gate/up matrix (with one share a wave owns a gate
// tile and its up tile); for a fused q/k/v projection bias, RoPE and the cache write.
#include "common.h"

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float f32x4 __attribute__((ext_vector_type(4)));

#define R64_SC 128
#define R64_UNITS (R64_SC / 8)
#define R64_ROWPAD 17
#define R64_MT 4
#define R64_DEPTH 2                          // steps of loads in flight per wave
#define R64_A_WEIGHT 1                       // a group's loads of A, in units of one wave's loads of W (cost model)
#define R64_PIECES (64 * R64_UNITS)          // 16-byte pieces of A per step
#define R64_MIN_WAVES 4
#define R64_MAX_WAVES 16
#define R64_CUS 256

__device__ __forceinline__ bf16x8 r64_frag(uint4 v) { return __builtin_bit_cast(bf16x8, v); }

// Loads of one step: this thread's P pieces of A and this lane's four W fragments.  Steps are
// clamped by the caller, so every address is valid; nothing here depends on the loaded data, so
// the loads stay in flight until the step that uses them.
template <int P, bool PAIR>
__device__ __forceinline__ void r64_issue(const bf16_t* const (&xp)[P], const uint4* w1, const uint4* w2, int step,
                                          int xunit, int K, int last_c, uint4 (&xo)[P], uint4 (&wo)[4],
                                          uint4 (&uo)[PAIR ? 4 : 1]) {
    // past K: the row's first unit, which lies inside the row whatever K is
    const int kbase = (step * R64_SC + xunit * 8 < K) ? step * R64_SC + xunit * 8 : 0;
#pragma unroll
    for (int i = 0; i < P; ++i) xo[i] = *reinterpret_cast<const uint4*>(xp[i] + kbase);
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        int c = step * 4 + i;
        if (c > last_c) c = last_c;
        wo[i] = tl_load_stream(w1 + (size_t)c * 64);
        if (PAIR) uo[i] = tl_load_stream(w2 + (size_t)c * 64);
    }
}

// P: pieces of A a thread loads per step; the group has at least 1024 / P threads (a multiple of
// 16, so that a thread's pieces all lie in one 16-byte column of the step).  Wave w of group x owns
// tile w * gridDim.x + x: groups differ by at most one live wave.  PAIR: W is a fused gate/up
// matrix of ntiles + ntiles tiles, a wave owns gate tile t and up tile ntiles + t and writes
// silu(gate) * up to C [M, N / 2] (one share only: the sums must be complete).
template <typename TO, int P, int THREADS, bool PAIR>
__global__ __launch_bounds__(THREADS) void gemm_rows64_kernel(
    const bf16_t* __restrict__ A, const uint4* __restrict__ Ws, const float* __restrict__ bias, TO* __restrict__ C,
    float* __restrict__ partial, int M, int N, int K, int K32, int lda, int ldc, int steps_per_share, int ntiles,
    TlNormArgs na) {
    constexpr int DEPTH = R64_DEPTH;
    __shared__ uint4 xs[2][R64_MT * R64_UNITS * R64_ROWPAD];
    __shared__ float sh_rstd[64];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int nthreads = blockDim.x;
    const int r = lane & 15, g = lane >> 4;
    const int nsc = (K32 + 3) / 4;
    const int s0 = blockIdx.y * steps_per_share;
    const int s1 = (s0 + steps_per_share < nsc) ? s0 + steps_per_share : nsc;
    int tile = wave * gridDim.x + blockIdx.x;
    const bool tile_live = tile < ntiles;
    if (!tile_live) tile = ntiles - 1;                       // loads stay in bounds; nothing is written
    const uint4* w1 = Ws + (size_t)tile * K32 * 64 + lane;
    const uint4* w2 = PAIR ? Ws + (size_t)(ntiles + tile) * K32 * 64 + lane : nullptr;
    const uint4 zero = make_uint4(0, 0, 0, 0);
    const int last_c = K32 - 1;

    f32x4 acc[R64_MT], acc2[PAIR ? R64_MT : 1];
#pragma unroll
    for (int i = 0; i < R64_MT; ++i) acc[i] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int i = 0; i < (PAIR ? R64_MT : 1); ++i) acc2[i] = f32x4{0.f, 0.f, 0.f, 0.f};

    // loader of A: 64 rows x 16 units = 1024 16-byte pieces, up to P per thread
    const bf16_t* xp[P];
    int xslot[P];
    bool xmine[P];
#pragma unroll
    for (int i = 0; i < P; ++i) {
        const int idx = tid + nthreads * i;
        xmine[i] = idx < R64_PIECES;
        const int row = xmine[i] ? idx >> 4 : 0, unit = idx & 15;
        xp[i] = A + (size_t)(row < M ? row : 0) * lda;       // the row's start: the unit (this thread's xunit) is part of the k offset
        xslot[i] = ((row >> 4) * R64_UNITS + unit) * R64_ROWPAD + (row & 15);
    }
    const int xunit = tid & 15;
    const int nst = s1 - s0;
    uint4 xa[DEPTH][P], wr[DEPTH][4], ur[DEPTH][PAIR ? 4 : 1];
#pragma unroll
    for (int j = 0; j < DEPTH; ++j) {
        const int st = (j < nst) ? s0 + j : s1 - 1;
        r64_issue<P, PAIR>(xp, w1, w2, st, xunit, K, last_c, xa[j], wr[j], ur[j]);
        __builtin_amdgcn_sched_barrier(0);                   // oldest slot first, as in the loop below
    }
    int cur = 0;
    for (int base = 0; base < nst; base += DEPTH) {
#pragma unroll
        for (int j = 0; j < DEPTH; ++j) {
            const int it = base + j;
            const int sc = (it < nst) ? s0 + it : s1 - 1;
            // No branch in here: a step past the share's end (the step count need not be a multiple
            // of DEPTH) runs on zeros.  Pieces of A past K count as zero too.
            const bool xlive = it < nst && sc * R64_SC + xunit * 8 < K;
#pragma unroll
            for (int i = 0; i < P; ++i) {
                uint4 x = xa[j][i];
                if (!xlive) x = zero;
                if (xmine[i]) xs[cur][xslot[i]] = x;
            }
            __syncthreads();
            // chunks past K32 multiply a clamped (valid) chunk of W with pieces of A that are zero
#pragma unroll
            for (int cc = 0; cc < 4; ++cc) {
#pragma unroll
                for (int mt = 0; mt < R64_MT; ++mt) {
                    const uint4 xf = xs[cur][(mt * R64_UNITS + cc * 4 + g) * R64_ROWPAD + r];
                    acc[mt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(r64_frag(wr[j][cc]), r64_frag(xf), acc[mt], 0, 0, 0);
                    if (PAIR)
                        acc2[mt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(r64_frag(ur[j][cc]), r64_frag(xf), acc2[mt], 0, 0, 0);
                }
            }
            // Refill this slot of the ring only now that its values are used up, so that the slot
            // keeps its registers over the whole loop and nothing has to wait for a copy.
            __builtin_amdgcn_sched_barrier(0);
            const int sn = (it + DEPTH < nst) ? s0 + it + DEPTH : s1 - 1;   // past the end: a step again, unused
            r64_issue<P, PAIR>(xp, w1, w2, sn, xunit, K, last_c, xa[j], wr[j], ur[j]);
            __builtin_amdgcn_sched_barrier(0);
            cur ^= 1;
        }
    }
    // An owed normalisation is applied here only when the sums are complete (one share): thread
    // (row, group) adds every ngroups-th partial of its row, one thread per row adds the groups in
    // order.  The staging buffers are done with and serve as scratch.
    const bool owed = na.ss_in != nullptr && partial == nullptr;
    if (owed) {
        __syncthreads();
        float* part_sh = reinterpret_cast<float*>(&xs[0][0]);    // [ngroups][64], ngroups <= 16
        const int row = tid & 63, grp = tid >> 6, ngroups = nthreads >> 6;
        float ssum = 0.f;
        if (row < M)
            for (int t = grp; t < na.ss_n; t += ngroups) ssum += na.ss_in[(size_t)t * na.ss_ld + row];
        part_sh[grp * 64 + row] = ssum;
        __syncthreads();
        if (tid < 64) {
            float tot = 0.f;
            for (int g2 = 0; g2 < ngroups; ++g2) tot += part_sh[g2 * 64 + tid];
            sh_rstd[tid] = 1.0f / sqrtf(tot / na.dim + na.eps);
        }
        __syncthreads();
    }
    if (!tile_live) return;
    // accumulator register i of lane l: C[m = mt*16 + l % 16][n = tile*16 + 4*(l / 16) + i]
    const int n0 = tile * 16 + 4 * g;
    const bool sink = na.resid != nullptr && partial == nullptr;
#pragma unroll
    for (int mt = 0; mt < R64_MT; ++mt) {
        const int m = mt * 16 + r;
        float sq = 0.f;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const int n = n0 + i;
            if (m >= M || n >= (PAIR ? N / 2 : N)) continue;
            if (partial) {
                partial[((size_t)blockIdx.y * M + m) * N + n] = acc[mt][i];
                continue;
            }
            float v = owed ? acc[mt][i] * sh_rstd[m] : acc[mt][i];
            if (PAIR) {
                const float u = owed ? acc2[mt][i] * sh_rstd[m] : acc2[mt][i];
                C[(size_t)m * ldc + n] = tl_from_float<TO>(v / (1.0f + expf(-v)) * u);
                continue;
            }
            if (bias) v += bias[n];
            if (sink) {
                float* rp = na.resid + (size_t)m * na.resid_ld + n;
                const float h = *rp + v;
                *rp = h;
                na.a_out[(size_t)m * na.a_ld + n] = tl_from_float<bf16_t>(h * na.next_weight[n]);
                sq += h * h;
            } else {
                C[(size_t)m * ldc + n] = tl_from_float<TO>(v);
            }
        }
        if (sink) {
            // the tile's sum of squares of row m: over this lane's four columns, then over the four lanes
            sq += __shfl_xor(sq, 16, TL_WAVE);
            sq += __shfl_xor(sq, 32, TL_WAVE);
            if (g == 0 && m < M) na.ss_out[(size_t)tile * na.ss_out_ld + m] = sq;
        }
    }
}

// out[m, n] = sum over shares of partial[share, m, n] (+ bias[n]); with swiglu: n < I and
// out[m, n] = silu(sum gate) * (sum up), gate at column n and up at column I + n of the partials.
// One group per (256 columns, row).  With an owed normalisation the sums are scaled by the row's
// 1/sqrt(sum of partials / dim + eps) first; with a residual sink the result is added into the
// residual, the next norm's input is written and the group's sum of squares becomes one partial.
template <typename TO>
__global__ __launch_bounds__(256) void gemm_rows64_reduce_kernel(const float* __restrict__ partial,
                                                                 const float* __restrict__ bias, TO* __restrict__ C,
                                                                 int M, int N, int n_out, int ldc, int shares,
                                                                 int swiglu, TlNormArgs na) {
    __shared__ float red[16];
    const int n = blockIdx.x * blockDim.x + threadIdx.x;
    const int m = blockIdx.y;
    float rs = 1.f;
    if (na.ss_in) {
        float ssum = 0.f;
        for (int t = threadIdx.x; t < na.ss_n; t += blockDim.x) ssum += na.ss_in[(size_t)t * na.ss_ld + m];
        rs = 1.0f / sqrtf(tl_block_sum(ssum, red) / na.dim + na.eps);
    }
    const bool live = n < n_out;
    float v = 0.f, u = 0.f;
    if (live) {
        for (int s = 0; s < shares; ++s) {
            const float* p = partial + ((size_t)s * M + m) * N;
            v += p[n];
            if (swiglu) u += p[n_out + n];
        }
        v *= rs;
        if (swiglu) v = v / (1.0f + expf(-v)) * (u * rs);
        else if (bias) v += bias[n];
    }
    if (na.resid) {
        float sq = 0.f;
        if (live) {
            float* rp = na.resid + (size_t)m * na.resid_ld + n;
            const float h = *rp + v;
            *rp = h;
            na.a_out[(size_t)m * na.a_ld + n] = tl_from_float<bf16_t>(h * na.next_weight[n]);
            sq = h * h;
        }
        const float tot = tl_block_sum(sq, red);
        if (threadIdx.x == 0) na.ss_out[(size_t)blockIdx.x * na.ss_out_ld + m] = tot;
        return;
    }
    if (live) C[(size_t)m * ldc + n] = tl_from_float<TO>(v);
}

// The second kernel of a fused q/k/v projection: sums of the shares (scaled by an owed
// normalisation), bias, rotate-half RoPE of query and key heads by the token's position (angle
// pos * inv_freq[i] in float, as tl_rope_store does), queries to q_out [M, nq*d], rotated keys and
// the values into the paged cache at slots[m] (k_cache [pages, page, nkv, d], v_cache
// [pages, nkv, d, page]; a negative slot stores nothing).  One thread per (row, head, pair of dims
// idx and idx + d/2); full-width rotation only.
__global__ __launch_bounds__(256) void gemm_rows64_reduce_qkv_kernel(
    const float* __restrict__ partial, const float* __restrict__ bias, int M, int N, int shares,
    const int32_t* __restrict__ pos, const float* __restrict__ inv_freq, const int32_t* __restrict__ slots,
    bf16_t* __restrict__ q_out, bf16_t* __restrict__ k_cache, bf16_t* __restrict__ v_cache, int nq, int nkv, int d,
    int bs, TlNormArgs na) {
    __shared__ float red[16];
    const int pi = blockIdx.x * blockDim.x + threadIdx.x;
    const int m = blockIdx.y;
    float rs = 1.f;
    if (na.ss_in) {
        float ssum = 0.f;
        for (int t = threadIdx.x; t < na.ss_n; t += blockDim.x) ssum += na.ss_in[(size_t)t * na.ss_ld + m];
        rs = 1.0f / sqrtf(tl_block_sum(ssum, red) / na.dim + na.eps);
    }
    const int half = d / 2;
    if (pi >= N / 2) return;
    const int head = pi / half, idx = pi - head * half;
    const int n1 = head * d + idx, n2 = n1 + half;
    float v = 0.f, u = 0.f;
    for (int s = 0; s < shares; ++s) {
        const float* p = partial + ((size_t)s * M + m) * N;
        v += p[n1];
        u += p[n2];
    }
    v *= rs;
    u *= rs;
    if (bias) {
        v += bias[n1];
        u += bias[n2];
    }
    const int slot = slots[m];
    if (head < nq + nkv) {
        float sn, cs;
        sincosf((float)pos[m] * inv_freq[idx], &sn, &cs);
        const float o1 = v * cs - u * sn, o2 = u * cs + v * sn;
        if (head < nq) {
            bf16_t* qp = q_out + (size_t)m * nq * d + (size_t)head * d + idx;
            qp[0] = tl_from_float<bf16_t>(o1);
            qp[half] = tl_from_float<bf16_t>(o2);
        } else if (slot >= 0) {
            bf16_t* kp = k_cache + ((size_t)slot * nkv + (head - nq)) * d + idx;
            kp[0] = tl_from_float<bf16_t>(o1);
            kp[half] = tl_from_float<bf16_t>(o2);
        }
    } else if (slot >= 0) {
        const int page = slot / bs, off = slot - page * bs;
        bf16_t* vp = v_cache + (((size_t)page * nkv + (head - nq - nkv)) * d + idx) * bs + off;
        vp[0] = tl_from_float<bf16_t>(v);
        vp[(size_t)half * bs] = tl_from_float<bf16_t>(u);
    }
}

// The cut of a [N, K] product with M rows: waves per group and shares of K.  The cost of a cut is
// the work of the busiest CU in units of one wave's step (4 KB of W): whole rounds of groups over
// the CUs, each group as slow as its waves are many, plus two steps of filling and draining per
// group, plus (with more than one share) the second kernel and the partial sums' traffic.  The
// group's loads of A weigh about as much as one more wave's loads of W.
struct R64Plan {
    int waves, shares, steps, groups_x;
};

static R64Plan r64_plan(int M, int N, int K) {
    const int ntiles = tl_ceil_div(N, 16);
    const int nsc = tl_ceil_div(tl_ceil_div(K, 32), 4);
    R64Plan best{R64_MIN_WAVES, 1, nsc, tl_ceil_div(ntiles, R64_MIN_WAVES)};
    double best_cost = 1e30;
    const int max_shares = nsc / 2 > 1 ? nsc / 2 : 1;
    for (int waves = R64_MIN_WAVES; waves <= R64_MAX_WAVES; ++waves) {
        const int gx = tl_ceil_div(ntiles, waves);
        const int live = tl_ceil_div(ntiles, gx);            // waves with a tile in the fullest group
        for (int want = 1; want <= max_shares && want <= 64; ++want) {
            const int steps = tl_ceil_div(nsc, want);
            const int shares = tl_ceil_div(nsc, steps);
            if (shares != want) continue;                     // the same cut as a smaller `want`
            const int rounds = tl_ceil_div(gx * shares, R64_CUS);
            double cost = (double)rounds * (live + R64_A_WEIGHT) * (steps + 2);
            if (shares > 1) cost += 25.0 + (double)shares * (M > 0 ? M : 1) * N * 8.0 / R64_CUS / 4096.0;
            if (cost < best_cost) {
                best_cost = cost;
                best = R64Plan{waves, shares, steps, gx};
            }
        }
    }
    return best;
}

// The cut for the paired gate/up form: one share, a wave per pair of tiles (it streams two tiles),
// at most 7 waves so that a thread's registers hold two rings of fragments.
static R64Plan r64_plan_pairs(int M, int npairs, int K) {
    const int nsc = tl_ceil_div(tl_ceil_div(K, 32), 4);
    R64Plan best{R64_MIN_WAVES, 1, nsc, tl_ceil_div(npairs, R64_MIN_WAVES)};
    double best_cost = 1e30;
    for (int waves = R64_MIN_WAVES; waves <= 7; ++waves) {
        const int gx = tl_ceil_div(npairs, waves);
        const int live = tl_ceil_div(npairs, gx);
        const double cost = (double)tl_ceil_div(gx, R64_CUS) * (2 * live + R64_A_WEIGHT) * (nsc + 2);
        if (cost < best_cost) {
            best_cost = cost;
            best = R64Plan{waves, 1, nsc, gx};
        }
    }
    return best;
}

// Number of shares K is cut into for a [N, K] matrix and M rows (the caller sizes the workspace by it).
extern "C" int tl_gemm_rows64_shares(int M, int N, int K) { return r64_plan(M, N, K).shares; }

template <typename TO>
static void r64_launch(const R64Plan& p, hipStream_t stream, const bf16_t* A, const uint4* Ws, const float* bias, TO* C,
                       float* part, int M, int N, int K, int K32, int lda, int ldc, int ntiles, const TlNormArgs& na) {
    dim3 grid(p.groups_x, p.shares), block(p.waves * 64);
    if (p.waves >= 16)
        hipLaunchKernelGGL((gemm_rows64_kernel<TO, 1, 1024, false>), grid, block, 0, stream, A, Ws, bias, C, part, M, N, K,
                           K32, lda, ldc, p.steps, ntiles, na);
    else if (p.waves >= 8)
        hipLaunchKernelGGL((gemm_rows64_kernel<TO, 2, 1024, false>), grid, block, 0, stream, A, Ws, bias, C, part, M, N, K,
                           K32, lda, ldc, p.steps, ntiles, na);
    else
        hipLaunchKernelGGL((gemm_rows64_kernel<TO, 4, 512, false>), grid, block, 0, stream, A, Ws, bias, C, part, M, N, K,
                           K32, lda, ldc, p.steps, ntiles, na);
}

// A: bfloat16 [M, K], 16 < M <= 64 is what it is for (any M from 1 to 64 works); Ws: shuffled copy of
// W [N, K]; C [M, n_out] bfloat16 or float.  shares = tl_gemm_rows64_shares(M, N, K); with shares > 1
// `partial` holds shares*M*N floats.  swiglu: W is a fused [2I, K] gate/up matrix (N = 2I), C is
// [M, I] = silu(gate) * up and bias is not used (with one share I must be a multiple of 16).  norm: null, or an owed
// normalisation of A's rows and / or a residual sink (TlNormArgs).  With a sink C is not written,
// swiglu is not allowed, and ss_out gets one partial per row and 16-column tile when shares is 1
// ([ceil(N/16), M]), per row and 256 columns otherwise ([ceil(N/256), M]).
extern "C" int tl_gemm_rows64(const void* A, const void* Ws, const float* bias, void* C, int c_dtype, float* partial,
                              int M, int N, int K, int lda, int ldc, int shares, int swiglu, const TlNormArgs* norm,
                              hipStream_t stream) {
    TL_CHECK_ARG(M >= 0 && M <= 64 && N > 0 && K > 0, "tl_gemm_rows64: bad sizes M=%d N=%d K=%d", M, N, K);
    TL_CHECK_ARG(K % 8 == 0 && lda % 8 == 0 && lda >= K, "tl_gemm_rows64: K=%d and the row stride %d must be multiples of 8", K, lda);
    TL_CHECK_ARG(((uintptr_t)A % 16) == 0 && ((uintptr_t)Ws % 16) == 0, "tl_gemm_rows64: operands must be 16-byte aligned");
    const R64Plan plan = r64_plan(M, N, K);
    TL_CHECK_ARG(shares == plan.shares, "tl_gemm_rows64: %d shares do not fit this shape", shares);
    TL_CHECK_ARG(shares == 1 || partial, "tl_gemm_rows64: shares need a workspace");
    TL_CHECK_ARG(!swiglu || (N % 2 == 0 && (shares > 1 || N % 32 == 0)),
                 "tl_gemm_rows64: the SwiGLU form needs N even, and N / 2 a multiple of 16 unless K is cut");
    const int n_out = swiglu ? N / 2 : N;
    TlNormArgs na = TlNormArgs();
    if (norm) na = *norm;
    if (na.ss_in)
        TL_CHECK_ARG(na.ss_n > 0 && na.ss_ld >= M && na.dim > 0.f && na.eps >= 0.f,
                     "tl_gemm_rows64: bad owed-norm arguments (partials %d, stride %d)", na.ss_n, na.ss_ld);
    if (na.resid)
        TL_CHECK_ARG(!swiglu && na.next_weight && na.a_out && na.ss_out && na.resid_ld >= N && na.a_ld >= N &&
                         na.ss_out_ld >= M,
                     "tl_gemm_rows64: bad residual-sink arguments for M=%d N=%d", M, N);
    TL_CHECK_ARG(na.resid || (ldc >= n_out && C), "tl_gemm_rows64: bad output");
    TL_CHECK_ARG(c_dtype == TL_F32 || c_dtype == TL_BF16, "tl_gemm_rows64: unknown output dtype %d", c_dtype);
    if (M == 0) return 0;
    const int K32 = tl_ceil_div(K, 32), ntiles = tl_ceil_div(N, 16);
    float* part = shares > 1 ? partial : nullptr;
    if (swiglu && shares == 1) {
        // complete sums in the first kernel: a wave owns a gate tile and its up tile
        TL_CHECK_ARG(c_dtype == TL_BF16, "tl_gemm_rows64: the paired SwiGLU form writes bfloat16");
        const int npairs = N / 32;
        const R64Plan pp = r64_plan_pairs(M, npairs, K);
        hipLaunchKernelGGL((gemm_rows64_kernel<bf16_t, 4, 512, true>), dim3(pp.groups_x, 1), dim3(pp.waves * 64), 0, stream,
                           (const bf16_t*)A, (const uint4*)Ws, nullptr, (bf16_t*)C, nullptr, M, N, K, K32, lda, ldc,
                           pp.steps, npairs, na);
        TL_CHECK_LAUNCH("tl_gemm_rows64 pairs");
        return 0;
    }
    if (c_dtype == TL_F32)
        r64_launch<float>(plan, stream, (const bf16_t*)A, (const uint4*)Ws, bias, (float*)C, part, M, N, K, K32, lda, ldc, ntiles, na);
    else
        r64_launch<bf16_t>(plan, stream, (const bf16_t*)A, (const uint4*)Ws, bias, (bf16_t*)C, part, M, N, K, K32, lda, ldc, ntiles, na);
    TL_CHECK_LAUNCH("tl_gemm_rows64");
    if (shares > 1) {
        dim3 rgrid(tl_ceil_div(n_out, 256), M), rblock(256);
        if (c_dtype == TL_F32)
            hipLaunchKernelGGL(gemm_rows64_reduce_kernel<float>, rgrid, rblock, 0, stream, partial, bias, (float*)C, M, N,
                               n_out, ldc, shares, swiglu, na);
        else
            hipLaunchKernelGGL(gemm_rows64_reduce_kernel<bf16_t>, rgrid, rblock, 0, stream, partial, bias, (bf16_t*)C, M, N,
                               n_out, ldc, shares, swiglu, na);
        TL_CHECK_LAUNCH("tl_gemm_rows64 reduce");
    }
    return 0;
}

// The fused q/k/v projection for 17 to 64 rows: the product above with K cut into shares, then
// gemm_rows64_reduce_qkv_kernel.  Ws is the shuffled copy of the [(nq + 2 nkv) d, K] matrix; shares
// = tl_gemm_rows64_shares(M, N, K) must be above 1 (the caller uses the separate kernels otherwise)
// and `partial` holds shares*M*N floats.  norm: null or an owed normalisation of A's rows.
extern "C" int tl_gemm_rows64_qkv_rope(const void* A, const void* Ws, const float* bias, const int32_t* pos,
                                       const float* inv_freq, const int32_t* slots, void* q_out, void* k_cache,
                                       void* v_cache, float* partial, int M, int K, int lda, int nq, int nkv, int d,
                                       int bs, int shares, const TlNormArgs* norm, hipStream_t stream) {
    TL_CHECK_ARG(nq > 0 && nkv > 0 && d > 0 && d % 2 == 0 && bs > 0, "tl_gemm_rows64_qkv_rope: bad sizes d=%d nq=%d nkv=%d page=%d", d, nq, nkv, bs);
    const int N = (nq + 2 * nkv) * d;
    TL_CHECK_ARG(M >= 0 && M <= 64 && K > 0, "tl_gemm_rows64_qkv_rope: bad sizes M=%d K=%d", M, K);
    TL_CHECK_ARG(K % 8 == 0 && lda % 8 == 0 && lda >= K, "tl_gemm_rows64_qkv_rope: K=%d and the row stride %d must be multiples of 8", K, lda);
    TL_CHECK_ARG(((uintptr_t)A % 16) == 0 && ((uintptr_t)Ws % 16) == 0, "tl_gemm_rows64_qkv_rope: operands must be 16-byte aligned");
    TL_CHECK_ARG(pos && inv_freq && slots && q_out && k_cache && v_cache && partial, "tl_gemm_rows64_qkv_rope: missing argument");
    const R64Plan plan = r64_plan(M, N, K);
    TL_CHECK_ARG(shares == plan.shares && shares > 1, "tl_gemm_rows64_qkv_rope: %d shares do not fit this shape, or K is not cut", shares);
    TlNormArgs na = TlNormArgs();
    if (norm) na = *norm;
    TL_CHECK_ARG(!na.resid, "tl_gemm_rows64_qkv_rope: a projection into the cache has no residual sink");
    if (na.ss_in)
        TL_CHECK_ARG(na.ss_n > 0 && na.ss_ld >= M && na.dim > 0.f && na.eps >= 0.f,
                     "tl_gemm_rows64_qkv_rope: bad owed-norm arguments (partials %d, stride %d)", na.ss_n, na.ss_ld);
    if (M == 0) return 0;
    const int K32 = tl_ceil_div(K, 32), ntiles = tl_ceil_div(N, 16);
    r64_launch<bf16_t>(plan, stream, (const bf16_t*)A, (const uint4*)Ws, nullptr, (bf16_t*)nullptr, partial, M, N, K, K32,
                       lda, N, ntiles, TlNormArgs());
    TL_CHECK_LAUNCH("tl_gemm_rows64_qkv_rope");
    dim3 rgrid(tl_ceil_div(N / 2, 256), M), rblock(256);
    hipLaunchKernelGGL(gemm_rows64_reduce_qkv_kernel, rgrid, rblock, 0, stream, partial, bias, M, N, shares, pos, inv_freq,
                       slots, (bf16_t*)q_out, (bf16_t*)k_cache, (bf16_t*)v_cache, nq, nkv, d, bs, na);
    TL_CHECK_LAUNCH("tl_gemm_rows64_qkv_rope second kernel");
    return 0;
}
