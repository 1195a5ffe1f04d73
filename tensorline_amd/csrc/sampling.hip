// Token selection from float logits: arg-max rows and temperature / top-p sampling rows.
//
// A row with temperature <= 0 is greedy (lowest index among equal maxima).  Otherwise the rule of
// the reference's sample() (tensorline/engine.py:42-51) is kept:
//   probs = softmax(logits / temperature)
//   with top_p < 1: sort descending, keep a token while the mass *before* it is < top_p
//   draw one token from the kept ones, renormalised.
// No sort is done: the smallest kept weight is found by a three-level radix selection over the
// weights' bit patterns (see the sampling section below).  The draw uses a uniform number u[row] in
// [0, 1) given by the caller: the token is the first in index order whose running kept mass
// exceeds u * kept_mass.
#include "common.h"
#include "argmax_static.h"

#include <mutex>

#define SM_THREADS 1024

struct ArgMax {
    float v;
    int i;
};

__device__ __forceinline__ ArgMax argmax_better(ArgMax a, ArgMax b) {
    // NaN never wins; ties go to the lower index
    if (b.v > a.v || (b.v == a.v && b.i < a.i)) return b;
    return a;
}

__device__ int block_argmax(const float* __restrict__ row, int V, ArgMax* sh) {
    ArgMax best;
    best.v = -INFINITY;
    best.i = 0x7fffffff;
    for (int c = threadIdx.x; c < V; c += blockDim.x) {
        ArgMax cur;
        cur.v = row[c];
        cur.i = c;
        best = argmax_better(best, cur);
    }
#pragma unroll
    for (int off = TL_WAVE / 2; off > 0; off >>= 1) {
        ArgMax o;
        o.v = __shfl_xor(best.v, off, TL_WAVE);
        o.i = __shfl_xor(best.i, off, TL_WAVE);
        best = argmax_better(best, o);
    }
    const int lane = threadIdx.x & (TL_WAVE - 1), wave = threadIdx.x / TL_WAVE;
    const int nwaves = (blockDim.x + TL_WAVE - 1) / TL_WAVE;
    if (lane == 0) sh[wave] = best;
    __syncthreads();
    ArgMax r = sh[0];
    for (int w = 1; w < nwaves; ++w) r = argmax_better(r, sh[w]);
    __syncthreads();
    if (r.i == 0x7fffffff) r.i = 0;  // a row of NaN or -inf
    return r.i;
}

__global__ __launch_bounds__(SM_THREADS) void argmax_kernel(const float* __restrict__ logits, int ld, int V,
                                                            int32_t* __restrict__ out) {
    __shared__ ArgMax sh[16];
    const int r = blockIdx.x;
    const int best = block_argmax(logits + (size_t)r * ld, V, sh);
    if (threadIdx.x == 0) out[r] = best;
}

// Wide rows are cut into chunks so that a few rows still fill the GPU: one work-group per (row,
// chunk) finds the chunk's best, a second kernel the row's best among them.  Ties go to the lower
// index in both steps, so the answer is that of the one-kernel form.
__global__ __launch_bounds__(256) void argmax_chunk_kernel(const float* __restrict__ logits, int ld, int V,
                                                                  int chunk, float* __restrict__ pval,
                                                                  int32_t* __restrict__ pidx) {
    __shared__ ArgMax sh[16];
    const int r = blockIdx.x, ch = blockIdx.y;
    const int c0 = ch * chunk;
    const int n = (V - c0 < chunk) ? V - c0 : chunk;
    const float* row = logits + (size_t)r * ld + c0;
    const int best = block_argmax(row, n, sh);
    if (threadIdx.x == 0) {
        pval[(size_t)r * gridDim.y + ch] = row[best];
        pidx[(size_t)r * gridDim.y + ch] = c0 + best;
    }
}

__global__ void argmax_final_kernel(const float* __restrict__ pval, const int32_t* __restrict__ pidx, int nch,
                                    int32_t* __restrict__ out) {
    const int r = blockIdx.x;
    ArgMax best;
    best.v = -INFINITY;
    best.i = 0x7fffffff;
    for (int c = threadIdx.x; c < nch; c += TL_WAVE) {
        ArgMax cur;
        cur.v = pval[(size_t)r * nch + c];
        cur.i = pidx[(size_t)r * nch + c];
        best = argmax_better(best, cur);
    }
#pragma unroll
    for (int off = TL_WAVE / 2; off > 0; off >>= 1) {
        ArgMax o;
        o.v = __shfl_xor(best.v, off, TL_WAVE);
        o.i = __shfl_xor(best.i, off, TL_WAVE);
        best = argmax_better(best, o);
    }
    if (threadIdx.x == 0) out[r] = (best.i == 0x7fffffff) ? 0 : best.i;
}

#define AM_CHUNKS 64
static_assert(AM_CHUNKS == TL_ARGMAX_STATIC_CHUNKS, "the static buffer is sized for the chunking of tl_argmax");
// scratch: room for R * 64 floats and R * 64 int32 when V > 8192 (may be null otherwise)
extern "C" int tl_argmax(const float* logits, int ld, int R, int V, int32_t* out, float* scratch_val,
                         int32_t* scratch_idx, hipStream_t stream) {
    TL_CHECK_ARG(R >= 0 && V > 0 && ld >= V, "tl_argmax: bad sizes R=%d V=%d ld=%d", R, V, ld);
    if (R == 0) return 0;
    if (V <= 8192 || !scratch_val || !scratch_idx || R > 65535) {
        hipLaunchKernelGGL(argmax_kernel, dim3(R), dim3(SM_THREADS), 0, stream, logits, ld, V, out);
        TL_CHECK_LAUNCH("tl_argmax");
        return 0;
    }
    const int chunk = tl_ceil_div(V, AM_CHUNKS);
    const int nch = tl_ceil_div(V, chunk);
    hipLaunchKernelGGL(argmax_chunk_kernel, dim3(R, nch), dim3(256), 0, stream, logits, ld, V, chunk, scratch_val,
                       scratch_idx);
    hipLaunchKernelGGL(argmax_final_kernel, dim3(R), dim3(TL_WAVE), 0, stream, scratch_val, scratch_idx, nch, out);
    TL_CHECK_LAUNCH("tl_argmax");
    return 0;
}

// ---- arg-max without an allocation ------------------------------------------------------------
// The partial results of wide rows live in this array: TL_ARGMAX_STATIC_MAX_ROWS * 64 floats (the
// chunks' best values), then as many int32 (their indices).  In host code the array's name is a
// stand-in, not a device address: hipGetSymbolAddress gives the address, once per GPU, because
// every GPU holds a copy of its own.  Kernels get that address as an argument.
static __device__ __align__(256) unsigned char scratch[TL_ARGMAX_STATIC_BYTES];

#define TL_MAX_DEVICES 64
static void* g_scratch_ptr[TL_MAX_DEVICES];
static std::mutex g_scratch_mutex;

static int argmax_static_ptr(void** ptr) {
    int dev = -1;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return tl_fail("tl_argmax_static: hipGetDevice failed: %s", hipGetErrorString(e));
    TL_CHECK_ARG(dev >= 0 && dev < TL_MAX_DEVICES, "tl_argmax_static: device %d is outside [0, %d)", dev, TL_MAX_DEVICES);
    std::lock_guard<std::mutex> lock(g_scratch_mutex);
    if (!g_scratch_ptr[dev]) {
        void* p = nullptr;
        e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
        if (e != hipSuccess || !p)
            return tl_fail("tl_argmax_static: hipGetSymbolAddress failed on device %d: %s", dev, hipGetErrorString(e));
        g_scratch_ptr[dev] = p;
    }
    *ptr = g_scratch_ptr[dev];
    return 0;
}

extern "C" int tl_argmax_static_setup(void) {
    void* p = nullptr;
    return argmax_static_ptr(&p);
}

extern "C" int tl_argmax_static(const float* logits, int ld, int R, int V, int32_t* out, hipStream_t stream) {
    TL_CHECK_ARG(R >= 0 && V > 0 && ld >= V, "tl_argmax_static: bad sizes R=%d V=%d ld=%d", R, V, ld);
    TL_CHECK_ARG(R <= TL_ARGMAX_STATIC_MAX_ROWS, "tl_argmax_static: %d rows exceed the %d the static buffer holds", R,
                 TL_ARGMAX_STATIC_MAX_ROWS);
    TL_CHECK_ARG(logits && out, "tl_argmax_static: null logits or output");
    if (R == 0) return 0;
    void* base = nullptr;
    if (int rc = argmax_static_ptr(&base)) return rc;
    float* pval = (float*)base;
    int32_t* pidx = (int32_t*)((unsigned char*)base + (size_t)TL_ARGMAX_STATIC_MAX_ROWS * TL_ARGMAX_STATIC_CHUNKS * 4);
    return tl_argmax(logits, ld, R, V, out, pval, pidx, stream);
}

// ---- temperature / top-p sampling ---------------------------------------------------------------
// A row is cut into chunks of SP_CHUNK logits, one work-group per (chunk, row), so that a few rows
// still use the whole GPU, and the work is a short chain of kernels.  Weights are
// w = exp((logit - max) / T) <= 1; every mass is a sum of weights in fixed point (w * 2^40 as a
// 64-bit integer), so sums are exact, do not depend on the order of addition, and integer atomics
// can build them: a row's result depends on its inputs only.
//   sp_max    chunk maxima
//   sp_sum    chunk masses; for rows with top_p < 1 a histogram of mass over the top 10 bits of the
//             weight's bit pattern (weights are positive floats: their order is that of their bits)
//   sp_level  (twice) finds the bucket the smallest kept weight w_t lies in and builds the histogram
//             of the next 10 bits inside it
//   sp_kept   w_t is known to the bit: per chunk, the mass strictly above it and the number of ties
//   sp_walk   the draw: target = u * kept mass; the chunk whose share of the kept mass holds the
//             target finds the first token, in index order, whose running kept mass exceeds it
// The rule for w_t: with P = top_p * Z, a weight is kept iff the mass of strictly larger weights is
// < P; in a histogram, w_t lies in the lowest non-empty bucket whose mass above is < P.  Of the
// tokens equal to w_t the first ceil((P - above) / w_t) in index order are kept, at least one.
#define SP_THREADS 256
#define SP_ROWS 16                           // element j of thread t in chunk c: c*SP_CHUNK + j*SP_THREADS + t
#define SP_CHUNK (SP_THREADS * SP_ROWS)
#define SP_BUCKETS 1024
#define SP_STATE (3 * SP_BUCKETS)            // per row: three mass histograms, then 8 state words
#define SP_ROW_WORDS (SP_STATE + 8)          // state: P, bucket and mass above of levels 1 and 2, w_t's bits, mass above w_t
typedef unsigned long long u64;
static_assert(SP_BUCKETS == 4 * SP_THREADS, "sp_find gives four buckets to a thread");

__device__ __forceinline__ u64 sp_fix(float w) { return (w > 0.f) ? (u64)(w * 1099511627776.0f) : 0ull; }

__device__ __forceinline__ float sp_weight(float x, float mx, float inv_t) {
    const float w = expf((x - mx) * inv_t);
    return (w <= 1.0f) ? w : 0.f;            // NaN (a row of -inf) counts as no weight
}

__device__ __forceinline__ u64 sp_wave_sum(u64 v) {
#pragma unroll
    for (int off = TL_WAVE / 2; off > 0; off >>= 1) {
        const unsigned lo = __shfl_xor((unsigned)v, off, TL_WAVE), hi = __shfl_xor((unsigned)(v >> 32), off, TL_WAVE);
        v += ((u64)hi << 32) | lo;
    }
    return v;
}

// sum over the block, returned to every thread; sh: room for 4 values; ends with a barrier
__device__ __forceinline__ u64 sp_block_sum(u64 v, u64* sh) {
    v = sp_wave_sum(v);
    if ((threadIdx.x & (TL_WAVE - 1)) == 0) sh[threadIdx.x / TL_WAVE] = v;
    __syncthreads();
    const u64 r = sh[0] + sh[1] + sh[2] + sh[3];
    __syncthreads();
    return r;
}

struct SpRow {
    float mx, inv_t;
    bool active, nucleus;
};

// what every kernel needs of its row: greedy rows (temperature <= 0) are not touched by these kernels
__device__ __forceinline__ SpRow sp_row(const float* temperature, const float* top_p, const float* pmax, int r, int C) {
    SpRow row;
    const float t = temperature[r];
    row.active = t > 0.f;
    row.nucleus = top_p[r] < 1.0f;
    row.inv_t = row.active ? 1.0f / t : 0.f;
    float mx = -INFINITY;
    if (pmax)
        for (int c = 0; c < C; ++c) mx = fmaxf(mx, pmax[(size_t)r * C + c]);
    row.mx = mx;
    return row;
}

__global__ __launch_bounds__(SP_THREADS) void sp_max_kernel(const float* __restrict__ logits, int ld, int V, int C,
                                                            const float* __restrict__ temperature,
                                                            float* __restrict__ pmax) {
    __shared__ float red[16];
    const int c = blockIdx.x, r = blockIdx.y;
    if (!(temperature[r] > 0.f)) return;
    const float* x = logits + (size_t)r * ld;
    float mx = -INFINITY;
#pragma unroll
    for (int j = 0; j < SP_ROWS; ++j) {
        const int i = c * SP_CHUNK + j * SP_THREADS + threadIdx.x;
        if (i < V) mx = fmaxf(mx, x[i]);
    }
    mx = tl_block_max(mx, red);
    if (threadIdx.x == 0) pmax[(size_t)r * C + c] = mx;
}

// P = top_p * Z of a row, Z the sum of its chunk masses
__device__ __forceinline__ u64 sp_mass_wanted(const u64* psum, int C, float top_p) {
    u64 Z = 0;
    for (int c = 0; c < C; ++c) Z += psum[c];
    return (u64)((double)Z * (double)top_p);
}

// In a histogram of SP_BUCKETS masses (buckets ordered by weight): the lowest non-empty bucket whose
// mass above (A0 + the buckets over it) is < P, and that mass; the highest non-empty bucket if none
// is (P == 0).  Every thread gets the answer.  sh: SP_THREADS values, shb: SP_THREADS ints.
__device__ void sp_find(const u64* __restrict__ hist, u64 P, u64 A0, u64* sh, int* shb, int& b_out, u64& A_out) {
    const int t = threadIdx.x;
    u64 m[4];
#pragma unroll
    for (int k = 0; k < 4; ++k) m[k] = hist[4 * t + k];
    const u64 s = m[0] + m[1] + m[2] + m[3];
    sh[t] = s;
    __syncthreads();
    for (int off = 1; off < SP_THREADS; off <<= 1) {            // inclusive suffix sums over the threads
        const u64 v = (t + off < SP_THREADS) ? sh[t + off] : 0ull;
        __syncthreads();
        sh[t] += v;
        __syncthreads();
    }
    u64 above = A0 + sh[t] - s;                                 // mass of the buckets above this thread's four
    int best = 0x7fffffff, top = -1;
    u64 best_a = 0, top_a = 0;
#pragma unroll
    for (int k = 3; k >= 0; --k) {
        if (m[k] != 0) {
            if (top < 0) {
                top = 4 * t + k;
                top_a = above;
            }
            if (above < P) {
                best = 4 * t + k;
                best_a = above;
            }
        }
        above += m[k];
    }
    __syncthreads();
    shb[t] = best;
    __syncthreads();
    for (int off = SP_THREADS / 2; off > 0; off >>= 1) {
        if (t < off) shb[t] = min(shb[t], shb[t + off]);
        __syncthreads();
    }
    int b = shb[0];
    __syncthreads();
    if (b == 0x7fffffff) {                                      // no bucket qualifies: the highest non-empty one
        shb[t] = top;
        __syncthreads();
        for (int off = SP_THREADS / 2; off > 0; off >>= 1) {
            if (t < off) shb[t] = max(shb[t], shb[t + off]);
            __syncthreads();
        }
        b = shb[0];
        __syncthreads();
        if (b < 0) b = 0;                                       // an empty histogram
        if (top == b) sh[0] = top_a;
    } else if (best == b) {
        sh[0] = best_a;
    }
    __syncthreads();
    b_out = b;
    A_out = (b >= 0 && hist[b] != 0) ? sh[0] : A0;
    __syncthreads();
}

// level 1: chunk masses and the first histogram
__global__ __launch_bounds__(SP_THREADS) void sp_sum_kernel(const float* __restrict__ logits, int ld, int V, int C,
                                                            const float* __restrict__ temperature,
                                                            const float* __restrict__ top_p,
                                                            const float* __restrict__ pmax, u64* __restrict__ ws) {
    __shared__ u64 hist[SP_BUCKETS];
    __shared__ u64 red[4];
    const int c = blockIdx.x, r = blockIdx.y;
    const SpRow row = sp_row(temperature, top_p, pmax, r, C);
    if (!row.active) return;
    u64* wr = ws + (size_t)r * (SP_ROW_WORDS + 3 * C);
    if (row.nucleus)
        for (int b = threadIdx.x; b < SP_BUCKETS; b += SP_THREADS) hist[b] = 0;
    __syncthreads();
    const float* x = logits + (size_t)r * ld;
    u64 sum = 0;
#pragma unroll
    for (int j = 0; j < SP_ROWS; ++j) {
        const int i = c * SP_CHUNK + j * SP_THREADS + threadIdx.x;
        if (i >= V) continue;
        const float w = sp_weight(x[i], row.mx, row.inv_t);
        const u64 f = sp_fix(w);
        sum += f;
        if (row.nucleus && f) atomicAdd(&hist[__float_as_uint(w) >> 20], f);
    }
    sum = sp_block_sum(sum, red);
    if (threadIdx.x == 0) wr[SP_ROW_WORDS + c] = sum;
    if (row.nucleus)
        for (int b = threadIdx.x; b < SP_BUCKETS; b += SP_THREADS)
            if (hist[b]) atomicAdd(&wr[b], hist[b]);
}

// levels 2 and 3: find the bucket(s) above, build the next histogram inside
__global__ __launch_bounds__(SP_THREADS) void sp_level_kernel(const float* __restrict__ logits, int ld, int V, int C,
                                                              const float* __restrict__ temperature,
                                                              const float* __restrict__ top_p,
                                                              const float* __restrict__ pmax, u64* __restrict__ ws,
                                                              int level) {
    __shared__ u64 hist[SP_BUCKETS];
    __shared__ u64 sh[SP_THREADS];
    __shared__ int shb[SP_THREADS];
    const int c = blockIdx.x, r = blockIdx.y;
    const SpRow row = sp_row(temperature, top_p, pmax, r, C);
    if (!row.active || !row.nucleus) return;
    u64* wr = ws + (size_t)r * (SP_ROW_WORDS + 3 * C);
    // one selection per kernel; chunk 0 leaves its result in the row's state for the kernels after it
    u64* st = wr + SP_STATE;
    unsigned prefix, shift;
    if (level == 2) {
        const u64 P = sp_mass_wanted(wr + SP_ROW_WORDS, C, top_p[r]);
        int b1;
        u64 A;
        sp_find(wr, P, 0, sh, shb, b1, A);
        if (c == 0 && threadIdx.x == 0) {
            st[0] = P;
            st[1] = (u64)b1;
            st[2] = A;
        }
        prefix = (unsigned)b1;
        shift = 10;
    } else {
        int b2;
        u64 A;
        sp_find(wr + SP_BUCKETS, st[0], st[2], sh, shb, b2, A);
        if (c == 0 && threadIdx.x == 0) {
            st[3] = (u64)b2;
            st[4] = A;
        }
        prefix = ((unsigned)st[1] << 10) | (unsigned)b2;
        shift = 0;
    }
    for (int b = threadIdx.x; b < SP_BUCKETS; b += SP_THREADS) hist[b] = 0;
    __syncthreads();
    const float* x = logits + (size_t)r * ld;
#pragma unroll
    for (int j = 0; j < SP_ROWS; ++j) {
        const int i = c * SP_CHUNK + j * SP_THREADS + threadIdx.x;
        if (i >= V) continue;
        const float w = sp_weight(x[i], row.mx, row.inv_t);
        const u64 f = sp_fix(w);
        const unsigned bits = __float_as_uint(w);
        if (!f || (bits >> (shift + 10)) != prefix) continue;
        atomicAdd(&hist[(bits >> shift) & (SP_BUCKETS - 1)], f);
    }
    __syncthreads();
    u64* out_hist = wr + (size_t)(level - 1) * SP_BUCKETS;
    for (int b = threadIdx.x; b < SP_BUCKETS; b += SP_THREADS)
        if (hist[b]) atomicAdd(&out_hist[b], hist[b]);
}

// per chunk: mass strictly above w_t and number of weights equal to it
__global__ __launch_bounds__(SP_THREADS) void sp_kept_kernel(const float* __restrict__ logits, int ld, int V, int C,
                                                             const float* __restrict__ temperature,
                                                             const float* __restrict__ top_p,
                                                             const float* __restrict__ pmax, u64* __restrict__ ws) {
    __shared__ u64 sh[SP_THREADS];
    __shared__ int shb[SP_THREADS];
    __shared__ u64 red[4];
    const int c = blockIdx.x, r = blockIdx.y;
    const SpRow row = sp_row(temperature, top_p, pmax, r, C);
    if (!row.active || !row.nucleus) return;
    u64* wr = ws + (size_t)r * (SP_ROW_WORDS + 3 * C);
    u64* st = wr + SP_STATE;
    int b3;
    u64 above;
    sp_find(wr + 2 * SP_BUCKETS, st[0], st[4], sh, shb, b3, above);
    const unsigned wt_bits = ((unsigned)st[1] << 20) | ((unsigned)st[3] << 10) | (unsigned)b3;
    if (c == 0 && threadIdx.x == 0) {
        st[5] = (u64)wt_bits;
        st[6] = above;
    }
    const float* x = logits + (size_t)r * ld;
    u64 mass = 0, ties = 0;
#pragma unroll
    for (int j = 0; j < SP_ROWS; ++j) {
        const int i = c * SP_CHUNK + j * SP_THREADS + threadIdx.x;
        if (i >= V) continue;
        const float w = sp_weight(x[i], row.mx, row.inv_t);
        const u64 f = sp_fix(w);
        const unsigned bits = __float_as_uint(w);
        if (!f) continue;
        if (bits > wt_bits) mass += f;
        else if (bits == wt_bits) ++ties;
    }
    mass = sp_block_sum(mass, red);
    ties = sp_block_sum(ties, red);
    if (threadIdx.x == 0) {
        wr[SP_ROW_WORDS + C + c] = mass;
        wr[SP_ROW_WORDS + 2 * C + c] = ties;
    }
}

// exclusive prefix sums of one value per thread, in thread order; sh: SP_THREADS values; the total
// comes back in `total`
__device__ u64 sp_block_scan(u64 v, u64* sh, u64& total) {
    const int t = threadIdx.x;
    sh[t] = v;
    __syncthreads();
    for (int off = 1; off < SP_THREADS; off <<= 1) {
        const u64 add = (t >= off) ? sh[t - off] : 0ull;
        __syncthreads();
        sh[t] += add;
        __syncthreads();
    }
    const u64 incl = sh[t];
    total = sh[SP_THREADS - 1];
    __syncthreads();
    return incl - v;
}

__global__ __launch_bounds__(SP_THREADS) void sp_walk_kernel(const float* __restrict__ logits, int ld, int V, int C,
                                                             const float* __restrict__ temperature,
                                                             const float* __restrict__ top_p,
                                                             const float* __restrict__ uniform,
                                                             const float* __restrict__ pmax, u64* __restrict__ ws,
                                                             int32_t* __restrict__ out) {
    __shared__ u64 kept[SP_CHUNK];                              // kept weight of each element, in index order
    __shared__ unsigned char is_tie[SP_CHUNK];
    __shared__ u64 sh[SP_THREADS];
    const int c = blockIdx.x, r = blockIdx.y;
    const SpRow row = sp_row(temperature, top_p, pmax, r, C);
    if (!row.active) return;
    const u64* wr = ws + (size_t)r * (SP_ROW_WORDS + 3 * C);
    const u64* psum = wr + SP_ROW_WORDS;
    // the kept mass of every chunk, in order: before this chunk, of this chunk, in total
    unsigned wt_bits = 0;
    u64 wt_fix = 0, keep_ties = 0, before = 0, mine = 0, total = 0, ties_before = 0;
    if (row.nucleus) {
        const u64 P = wr[SP_STATE], above = wr[SP_STATE + 6];
        wt_bits = (unsigned)wr[SP_STATE + 5];
        wt_fix = sp_fix(__uint_as_float(wt_bits));
        keep_ties = (P > above && wt_fix) ? (P - above + wt_fix - 1) / wt_fix : 1;
        if (keep_ties < 1) keep_ties = 1;
        u64 ties_seen = 0;
        for (int k = 0; k < C; ++k) {
            const u64 t = psum[2 * C + k];
            const u64 room = keep_ties > ties_seen ? keep_ties - ties_seen : 0;
            const u64 kc = psum[C + k] + (t < room ? t : room) * wt_fix;
            if (k < c) before += kc;
            if (k == c) {
                mine = kc;
                ties_before = ties_seen;
            }
            total += kc;
            ties_seen += t;
        }
    } else {
        for (int k = 0; k < C; ++k) {
            const u64 kc = psum[k];
            if (k < c) before += kc;
            if (k == c) mine = kc;
            total += kc;
        }
    }
    if (total == 0) {                                           // a row without any weight
        if (c == 0 && threadIdx.x == 0) out[r] = 0;
        return;
    }
    u64 target = (u64)((double)total * (double)uniform[r]);
    if (target >= total) target = total - 1;
    if (target < before || target >= before + mine) return;    // another chunk holds the target
    target -= before;
    // this chunk, element by element in index order
    const float* x = logits + (size_t)r * ld;
#pragma unroll 4
    for (int j = 0; j < SP_ROWS; ++j) {
        const int e = j * SP_THREADS + threadIdx.x, i = c * SP_CHUNK + e;
        u64 f = 0;
        bool tie = false;
        if (i < V) {
            const float w = sp_weight(x[i], row.mx, row.inv_t);
            const u64 v = sp_fix(w);
            const unsigned bits = __float_as_uint(w);
            if (!row.nucleus || bits > wt_bits) f = v;
            else if (v && bits == wt_bits) tie = true;
        }
        kept[e] = f;
        is_tie[e] = tie ? 1 : 0;
    }
    __syncthreads();
    const int e0 = threadIdx.x * SP_ROWS;                       // this thread's run of consecutive elements
    u64 all;
    if (row.nucleus) {
        // of the weights equal to w_t the first keep_ties in index order are kept
        u64 mine_ties = 0;
#pragma unroll 1
        for (int k = 0; k < SP_ROWS; ++k) mine_ties += is_tie[e0 + k];
        u64 rank = ties_before + sp_block_scan(mine_ties, sh, all);
#pragma unroll 1
        for (int k = 0; k < SP_ROWS; ++k) {
            if (is_tie[e0 + k]) {
                if (rank < keep_ties) kept[e0 + k] = wt_fix;
                ++rank;
            }
        }
        __syncthreads();
    }
    u64 sum = 0;
#pragma unroll 1
    for (int k = 0; k < SP_ROWS; ++k) sum += kept[e0 + k];
    u64 run = sp_block_scan(sum, sh, all);
    if (target < run || target >= run + sum) return;           // another thread's run holds the target
#pragma unroll 1
    for (int k = 0; k < SP_ROWS; ++k) {
        const u64 v = kept[e0 + k];
        if (v && target < run + v) {
            out[r] = c * SP_CHUNK + e0 + k;
            return;
        }
        run += v;
    }
}

// chunks a row of V logits is cut into, and the workspace tl_sample needs: pmax holds R * chunks
// floats, ws R * (3080 + 3 * chunks) 64-bit words that must be zero when the call starts.  any_greedy /
// any_top_p: whether some row has temperature <= 0 / top_p < 1 (saying yes is always right)
extern "C" int tl_sample_chunks(int V) { return tl_ceil_div(V, SP_CHUNK); }

extern "C" int tl_sample(const float* logits, int ld, int R, int V, const float* temperature, const float* top_p,
                         const float* uniform, int32_t* out, float* pmax, void* ws, int any_greedy, int any_top_p,
                         hipStream_t stream) {
    TL_CHECK_ARG(R >= 0 && V > 0 && ld >= V, "tl_sample: bad sizes R=%d V=%d ld=%d", R, V, ld);
    TL_CHECK_ARG(R <= 65535, "tl_sample: %d rows are more than a launch takes", R);
    TL_CHECK_ARG(pmax && ws && ((uintptr_t)ws % 8) == 0, "tl_sample: missing or misaligned workspace");
    if (R == 0) return 0;
    // greedy rows: the arg-max (of every row: the kernels below overwrite the others and leave these alone)
    if (any_greedy) hipLaunchKernelGGL(argmax_kernel, dim3(R), dim3(SM_THREADS), 0, stream, logits, ld, V, out);
    const int C = tl_ceil_div(V, SP_CHUNK);
    dim3 grid(C, R), block(SP_THREADS);
    u64* w = (u64*)ws;
    hipLaunchKernelGGL(sp_max_kernel, grid, block, 0, stream, logits, ld, V, C, temperature, pmax);
    hipLaunchKernelGGL(sp_sum_kernel, grid, block, 0, stream, logits, ld, V, C, temperature, top_p, pmax, w);
    if (any_top_p) {
        hipLaunchKernelGGL(sp_level_kernel, grid, block, 0, stream, logits, ld, V, C, temperature, top_p, pmax, w, 2);
        hipLaunchKernelGGL(sp_level_kernel, grid, block, 0, stream, logits, ld, V, C, temperature, top_p, pmax, w, 3);
        hipLaunchKernelGGL(sp_kept_kernel, grid, block, 0, stream, logits, ld, V, C, temperature, top_p, pmax, w);
    }
    hipLaunchKernelGGL(sp_walk_kernel, grid, block, 0, stream, logits, ld, V, C, temperature, top_p, uniform, pmax, w, out);
    TL_CHECK_LAUNCH("tl_sample");
    return 0;
}
