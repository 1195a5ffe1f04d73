// Token selection from float logits: arg-max rows and temperature / top-p sampling rows.
//
// One work-group per row.  A row with temperature <= 0 is greedy (lowest index among equal
// maxima).  Otherwise the rule of the reference's sample() (tensorline/engine.py:42-51) is kept:
//   probs = softmax(logits / temperature)
//   with top_p < 1: sort descending, keep a token while the mass *before* it is < top_p
//   draw one token from the kept ones, renormalised.
// No sort is done.  With weights w = exp((logit - max) / T) and Z their sum, a token is kept iff
// the mass of strictly larger weights is < top_p * Z; the smallest kept weight w_t is found by a
// binary search over float bit patterns, and of the tokens equal to w_t only as many as the rule
// admits are kept (lowest indices first).  The draw uses a uniform number u[row] in [0, 1) given
// by the caller: the token is the first in index order whose running kept mass exceeds
// u * kept_mass.  Every sum has a fixed order, so a row's result depends only on its inputs.
#include "common.h"

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

// mass of the weights strictly above `thr`
__device__ __forceinline__ float mass_above(const float* __restrict__ row, int V, float mx, float inv_t, float thr,
                                            float* red) {
    float s = 0.f;
    for (int c = threadIdx.x; c < V; c += blockDim.x) {
        const float w = expf((row[c] - mx) * inv_t);
        if (w > thr) s += w;
    }
    return tl_block_sum(s, red);
}

__global__ __launch_bounds__(SM_THREADS) void sample_kernel(const float* __restrict__ logits, int ld, int V,
                                                            const float* __restrict__ temperature,
                                                            const float* __restrict__ top_p,
                                                            const float* __restrict__ uniform,
                                                            int32_t* __restrict__ out) {
    __shared__ ArgMax sh[16];
    __shared__ float red[16];
    __shared__ float th_mass[SM_THREADS];
    __shared__ int th_ties[SM_THREADS];
    __shared__ int winner;
    __shared__ float winner_base;

    const int r = blockIdx.x;
    const float* row = logits + (size_t)r * ld;
    const float temp = temperature[r];
    if (!(temp > 0.f)) {
        const int best = block_argmax(row, V, sh);
        if (threadIdx.x == 0) out[r] = best;
        return;
    }
    const float inv_t = 1.0f / temp;
    float mx = -INFINITY;
    for (int c = threadIdx.x; c < V; c += blockDim.x) mx = fmaxf(mx, row[c]);
    mx = tl_block_max(mx, red);
    const float Z = mass_above(row, V, mx, inv_t, -1.0f, red);

    const float tp = top_p[r];
    float w_t = 0.f;          // smallest kept weight; 0 keeps everything
    float above = 0.f;        // mass strictly above w_t
    int keep_ties = 0x7fffffff;
    if (tp < 1.0f) {
        const float P = tp * Z;
        // smallest bit pattern b with mass_above(float(b)) < P; the weight of the maximum is 1.0
        uint32_t lo = 0u, hi = 0x3f800000u;
        while (lo < hi) {
            const uint32_t mid = lo + ((hi - lo) >> 1);
            const float f = mass_above(row, V, mx, inv_t, __uint_as_float(mid), red);
            if (f < P) hi = mid; else lo = mid + 1u;
        }
        const float b = __uint_as_float(lo);
        float wmin = INFINITY;
        for (int c = threadIdx.x; c < V; c += blockDim.x) {
            const float w = expf((row[c] - mx) * inv_t);
            if (w >= b) wmin = fminf(wmin, w);
        }
        w_t = -tl_block_max(-wmin, red);
        above = mass_above(row, V, mx, inv_t, w_t, red);
        // ties at w_t are kept while the mass before them is < P
        const float room = (P - above) / w_t;
        keep_ties = (int)ceilf(room);
        if (keep_ties < 1) keep_ties = 1;
    }

    // Walk in index order: thread i owns the contiguous range [i*chunk, (i+1)*chunk).
    const int chunk = (V + blockDim.x - 1) / blockDim.x;
    const int c0 = threadIdx.x * chunk;
    const int c1 = (c0 + chunk < V) ? c0 + chunk : V;
    float my_mass = 0.f;
    int my_ties = 0;
    for (int c = c0; c < c1; ++c) {
        const float w = expf((row[c] - mx) * inv_t);
        if (w > w_t) my_mass += w;
        else if (w == w_t) ++my_ties;
    }
    th_mass[threadIdx.x] = my_mass;
    th_ties[threadIdx.x] = my_ties;
    __syncthreads();
    if (threadIdx.x == 0) {
        // exclusive prefix of kept ties and of kept mass; pick the thread whose range holds the target
        int ties_before = 0;
        float total = 0.f;
        for (int i = 0; i < (int)blockDim.x; ++i) {
            int kt = keep_ties - ties_before;
            if (kt < 0) kt = 0;
            if (kt > th_ties[i]) kt = th_ties[i];
            ties_before += th_ties[i];
            th_ties[i] = kt;                       // now: ties this thread keeps
            th_mass[i] += (float)kt * w_t;
            total += th_mass[i];
        }
        const float target = uniform[r] * total;
        float run = 0.f;
        int win = -1, last = 0;
        float base = 0.f, last_base = 0.f;
        for (int i = 0; i < (int)blockDim.x; ++i) {
            if (th_mass[i] > 0.f) {
                last = i;
                last_base = run;
            }
            if (win < 0 && run + th_mass[i] > target && th_mass[i] > 0.f) {
                win = i;
                base = run;
            }
            run += th_mass[i];
        }
        if (win < 0) {
            win = last;
            base = last_base;
        }
        winner = win;
        winner_base = base;
        red[0] = target;
    }
    __syncthreads();
    if ((int)threadIdx.x == winner) {
        const float target = red[0];
        float run = winner_base;
        int ties_left = th_ties[threadIdx.x];
        int chosen = -1, last_kept = -1;
        for (int c = c0; c < c1; ++c) {
            const float w = expf((row[c] - mx) * inv_t);
            bool kept = w > w_t;
            if (!kept && w == w_t && ties_left > 0) {
                kept = true;
                --ties_left;
            }
            if (!kept) continue;
            last_kept = c;
            run += w;
            if (run > target) {
                chosen = c;
                break;
            }
        }
        if (chosen < 0) chosen = last_kept >= 0 ? last_kept : c0;
        out[r] = chosen;
    }
}

extern "C" int tl_sample(const float* logits, int ld, int R, int V, const float* temperature, const float* top_p,
                         const float* uniform, int32_t* out, hipStream_t stream) {
    TL_CHECK_ARG(R >= 0 && V > 0 && ld >= V, "tl_sample: bad sizes R=%d V=%d ld=%d", R, V, ld);
    if (R == 0) return 0;
    hipLaunchKernelGGL(sample_kernel, dim3(R), dim3(SM_THREADS), 0, stream, logits, ld, V, temperature, top_p,
                       uniform, out);
    TL_CHECK_LAUNCH("tl_sample");
    return 0;
}
