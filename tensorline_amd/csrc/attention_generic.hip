// Causal attention of the step's tokens over the paged cache, for any head size, group size and
// storage type.  One work-group per (token, key/value head); the query heads that share the
// key/value head are handled together, up to AG_GC at a time.
//
// A token at position p of sequence s attends to keys [lo, p] of that sequence, lo = 0 or
// p - window + 1 for a windowed layer, found through the sequence's row of the page table.  The
// keys of the step's own tokens are already in the cache when this runs.  k_cache is
// [pages, page, nkv, d]; v_cache is [pages, nkv, d, page].  Scores, the running
// maximum, the sum and the accumulator are float (reference: tensorline/paged_attn.py:25-58,
// tensorline/paged.py:233-238).  Key tiles start at lo, so the result for a position does not
// depend on how the sequence was cut into steps.
#include "common.h"

#define AG_THREADS 256
#define AG_TILE 256   // keys per tile, one per thread in the score phase
#define AG_GC 8       // query heads per pass

template <typename T>
__global__ __launch_bounds__(AG_THREADS) void attn_generic_kernel(
    const T* __restrict__ q, int q_stride, const T* __restrict__ k_cache, const T* __restrict__ v_cache,
    const int32_t* __restrict__ tables, int NB, const int32_t* __restrict__ seq_of_token,
    const int32_t* __restrict__ pos, T* __restrict__ out, int out_stride, int nq, int nkv, int d, int dpad, int bs,
    int window, float scale) {
    extern __shared__ float smem[];
    float* q_s = smem;                         // [AG_GC][d]
    float* s_s = q_s + AG_GC * d;              // [AG_GC][AG_TILE]
    float* red = s_s + AG_GC * AG_TILE;        // [16]
    float* acc_s = red + 16;                   // [AG_THREADS] for the final cross-subset sum
    int* blk_s = (int*)(acc_s + AG_THREADS);   // [AG_TILE] cache row index of each key of the tile

    const int tid = threadIdx.x;
    const int t = blockIdx.x, kvh = blockIdx.y;
    const int s = seq_of_token[t];
    const int p = pos[t];
    const int lo = (window > 0 && p - window + 1 > 0) ? p - window + 1 : 0;
    const int hi = p + 1;
    const int G = nq / nkv;
    const int32_t* table = tables + (size_t)s * NB;

    // value phase mapping: thread = (dim c, key subset sub)
    const int nsub = AG_THREADS / dpad;
    const int c = tid % dpad, sub = tid / dpad;

    for (int g0 = 0; g0 < G; g0 += AG_GC) {
        const int gc = (G - g0 < AG_GC) ? G - g0 : AG_GC;
        for (int i = tid; i < gc * d; i += AG_THREADS) {
            const int g = i / d, cc = i - g * d;
            q_s[g * d + cc] = tl_to_float(q[(size_t)t * q_stride + (size_t)(kvh * G + g0 + g) * d + cc]) * scale;
        }
        float m[AG_GC], l[AG_GC], acc[AG_GC];
#pragma unroll
        for (int g = 0; g < AG_GC; ++g) {
            m[g] = -INFINITY;
            l[g] = 0.f;
            acc[g] = 0.f;
        }
        __syncthreads();

        for (int k0 = lo; k0 < hi; k0 += AG_TILE) {
            const int key = k0 + tid;
            const bool valid = key < hi;
            float sc[AG_GC];
#pragma unroll
            for (int g = 0; g < AG_GC; ++g) sc[g] = 0.f;
            if (valid) {
                const int blk = table[key / bs];
                const int row = blk * bs + key % bs;
                blk_s[tid] = row;
                const T* kr = k_cache + ((size_t)row * nkv + kvh) * d;
                for (int cc = 0; cc < d; ++cc) {
                    const float kv = tl_to_float(kr[cc]);
#pragma unroll
                    for (int g = 0; g < AG_GC; ++g)
                        if (g < gc) sc[g] = fmaf(q_s[g * d + cc], kv, sc[g]);
                }
            } else {
                blk_s[tid] = 0;
            }
#pragma unroll
            for (int g = 0; g < AG_GC; ++g) {
                if (g >= gc) break;
                const float sv = valid ? sc[g] : -INFINITY;
                const float mx = tl_block_max(sv, red);
                const float m_new = fmaxf(m[g], mx);
                const float alpha = expf(m[g] - m_new);   // exp(-inf) = 0 on the first tile
                const float pe = valid ? expf(sv - m_new) : 0.f;
                s_s[g * AG_TILE + tid] = pe;
                const float psum = tl_block_sum(pe, red);
                l[g] = l[g] * alpha + psum;
                acc[g] *= alpha;
                m[g] = m_new;
            }
            __syncthreads();
            const int nkeys = (hi - k0 < AG_TILE) ? hi - k0 : AG_TILE;
            if (c < d) {
                for (int j = sub; j < nkeys; j += nsub) {
                    const int vrow = blk_s[j];
                    const float vv = tl_to_float(v_cache[(((size_t)(vrow / bs) * nkv + kvh) * d + c) * bs + vrow % bs]);
#pragma unroll
                    for (int g = 0; g < AG_GC; ++g)
                        if (g < gc) acc[g] = fmaf(s_s[g * AG_TILE + j], vv, acc[g]);
                }
            }
            __syncthreads();
        }
        // sum the key subsets and write
        for (int g = 0; g < gc; ++g) {
            acc_s[tid] = acc[g];
            __syncthreads();
            if (sub == 0 && c < d) {
                float v = 0.f;
                for (int u = 0; u < nsub; ++u) v += acc_s[u * dpad + c];
                out[(size_t)t * out_stride + (size_t)(kvh * G + g0 + g) * d + c] = tl_from_float<T>(v / l[g]);
            }
            __syncthreads();
        }
    }
}

extern "C" int tl_attention_generic(const void* q, int q_stride, const void* k_cache, const void* v_cache,
                                    const int32_t* tables, int NB, const int32_t* seq_of_token, const int32_t* pos,
                                    void* out, int out_stride, int dtype, int T, int nq, int nkv, int d, int bs,
                                    int window, float scale, hipStream_t stream) {
    TL_CHECK_ARG(T >= 0 && nq > 0 && nkv > 0 && d > 0 && bs > 0 && NB > 0,
                 "tl_attention_generic: bad sizes T=%d nq=%d nkv=%d d=%d page=%d NB=%d", T, nq, nkv, d, bs, NB);
    TL_CHECK_ARG(nq % nkv == 0, "tl_attention_generic: %d query heads are not a multiple of %d key/value heads", nq, nkv);
    TL_CHECK_ARG(d <= 256, "tl_attention_generic: head size %d is above the supported 256", d);
    TL_CHECK_ARG(nkv <= 65535, "tl_attention_generic: too many key/value heads %d", nkv);
    TL_CHECK_ARG(q_stride >= nq * d && out_stride >= nq * d, "tl_attention_generic: row strides too small");
    if (T == 0) return 0;
    int dpad = 1;
    while (dpad < d) dpad <<= 1;
    const size_t smem = sizeof(float) * ((size_t)AG_GC * d + (size_t)AG_GC * AG_TILE + 16 + AG_THREADS) + sizeof(int) * AG_TILE;
    dim3 grid(T, nkv), block(AG_THREADS);
    if (dtype == TL_F32)
        hipLaunchKernelGGL(attn_generic_kernel<float>, grid, block, smem, stream, (const float*)q, q_stride,
                           (const float*)k_cache, (const float*)v_cache, tables, NB, seq_of_token, pos, (float*)out,
                           out_stride, nq, nkv, d, dpad, bs, window, scale);
    else if (dtype == TL_BF16)
        hipLaunchKernelGGL(attn_generic_kernel<bf16_t>, grid, block, smem, stream, (const bf16_t*)q, q_stride,
                           (const bf16_t*)k_cache, (const bf16_t*)v_cache, tables, NB, seq_of_token, pos, (bf16_t*)out,
                           out_stride, nq, nkv, d, dpad, bs, window, scale);
    else
        return tl_fail("tl_attention_generic: unknown dtype %d", dtype);
    TL_CHECK_LAUNCH("tl_attention_generic");
    return 0;
}
