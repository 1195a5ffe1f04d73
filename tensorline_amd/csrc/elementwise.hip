// Row-wise and element-wise kernels: embedding gather, residual add + RMSNorm, rotary position
// encoding fused with the write into the paged cache, SiLU-multiply.
//
// The residual stream is float in every mode; the kernels that read or write activations take
// the storage type (float or bfloat16) as a template argument and compute in float.
#include "common.h"

#include <math.h>
#include <stdarg.h>
#include <stdio.h>

// ---- error reporting -----------------------------------------------------------------------
static thread_local char g_tl_error[512] = "";

int tl_fail(const char* fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_tl_error, sizeof(g_tl_error), fmt, ap);
    va_end(ap);
    return 1;
}

extern "C" const char* tl_last_error() { return g_tl_error; }

extern "C" int tl_abi_version() { return 1; }

// ---- embedding gather ----------------------------------------------------------------------
// x[t, :] = float(table[ids[t], :]).  An id outside [0, V) gives a row of NaN instead of a fault;
// callers validate ids on the host.
template <typename T>
__global__ void embed_kernel(const int32_t* __restrict__ ids, const T* __restrict__ table,
                             float* __restrict__ x, int H, int V) {
    const int t = blockIdx.x;
    const int id = ids[t];
    float* xr = x + (size_t)t * H;
    if (id < 0 || id >= V) {
        for (int c = threadIdx.x; c < H; c += blockDim.x) xr[c] = NAN;
        return;
    }
    const T* row = table + (size_t)id * H;
    for (int c = threadIdx.x; c < H; c += blockDim.x) xr[c] = tl_to_float(row[c]);
}

extern "C" int tl_embed(const int32_t* ids, const void* table, int table_dtype, float* x, int T, int H, int V,
                        hipStream_t stream) {
    TL_CHECK_ARG(T >= 0 && H > 0 && V > 0, "tl_embed: bad sizes T=%d H=%d V=%d", T, H, V);
    if (T == 0) return 0;
    dim3 grid(T), block(256);
    if (table_dtype == TL_F32)
        hipLaunchKernelGGL(embed_kernel<float>, grid, block, 0, stream, ids, (const float*)table, x, H, V);
    else if (table_dtype == TL_BF16)
        hipLaunchKernelGGL(embed_kernel<bf16_t>, grid, block, 0, stream, ids, (const bf16_t*)table, x, H, V);
    else
        return tl_fail("tl_embed: unknown dtype %d", table_dtype);
    TL_CHECK_LAUNCH("tl_embed");
    return 0;
}

// ---- residual add + RMSNorm ----------------------------------------------------------------
// Without `rows`: x[r] += residual[r] (written back, float), out[r] = x[r] * rstd * w.
// With `rows`:    out[r] = norm(x[rows[r]] + residual[rows[r]]); x is left as it is.
// The residual may come in `parts` slices `pstride` elements apart (the K shares of a product):
// it is then their sum in ascending order, formed first and added to x as one number.
// The sum, the mean of squares and the scaling are float (reference: tensorline/fused.py:19-32).
template <typename R, typename O, bool HAS_RES, bool HAS_ROWS>
__global__ void add_rmsnorm_kernel(float* __restrict__ x, const R* __restrict__ res, const float* __restrict__ w,
                                   O* __restrict__ out, const int32_t* __restrict__ rows, int H, float eps, int parts,
                                   size_t pstride) {
    __shared__ float red[16];
    const int r = blockIdx.x;
    const size_t src = HAS_ROWS ? (size_t)rows[r] : (size_t)r;
    float* xr = x + src * H;
    const R* rr = HAS_RES ? res + src * H : nullptr;
    O* orow = out + (size_t)r * H;

    float ss = 0.f;
    for (int c = threadIdx.x; c < H; c += blockDim.x) {
        float v = xr[c];
        if (HAS_RES) {
            float b = tl_to_float(rr[c]);
            for (int p = 1; p < parts; ++p) b += tl_to_float(rr[c + p * pstride]);
            v += b;
            if (!HAS_ROWS) xr[c] = v;
        }
        ss += v * v;
    }
    ss = tl_block_sum(ss, red);
    const float rstd = 1.0f / sqrtf(ss / (float)H + eps);
    for (int c = threadIdx.x; c < H; c += blockDim.x) {
        float v = xr[c];
        if (HAS_RES && HAS_ROWS) {
            float b = tl_to_float(rr[c]);
            for (int p = 1; p < parts; ++p) b += tl_to_float(rr[c + p * pstride]);
            v += b;
        }
        orow[c] = tl_from_float<O>(v * rstd * w[c]);
    }
}

// The same for H a multiple of 4 and at most 16384: one pass, 16-byte accesses, the row kept in
// registers between the sum of squares and the scaling.
__device__ __forceinline__ float4 tl_load4(const float* p) { return *reinterpret_cast<const float4*>(p); }
__device__ __forceinline__ float4 tl_load4(const bf16_t* p) {
    const uint2 u = *reinterpret_cast<const uint2*>(p);
    return make_float4(__uint_as_float(u.x << 16), __uint_as_float(u.x & 0xffff0000u), __uint_as_float(u.y << 16),
                       __uint_as_float(u.y & 0xffff0000u));
}
__device__ __forceinline__ void tl_store4(float* p, float4 v) { *reinterpret_cast<float4*>(p) = v; }
__device__ __forceinline__ void tl_store4(bf16_t* p, float4 v) {
    uint2 u;
    u.x = (uint32_t)tl_f2bf_bits(v.x) | ((uint32_t)tl_f2bf_bits(v.y) << 16);
    u.y = (uint32_t)tl_f2bf_bits(v.z) | ((uint32_t)tl_f2bf_bits(v.w) << 16);
    *reinterpret_cast<uint2*>(p) = u;
}

#define NORM_VPT 4   // float4 per thread at most
template <typename R, typename O, bool HAS_RES, bool HAS_ROWS>
__global__ __launch_bounds__(1024) void add_rmsnorm_vec_kernel(float* __restrict__ x, const R* __restrict__ res,
                                                               const float* __restrict__ w, O* __restrict__ out,
                                                               const int32_t* __restrict__ rows, int H, float eps,
                                                               int parts, size_t pstride) {
    __shared__ float red[16];
    const int r = blockIdx.x;
    const size_t src = HAS_ROWS ? (size_t)rows[r] : (size_t)r;
    float* xr = x + src * H;
    const R* rr = HAS_RES ? res + src * H : nullptr;
    O* orow = out + (size_t)r * H;
    const int n4 = H >> 2;
    float4 v[NORM_VPT];
    float ss = 0.f;
#pragma unroll
    for (int i = 0; i < NORM_VPT; ++i) {
        const int c4 = threadIdx.x + i * blockDim.x;
        if (c4 < n4) {
            float4 a = tl_load4(xr + 4 * c4);
            if (HAS_RES) {
                float4 b = tl_load4(rr + 4 * c4);
                for (int p = 1; p < parts; ++p) {
                    const float4 e = tl_load4(rr + 4 * c4 + p * pstride);
                    b.x += e.x;
                    b.y += e.y;
                    b.z += e.z;
                    b.w += e.w;
                }
                a.x += b.x;
                a.y += b.y;
                a.z += b.z;
                a.w += b.w;
                if (!HAS_ROWS) tl_store4(xr + 4 * c4, a);
            }
            v[i] = a;
            ss += a.x * a.x;
            ss += a.y * a.y;
            ss += a.z * a.z;
            ss += a.w * a.w;
        }
    }
    ss = tl_block_sum(ss, red);
    const float rstd = 1.0f / sqrtf(ss / (float)H + eps);
#pragma unroll
    for (int i = 0; i < NORM_VPT; ++i) {
        const int c4 = threadIdx.x + i * blockDim.x;
        if (c4 < n4) {
            const float4 g = tl_load4(w + 4 * c4);
            float4 o;
            o.x = v[i].x * rstd * g.x;
            o.y = v[i].y * rstd * g.y;
            o.z = v[i].z * rstd * g.z;
            o.w = v[i].w * rstd * g.w;
            tl_store4(orow + 4 * c4, o);
        }
    }
}

template <typename R, typename O>
static void launch_add_rmsnorm(float* x, const R* res, const float* w, O* out, const int32_t* rows, int n_rows,
                               int H, float eps, int parts, size_t pstride, hipStream_t stream) {
    if (H % 4 == 0 && H <= 1024 * 4 * NORM_VPT && pstride % 4 == 0) {
        int threads = ((H / 4 + 63) / 64) * 64;
        if (threads > 1024) threads = 1024;
        dim3 grid(n_rows), block(threads);
        if (res && rows)
            hipLaunchKernelGGL((add_rmsnorm_vec_kernel<R, O, true, true>), grid, block, 0, stream, x, res, w, out, rows, H, eps, parts, pstride);
        else if (res)
            hipLaunchKernelGGL((add_rmsnorm_vec_kernel<R, O, true, false>), grid, block, 0, stream, x, res, w, out, rows, H, eps, parts, pstride);
        else if (rows)
            hipLaunchKernelGGL((add_rmsnorm_vec_kernel<R, O, false, true>), grid, block, 0, stream, x, res, w, out, rows, H, eps, parts, pstride);
        else
            hipLaunchKernelGGL((add_rmsnorm_vec_kernel<R, O, false, false>), grid, block, 0, stream, x, res, w, out, rows, H, eps, parts, pstride);
        return;
    }
    dim3 grid(n_rows), block(H >= 2048 ? 512 : 256);
    if (res && rows)
        hipLaunchKernelGGL((add_rmsnorm_kernel<R, O, true, true>), grid, block, 0, stream, x, res, w, out, rows, H, eps, parts, pstride);
    else if (res)
        hipLaunchKernelGGL((add_rmsnorm_kernel<R, O, true, false>), grid, block, 0, stream, x, res, w, out, rows, H, eps, parts, pstride);
    else if (rows)
        hipLaunchKernelGGL((add_rmsnorm_kernel<R, O, false, true>), grid, block, 0, stream, x, res, w, out, rows, H, eps, parts, pstride);
    else
        hipLaunchKernelGGL((add_rmsnorm_kernel<R, O, false, false>), grid, block, 0, stream, x, res, w, out, rows, H, eps, parts, pstride);
}

extern "C" int tl_add_rmsnorm(float* x, const void* residual, int res_dtype, int res_parts, long long res_part_stride,
                              const float* w, void* out, int out_dtype, const int32_t* rows, int n_rows, int H,
                              float eps, hipStream_t stream) {
    TL_CHECK_ARG(n_rows >= 0 && H > 0, "tl_add_rmsnorm: bad sizes rows=%d H=%d", n_rows, H);
    TL_CHECK_ARG(res_parts >= 1 && res_parts <= 64 && (res_parts == 1 || (residual && res_part_stride > 0)),
                 "tl_add_rmsnorm: bad residual parts %d (stride %lld)", res_parts, res_part_stride);
    TL_CHECK_ARG(eps >= 0.f, "tl_add_rmsnorm: eps must be >= 0");
    if (n_rows == 0) return 0;
    if (!residual) res_dtype = TL_F32;
#define TL_NORM_CASE(RD, RT, OD, OT)                                                                     \
    if (res_dtype == RD && out_dtype == OD) {                                                            \
        launch_add_rmsnorm<RT, OT>(x, (const RT*)residual, w, (OT*)out, rows, n_rows, H, eps, res_parts, \
                                   (size_t)res_part_stride, stream);                                     \
        TL_CHECK_LAUNCH("tl_add_rmsnorm");                                                               \
        return 0;                                                                                        \
    }
    TL_NORM_CASE(TL_F32, float, TL_F32, float)
    TL_NORM_CASE(TL_F32, float, TL_BF16, bf16_t)
    TL_NORM_CASE(TL_BF16, bf16_t, TL_F32, float)
    TL_NORM_CASE(TL_BF16, bf16_t, TL_BF16, bf16_t)
#undef TL_NORM_CASE
    return tl_fail("tl_add_rmsnorm: unknown dtypes residual=%d out=%d", res_dtype, out_dtype);
}

// ---- rotary position encoding + cache write ------------------------------------------------
// qkv: [T, (nq + 2 nkv) * d] as the fused projection leaves it.  Query heads are rotated in place;
// key heads are rotated and written to k_cache at the token's slot; value heads are copied to
// v_cache, which is transposed within a page so that the keys of one page are contiguous for each
// head dim (what the matrix cores want for the P*V product).  Rotate-half layout over the first
// `rot` dims of a head (reference: fused.py:34-51):
//   out[i]         = a*cos(theta_i) - b*sin(theta_i)       a = x[i], b = x[i + rot/2]
//   out[i + rot/2] = b*cos(theta_i) + a*sin(theta_i)       theta_i = pos * inv_freq[i]
// The angle, sine and cosine are float.  A negative slot skips the cache write of that token.
// k_cache is [pages, page, nkv, d] (addressed as [slot, nkv, d]); v_cache is [pages, nkv, d, page].
template <typename T>
__global__ void rope_store_kernel(T* __restrict__ qkv, const int32_t* __restrict__ pos,
                                  const float* __restrict__ inv_freq, T* __restrict__ k_cache, T* __restrict__ v_cache,
                                  const int32_t* __restrict__ slots, int nq, int nkv, int d, int rot, int write_kv,
                                  int bs, const float* __restrict__ bias, int vec8) {
    __shared__ float cs_s[256], sn_s[256];          // one sine and cosine per rotated pair of the token
    const int t = blockIdx.x;
    const int half = rot / 2;
    const float p = (float)pos[t];
    const int slot = write_kv ? slots[t] : -1;
    T* row = qkv + (size_t)t * (nq + 2 * nkv) * d;
    const int nrot = nq + nkv;  // heads that are rotated: q then k
    for (int i = threadIdx.x; i < half; i += blockDim.x) sincosf(p * inv_freq[i], &sn_s[i], &cs_s[i]);
    __syncthreads();
    // rotated pairs; bfloat16 with eight pairs to a thread where the sizes allow 16-byte accesses
    if (vec8) {
        if constexpr (sizeof(T) == 2) {
            const int per_head = half >> 3;
            for (int idx = threadIdx.x; idx < nrot * per_head; idx += blockDim.x) {
                const int h = idx / per_head, i = (idx - h * per_head) * 8;
                bf16_t* hp = reinterpret_cast<bf16_t*>(row) + (size_t)h * d;
                const uint4 lo = *reinterpret_cast<const uint4*>(hp + i);
                const uint4 hi = *reinterpret_cast<const uint4*>(hp + i + half);
                const uint32_t lw[4] = {lo.x, lo.y, lo.z, lo.w}, hw[4] = {hi.x, hi.y, hi.z, hi.w};
                uint32_t o1[4], o2[4];
#pragma unroll
                for (int k = 0; k < 4; ++k) {
                    float a0 = __uint_as_float(lw[k] << 16), a1 = __uint_as_float(lw[k] & 0xffff0000u);
                    float b0 = __uint_as_float(hw[k] << 16), b1 = __uint_as_float(hw[k] & 0xffff0000u);
                    if (bias) {
                        a0 += bias[h * d + i + 2 * k], a1 += bias[h * d + i + 2 * k + 1];
                        b0 += bias[h * d + i + half + 2 * k], b1 += bias[h * d + i + half + 2 * k + 1];
                    }
                    const float c0 = cs_s[i + 2 * k], c1 = cs_s[i + 2 * k + 1];
                    const float s0 = sn_s[i + 2 * k], s1 = sn_s[i + 2 * k + 1];
                    o1[k] = (uint32_t)tl_f2bf_bits(a0 * c0 - b0 * s0) | ((uint32_t)tl_f2bf_bits(a1 * c1 - b1 * s1) << 16);
                    o2[k] = (uint32_t)tl_f2bf_bits(b0 * c0 + a0 * s0) | ((uint32_t)tl_f2bf_bits(b1 * c1 + a1 * s1) << 16);
                }
                bf16_t* dst = hp;
                if (h >= nq) {
                    if (slot < 0) continue;
                    dst = reinterpret_cast<bf16_t*>(k_cache) + ((size_t)slot * nkv + (h - nq)) * d;
                }
                *reinterpret_cast<uint4*>(dst + i) = make_uint4(o1[0], o1[1], o1[2], o1[3]);
                *reinterpret_cast<uint4*>(dst + i + half) = make_uint4(o2[0], o2[1], o2[2], o2[3]);
            }
        }
    } else
    for (int idx = threadIdx.x; idx < nrot * half; idx += blockDim.x) {
        const int h = idx / half, i = idx - h * half;
        const float sn = sn_s[i], cs = cs_s[i];
        T* hp = row + (size_t)h * d;
        float a = tl_to_float(hp[i]), b = tl_to_float(hp[i + half]);
        if (bias) {
            a += bias[h * d + i];
            b += bias[h * d + i + half];
        }
        const T o1 = tl_from_float<T>(a * cs - b * sn);
        const T o2 = tl_from_float<T>(b * cs + a * sn);
        if (h < nq) {
            hp[i] = o1;
            hp[i + half] = o2;
        } else if (slot >= 0) {
            T* kp = k_cache + ((size_t)slot * nkv + (h - nq)) * d;
            kp[i] = o1;
            kp[i + half] = o2;
        }
    }
    // dims beyond the rotated part pass through: query dims only change when a bias is owed
    const int tail = d - rot;
    if (bias) {
        for (int idx = threadIdx.x; idx < nq * tail; idx += blockDim.x) {
            const int h = idx / tail, i = rot + (idx - h * tail);
            row[(size_t)h * d + i] = tl_from_float<T>(tl_to_float(row[(size_t)h * d + i]) + bias[h * d + i]);
        }
    }
    if (slot < 0) return;
    for (int idx = threadIdx.x; idx < nkv * tail; idx += blockDim.x) {
        const int h = idx / tail, i = rot + (idx - h * tail);
        const T v = row[(size_t)(nq + h) * d + i];
        k_cache[((size_t)slot * nkv + h) * d + i] = bias ? tl_from_float<T>(tl_to_float(v) + bias[(nq + h) * d + i]) : v;
    }
    // values
    const T* vrow = row + (size_t)(nq + nkv) * d;
    const float* vbias = bias ? bias + (size_t)(nq + nkv) * d : nullptr;
    const int page = slot / bs, off = slot - page * bs;
    T* vdst = v_cache + (size_t)page * nkv * d * bs + off;
    for (int idx = threadIdx.x; idx < nkv * d; idx += blockDim.x)
        vdst[(size_t)idx * bs] = vbias ? tl_from_float<T>(tl_to_float(vrow[idx]) + vbias[idx]) : vrow[idx];
}

extern "C" int tl_rope_store(void* qkv, int dtype, const int32_t* pos, const float* inv_freq, void* k_cache,
                             void* v_cache, const int32_t* slots, int T, int nq, int nkv, int d, int rot,
                             int write_kv, int bs, const float* bias, hipStream_t stream) {
    TL_CHECK_ARG(T >= 0 && nq > 0 && nkv >= 0 && d > 0, "tl_rope_store: bad sizes T=%d nq=%d nkv=%d d=%d", T, nq, nkv, d);
    TL_CHECK_ARG(rot >= 0 && rot <= d && rot % 2 == 0, "tl_rope_store: rotary width %d must be even and <= head size %d", rot, d);
    TL_CHECK_ARG(rot <= 512, "tl_rope_store: rotary width %d is above the supported 512", rot);
    TL_CHECK_ARG(!write_kv || (k_cache && v_cache && slots && bs > 0), "tl_rope_store: cache write asked for without a cache");
    if (T == 0) return 0;
    dim3 grid(T), block(256);
    // 16-byte accesses: every head and both halves of the rotated part start at a multiple of 8 values
    const int vec8 = dtype == TL_BF16 && d % 8 == 0 && rot % 16 == 0 && rot > 0 && ((uintptr_t)qkv % 16) == 0 &&
                     (!write_kv || ((uintptr_t)k_cache % 16) == 0);
    if (dtype == TL_F32)
        hipLaunchKernelGGL(rope_store_kernel<float>, grid, block, 0, stream, (float*)qkv, pos, inv_freq,
                           (float*)k_cache, (float*)v_cache, slots, nq, nkv, d, rot, write_kv, bs, bias, 0);
    else if (dtype == TL_BF16)
        hipLaunchKernelGGL(rope_store_kernel<bf16_t>, grid, block, 0, stream, (bf16_t*)qkv, pos, inv_freq,
                           (bf16_t*)k_cache, (bf16_t*)v_cache, slots, nq, nkv, d, rot, write_kv, bs, bias, vec8);
    else
        return tl_fail("tl_rope_store: unknown dtype %d", dtype);
    TL_CHECK_LAUNCH("tl_rope_store");
    return 0;
}

// ---- SiLU(gate) * up ------------------------------------------------------------------------
// gu: [T, 2 I] with the gate in the first I columns and the up projection in the last I.
template <typename T>
__global__ void silu_mul_kernel(const T* __restrict__ gu, T* __restrict__ out, int I) {
    const int t = blockIdx.y;
    const int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= I) return;
    const T* row = gu + (size_t)t * 2 * I;
    const float g = tl_to_float(row[i]), u = tl_to_float(row[I + i]);
    out[(size_t)t * I + i] = tl_from_float<T>(g / (1.0f + expf(-g)) * u);
}

// bfloat16 with I a multiple of 8: 16 bytes of gate and of up per thread
__global__ void silu_mul_bf16x8_kernel(const bf16_t* __restrict__ gu, bf16_t* __restrict__ out, int I) {
    const int t = blockIdx.y;
    const int i8 = blockIdx.x * blockDim.x + threadIdx.x;
    if (i8 * 8 >= I) return;
    const bf16_t* row = gu + (size_t)t * 2 * I;
    const uint4 gv = *reinterpret_cast<const uint4*>(row + i8 * 8);
    const uint4 uv = *reinterpret_cast<const uint4*>(row + I + i8 * 8);
    const uint32_t gw[4] = {gv.x, gv.y, gv.z, gv.w}, uw[4] = {uv.x, uv.y, uv.z, uv.w};
    uint32_t ow[4];
#pragma unroll
    for (int k = 0; k < 4; ++k) {
        const float g0 = __uint_as_float(gw[k] << 16), g1 = __uint_as_float(gw[k] & 0xffff0000u);
        const float u0 = __uint_as_float(uw[k] << 16), u1 = __uint_as_float(uw[k] & 0xffff0000u);
        const float o0 = g0 / (1.0f + expf(-g0)) * u0, o1 = g1 / (1.0f + expf(-g1)) * u1;
        ow[k] = (uint32_t)tl_f2bf_bits(o0) | ((uint32_t)tl_f2bf_bits(o1) << 16);
    }
    *reinterpret_cast<uint4*>(out + (size_t)t * I + i8 * 8) = make_uint4(ow[0], ow[1], ow[2], ow[3]);
}

extern "C" int tl_silu_mul(const void* gu, void* out, int dtype, int T, int I, hipStream_t stream) {
    TL_CHECK_ARG(T >= 0 && I > 0, "tl_silu_mul: bad sizes T=%d I=%d", T, I);
    TL_CHECK_ARG(T <= 65535 * 64, "tl_silu_mul: too many rows %d", T);
    if (T == 0) return 0;
    // grid.y is limited to 65535: rows beyond that are covered by repeated launches.
    for (int t0 = 0; t0 < T; t0 += 65535) {
        const int tn = (T - t0 < 65535) ? T - t0 : 65535;
        dim3 grid(tl_ceil_div(I, 256), tn), block(256);
        if (dtype == TL_BF16 && I % 8 == 0 && ((uintptr_t)gu % 16) == 0 && ((uintptr_t)out % 16) == 0) {
            hipLaunchKernelGGL(silu_mul_bf16x8_kernel, dim3(tl_ceil_div(I / 8, 256), tn), block, 0, stream,
                               (const bf16_t*)gu + (size_t)t0 * 2 * I, (bf16_t*)out + (size_t)t0 * I, I);
            continue;
        }
        if (dtype == TL_F32)
            hipLaunchKernelGGL(silu_mul_kernel<float>, grid, block, 0, stream, (const float*)gu + (size_t)t0 * 2 * I,
                               (float*)out + (size_t)t0 * I, I);
        else if (dtype == TL_BF16)
            hipLaunchKernelGGL(silu_mul_kernel<bf16_t>, grid, block, 0, stream, (const bf16_t*)gu + (size_t)t0 * 2 * I,
                               (bf16_t*)out + (size_t)t0 * I, I);
        else
            return tl_fail("tl_silu_mul: unknown dtype %d", dtype);
    }
    TL_CHECK_LAUNCH("tl_silu_mul");
    return 0;
}
