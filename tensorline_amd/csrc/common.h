// Shared device helpers for the gfx950 kernels: storage types, wave and block reductions,
// error reporting of the C entry points.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#define TL_WAVE 64

// ---- storage types -------------------------------------------------------------------------
// bfloat16 is handled as raw 16 bits; conversion is a shift one way and round-to-nearest-even
// the other.  All arithmetic is done in float.
struct bf16_t {
    uint16_t bits;
};

__device__ __forceinline__ float tl_to_float(float v) { return v; }
__device__ __forceinline__ float tl_to_float(bf16_t v) { return __uint_as_float(((uint32_t)v.bits) << 16); }

__device__ __forceinline__ uint16_t tl_f2bf_bits(float f) {
    uint32_t u = __float_as_uint(f);
    if ((u & 0x7fffffffu) > 0x7f800000u) return (uint16_t)((u >> 16) | 0x0040u);  // quiet NaN
    u += 0x7fffu + ((u >> 16) & 1u);
    return (uint16_t)(u >> 16);
}

// 16 bytes that are read once and not again soon (the weights of a decode step's products): a
// non-temporal load.  Such data then does not displace what the caches hold for reuse, and the long
// products of a decode step stream 5 to 10% faster (lm_head of a 7B model at 8 rows: 195 -> 176 us,
// 6.2 TB/s).  Decode attention gains nothing from it for its keys and values (batch 64) or loses
// (batch 8: 16.4 -> 17.6 us per layer) and reads them with plain loads.
typedef unsigned tl_u32x4 __attribute__((ext_vector_type(4)));
__device__ __forceinline__ uint4 tl_load_stream(const uint4* p) {
    return __builtin_bit_cast(uint4, __builtin_nontemporal_load(reinterpret_cast<const tl_u32x4*>(p)));
}

template <typename T> __device__ __forceinline__ T tl_from_float(float v);
template <> __device__ __forceinline__ float tl_from_float<float>(float v) { return v; }
template <> __device__ __forceinline__ bf16_t tl_from_float<bf16_t>(float v) {
    bf16_t r;
    r.bits = tl_f2bf_bits(v);
    return r;
}

// ---- reductions ----------------------------------------------------------------------------
__device__ __forceinline__ float tl_wave_sum(float v) {
#pragma unroll
    for (int off = TL_WAVE / 2; off > 0; off >>= 1) v += __shfl_xor(v, off, TL_WAVE);
    return v;
}

__device__ __forceinline__ float tl_wave_max(float v) {
#pragma unroll
    for (int off = TL_WAVE / 2; off > 0; off >>= 1) v = fmaxf(v, __shfl_xor(v, off, TL_WAVE));
    return v;
}

// Block-wide reductions for blocks of up to 1024 threads (16 waves).  `scratch` is LDS with room
// for 16 floats.  The value is returned to every thread; the combination order is fixed, so the
// result does not depend on timing.  Both end with a barrier, so `scratch` can be reused at once.
__device__ __forceinline__ float tl_block_sum(float v, float* scratch) {
    const int lane = threadIdx.x & (TL_WAVE - 1), wave = threadIdx.x / TL_WAVE;
    const int nwaves = (blockDim.x + TL_WAVE - 1) / TL_WAVE;
    v = tl_wave_sum(v);
    if (lane == 0) scratch[wave] = v;
    __syncthreads();
    float r = 0.f;
    for (int w = 0; w < nwaves; ++w) r += scratch[w];
    __syncthreads();
    return r;
}

__device__ __forceinline__ float tl_block_max(float v, float* scratch) {
    const int lane = threadIdx.x & (TL_WAVE - 1), wave = threadIdx.x / TL_WAVE;
    const int nwaves = (blockDim.x + TL_WAVE - 1) / TL_WAVE;
    v = tl_wave_max(v);
    if (lane == 0) scratch[wave] = v;
    __syncthreads();
    float r = -INFINITY;
    for (int w = 0; w < nwaves; ++w) r = fmaxf(r, scratch[w]);
    __syncthreads();
    return r;
}

// What a matrix product does for the RMS norms around it (gemm_skinny.hip, gemm_rows64.hip);
// bfloat16 activations.  Passed by the caller as a pointer (null: nothing).
struct TlNormArgs {
    // owed normalisation of A's rows (null: none): ss_in [ss_n, ss_ld] holds ss_n partial sums per
    // row, row m in column m (a wave reads four partials of all rows from one stretch of memory)
    const float* ss_in;
    int ss_ld, ss_n;
    float dim, eps;            // result rows are scaled by 1/sqrt(sum / dim + eps)
    // residual add and next norm's input (MODE_PLAIN; null: none)
    float* resid;              // [M, resid_ld] float, updated in place
    int resid_ld;
    const float* next_weight;  // [N]
    bf16_t* a_out;             // [M, a_ld] = resid * next_weight
    int a_ld;
    float* ss_out;             // [tiles, ss_out_ld]: row `tile` gets the tile's sums of resid^2, one per row
    int ss_out_ld;
};

// ---- host side -----------------------------------------------------------------------------
// Every C entry point returns 0 on success.  On failure it returns a non-zero code and leaves a
// message that tl_last_error() hands out; nothing is launched in that case.
int tl_fail(const char* fmt, ...);

#define TL_CHECK_ARG(cond, ...)                  \
    do {                                         \
        if (!(cond)) return tl_fail(__VA_ARGS__); \
    } while (0)

#define TL_CHECK_LAUNCH(name)                                                              \
    do {                                                                                   \
        hipError_t e__ = hipGetLastError();                                                \
        if (e__ != hipSuccess) return tl_fail("%s: launch failed: %s", name, hipGetErrorString(e__)); \
    } while (0)

enum TlDtype { TL_F32 = 0, TL_BF16 = 1 };

static inline int tl_ceil_div(int a, int b) { return (a + b - 1) / b; }
