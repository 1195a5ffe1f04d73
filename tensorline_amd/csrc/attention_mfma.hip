// Causal grouped-query attention over the paged cache on the matrix cores (bfloat16, gfx950),
// for prompt portions and decoded tokens alike, with the key range optionally split over several
// waves (split-KV) and a second kernel that merges the splits.
//
// Work of one wave: NT tiles of 16 "columns" of one (sequence, key/value head).  A column is a
// (query token, query head of the group) pair; columns are numbered token-major, so a decoded
// token with a group of 7 fills 7 of the 16 columns of one tile and a prompt portion fills whole
// tiles.  The wave walks its share of the keys in blocks of 32 and keeps, per column, the running
// maximum, the running sum and the output accumulator in float (online softmax; reference:
// tensorline/paged_attn.py:25-58).  In the first kernel (decoded tokens, key splits) waves never
// talk to each other: no LDS, no barriers.  The second (attn_tile_kernel, steps with prompt
// portions) shares tiles of keys and values among the eight waves of a work-group through LDS.
//
// Matrix-core mapping (v_mfma_f32_16x16x32_bf16, D = A*B, lane l: c = l % 16, g = l / 16):
//   scores^T [keys x columns] = K [keys x d] * Q^T [d x columns]
//       A = K: lane holds 8 dims of key row c;  B = Q^T: lane holds the same 8 dims of column c.
//       The accumulator register i of lane l is (key row 4g + i, column c).
//   out^T [d x columns] += V^T [d x keys] * P^T [keys x columns]
//       A = V^T: lane holds 8 keys of dim c;     B = P^T: lane holds the same 8 keys of column c.
// Which key a key row stands for is free.  The two score tiles of a 32-key block use rows
//   tile 0: row 4g + i  <->  key 8g + i          tile 1: row 4g + i  <->  key 8g + 4 + i
// so that after both tiles lane (c, g) holds exactly the probabilities of keys 8g .. 8g+7 of
// column c: the B fragment of the second product, with no exchange between lanes.  The matching A
// fragment, 8 consecutive keys of one dim, is one 16-byte load because the value cache is stored
// transposed within a page: [pages, nkv, d, page].  The key cache is [pages, page, nkv, d].
//
// Key blocks are aligned to absolute positions (block b holds keys 32b .. 32b+31), and so are the
// splits (split s holds blocks s*SB .. s*SB + SB - 1): which keys are summed together does not
// depend on the context length, on the launch's number of splits or on how the sequence was cut
// into steps.  A wave whose split holds none of its keys writes nothing; the merge kernel visits
// exactly the splits that hold keys of a token.
#include "common.h"

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float f32x4 __attribute__((ext_vector_type(4)));

__device__ __forceinline__ bf16x8 am_frag(uint4 v) { return __builtin_bit_cast(bf16x8, v); }

typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
typedef float f32x2 __attribute__((ext_vector_type(2)));

// two floats -> two bfloat16 (round to nearest even) in one register: v_cvt_pk_bf16_f32
__device__ __forceinline__ uint32_t am_pack2(float a, float b) {
    const f32x2 v = {a, b};
    return __builtin_bit_cast(uint32_t, __builtin_convertvector(v, bf16x2));
}

// max(a, b, c) of numbers that are not NaN as the one instruction it is (fmaxf first quiets each
// operand with an instruction of its own)
__device__ __forceinline__ float am_max3(float a, float b, float c) {
    float r;
    asm("v_max3_f32 %0, %1, %2, %3" : "=v"(r) : "v"(a), "v"(b), "v"(c));
    return r;
}

// The maximum over the four lanes that hold one column (lanes c, c + 16, c + 32, c + 48), in all
// four: two swaps of 16- and 32-lane halves between registers instead of two trips through LDS.
typedef unsigned int am_u32x2 __attribute__((ext_vector_type(2)));
__device__ __forceinline__ float am_column_max(float v) {
    am_u32x2 sw = __builtin_amdgcn_permlane16_swap(__float_as_uint(v), __float_as_uint(v), false, false);
    v = am_max3(v, __uint_as_float(sw[0]), __uint_as_float(sw[1]));
    sw = __builtin_amdgcn_permlane32_swap(__float_as_uint(v), __float_as_uint(v), false, false);
    return am_max3(v, __uint_as_float(sw[0]), __uint_as_float(sw[1]));
}

#define AM_LOG2E 1.4426950408889634f
#define AM_LAZY 8.0f                 // how far a block's maximum may exceed the running one before it moves
#define AM_NO_COLUMN 0x7fffffff      // position of a lane without a column: never masks, never written

// One block of 32 keys for the NT column tiles of a wave: scores, online softmax, P*V.
// Scores and the running maximum are kept in the base-2 domain (score * scale * log2 e), so the
// exponential is one v_exp_f32; sums and accumulators are float.  Masking is skipped when every
// key of the block is visible to every column of the wave, the rescaling of the accumulator when
// no running maximum moved.
template <int DC, int NT>
__device__ __forceinline__ void am_block(const uint4* kf0, const uint4* kf1, const uint4* vf, const uint4 (*qf)[DC],
                                         const int* p_col, const int* lo_col, int kb, int g, float scale2,
                                         float* m_run, float* l_run, f32x4 (*acc)[DC * 2]) {
    constexpr int DB = DC * 2;
    const int key_base = kb + 8 * g;
#pragma unroll
    for (int j = 0; j < NT; ++j) {
        f32x4 st0 = f32x4{0.f, 0.f, 0.f, 0.f}, st1 = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int dc = 0; dc < DC; ++dc) {
            st0 = __builtin_amdgcn_mfma_f32_16x16x32_bf16(am_frag(kf0[dc]), am_frag(qf[j][dc]), st0, 0, 0, 0);
            st1 = __builtin_amdgcn_mfma_f32_16x16x32_bf16(am_frag(kf1[dc]), am_frag(qf[j][dc]), st1, 0, 0, 0);
        }
        float sv[8];
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            sv[i] = st0[i] * scale2;
            sv[4 + i] = st1[i] * scale2;
        }
        const bool edge = (kb + 31 > p_col[j]) || (kb < lo_col[j]);
        if (__any(edge)) {
#pragma unroll
            for (int i = 0; i < 8; ++i) {
                const int key = key_base + i;
                if (key > p_col[j] || key < lo_col[j]) sv[i] = -INFINITY;
            }
        }
        const float bmax = am_column_max(am_max3(am_max3(sv[0], sv[1], sv[2]), am_max3(sv[3], sv[4], sv[5]), am_max3(sv[6], sv[7], sv[7])));
        const float m_new = fmaxf(m_run[j], bmax);
        const float m_safe = (m_new == -INFINITY) ? 0.f : m_new;
        const bool moved = m_new > m_run[j];
        float pr[8], psum = 0.f;
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            pr[i] = __builtin_amdgcn_exp2f(sv[i] - m_safe);
            psum += pr[i];
        }
        uint4 pf;
        pf.x = am_pack2(pr[0], pr[1]);
        pf.y = am_pack2(pr[2], pr[3]);
        pf.z = am_pack2(pr[4], pr[5]);
        pf.w = am_pack2(pr[6], pr[7]);
        if (__any(moved)) {
            const float alpha = __builtin_amdgcn_exp2f(m_run[j] - m_safe);
            l_run[j] = l_run[j] * alpha + psum;
#pragma unroll
            for (int db = 0; db < DB; ++db) {
                f32x4 a = acc[j][db];
                a[0] *= alpha;
                a[1] *= alpha;
                a[2] *= alpha;
                a[3] *= alpha;
                acc[j][db] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(am_frag(vf[db]), am_frag(pf), a, 0, 0, 0);
            }
        } else {
            l_run[j] += psum;
#pragma unroll
            for (int db = 0; db < DB; ++db)
                acc[j][db] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(am_frag(vf[db]), am_frag(pf), acc[j][db], 0, 0, 0);
        }
        m_run[j] = m_new;
    }
}

// index of the page that holds key k: a shift for pages of a power of two of tokens
__device__ __forceinline__ int am_page_index(int k, int bs, int bs_shift) {
    return bs_shift >= 0 ? k >> bs_shift : k / bs;
}

template <int DC, int NT>
__global__ __launch_bounds__(256) void attn_mfma_kernel(
    const bf16_t* __restrict__ q, int q_stride, const bf16_t* __restrict__ kc, const bf16_t* __restrict__ vc,
    const int32_t* __restrict__ tables, int NB, const int32_t* __restrict__ q_start,
    const int32_t* __restrict__ ctx_start, bf16_t* __restrict__ out, int out_stride, float* __restrict__ ws_o,
    float* __restrict__ ws_ml, int nq, int nkv, int bs, int bs_shift, int window, float scale, int nsplit,
    int split_blocks, const int32_t* __restrict__ seq_list, int skip_single) {
    constexpr int D = DC * 32;
    constexpr int DB = D / 16;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int c = lane & 15, g = lane >> 4;
    // With a list the grid runs over the listed sequences only (one-token sequences of a step that
    // also holds prompt portions), and their partial results lie in the workspace by list place.
    const int s = seq_list ? seq_list[blockIdx.x] : (int)blockIdx.x, kvh = blockIdx.y;
    const int widx = blockIdx.z * (blockDim.x >> 6) + wave;    // one to four waves per work-group
    const int tg = widx / nsplit, sp = widx - tg * nsplit;
    const int G = nq / nkv;
    const float scale2 = scale * AM_LOG2E;
    const int r0 = q_start[s];
    const int n = q_start[s + 1] - r0;
    const int start = ctx_start[s];
    const int ncols = n * G;
    const int col0 = tg * NT * 16;
    if (col0 >= ncols) return;
    if (seq_list ? n != 1 : (skip_single && n == 1)) return;   // another launch of the step owns it
    const int ws_shift = seq_list ? (int)blockIdx.x - r0 : 0;
    const int32_t* table = tables + (size_t)s * NB;

    // ---- this lane's column of each tile ----
    uint4 qf[NT][DC];
    int p_col[NT], lo_col[NT], row_col[NT], head_col[NT];
    bool has_col[NT];
#pragma unroll
    for (int j = 0; j < NT; ++j) {
        const int col = col0 + j * 16 + c;
        const bool valid = col < ncols;
        const int tok = valid ? col / G : 0;
        const int gh = valid ? col - tok * G : 0;
        row_col[j] = r0 + tok;
        head_col[j] = kvh * G + gh;
        has_col[j] = valid;
        p_col[j] = valid ? start + tok : AM_NO_COLUMN;
        lo_col[j] = (valid && window > 0 && p_col[j] - window + 1 > 0) ? p_col[j] - window + 1 : 0;
        const bf16_t* qp = q + (size_t)row_col[j] * q_stride + (size_t)head_col[j] * D + g * 8;
#pragma unroll
        for (int dc = 0; dc < DC; ++dc)
            qf[j][dc] = valid ? *reinterpret_cast<const uint4*>(qp + dc * 32) : make_uint4(0, 0, 0, 0);
    }

    // ---- key range of the wave, in blocks of 32, and this split's share ----
    const int last_col = ((col0 + NT * 16 < ncols) ? col0 + NT * 16 : ncols) - 1;
    const int khi = start + last_col / G;                      // last key any column of the wave sees
    int klo = 0;
    if (window > 0) {
        klo = start + col0 / G - window + 1;
        if (klo < 0) klo = 0;
    }
    const int b_lo = klo >> 5, b_hi = khi >> 5;
    int bb = b_lo, be = b_hi + 1;
    if (nsplit > 1) {
        if (sp * split_blocks > bb) bb = sp * split_blocks;
        if ((sp + 1) * split_blocks < be) be = (sp + 1) * split_blocks;
        if (bb >= be) return;
    }

    float m_run[NT], l_run[NT];
    f32x4 acc[NT][DB];
#pragma unroll
    for (int j = 0; j < NT; ++j) {
        m_run[j] = -INFINITY;
        l_run[j] = 0.f;
#pragma unroll
        for (int db = 0; db < DB; ++db) acc[j][db] = f32x4{0.f, 0.f, 0.f, 0.f};
    }

    // The page ids of the wave's keys, one per lane, when they are at most 64 (a split of a decode
    // step always is): a block's addresses then come from a lane exchange instead of a load from
    // memory that the loads of keys and values would have to wait for.
    const int page_lo = am_page_index(bb << 5, bs, bs_shift);
    const int last_key = ((be << 5) - 1 < khi) ? (be << 5) - 1 : khi;
    const int npages = am_page_index(last_key, bs, bs_shift) - page_lo + 1;
    const bool pages_in_lanes = npages <= 64;
    const int my_page = pages_in_lanes ? table[page_lo + (lane < npages ? lane : npages - 1)] : 0;
    const int krow_in_block0 = 8 * (c >> 2) + (c & 3);         // key of row c in tile 0; tile 1: + 4
    // One block ahead: while block b is multiplied, the fragments of block b + 1 are in flight
    // (past the last block the same block is requested again and not used).
    uint4 kf0[DC], kf1[DC], vf[DB], kn0[DC], kn1[DC], vn[DB];
#define AM_LOAD_BLOCK(B, K0, K1, V)                                                                          \
    {                                                                                                        \
        const int kb_ = (B) << 5;                                                                            \
        /* keys past khi are masked for every column; their addresses are clamped to stay on pages the */    \
        /* sequence owns */                                                                                  \
        int k0_ = kb_ + krow_in_block0, k1_ = k0_ + 4;                                                       \
        if (k0_ > khi) k0_ = khi;                                                                            \
        if (k1_ > khi) k1_ = khi;                                                                            \
        const int i0_ = am_page_index(k0_, bs, bs_shift), i1_ = am_page_index(k1_, bs, bs_shift);            \
        const int p0_ = pages_in_lanes ? __shfl(my_page, i0_ - page_lo, TL_WAVE) : table[i0_];               \
        const int p1_ = pages_in_lanes ? __shfl(my_page, i1_ - page_lo, TL_WAVE) : table[i1_];               \
        const bf16_t* kp0_ = kc + ((size_t)(p0_ * bs + k0_ - i0_ * bs) * nkv + kvh) * D + g * 8;             \
        const bf16_t* kp1_ = kc + ((size_t)(p1_ * bs + k1_ - i1_ * bs) * nkv + kvh) * D + g * 8;             \
        _Pragma("unroll") for (int dc = 0; dc < DC; ++dc) {                                                  \
            K0[dc] = *reinterpret_cast<const uint4*>(kp0_ + dc * 32);                                        \
            K1[dc] = *reinterpret_cast<const uint4*>(kp1_ + dc * 32);                                        \
        }                                                                                                    \
        int vk_ = kb_ + 8 * g;                                                                               \
        if (vk_ > khi) vk_ = khi & ~7;                                                                       \
        const int iv_ = am_page_index(vk_, bs, bs_shift);                                                    \
        const int pv_ = pages_in_lanes ? __shfl(my_page, iv_ - page_lo, TL_WAVE) : table[iv_];               \
        const bf16_t* vp_ = vc + (((size_t)pv_ * nkv + kvh) * D + c) * bs + vk_ - iv_ * bs;                  \
        _Pragma("unroll") for (int db = 0; db < DB; ++db)                                                    \
            V[db] = *reinterpret_cast<const uint4*>(vp_ + (size_t)db * 16 * bs);                             \
    }
    AM_LOAD_BLOCK(bb, kf0, kf1, vf)
    for (int b = bb; b < be; ++b) {
        const int kb = b << 5;
        const int b_next = (b + 1 < be) ? b + 1 : b;
        AM_LOAD_BLOCK(b_next, kn0, kn1, vn)

        am_block<DC, NT>(kf0, kf1, vf, qf, p_col, lo_col, kb, g, scale2, m_run, l_run, acc);
#pragma unroll
        for (int dc = 0; dc < DC; ++dc) {
            kf0[dc] = kn0[dc];
            kf1[dc] = kn1[dc];
        }
#pragma unroll
        for (int db = 0; db < DB; ++db) vf[db] = vn[db];
    }

#undef AM_LOAD_BLOCK
    // ---- write: accumulator register i of lane (c, g) is (dim db*16 + 4g + i, column c) ----
#pragma unroll
    for (int j = 0; j < NT; ++j) {
        if (!has_col[j]) continue;
        float l_tot = l_run[j];
        l_tot += __shfl_xor(l_tot, 16, TL_WAVE);
        l_tot += __shfl_xor(l_tot, 32, TL_WAVE);
        if (nsplit == 1) {
            const float inv = 1.0f / l_tot;
            bf16_t* op = out + (size_t)row_col[j] * out_stride + (size_t)head_col[j] * D + 4 * g;
#pragma unroll
            for (int db = 0; db < DB; ++db) {
                uint2 w;
                w.x = am_pack2(acc[j][db][0] * inv, acc[j][db][1] * inv);
                w.y = am_pack2(acc[j][db][2] * inv, acc[j][db][3] * inv);
                *reinterpret_cast<uint2*>(op + db * 16) = w;
            }
        } else {
            const size_t part = ((size_t)(row_col[j] + ws_shift) * nq + head_col[j]) * nsplit + sp;
            float* wp = ws_o + part * D + 4 * g;
#pragma unroll
            for (int db = 0; db < DB; ++db)
                *reinterpret_cast<f32x4*>(wp + db * 16) = acc[j][db];
            if (g == 0) {
                ws_ml[part * 2] = m_run[j];
                ws_ml[part * 2 + 1] = l_tot;
            }
        }
    }
}

// The same block of 32 keys (half `half` of a 64-key tile) with the fragments taken from LDS where
// they are used.  kt is the tile's 64 key rows of 4 DC units in matrix-core order (row c of score
// tile r, which is key 32 (r / 2) + 8 (c / 4) + 4 (r % 2) + c % 4 of the tile, in LDS row 16 r + c), vt
// its 32 DC dim rows of 8 units (8 keys each).  Rows are not padded: unit u of a row lies at u ^ kx
// (keys) or u ^ vx (values), kx and vx depending on the row so that the 16 lanes of a read, which
// take the same unit of 16 consecutive rows, are spread over all banks (at_k_swizzle, at_v_swizzle).
// All score tiles first, then the softmax of each column tile, then all P*V products, so that key
// fragments are dead before value fragments are read: few registers are live at once.
template <int DC, int NT>
__device__ __forceinline__ void am_block_lds(const uint4* kt, const uint4* vt, int kx, int vx, int half,
                                             const uint4 (*qf)[DC], const int* p_col, const int* lo_col, int kb, int c,
                                             int g, float scale2, float* m_run, float* l_run, f32x4 (*acc)[DC * 2]) {
    constexpr int DB = DC * 2;
    constexpr int UPK = DC * 4;
    const int key_base = kb + 8 * g;
    f32x4 st0[NT], st1[NT];
#pragma unroll
    for (int j = 0; j < NT; ++j) st0[j] = st1[j] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int dc = 0; dc < DC; ++dc) {
        const uint4 k0 = kt[(32 * half + c) * UPK + ((dc * 4 + g) ^ kx)];
        const uint4 k1 = kt[(32 * half + 16 + c) * UPK + ((dc * 4 + g) ^ kx)];
#pragma unroll
        for (int j = 0; j < NT; ++j) {
            st0[j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(am_frag(k0), am_frag(qf[j][dc]), st0[j], 0, 0, 0);
            st1[j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(am_frag(k1), am_frag(qf[j][dc]), st1[j], 0, 0, 0);
        }
    }
    uint4 pf[NT];
#pragma unroll
    for (int j = 0; j < NT; ++j) {
        float sv[8];
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            sv[i] = st0[j][i] * scale2;
            sv[4 + i] = st1[j][i] * scale2;
        }
        const bool edge = (kb + 31 > p_col[j]) || (kb < lo_col[j]);
        if (__any(edge)) {
#pragma unroll
            for (int i = 0; i < 8; ++i) {
                const int key = key_base + i;
                if (key > p_col[j] || key < lo_col[j]) sv[i] = -INFINITY;
            }
        }
        const float bmax = am_column_max(am_max3(am_max3(sv[0], sv[1], sv[2]), am_max3(sv[3], sv[4], sv[5]), am_max3(sv[6], sv[7], sv[7])));
        // The running maximum follows the true one lazily: it moves only when the block's maximum
        // exceeds it by more than AM_LAZY (in the base-2 domain), so probabilities stay below
        // 2^AM_LAZY and the accumulator is rescaled in few blocks instead of most.  Sums and
        // accumulators stay relative to the same running maximum, so the result is the same.
        const bool moved = bmax > m_run[j] + AM_LAZY;         // also the first keys: -inf + AM_LAZY is -inf
        const float m_new = moved ? bmax : m_run[j];
        const float m_safe = (m_new == -INFINITY) ? 0.f : m_new;
        float pr[8], psum = 0.f;
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            pr[i] = __builtin_amdgcn_exp2f(sv[i] - m_safe);
            psum += pr[i];
        }
        pf[j].x = am_pack2(pr[0], pr[1]);
        pf[j].y = am_pack2(pr[2], pr[3]);
        pf[j].z = am_pack2(pr[4], pr[5]);
        pf[j].w = am_pack2(pr[6], pr[7]);
        if (__any(moved)) {
            const float alpha = __builtin_amdgcn_exp2f(m_run[j] - m_safe);
            l_run[j] = l_run[j] * alpha + psum;
#pragma unroll
            for (int db = 0; db < DB; ++db) {
                acc[j][db][0] *= alpha;
                acc[j][db][1] *= alpha;
                acc[j][db][2] *= alpha;
                acc[j][db][3] *= alpha;
            }
        } else {
            l_run[j] += psum;
        }
        m_run[j] = m_new;
    }
#pragma unroll
    for (int db = 0; db < DB; ++db) {
        const uint4 v = vt[(db * 16 + c) * 8 + ((4 * half + g) ^ vx)];
#pragma unroll
        for (int j = 0; j < NT; ++j)
            acc[j][db] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(am_frag(v), am_frag(pf[j]), acc[j][db], 0, 0, 0);
    }
}

// A whole tile of 64 keys for one column tile of a wave, all of whose keys some column of the wave
// sees: the same arithmetic as two calls of am_block_lds with one softmax step instead of two (one
// maximum, one decision to move the running maximum), the scale folded into the exponent's
// argument, and the LDS reads ahead of the products that use them: the key fragments of two
// 32-wide slices of the head are in flight while the products of the slice before run, the value
// fragments of the first 32 keys while the softmax is computed.
template <int DC>
__device__ __forceinline__ void am_tile_lds(const uint4* kt, const uint4* vt, int kx, int vx, const uint4* qf,
                                            int p_col, int lo_col, int kb, int c, int g, float scale2, float& m_run,
                                            float& l_run, f32x4* acc) {
    constexpr int DB = DC * 2;
    constexpr int UPK = DC * 4;
    f32x4 st[4];
#pragma unroll
    for (int r = 0; r < 4; ++r) st[r] = f32x4{0.f, 0.f, 0.f, 0.f};
    {
        // a ring of four fragments: each is replaced, right behind the product that used it, by
        // the one needed four products later
        uint4 kf[4];
#pragma unroll
        for (int r = 0; r < 4; ++r) kf[r] = kt[(16 * r + c) * UPK + (g ^ kx)];
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int dc = 0; dc < DC; ++dc) {
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                st[r] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(am_frag(kf[r]), am_frag(qf[dc]), st[r], 0, 0, 0);
                if (dc + 1 < DC) kf[r] = kt[(16 * r + c) * UPK + (((dc + 1) * 4 + g) ^ kx)];
                __builtin_amdgcn_sched_barrier(0);
            }
        }
    }
    // The value fragments in the order of their products: those of the first 32 keys for every 16
    // dims, then those of the last 32.  The first four are on their way during the softmax.
    uint4 vf[4];
#define AM_VFRAG(I) vt[((((I) % DB) * 16 + c) * 8) + ((4 * ((I) / DB) + g) ^ vx)]
#pragma unroll
    for (int i = 0; i < 4; ++i) vf[i] = AM_VFRAG(i);
    // A vector instruction may read what a matrix-core instruction wrote only a number of cycles
    // later, and the compiler puts that wait before instructions it knows.  The first readers of
    // the scores below are written as assembly (am_max3), which it does not look into: so the first
    // read is this one, of a register of each of the four last products, and nothing that follows
    // may be moved ahead of it.
    {
        const float first_read = fmaxf(fmaxf(st[0][3], st[1][3]), fmaxf(st[2][3], st[3][3]));
        asm volatile("" ::"v"(first_read));
    }
    __builtin_amdgcn_sched_barrier(0);
    // lane (c, g) holds, of column c, keys kb + 32 h + 8 g + 4 r + i in st[2 h + r][i]
    float sv[16];
#pragma unroll
    for (int r = 0; r < 4; ++r)
#pragma unroll
        for (int i = 0; i < 4; ++i) sv[4 * r + i] = st[r][i];
    const bool edge = (kb + 63 > p_col) || (kb < lo_col);
    if (__any(edge)) {
#pragma unroll
        for (int h = 0; h < 2; ++h)
#pragma unroll
            for (int i = 0; i < 8; ++i) {
                const int key = kb + 32 * h + 8 * g + i;
                if (key > p_col || key < lo_col) sv[8 * h + i] = -INFINITY;
            }
    }
    float bmax = am_max3(am_max3(am_max3(sv[0], sv[1], sv[2]), am_max3(sv[3], sv[4], sv[5]), sv[6]),
                         am_max3(am_max3(sv[7], sv[8], sv[9]), am_max3(sv[10], sv[11], sv[12]), sv[13]), am_max3(sv[14], sv[15], sv[15]));
    bmax = am_column_max(bmax);
    bmax *= scale2;                                          // the scale is positive: the order is the same
    const bool moved = bmax > m_run + AM_LAZY;               // also the first keys: -inf + AM_LAZY is -inf
    const float m_new = moved ? bmax : m_run;
    const float neg_m = (m_new == -INFINITY) ? 0.f : -m_new;
    float pr[16];
#pragma unroll
    for (int i = 0; i < 16; ++i) pr[i] = __builtin_amdgcn_exp2f(__builtin_fmaf(sv[i], scale2, neg_m));
    const float psum = (((pr[0] + pr[1]) + (pr[2] + pr[3])) + ((pr[4] + pr[5]) + (pr[6] + pr[7]))) +
                       (((pr[8] + pr[9]) + (pr[10] + pr[11])) + ((pr[12] + pr[13]) + (pr[14] + pr[15])));
    uint4 pf[2];
#pragma unroll
    for (int h = 0; h < 2; ++h) {
        pf[h].x = am_pack2(pr[8 * h + 0], pr[8 * h + 1]);
        pf[h].y = am_pack2(pr[8 * h + 2], pr[8 * h + 3]);
        pf[h].z = am_pack2(pr[8 * h + 4], pr[8 * h + 5]);
        pf[h].w = am_pack2(pr[8 * h + 6], pr[8 * h + 7]);
    }
    if (__any(moved)) {
        const float alpha = __builtin_amdgcn_exp2f(m_run + neg_m);
        l_run = l_run * alpha + psum;
#pragma unroll
        for (int db = 0; db < DB; ++db) {
            acc[db][0] *= alpha;
            acc[db][1] *= alpha;
            acc[db][2] *= alpha;
            acc[db][3] *= alpha;
        }
    } else {
        l_run += psum;
    }
    m_run = m_new;
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int i = 0; i < 2 * DB; ++i) {
        acc[i % DB] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(am_frag(vf[i % 4]), am_frag(pf[i / DB]), acc[i % DB], 0, 0, 0);
        if (i + 4 < 2 * DB) vf[i % 4] = AM_VFRAG(i + 4);
        __builtin_amdgcn_sched_barrier(0);
    }
#undef AM_VFRAG
}

// The kernel for steps with prompt portions.  A work-group owns 128 consecutive columns of one
// (sequence, key/value head), 16 * NT per wave, and walks the keys together in tiles of 64.  A
// tile is brought into LDS once and every wave takes its MFMA fragments from there: keys and
// values are read from the cache once per 128 columns, and a wave holds no copy of them in
// registers, so two work-groups (sixteen waves) fit on a CU and some compute while others wait.
// The tile goes from memory straight into LDS (global_load_lds_dwordx4: each lane brings 16 bytes,
// a wave's 64 lanes fill 1 KB of consecutive LDS), so it passes through no registers either: which
// 16 bytes a lane asks for is chosen so that the consecutive LDS image is the swizzled layout the
// fragment reads expect.  Two LDS buffers: the loads of tile t + 1 are in flight while tile t is
// multiplied; every wave waits for its own loads before the one barrier of the iteration.  The
// sequence's page ids are copied to LDS first, so a tile's addresses depend on no load from
// memory.  Pages must hold a power of two of tokens (at least 8; 2^bs_shift): an 8-key run of V^T
// then lies in one page and a page id is a shift away.  No key split: a step with prompt portions
// has columns enough.
#define AT_KEYS 64
#define AT_CUS 256                   // compute units of the GPU
#define AT_NT 1                      // column tiles per wave; 8 / AT_NT waves in a work-group
// The key of a tile that LDS row `row` holds (see am_block_lds); key k lies in row
// (k & 32) + ((k & 4) << 2) + ((k & 24) >> 1) + (k & 3).
__device__ __forceinline__ int at_lds_key(int row) {
    return (row & 35) + ((row & 16) >> 2) + ((row & 12) << 1);
}
// Where unit u of a row lies in it: u ^ swizzle(row).  A K row has UPK = 4, 8 or 16 units, so 16 /
// UPK rows span the 256 bytes over which the banks repeat; the swizzle steps once per such span.  A
// V^T row has 8 units.  Both depend only on the row modulo 16 (the lane's c in a fragment read).
template <int UPK>
__device__ __forceinline__ int at_k_swizzle(int row) { return ((row & 15) * UPK) >> 4; }
__device__ __forceinline__ int at_v_swizzle(int row) { return (row >> 1) & 7; }

// 16 bytes per lane from memory straight into LDS at lds_base + 16 * lane (lds_base is the same for
// the whole wave).  Written as assembly so that the compiler does not make every later LDS read wait
// for it: a load is waited for only where AT_LANDED says so.  M0 holds the LDS base for the
// instruction and is put back.
__device__ __forceinline__ void at_load_to_lds_at(const void* g, uint32_t lds_base) {
    uint32_t saved;
    asm volatile(
        "s_mov_b32 %0, m0\n\ts_mov_b32 m0, %1\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %2, off\n\ts_mov_b32 m0, %0"
        : "=&s"(saved)
        : "s"(lds_base), "v"(g)
        : "memory");
}
__device__ __forceinline__ void at_load_to_lds(const void* g, void* lds_base) {
    at_load_to_lds_at(g, (uint32_t)(uintptr_t)(__attribute__((address_space(3))) void*)lds_base);
}

// CH = 2 ("two chains"): a work-group of twice the waves, whose second half takes every other tile of
// the same columns, with tile buffers, running maximum, sum and accumulator of its own; at the end
// the halves are put together through LDS as two splits of the keys are.  For steps with at most one
// work-group per CU (a short portion behind a long context), where the longest walk sets the time and
// a lone work-group leaves part of its CU unused.  The chains share the barrier, so they pass a
// tile's phases together and gain less than two work-groups that drift apart would: 10 to 17%.
template <int DC, int NT, int WAVES, int CH>
__global__ __launch_bounds__(CH * WAVES * 64, 32 / WAVES) void attn_tile_kernel(
    const bf16_t* __restrict__ q, int q_stride, const bf16_t* __restrict__ kc, const bf16_t* __restrict__ vc,
    const int32_t* __restrict__ tables, int NB, const int32_t* __restrict__ q_start,
    const int32_t* __restrict__ ctx_start, bf16_t* __restrict__ out, int out_stride, int S, int nq, int nkv, int bs,
    int bs_shift, int window, float scale, int skip_single) {
    constexpr int THREADS = CH * WAVES * 64;
    constexpr int WCOLS = NT * 16;                       // columns of a wave; WAVES * WCOLS = 128 per work-group
    constexpr int D = DC * 32;
    constexpr int DB = D / 16;
    constexpr int UPK = D / 8;                // uint4 per key row; also the wave-loads of a K tile and of a V^T tile
    constexpr int TILE = AT_KEYS * UPK;       // uint4 of a K tile, and of a V^T tile (D rows of 8)
    extern __shared__ uint4 at_smem[];
    const int tid = threadIdx.x, lane = tid & 63;
    const int chain = CH > 1 ? __builtin_amdgcn_readfirstlane((tid >> 6) / WAVES) : 0;
    const int wave = (tid >> 6) - chain * WAVES;           // which 16 NT columns of the 128
    uint4* ks = at_smem + chain * 4 * TILE;                // [2][TILE], per chain
    uint4* vs = ks + 2 * TILE;                             // [2][TILE]
    // with two chains: the tiles' LDS addresses for the loads, the same in every lane of a wave and said so,
    // so that they and what is added to them stay in scalar registers
    const uint32_t ks_lds = CH > 1 ? (uint32_t)__builtin_amdgcn_readfirstlane(
        (int)(uint32_t)(uintptr_t)(__attribute__((address_space(3))) void*)ks) : 0u;
    const uint32_t vs_lds = ks_lds + 2 * TILE * 16;
    int* tab = reinterpret_cast<int*>(at_smem + CH * 4 * TILE);   // page ids of the sequence, as far as needed (NB ints)
    int* qst = tab + NB;                                   // q_start of the step (S + 1 ints)
    const int c = lane & 15, g = lane >> 4;
    const int kvh = blockIdx.x;                            // fastest: the heads of a group start together
    const int G = nq / nkv;
    const float scale2 = scale * AM_LOG2E;
    // Which (sequence, group of 128 columns) this work-group owns: the grid has one work-group per
    // group that exists (a step mixes a long prompt portion with many one-token sequences, and a
    // grid of sequences x most groups would be nearly all empty work-groups).  Within a sequence
    // the groups with the most keys (the last columns) come first.
    for (int i = tid; i <= S; i += THREADS) qst[i] = q_start[i];
    __syncthreads();
    int s = 0, flat = blockIdx.y, ngroups = 0;
    for (; s < S; ++s) {
        const int nn = qst[s + 1] - qst[s];
        ngroups = (skip_single && nn == 1) ? 0 : (nn * G + 127) / 128;   // one-token sequences: another launch's
        if (flat < ngroups) break;
        flat -= ngroups;
    }
    if (s >= S) return;                       // the whole work-group leaves: no barrier is missed
    const int r0 = qst[s];
    const int n = qst[s + 1] - r0;
    const int start = ctx_start[s];
    const int ncols = n * G;
    // Loader.  A K tile is 64 rows x UPK units of 16 bytes, a V^T tile D rows x 8 units (8 keys
    // each): UPK wave-loads of 64 consecutive units each, dealt round-robin to the waves.  For its
    // load number i a lane knows which key and unit (K) and which dim and first key (V^T) the LDS
    // place it fills holds.
    constexpr int NI = (UPK + WAVES - 1) / WAVES;
    const int wave_u = __builtin_amdgcn_readfirstlane(wave);
    int k_key[NI], v_key[NI];                  // K: the lane's key of the tile; V^T: the first key of its unit
    const char *k_base[NI], *v_base[NI];       // where that unit lies in slot 0 (K), in page 0 at offset 0 (V^T)
#pragma unroll
    for (int i = 0; i < NI; ++i) {
        int w = wave_u + i * WAVES;
        if (w >= UPK) w = UPK - 1;                           // not issued
        const int idx = w * 64 + lane;
        const int krow = idx / UPK, kpu = idx % UPK;
        k_key[i] = at_lds_key(krow);
        k_base[i] = reinterpret_cast<const char*>(kc + (size_t)kvh * D + (kpu ^ at_k_swizzle<UPK>(krow)) * 8);
        const int vrow = idx >> 3, vpu = idx & 7;
        v_key[i] = (vpu ^ at_v_swizzle(vrow)) * 8;
        v_base[i] = reinterpret_cast<const char*>(vc + ((size_t)kvh * D + vrow) * bs);
    }
    const uint32_t k_stride = (uint32_t)nkv * D * 2;         // bytes from a slot to the next
    const uint32_t v_stride = (uint32_t)nkv * D * bs * 2;    // bytes from a page to the next
    const int kx = at_k_swizzle<UPK>(c), vx = at_v_swizzle(c);
    // Which of its sequence's groups: the one with the most keys first.  The hardware places
    // work-group i + 256 on the CU of work-group i (256 CUs, two work-groups each), so when the
    // grid has more than 256 and at most 512 work-groups the groups after the first 256 / nkv are
    // taken from the light end instead: the heaviest shares its CU with the lightest, and the CUs
    // finish together instead of the first ones last.
    int group = ngroups - 1 - flat;
    {
        const int total = (int)(gridDim.x * gridDim.y), first = AT_CUS / (int)gridDim.x;
        if (CH == 1 && total > AT_CUS && total <= 2 * AT_CUS && flat >= first) group = flat - first;
    }
    const int wg_col0 = group * 128;
    const int col0 = wg_col0 + wave * WCOLS;
    const bool wave_active = col0 < ncols;

    // key range of the work-group and of this wave
    const int wg_last = ((wg_col0 + 128 < ncols) ? wg_col0 + 128 : ncols) - 1;
    const int khi = start + wg_last / G;
    int klo = 0;
    if (window > 0) {
        klo = start + wg_col0 / G - window + 1;
        if (klo < 0) klo = 0;
    }
    const int t_lo = klo / AT_KEYS, t_hi = khi / AT_KEYS;
    int wk_lo = 1, wk_hi = 0;                 // empty for a wave without columns
    if (wave_active) {
        const int w_last = ((col0 + WCOLS < ncols) ? col0 + WCOLS : ncols) - 1;
        wk_hi = start + w_last / G;
        wk_lo = 0;
        if (window > 0) {
            wk_lo = start + col0 / G - window + 1;
            if (wk_lo < 0) wk_lo = 0;
        }
    }
    // page ids into LDS
    {
        const int32_t* table = tables + (size_t)s * NB;
        const int npages = (khi >> bs_shift) + 1;
        for (int i = tid; i < npages; i += THREADS) tab[i] = table[i];
    }

    uint4 qf[NT][DC];
    int p_col[NT], lo_col[NT], row_col[NT], head_col[NT];
    bool has_col[NT];
#pragma unroll
    for (int j = 0; j < NT; ++j) {
        const int col = col0 + j * 16 + c;
        const bool valid = col < ncols;
        const int tok = valid ? col / G : 0;
        const int gh = valid ? col - tok * G : 0;
        row_col[j] = r0 + tok;
        head_col[j] = kvh * G + gh;
        has_col[j] = valid;
        p_col[j] = valid ? start + tok : AM_NO_COLUMN;
        lo_col[j] = (valid && window > 0 && p_col[j] - window + 1 > 0) ? p_col[j] - window + 1 : 0;
        const bf16_t* qp = q + (size_t)row_col[j] * q_stride + (size_t)head_col[j] * D + g * 8;
#pragma unroll
        for (int dc = 0; dc < DC; ++dc)
            qf[j][dc] = valid ? *reinterpret_cast<const uint4*>(qp + dc * 32) : make_uint4(0, 0, 0, 0);
    }

    float m_run[NT], l_run[NT];
    f32x4 acc[NT][DB];
#pragma unroll
    for (int j = 0; j < NT; ++j) {
        m_run[j] = -INFINITY;
        l_run[j] = 0.f;
#pragma unroll
        for (int db = 0; db < DB; ++db) acc[j][db] = f32x4{0.f, 0.f, 0.f, 0.f};
    }

    // Tile T into buffer BUF: nothing comes back into registers.  All addresses first (their page
    // ids come from LDS), then the loads.  A key past the last one any column sees is masked for
    // every column: it is read from the last key's place, which stays on pages the sequence owns.
#define AT_FETCH(T, BUF)                                                                                       \
    {                                                                                                         \
        const int kb_ = (T) * AT_KEYS;                                                                        \
        const char *gk_[NI], *gv_[NI];                                                                        \
        _Pragma("unroll") for (int i = 0; i < NI; ++i) {                                                      \
            int key_ = kb_ + k_key[i];                                                                        \
            if (key_ > khi) key_ = khi;                                                                       \
            const uint32_t slot_ = ((uint32_t)tab[key_ >> bs_shift] << bs_shift) + (key_ & (bs - 1));         \
            gk_[i] = k_base[i] + (uint64_t)slot_ * k_stride;                                                  \
            int vk_ = kb_ + v_key[i];                                                                         \
            if (vk_ > khi) vk_ = khi & ~7;                                                                    \
            gv_[i] = v_base[i] + (uint64_t)(uint32_t)tab[vk_ >> bs_shift] * v_stride + (vk_ & (bs - 1)) * 2;  \
        }                                                                                                     \
        const uint32_t buf_ = CH > 1 ? (uint32_t)__builtin_amdgcn_readfirstlane((BUF) * TILE * 16) : 0u;      \
        _Pragma("unroll") for (int i = 0; i < NI; ++i) {                                                      \
            const int w_ = wave_u + i * WAVES;                                                                \
            if (w_ < UPK) {                                                                                   \
                if (CH > 1) {                                                                                 \
                    at_load_to_lds_at(gk_[i], ks_lds + buf_ + w_ * 1024);                                     \
                    at_load_to_lds_at(gv_[i], vs_lds + buf_ + w_ * 1024);                                     \
                } else {                                                                                      \
                    at_load_to_lds(gk_[i], ks + (BUF) * TILE + w_ * 64);                                      \
                    at_load_to_lds(gv_[i], vs + (BUF) * TILE + w_ * 64);                                      \
                }                                                                                             \
            }                                                                                                 \
        }                                                                                                     \
    }
    // every load of this wave has landed (vmcnt 0; the other counters are left alone)
#define AT_LANDED() __builtin_amdgcn_s_waitcnt(0x0f70)

    __syncthreads();                                         // the page ids are in LDS
#define AT_TILE(T)                                                                                             \
    {                                                                                                         \
        const uint4* kt = ks + cur * TILE;                                                                    \
        const uint4* vt = vs + cur * TILE;                                                                    \
        if (NT == 1 && (T) * AT_KEYS + 32 <= wk_hi && (T) * AT_KEYS + 31 >= wk_lo) {                          \
            /* both halves hold keys of the wave: the whole tile at once */                                   \
            am_tile_lds<DC>(kt, vt, kx, vx, qf[0], p_col[0], lo_col[0], (T) * AT_KEYS, c, g, scale2, m_run[0], \
                            l_run[0], acc[0]);                                                                \
        } else {                                                                                              \
            _Pragma("unroll") for (int half = 0; half < 2; ++half) {                                          \
                const int kb = (T) * AT_KEYS + half * 32;                                                     \
                if (kb > wk_hi || kb + 31 < wk_lo) continue; /* the same for the whole wave */                \
                am_block_lds<DC, NT>(kt, vt, kx, vx, half, qf, p_col, lo_col, kb, c, g, scale2, m_run, l_run, acc); \
            }                                                                                                 \
        }                                                                                                     \
    }
    int cur = 0;
    if (CH == 1) {
        AT_FETCH(t_lo, 0)
        AT_LANDED();
        __syncthreads();
        for (int t = t_lo; t <= t_hi; ++t) {
            if (t < t_hi) AT_FETCH(t + 1, cur ^ 1)
            AT_TILE(t)
            AT_LANDED();
            __syncthreads();
            cur ^= 1;
        }
    } else {
        // chain c takes tiles t_lo + c, t_lo + c + CH, ...; every wave passes the same barriers, a chain
        // whose tile lies past the last one loads that one again and computes nothing
        const int iters = (t_hi - t_lo + CH) / CH;
        int t = t_lo + chain;
        AT_FETCH((t <= t_hi ? t : t_hi), 0)
        AT_LANDED();
        __syncthreads();
        for (int it = 0; it < iters; ++it, t += CH) {
            if (it + 1 < iters) AT_FETCH((t + CH <= t_hi ? t + CH : t_hi), cur ^ 1)
            if (t <= t_hi) AT_TILE(t)
            AT_LANDED();
            __syncthreads();
            cur ^= 1;
        }
    }
#undef AT_TILE

    if (CH > 1) {
        // The second chain hands its running maximum, sum and accumulator over through LDS (the tiles
        // are done with: every wave has passed the last barrier), lane to lane: the same lane of the
        // same wave number holds the same columns and dims in both chains.
        constexpr int PER = DB * 4 + 2;
        float* hand = reinterpret_cast<float*>(at_smem) + (size_t)wave * NT * PER * 64 + lane;
        if (chain == 1) {
#pragma unroll
            for (int j = 0; j < NT; ++j) {
                hand[(j * PER + 0) * 64] = m_run[j];
                hand[(j * PER + 1) * 64] = l_run[j];
#pragma unroll
                for (int db = 0; db < DB; ++db)
#pragma unroll
                    for (int i = 0; i < 4; ++i) hand[(j * PER + 2 + db * 4 + i) * 64] = acc[j][db][i];
            }
        }
        __syncthreads();
        if (chain == 1) return;                              // no barrier follows
#pragma unroll
        for (int j = 0; j < NT; ++j) {
            const float m1 = hand[(j * PER + 0) * 64], l1 = hand[(j * PER + 1) * 64];
            const float mm = fmaxf(m_run[j], m1);            // base-2 domain, as in the loop
            const float w0 = (m_run[j] > -INFINITY) ? exp2f(m_run[j] - mm) : 0.f;
            const float w1 = (m1 > -INFINITY) ? exp2f(m1 - mm) : 0.f;
            l_run[j] = l_run[j] * w0 + l1 * w1;
#pragma unroll
            for (int db = 0; db < DB; ++db)
#pragma unroll
                for (int i = 0; i < 4; ++i) acc[j][db][i] = acc[j][db][i] * w0 + hand[(j * PER + 2 + db * 4 + i) * 64] * w1;
        }
    }

#pragma unroll
    for (int j = 0; j < NT; ++j) {
        if (!has_col[j]) continue;
        float l_tot = l_run[j];
        l_tot += __shfl_xor(l_tot, 16, TL_WAVE);
        l_tot += __shfl_xor(l_tot, 32, TL_WAVE);
        const float inv = 1.0f / l_tot;
        bf16_t* op = out + (size_t)row_col[j] * out_stride + (size_t)head_col[j] * D + 4 * g;
#pragma unroll
        for (int db = 0; db < DB; ++db) {
            uint2 w;
            w.x = am_pack2(acc[j][db][0] * inv, acc[j][db][1] * inv);
            w.y = am_pack2(acc[j][db][2] * inv, acc[j][db][3] * inv);
            *reinterpret_cast<uint2*>(op + db * 16) = w;
        }
    }
}

#undef AT_FETCH
#undef AT_LANDED

// LDS of the tile kernel for head size 32 * DC, a table of `pages` page ids and S sequences: 64 KB of tiles at
// head size 128, so two work-groups share a CU's 160 KB up to some 8,000 pages per sequence and one
// work-group has it alone beyond that
static size_t at_lds_bytes(int DC, int pages, int S, int chains = 1) {
    return (size_t)chains * (4 * AT_KEYS * DC * 4) * sizeof(uint4) + (size_t)(pages + S + 1) * sizeof(int);
}

// Merge the splits of one (token, head): M = max m_s, out = sum acc_s e^(m_s - M) / sum l_s e^(m_s - M),
// over the splits that hold keys of the token.  One work-group of 128 or 256 threads: a thread per split for
// the weights, and (a float4 of the head, a group of splits) per thread for the sum, whose first eight
// loads are in flight while the weights are found.
#define AM_MAX_SPLITS 1024
#define AM_MERGE_AHEAD 8
template <int AM_MERGE_THREADS>
__global__ __launch_bounds__(AM_MERGE_THREADS) void attn_merge_kernel(
    const float* __restrict__ ws_o, const float* __restrict__ ws_ml, const int32_t* __restrict__ pos,
    bf16_t* __restrict__ out, int out_stride, int nq, int D, int nsplit, int split_blocks, int window,
    const int32_t* __restrict__ seq_list, const int32_t* __restrict__ q_start) {
    __shared__ float wgt[AM_MAX_SPLITS];
    __shared__ float red_m[AM_MERGE_THREADS / 64], red_l[AM_MERGE_THREADS / 64];
    __shared__ float4 part[AM_MERGE_THREADS];
    const int wrow = blockIdx.x, h = blockIdx.y, tid = threadIdx.x;
    const int t = seq_list ? q_start[seq_list[wrow]] : wrow;   // listed one-token sequences: their row of the step
    const int p = pos[t];
    const int lo = (window > 0 && p - window + 1 > 0) ? p - window + 1 : 0;
    const int s_lo = (lo >> 5) / split_blocks, s_hi = (p >> 5) / split_blocks;
    const int ns = s_hi - s_lo + 1;
    const size_t base = ((size_t)wrow * nq + h) * nsplit + s_lo;
    const int D4 = D >> 2, SG = AM_MERGE_THREADS / D4;      // D is 32, 64 or 128
    const int d4 = tid % D4, sg = tid / D4;
    const float4* acc4 = reinterpret_cast<const float4*>(ws_o) + base * D4 + d4;
    const float2* ml2 = reinterpret_cast<const float2*>(ws_ml) + base;
    const float4 zero4 = make_float4(0.f, 0.f, 0.f, 0.f);
    float4 a[AM_MERGE_AHEAD];
#pragma unroll
    for (int k = 0; k < AM_MERGE_AHEAD; ++k) {
        const int s = sg + k * SG;
        a[k] = zero4;
        if (s < ns) a[k] = acc4[(size_t)s * D4];
    }
    float2 ml[AM_MAX_SPLITS / AM_MERGE_THREADS];
    float mx = -INFINITY;
#pragma unroll
    for (int j = 0; j < AM_MAX_SPLITS / AM_MERGE_THREADS; ++j) {
        const int s = tid + j * AM_MERGE_THREADS;
        ml[j] = make_float2(-INFINITY, 0.f);
        if (s < ns) ml[j] = ml2[s];
        mx = fmaxf(mx, ml[j].x);
    }
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) mx = fmaxf(mx, __shfl_xor(mx, o));
    if ((tid & 63) == 0) red_m[tid >> 6] = mx;
    __syncthreads();
    float M = red_m[0];
#pragma unroll
    for (int w = 1; w < AM_MERGE_THREADS / 64; ++w) M = fmaxf(M, red_m[w]);
    float ls = 0.f;                                          // maxima are kept in the base-2 domain
#pragma unroll
    for (int j = 0; j < AM_MAX_SPLITS / AM_MERGE_THREADS; ++j) {
        const int s = tid + j * AM_MERGE_THREADS;
        const float w = (ml[j].x > -INFINITY) ? exp2f(ml[j].x - M) : 0.f;
        if (s < ns) wgt[s] = w;
        ls += ml[j].y * w;
    }
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) ls += __shfl_xor(ls, o);
    if ((tid & 63) == 0) red_l[tid >> 6] = ls;
    __syncthreads();
    float L = red_l[0];
#pragma unroll
    for (int w = 1; w < AM_MERGE_THREADS / 64; ++w) L += red_l[w];
    float4 o4 = zero4;
#pragma unroll
    for (int k = 0; k < AM_MERGE_AHEAD; ++k) {
        const int s = sg + k * SG;
        if (s < ns) {
            const float w = wgt[s];
            o4.x += a[k].x * w, o4.y += a[k].y * w, o4.z += a[k].z * w, o4.w += a[k].w * w;
        }
    }
    for (int s = sg + AM_MERGE_AHEAD * SG; s < ns; s += SG) {
        const float4 v = acc4[(size_t)s * D4];
        const float w = wgt[s];
        o4.x += v.x * w, o4.y += v.y * w, o4.z += v.z * w, o4.w += v.w * w;
    }
    part[tid] = o4;
    __syncthreads();
    if (tid < D4) {
        float4 r = part[tid];
        for (int g = 1; g < SG; ++g) {
            const float4 v = part[g * D4 + tid];
            r.x += v.x, r.y += v.y, r.z += v.z, r.w += v.w;
        }
        const float inv_l = 1.0f / L;
        bf16_t* dst = out + (size_t)t * out_stride + (size_t)h * D + tid * 4;
        dst[0] = tl_from_float<bf16_t>(r.x * inv_l);
        dst[1] = tl_from_float<bf16_t>(r.y * inv_l);
        dst[2] = tl_from_float<bf16_t>(r.z * inv_l);
        dst[3] = tl_from_float<bf16_t>(r.w * inv_l);
    }
}

template <int DC>
static void launch_attn(int NT, dim3 grid, int wg_waves, hipStream_t stream, const bf16_t* q, int q_stride, const bf16_t* kc,
                        const bf16_t* vc, const int32_t* tables, int NB, const int32_t* q_start,
                        const int32_t* ctx_start, bf16_t* out, int out_stride, float* ws_o, float* ws_ml, int nq, int nkv,
                        int bs, int window, float scale, int nsplit, int split_blocks, const int32_t* seq_list,
                        int skip_single) {
    int bs_shift = -1;                               // pages of a power of two of tokens: a shift finds the page
    if ((bs & (bs - 1)) == 0)
        for (bs_shift = 0; (1 << bs_shift) < bs;) ++bs_shift;
    if (NT == 1)
        hipLaunchKernelGGL((attn_mfma_kernel<DC, 1>), grid, dim3(64 * wg_waves), 0, stream, q, q_stride, kc, vc, tables, NB, q_start,
                           ctx_start, out, out_stride, ws_o, ws_ml, nq, nkv, bs, bs_shift, window, scale, nsplit,
                           split_blocks, seq_list, skip_single);
    else
        hipLaunchKernelGGL((attn_mfma_kernel<DC, 2>), grid, dim3(64 * wg_waves), 0, stream, q, q_stride, kc, vc, tables, NB, q_start,
                           ctx_start, out, out_stride, ws_o, ws_ml, nq, nkv, bs, bs_shift, window, scale, nsplit,
                           split_blocks, seq_list, skip_single);
}

// q: bfloat16 [T, >= nq*d] (row stride q_stride); k_cache [pages, page, nkv, d]; v_cache
// [pages, nkv, d, page]; tables int32 [S, NB]; q_start int32 [S+1]; ctx_start int32 [S]; out
// bfloat16 [T, nq*d] (row stride out_stride).  NT (1 or 2) column tiles per wave; max_tile_groups =
// the largest ceil(n_s * G / (16 NT)) over the sequences.  With nsplit > 1 a split is split_blocks
// blocks of 32 keys, nsplit * split_blocks * 32 must cover the longest context, pos is int32 [T]
// (the tokens' positions), ws_o holds T*nq*nsplit*d floats and ws_ml T*nq*nsplit*2.  shared != 0
// runs unsplit steps with prompt portions on the kernel that shares keys and values through LDS
// (when the page size and the table length allow it), shared == 2 with two chains of tiles per
// work-group where their buffers fit; shared == 0 keeps them on independent waves.
// A step that holds prompt portions and one-token sequences with long contexts may be run as two
// calls: one with seq_list (int32 [n_list], the indices of one-token sequences; only they are
// computed, with split keys, and the workspace then holds n_list rows instead of T), and one
// with skip_single != 0, which leaves sequences of one token out.
// total_groups128: the sum over the sequences of ceil(n_s * G / 128), that kernel's grid.
extern "C" int tl_attention_mfma(const void* q, int q_stride, const void* k_cache, const void* v_cache,
                                 const int32_t* tables, int NB, const int32_t* q_start, const int32_t* ctx_start,
                                 const int32_t* pos, void* out, int out_stride, float* ws_o, float* ws_ml, int T, int S,
                                 int nq, int nkv, int d, int bs, int window, float scale, int NT, int max_tile_groups,
                                 int nsplit, int split_blocks, int shared, int total_groups128,
                                 const int32_t* seq_list, int n_list, int skip_single, hipStream_t stream) {
    TL_CHECK_ARG(T >= 0 && S >= 0 && nq > 0 && nkv > 0 && NB > 0, "tl_attention_mfma: bad sizes T=%d S=%d nq=%d nkv=%d NB=%d", T, S, nq, nkv, NB);
    TL_CHECK_ARG(nq % nkv == 0, "tl_attention_mfma: %d query heads are not a multiple of %d key/value heads", nq, nkv);
    TL_CHECK_ARG(d == 32 || d == 64 || d == 128, "tl_attention_mfma: head size %d is not one of 32, 64, 128", d);
    TL_CHECK_ARG(bs >= 8 && bs % 8 == 0, "tl_attention_mfma: page size %d must be a multiple of 8", bs);
    TL_CHECK_ARG(NT == 1 || NT == 2, "tl_attention_mfma: NT=%d must be 1 or 2", NT);
    TL_CHECK_ARG(nsplit >= 1 && nsplit <= AM_MAX_SPLITS && max_tile_groups >= 1,
                 "tl_attention_mfma: bad split count %d (at most %d) or group count", nsplit, AM_MAX_SPLITS);
    TL_CHECK_ARG(nsplit == 1 || (ws_o && ws_ml && pos && split_blocks >= 1),
                 "tl_attention_mfma: split keys need a workspace, positions and a split length");
    TL_CHECK_ARG(q_stride % 8 == 0 && out_stride % 4 == 0 && q_stride >= nq * d && out_stride >= nq * d,
                 "tl_attention_mfma: bad row strides %d, %d", q_stride, out_stride);
    TL_CHECK_ARG(((uintptr_t)q % 16) == 0 && ((uintptr_t)k_cache % 16) == 0 && ((uintptr_t)v_cache % 16) == 0 &&
                     ((uintptr_t)out % 8) == 0, "tl_attention_mfma: operands must be 16-byte aligned");
    TL_CHECK_ARG(nsplit == 1 || (((uintptr_t)ws_o % 16) == 0 && ((uintptr_t)ws_ml % 8) == 0),
                 "tl_attention_mfma: the split workspace must be 16-byte aligned");
    TL_CHECK_ARG(nkv <= 65535, "tl_attention_mfma: too many key/value heads");
    TL_CHECK_ARG(scale > 0.f, "tl_attention_mfma: the score scale %g must be positive", (double)scale);
    TL_CHECK_ARG(!seq_list || (n_list >= 0 && n_list <= S && !skip_single),
                 "tl_attention_mfma: a list of %d sequences does not fit %d sequences, or it comes with skip_single", n_list, S);
    if (T == 0 || S == 0 || (seq_list && n_list == 0)) return 0;
    const int S_run = seq_list ? n_list : S;               // sequences the grid runs over
    const long waves = (long)max_tile_groups * nsplit;
    // The waves are independent: four to a work-group, fewer when that would leave compute units without one.
    int wg_waves = 4;
    while (wg_waves > 1 && (long)S_run * nkv * ((waves + wg_waves - 1) / wg_waves) < 256) wg_waves >>= 1;
    TL_CHECK_ARG((waves + wg_waves - 1) / wg_waves <= 65535, "tl_attention_mfma: too many tile groups x splits (%ld)", waves);
    dim3 grid(S_run, nkv, (unsigned)((waves + wg_waves - 1) / wg_waves));
    const bf16_t *qq = (const bf16_t*)q, *kk = (const bf16_t*)k_cache, *vv = (const bf16_t*)v_cache;
    const bool pow2 = (bs & (bs - 1)) == 0;
    if (NT == 2 && nsplit == 1 && shared && pow2 && !seq_list && total_groups128 > 0 &&
        at_lds_bytes(d / 32, NB, S) <= 160 * 1024) {
        // 128 columns per work-group, keys and values shared through LDS; shared == 2 asks for two
        // chains per work-group where their tiles fit LDS
        int bs_shift = 0;
        while ((1 << bs_shift) < bs) ++bs_shift;
        TL_CHECK_ARG(total_groups128 <= 65535, "tl_attention_mfma: %d column groups are more than a launch takes", total_groups128);
        dim3 sgrid(nkv, (unsigned)total_groups128, 1);
        const int chains = (shared == 2 && at_lds_bytes(d / 32, NB, S, 2) <= 160 * 1024) ? 2 : 1;
        const size_t lds = at_lds_bytes(d / 32, NB, S, chains);
#define TL_TILE_CASE(DCV)                                                                                             \
    do {                                                                                                              \
        if (chains == 2)                                                                                              \
            hipLaunchKernelGGL((attn_tile_kernel<DCV, AT_NT, 8 / AT_NT, 2>), sgrid, dim3(2 * 64 * 8 / AT_NT), lds,    \
                               stream, qq, q_stride, kk, vv, tables, NB, q_start, ctx_start, (bf16_t*)out, out_stride, \
                               S, nq, nkv, bs, bs_shift, window, scale, skip_single);                                 \
        else                                                                                                          \
            hipLaunchKernelGGL((attn_tile_kernel<DCV, AT_NT, 8 / AT_NT, 1>), sgrid, dim3(64 * 8 / AT_NT), lds,        \
                               stream, qq, q_stride, kk, vv, tables, NB, q_start, ctx_start, (bf16_t*)out, out_stride, \
                               S, nq, nkv, bs, bs_shift, window, scale, skip_single);                                 \
    } while (0)
        if (d == 32) TL_TILE_CASE(1);
        else if (d == 64) TL_TILE_CASE(2);
        else TL_TILE_CASE(4);
#undef TL_TILE_CASE
        TL_CHECK_LAUNCH("tl_attention_mfma tiles");
        return 0;
    }
    if (d == 32)
        launch_attn<1>(NT, grid, wg_waves, stream, qq, q_stride, kk, vv, tables, NB, q_start, ctx_start, (bf16_t*)out, out_stride,
                       ws_o, ws_ml, nq, nkv, bs, window, scale, nsplit, split_blocks, seq_list, skip_single);
    else if (d == 64)
        launch_attn<2>(NT, grid, wg_waves, stream, qq, q_stride, kk, vv, tables, NB, q_start, ctx_start, (bf16_t*)out, out_stride,
                       ws_o, ws_ml, nq, nkv, bs, window, scale, nsplit, split_blocks, seq_list, skip_single);
    else
        launch_attn<4>(NT, grid, wg_waves, stream, qq, q_stride, kk, vv, tables, NB, q_start, ctx_start, (bf16_t*)out, out_stride,
                       ws_o, ws_ml, nq, nkv, bs, window, scale, nsplit, split_blocks, seq_list, skip_single);
    TL_CHECK_LAUNCH("tl_attention_mfma");
    if (nsplit > 1) {
        const int merge_rows = seq_list ? n_list : T;
        if (nsplit > 32)
            hipLaunchKernelGGL(attn_merge_kernel<256>, dim3(merge_rows, nq), dim3(256), 0, stream, ws_o, ws_ml, pos,
                               (bf16_t*)out, out_stride, nq, d, nsplit, split_blocks, window, seq_list, q_start);
        else
            hipLaunchKernelGGL(attn_merge_kernel<128>, dim3(merge_rows, nq), dim3(128), 0, stream, ws_o, ws_ml, pos,
                               (bf16_t*)out, out_stride, nq, d, nsplit, split_blocks, window, seq_list, q_start);
        TL_CHECK_LAUNCH("tl_attention_mfma merge");
    }
    return 0;
}
