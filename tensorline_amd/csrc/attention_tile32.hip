// Causal grouped-query attention of prompt portions over the paged cache on the 32x32 matrix-core
// instruction (v_mfma_f32_32x32x16_bf16, bfloat16, gfx950): the kernel for steps that hold prompt
// portions when the head size is 64 or 128 and a page holds a power of two of tokens.
//
// A wave owns 32 "columns" of one (sequence, key/value head); a column is a (query token, query
// head of the group) pair, numbered token-major.  A work-group of WAVES waves owns WAVES * 32
// consecutive columns and walks the keys together in tiles of 64, which go from the cache straight
// into LDS (global_load_lds_dwordx4), double-buffered, one barrier per tile.  Per tile a wave
// computes
//   scores^T [64 keys x 32 columns] = K [64 x d] * Q^T [d x 32]         2 row tiles x d/16 products
//   out^T    [d x 32 columns]      += V^T [d x 64 keys] * P^T [64 x 32]  d/32 row tiles x 4 products
// with the online softmax (base-2 domain, float) between them.  With 32 columns a fragment of K or
// V^T read from LDS (1 KB per wave) feeds a product of 32 matrix-core cycles, where 16 columns on
// the 16x16x32 instruction feed one of 16: half the LDS traffic, half the loader's work and half
// the per-tile bookkeeping per column, and a wave's softmax (32 exponentials and about a hundred
// other vector instructions per tile) takes about as long as its 32 products instead of twice as
// long.  A wave uses up to 256 registers, so a CU holds eight waves: one work-group of eight or two of
// four (64 KB of LDS each).
//
// Operands of D = A * B (lane l: n = l % 32, h = l / 32): A is row n, eight k at 8h..8h+7; B is
// column n, the same eight k; D register r of lane l is row 8 (r / 4) + 4 h + r % 4 of column n.
// Which key a row of the score tile stands for is free, and is chosen so that what a lane holds
// after the two score tiles is, eight registers at a time, the B operand of a P*V product:
//   score tile t, row 8 b + 4 h + i   <->   key 32 t + 16 (b / 2) + 8 h + 4 (b % 2) + i
// so registers 8 kk .. 8 kk + 7 of a lane (kk = 0..3 over both tiles) are keys 16 kk + 8 h .. + 7
// of its column: the eight k of lane half h in product kk.  No value moves between lanes; the
// maximum of a column is one swap of the wave's halves (v_permlane32_swap).  The matching A
// fragment of V^T, eight consecutive keys of one dim, is one 16-byte read because values are paged
// transposed: [pages, nkv, d, page]; keys are paged [pages, page, nkv, d].
//
// Tiles are aligned to absolute positions (tile t holds keys 64 t .. 64 t + 63) and a tile's keys
// are summed in one fixed order, so which keys are summed together depends neither on the context
// length nor on how the sequence was cut into steps (reference: tensorline/paged_attn.py:25-58
// for the online softmax, tensorline/paged.py:233-238 for the mask).
#include "common.h"

typedef __bf16 t32_bf16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 t32_bf16x2 __attribute__((ext_vector_type(2)));
typedef float t32_f32x2 __attribute__((ext_vector_type(2)));
typedef float t32_f32x16 __attribute__((ext_vector_type(16)));
typedef unsigned int t32_u32x2 __attribute__((ext_vector_type(2)));

#define T32_KEYS 64
#define T32_CUS 256
#define T32_LOG2E 1.4426950408889634f
#define T32_LAZY 8.0f                 // how far a tile's maximum may exceed the running one before it moves
#define T32_NO_COLUMN 0x7fffffff      // position of a lane without a column: never masked, never written

__device__ __forceinline__ t32_bf16x8 t32_frag(uint4 v) { return __builtin_bit_cast(t32_bf16x8, v); }

// two floats -> two bfloat16 (round to nearest even) in one register
__device__ __forceinline__ uint32_t t32_pack2(float a, float b) {
    const t32_f32x2 v = {a, b};
    return __builtin_bit_cast(uint32_t, __builtin_convertvector(v, t32_bf16x2));
}

// max(a, b, c): the compiler makes one v_max3_f32 of it.  (Not written as assembly: the compiler
// keeps the waits that the hardware needs between a matrix-core or transcendental instruction and a
// reader of its result only for instructions it knows.)
__device__ __forceinline__ float t32_max3(float a, float b, float c) { return fmaxf(fmaxf(a, b), c); }

// Lanes l and l + 32 hold the two halves of a column's keys: both get the maximum / the sum of the two.
__device__ __forceinline__ float t32_halves_max(float v) {
    const t32_u32x2 sw = __builtin_amdgcn_permlane32_swap(__float_as_uint(v), __float_as_uint(v), false, false);
    return t32_max3(v, __uint_as_float(sw[0]), __uint_as_float(sw[1]));
}
__device__ __forceinline__ float t32_halves_sum(float v) {
    const t32_u32x2 sw = __builtin_amdgcn_permlane32_swap(__float_as_uint(v), __float_as_uint(v), false, false);
    return __uint_as_float(sw[0]) + __uint_as_float(sw[1]);
}

// Where unit u (16 bytes) of a row lies within the row in LDS: u ^ swizzle(row).  A K row has UPK =
// 8 or 16 units and 16 / UPK rows span the 256 bytes over which the banks repeat; a V^T row has 8.
template <int UPK>
__device__ __forceinline__ int t32_k_swizzle(int row) { return ((row & 15) * UPK) >> 4; }
__device__ __forceinline__ int t32_v_swizzle(int row) { return (row >> 1) & 7; }

// The key of a 32-key score tile that row `row` of the tile stands for (see the head of the file).
__device__ __forceinline__ int t32_row_key(int row) {
    const int b = row >> 3, h = (row >> 2) & 1, i = row & 3;
    return 16 * (b >> 1) + 8 * h + 4 * (b & 1) + i;
}

// 16 bytes per lane from memory straight into LDS at lds_base + 16 * lane (lds_base is the same for
// the whole wave).  Written as assembly so that the compiler does not make every later LDS read
// wait for it: a load is waited for only where T32_LANDED says so.  M0 holds the LDS base for the
// instruction and is put back.  Two forms: a 64-bit address per lane, and a wave-wide 64-bit base
// in scalar registers plus a 32-bit offset per lane.
__device__ __forceinline__ void t32_load_to_lds(const void* g, void* lds_base) {
    const uint32_t base = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) void*)lds_base;
    uint32_t saved;
    asm volatile(
        "s_mov_b32 %0, m0\n\ts_mov_b32 m0, %1\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %2, off\n\ts_mov_b32 m0, %0"
        : "=&s"(saved)
        : "s"(base), "v"(g)
        : "memory");
}
__device__ __forceinline__ void t32_load_to_lds_based(const void* wave_base, uint32_t voff, void* lds_base) {
    const uint32_t base = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) void*)lds_base;
    // the base is the same in every lane; said so explicitly, it lives in scalar registers
    const uint64_t a = (uint64_t)(uintptr_t)wave_base;
    const uint64_t sbase = ((uint64_t)(uint32_t)__builtin_amdgcn_readfirstlane((int)(a >> 32)) << 32) |
                           (uint32_t)__builtin_amdgcn_readfirstlane((int)(uint32_t)a);
    uint32_t saved;
    asm volatile(
        "s_mov_b32 %0, m0\n\ts_mov_b32 m0, %1\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %2, %3\n\ts_mov_b32 m0, %0"
        : "=&s"(saved)
        : "s"(base), "v"(voff), "s"(sbase)
        : "memory");
}

// The three stages of a tile of 64 keys for the 32 columns of a wave.  kt, vt: a tile's keys and
// values in LDS; koff[s] / voff[kk]: where the lane's fragment of step s of the score products (row
// tile 0; row tile 1 lies 32 * UPK units further) and of step kk of the P*V products (row tile 0;
// row tile m lies 256 m units further) is.
#define T32_KFRAG(I) kt[koff[(I) >> 1] + ((I) & 1) * 32 * UPK]
#define T32_VFRAG(I) vt[voff[(I) / DT] + ((I) % DT) * 256]

// scores^T of a tile: sc[t][r] is, of the lane's column, key 32 t + 16 (r / 8) + 8 h + r % 8.  The
// fragment reads run four products ahead of their products in a ring of registers.
template <int DC>
__device__ __forceinline__ void t32_scores(const uint4* kt, const int* koff, const uint4* qf, t32_f32x16* sc) {
    constexpr int D = DC * 32, KS = D / 16, UPK = D / 8;
#pragma unroll
    for (int t = 0; t < 2; ++t)
#pragma unroll
        for (int r = 0; r < 16; ++r) sc[t][r] = 0.f;
    uint4 kf[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) kf[i] = T32_KFRAG(i);
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int i = 0; i < 2 * KS; ++i) {
        sc[i & 1] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(t32_frag(kf[i % 4]), t32_frag(qf[i >> 1]), sc[i & 1], 0, 0, 0);
        if (i + 4 < 2 * KS) kf[i % 4] = T32_KFRAG(i + 4);
        __builtin_amdgcn_sched_barrier(0);
    }
}

// out^T += V^T P^T for a tile whose probabilities are pf.
template <int DC>
__device__ __forceinline__ void t32_weighted_sum(const uint4* vt, const int* voff, const uint4* pf, t32_f32x16* acc) {
    constexpr int DT = DC;
    uint4 vf[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) vf[i] = T32_VFRAG(i);
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int i = 0; i < 4 * DT; ++i) {
        acc[i % DT] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(t32_frag(vf[i % 4]), t32_frag(pf[i / DT]), acc[i % DT], 0, 0, 0);
        if (i + 4 < 4 * DT) vf[i % 4] = T32_VFRAG(i + 4);
        __builtin_amdgcn_sched_barrier(0);
    }
}

// The online softmax of a tile (base-2 domain): from the scores sc to the probabilities pf in the
// operand layout of the P*V products, the running maximum and sum brought up to date.  Returns the
// factor the accumulator of the tiles before has to be scaled by before this tile's P*V is added
// (1 unless the running maximum moved).
// The running maximum follows the true one lazily: it moves only when the tile's maximum exceeds it
// by more than T32_LAZY, so probabilities stay below 2^T32_LAZY and the accumulator is rescaled in
// few tiles instead of most.  Sums and accumulators stay relative to the same running maximum, so
// the result is the same.
__device__ __forceinline__ float t32_softmax(const t32_f32x16* sc, bool edge, int p_col, int lo_col, int kb, int h,
                                             float scale2, float& m_run, float& l_run, uint4* pf) {
    float sv[32];
#pragma unroll
    for (int t = 0; t < 2; ++t)
#pragma unroll
        for (int r = 0; r < 16; ++r) sv[16 * t + r] = sc[t][r];
    if (edge) {                                              // some key of the tile is hidden from some column of the wave
#pragma unroll
        for (int x = 0; x < 32; ++x) {
            const int key = kb + 16 * (x >> 3) + 8 * h + (x & 7);
            if (key > p_col || key < lo_col) sv[x] = -INFINITY;
            asm volatile("" : "+v"(sv[x]));                  // in place and under the branch: most tiles skip all of it
        }
    }
    float mx[11];
#pragma unroll
    for (int i = 0; i < 10; ++i) mx[i] = t32_max3(sv[3 * i], sv[3 * i + 1], sv[3 * i + 2]);
    mx[10] = fmaxf(sv[30], sv[31]);
    float bmax = t32_max3(t32_max3(mx[0], mx[1], mx[2]), t32_max3(mx[3], mx[4], mx[5]), t32_max3(mx[6], mx[7], mx[8]));
    bmax = t32_max3(bmax, mx[9], mx[10]);
    bmax = t32_halves_max(bmax);
    bmax *= scale2;                                          // the scale is positive: the order is the same
    const bool moved = bmax > m_run + T32_LAZY;              // also the first keys: -inf + T32_LAZY is -inf
    const float m_new = moved ? bmax : m_run;
    const float neg_m = (m_new == -INFINITY) ? 0.f : -m_new;
    float pr[32];
#pragma unroll
    for (int x = 0; x < 32; ++x) pr[x] = __builtin_amdgcn_exp2f(__builtin_fmaf(sv[x], scale2, neg_m));
    float ps[8];
#pragma unroll
    for (int x = 0; x < 8; ++x) ps[x] = (pr[4 * x] + pr[4 * x + 1]) + (pr[4 * x + 2] + pr[4 * x + 3]);
    const float psum = ((ps[0] + ps[1]) + (ps[2] + ps[3])) + ((ps[4] + ps[5]) + (ps[6] + ps[7]));
#pragma unroll
    for (int kk = 0; kk < 4; ++kk) {
        pf[kk].x = t32_pack2(pr[8 * kk + 0], pr[8 * kk + 1]);
        pf[kk].y = t32_pack2(pr[8 * kk + 2], pr[8 * kk + 3]);
        pf[kk].z = t32_pack2(pr[8 * kk + 4], pr[8 * kk + 5]);
        pf[kk].w = t32_pack2(pr[8 * kk + 6], pr[8 * kk + 7]);
    }
    // (nothing has been summed before a column's first keys: no factor then, though its maximum moves)
    const float alpha = (moved && m_run != -INFINITY) ? __builtin_amdgcn_exp2f(m_run + neg_m) : 1.0f;
    l_run = l_run * alpha + psum;
    m_run = m_new;
    return alpha;
}

#undef T32_KFRAG
#undef T32_VFRAG

// q: [T, >= nq * D] (row stride q_stride); kc [pages, bs, nkv, D]; vc [pages, nkv, D, bs]; tables
// [S, NB]; q_start [S + 1]; ctx_start [S]; out [T, nq * D] (row stride out_stride).  Grid: (nkv,
// sum over the sequences of ceil(n_s * G / (32 WAVES))): one work-group per group of columns that
// exists.  bs = 2^bs_shift >= 8.  skip_single: sequences of one token belong to another launch.
template <int DC, int WAVES>
__global__ __launch_bounds__(WAVES * 64, 2) void attn_tile32_kernel(
    const bf16_t* __restrict__ q, int q_stride, const bf16_t* __restrict__ kc, const bf16_t* __restrict__ vc,
    const int32_t* __restrict__ tables, int NB, const int32_t* __restrict__ q_start,
    const int32_t* __restrict__ ctx_start, bf16_t* __restrict__ out, int out_stride, int S, int nq, int nkv, int bs,
    int bs_shift, int window, float scale, int skip_single) {
    constexpr int THREADS = WAVES * 64;
    constexpr int WGC = WAVES * 32;           // columns of a work-group
    constexpr int D = DC * 32, KS = D / 16, DT = D / 32;
    constexpr int UPK = D / 8;                // 16-byte units of a key row; also the wave-loads of a K tile and of a V^T tile
    constexpr int TILE = T32_KEYS * UPK;      // units of a K tile, and of a V^T tile (D rows of 8)
    constexpr int NL = UPK / WAVES;           // wave-loads of each a wave issues per tile
    constexpr int KPL = 64 / UPK;             // keys a wave-load of K covers (4 or 8): they lie in one page
    static_assert(UPK % WAVES == 0 && NL >= 1, "a tile's wave-loads are dealt evenly to the waves");
    extern __shared__ uint4 t32_smem[];
    uint4* ks = t32_smem;                                  // [2][TILE]
    uint4* vs = t32_smem + 2 * TILE;                       // [2][TILE]
    int* tab = reinterpret_cast<int*>(vs + 2 * TILE);      // page ids of the sequence, as far as needed (NB ints)
    int* qst = tab + NB;                                   // q_start of the step (S + 1 ints)
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int n32 = lane & 31, h = lane >> 5;
    const int kvh = blockIdx.x;                            // fastest: the heads of a group start together
    const int G = nq / nkv;
    const float scale2 = scale * T32_LOG2E;
    // Which (sequence, group of WGC columns) this work-group owns.  Within a sequence the groups
    // with the most keys (the last columns) come first.
    for (int i = tid; i <= S; i += THREADS) qst[i] = q_start[i];
    __syncthreads();
    int s = 0, flat = blockIdx.y, ngroups = 0;
    for (; s < S; ++s) {
        const int nn = qst[s + 1] - qst[s];
        ngroups = (skip_single && nn == 1) ? 0 : (nn * G + WGC - 1) / WGC;
        if (flat < ngroups) break;
        flat -= ngroups;
    }
    if (s >= S) return;                       // the whole work-group leaves: no barrier is missed
    // the same in every lane: said so, they and all that follows from them live in scalar registers
    s = __builtin_amdgcn_readfirstlane(s);
    flat = __builtin_amdgcn_readfirstlane(flat);
    ngroups = __builtin_amdgcn_readfirstlane(ngroups);
    const int r0 = __builtin_amdgcn_readfirstlane(qst[s]);
    const int n = __builtin_amdgcn_readfirstlane(qst[s + 1]) - r0;
    const int start = __builtin_amdgcn_readfirstlane(ctx_start[s]);
    const int ncols = n * G;
    // The hardware places work-group i + 256 on the CU of work-group i (256 CUs, two work-groups
    // each), so when the grid has more than 256 and at most 512 work-groups the groups after the
    // first 256 / nkv are taken from the light end: the heaviest shares its CU with the lightest.
    int group = ngroups - 1 - flat;
    {
        const int total = (int)(gridDim.x * gridDim.y), first = T32_CUS / (int)gridDim.x;
        if (total > T32_CUS && total <= 2 * T32_CUS && flat >= first) group = flat - first;
    }
    const int wg_col0 = group * WGC;
    const int col0 = wg_col0 + wave * 32;
    const bool wave_active = col0 < ncols;

    // key range of the work-group and of this wave
    const int wg_last = ((wg_col0 + WGC < ncols) ? wg_col0 + WGC : ncols) - 1;
    const int khi = start + wg_last / G;
    int klo = 0;
    if (window > 0) {
        klo = start + wg_col0 / G - window + 1;
        if (klo < 0) klo = 0;
    }
    const int t_lo = klo / T32_KEYS, t_hi = khi / T32_KEYS;
    int wk_lo = 1, wk_hi = 0, wk_full_hi = -1, wk_full_lo = 0;   // empty for a wave without columns
    if (wave_active) {
        const int w_last = ((col0 + 32 < ncols) ? col0 + 32 : ncols) - 1;
        wk_hi = start + w_last / G;           // the last key any column of the wave sees
        wk_full_hi = start + col0 / G;        // the last key every column of the wave sees
        wk_lo = 0;
        if (window > 0) {
            wk_lo = start + col0 / G - window + 1;
            if (wk_lo < 0) wk_lo = 0;
            wk_full_lo = start + w_last / G - window + 1;     // the first key every column sees
            if (wk_full_lo < 0) wk_full_lo = 0;
        }
    }
    // page ids into LDS
    {
        const int32_t* table = tables + (size_t)s * NB;
        const int npages = (khi >> bs_shift) + 1;
        for (int i = tid; i < npages; i += THREADS) tab[i] = table[i];
    }

    // Loader.  A K tile is 64 rows x UPK units, a V^T tile D rows x 8 units: UPK wave-loads of 64
    // consecutive units each, wave w issuing numbers w, w + WAVES, ...  Load number L of K holds
    // keys KPL * L .. + KPL - 1 of the tile, which share a page: their slot comes from scalar
    // registers and the lane adds an offset that is the same for all its loads (the swizzle of a
    // row depends on the row modulo 16, and the rows of a lane's loads lie multiples of 16 apart).
    // Load number L of V^T holds dims 8 L .. 8 L + 7; which eight keys of the tile a lane brings is
    // again the same for all its loads, so one page id per lane and tile serves them.
    const uint32_t k_stride = (uint32_t)nkv * D * 2;         // bytes from a slot to the next
    const uint64_t v_stride = (uint64_t)nkv * D * bs * 2;    // bytes from a page to the next
    const int k_row = lane / UPK;                            // the lane's key within a K wave-load
    const uint32_t k_voff = (uint32_t)k_row * k_stride + (uint32_t)kvh * D * 2 +
                            (uint32_t)((lane % UPK) ^ t32_k_swizzle<UPK>(KPL * wave + k_row)) * 16;
    const int v_key = ((lane & 7) ^ t32_v_swizzle(8 * wave + (lane >> 3))) * 8;   // first of the lane's eight keys in the tile
    const char* v_base = reinterpret_cast<const char*>(vc) + ((size_t)kvh * D + (lane >> 3)) * bs * 2;
    const uint32_t v_lstep = (uint32_t)8 * bs * 2;           // bytes from a V^T wave-load to the next (8 dims)
    const char* kc_bytes = reinterpret_cast<const char*>(kc);

    // where the lane's fragments lie in a tile (units of 16 bytes)
    int koff[KS], voff[4];
    {
        const int key0 = t32_row_key(n32);
#pragma unroll
        for (int st = 0; st < KS; ++st) koff[st] = key0 * UPK + ((2 * st + h) ^ t32_k_swizzle<UPK>(key0));
#pragma unroll
        for (int kk = 0; kk < 4; ++kk) voff[kk] = n32 * 8 + ((2 * kk + h) ^ t32_v_swizzle(n32));
    }

    // the lane's column: queries in operand layout, position, output place
    const int col = col0 + n32;
    const bool valid = col < ncols;
    const int tok = valid ? col / G : 0;
    const int gh = valid ? col - tok * G : 0;
    const int row_out = r0 + tok, head = kvh * G + gh;
    const int p_col = valid ? start + tok : T32_NO_COLUMN;
    const int lo_col = (valid && window > 0 && p_col - window + 1 > 0) ? p_col - window + 1 : 0;
    uint4 qf[KS];
    {
        const bf16_t* qp = q + (size_t)row_out * q_stride + (size_t)head * D + h * 8;
#pragma unroll
        for (int st = 0; st < KS; ++st)
            qf[st] = valid ? *reinterpret_cast<const uint4*>(qp + st * 16) : make_uint4(0, 0, 0, 0);
    }
    float m_run = -INFINITY, l_run = 0.f;
    t32_f32x16 acc[DT];
#pragma unroll
    for (int m = 0; m < DT; ++m)
#pragma unroll
        for (int r = 0; r < 16; ++r) acc[m][r] = 0.f;
    // Tile T into buffer BUF: nothing comes back into registers.  A key past the last one any column
    // sees is masked for every column: it is read from the place of the last keys, which stay on
    // pages the sequence owns.  The page ids a tile's loads need are read from LDS a step ahead
    // (T32_PAGES), so that a wave does not start its step waiting for them.
    int k_page[NL], v_page;
#define T32_PAGES(T)                                                                                           \
    {                                                                                                          \
        const int kb_ = (T) * T32_KEYS;                                                                        \
        int vk_ = kb_ + v_key;                                                                                 \
        if (vk_ > khi) vk_ = khi & ~7;                                                                         \
        v_page = tab[vk_ >> bs_shift];                                                                         \
        _Pragma("unroll") for (int i = 0; i < NL; ++i) {                                                       \
            int k0_ = kb_ + (wave + i * WAVES) * KPL;                                                          \
            if (k0_ > khi) k0_ = khi & ~(KPL - 1);                                                             \
            k_page[i] = tab[k0_ >> bs_shift];                                                                  \
        }                                                                                                      \
    }
#define T32_FETCH(T, BUF)                                                                                      \
    {                                                                                                          \
        const int kb_ = (T) * T32_KEYS;                                                                        \
        int vk_ = kb_ + v_key;                                                                                 \
        if (vk_ > khi) vk_ = khi & ~7;                                                                         \
        const char* gv_ = v_base + (uint64_t)(uint32_t)v_page * v_stride + (vk_ & (bs - 1)) * 2;               \
        _Pragma("unroll") for (int i = 0; i < NL; ++i) {                                                       \
            const int L_ = wave + i * WAVES;                                                                   \
            int k0_ = kb_ + L_ * KPL;                                                                          \
            if (k0_ > khi) k0_ = khi & ~(KPL - 1);                                                             \
            const uint32_t page_ = (uint32_t)__builtin_amdgcn_readfirstlane(k_page[i]);                       \
            const char* sk_ = kc_bytes + (uint64_t)((page_ << bs_shift) + (uint32_t)(k0_ & (bs - 1))) * k_stride; \
            t32_load_to_lds_based(sk_, k_voff, ks + (BUF) * TILE + L_ * 64);                                   \
            t32_load_to_lds(gv_ + (uint64_t)L_ * v_lstep, vs + (BUF) * TILE + L_ * 64);                        \
        }                                                                                                      \
    }
    // every load of this wave has landed (vmcnt 0; the other counters are left alone)
#define T32_LANDED() __builtin_amdgcn_s_waitcnt(0x0f70)

    __syncthreads();                                         // the page ids are in LDS
    T32_PAGES(t_lo)
    T32_FETCH(t_lo, 0)
    T32_PAGES(t_lo < t_hi ? t_lo + 1 : t_hi)
    T32_LANDED();
    __syncthreads();
    int cur = 0;
    for (int t = t_lo; t <= t_hi; ++t) {
        if (t < t_hi) {
            T32_FETCH(t + 1, cur ^ 1)
            T32_PAGES(t + 2 <= t_hi ? t + 2 : t_hi)
        }
        const int kb = t * T32_KEYS;
        if (kb <= wk_hi && kb + T32_KEYS - 1 >= wk_lo) {     // the same for the whole wave
            const bool edge = kb + T32_KEYS - 1 > wk_full_hi || kb < wk_full_lo;
            t32_f32x16 sc[2];
            uint4 pf[4];
            t32_scores<DC>(ks + cur * TILE, koff, qf, sc);
            const float factor = t32_softmax(sc, edge, p_col, lo_col, kb, h, scale2, m_run, l_run, pf);
            if (__any(factor != 1.0f)) {                     // some column's maximum moved
#pragma unroll
                for (int m = 0; m < DT; ++m)
#pragma unroll
                    for (int r = 0; r < 16; ++r) acc[m][r] *= factor;
            }
            t32_weighted_sum<DC>(vs + cur * TILE, voff, pf, acc);
        }
        T32_LANDED();
        __syncthreads();
        cur ^= 1;
    }
#undef T32_FETCH
#undef T32_PAGES
#undef T32_LANDED

    if (!valid) return;
    const float inv = 1.0f / t32_halves_sum(l_run);
    // register r of row tile m is dim 32 m + 8 (r / 4) + 4 h + r % 4: four consecutive dims per store
    bf16_t* op = out + (size_t)row_out * out_stride + (size_t)head * D + 4 * h;
#pragma unroll
    for (int m = 0; m < DT; ++m)
#pragma unroll
        for (int b = 0; b < 4; ++b) {
            uint2 w;
            w.x = t32_pack2(acc[m][4 * b + 0] * inv, acc[m][4 * b + 1] * inv);
            w.y = t32_pack2(acc[m][4 * b + 2] * inv, acc[m][4 * b + 3] * inv);
            *reinterpret_cast<uint2*>(op + 32 * m + 8 * b) = w;
        }
}

// LDS of the kernel for head size d, a table of `pages` page ids and S sequences: 64 KB of tiles
// at a head size of 128
static size_t t32_lds_bytes(int d, int pages, int S) {
    return (size_t)(4 * T32_KEYS * (d / 8)) * sizeof(uint4) + (size_t)(pages + S + 1) * sizeof(int);
}

// Whether the kernel takes a step: head size 64 or 128, pages of a power of two of at least 8
// tokens, and a page table that fits LDS beside the tiles.
extern "C" int tl_attention_tile32_takes(int d, int bs, int NB, int S, int waves) {
    return (d == 64 || d == 128) && bs >= 8 && (bs & (bs - 1)) == 0 && NB > 0 && S >= 0 && (waves == 4 || waves == 8) &&
           t32_lds_bytes(d, NB, S) <= 160 * 1024;
}

// Columns of a work-group of `waves` waves (4 or 8): the caller sizes the grid with it (total_groups =
// the sum over the sequences of ceil(n_s * G / columns), leaving out one-token sequences with skip_single).
extern "C" int tl_attention_tile32_columns(int waves) { return 32 * waves; }

extern "C" int tl_attention_tile32(const void* q, int q_stride, const void* k_cache, const void* v_cache,
                                   const int32_t* tables, int NB, const int32_t* q_start, const int32_t* ctx_start,
                                   void* out, int out_stride, int T, int S, int nq, int nkv, int d, int bs, int window,
                                   float scale, int waves, int total_groups, int skip_single, hipStream_t stream) {
    TL_CHECK_ARG(T >= 0 && S >= 0 && nq > 0 && nkv > 0 && NB > 0, "tl_attention_tile32: bad sizes T=%d S=%d nq=%d nkv=%d NB=%d", T, S, nq, nkv, NB);
    TL_CHECK_ARG(nq % nkv == 0, "tl_attention_tile32: %d query heads are not a multiple of %d key/value heads", nq, nkv);
    TL_CHECK_ARG(tl_attention_tile32_takes(d, bs, NB, S, waves),
                 "tl_attention_tile32: head size %d, page size %d or a page table of %d entries is not served", d, bs, NB);
    TL_CHECK_ARG(q_stride % 8 == 0 && out_stride % 4 == 0 && q_stride >= nq * d && out_stride >= nq * d,
                 "tl_attention_tile32: bad row strides %d, %d", q_stride, out_stride);
    TL_CHECK_ARG(((uintptr_t)q % 16) == 0 && ((uintptr_t)k_cache % 16) == 0 && ((uintptr_t)v_cache % 16) == 0 &&
                     ((uintptr_t)out % 8) == 0, "tl_attention_tile32: operands must be 16-byte aligned");
    TL_CHECK_ARG(nkv <= 65535 && total_groups >= 0 && total_groups <= 65535,
                 "tl_attention_tile32: %d key/value heads or %d column groups are more than a launch takes", nkv, total_groups);
    TL_CHECK_ARG(scale > 0.f, "tl_attention_tile32: the score scale %g must be positive", (double)scale);
    TL_CHECK_ARG((uint64_t)nkv * d * 2 * 8 < (1ull << 31), "tl_attention_tile32: a cache slot of %d heads is too wide", nkv);
    if (T == 0 || S == 0 || total_groups == 0) return 0;
    int bs_shift = 0;
    while ((1 << bs_shift) < bs) ++bs_shift;
    const size_t lds = t32_lds_bytes(d, NB, S);
    dim3 grid(nkv, (unsigned)total_groups, 1);
    const bf16_t *qq = (const bf16_t*)q, *kk = (const bf16_t*)k_cache, *vv = (const bf16_t*)v_cache;
#define T32_LAUNCH(DCV, WV)                                                                                             \
    hipLaunchKernelGGL((attn_tile32_kernel<DCV, WV>), grid, dim3(64 * WV), lds, stream, qq, q_stride, kk, vv, tables, NB, \
                       q_start, ctx_start, (bf16_t*)out, out_stride, S, nq, nkv, bs, bs_shift, window, scale, skip_single)
    if (d == 64 && waves == 4) T32_LAUNCH(2, 4);
    else if (d == 64) T32_LAUNCH(2, 8);
    else if (waves == 4) T32_LAUNCH(4, 4);
    else T32_LAUNCH(4, 8);
#undef T32_LAUNCH
    TL_CHECK_LAUNCH("tl_attention_tile32");
    return 0;
}
