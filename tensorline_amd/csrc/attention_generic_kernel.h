// Causal attention of the step's tokens over the paged cache, for any head size that is a multiple
// of 16 up to 256, any group size, any page size and both storage types; all arithmetic in float.
// Products run on the matrix cores' float instruction (v_mfma_f32_16x16x4_f32: float in, float
// out, no reduced precision anywhere): this is the attention of the true 32-bit path, and of
// bfloat16 shapes the bfloat16 matrix-core kernel does not take.
//
// A token at position p of sequence s attends to keys [lo, p] of that sequence, lo = 0 or
// p - window + 1 for a windowed layer, found through the sequence's row of the page table.  The
// keys of the step's own tokens are already in the cache when this runs.  k_cache is
// [pages, page, nkv, d]; v_cache is [pages, nkv, d, page] (reference: tensorline/paged_attn.py:25-58,
// tensorline/paged.py:233-238).
//
// One work-group of four waves takes up to AG_ROWS = 64 rows: the (token, query head) pairs of a run
// of consecutive tokens of one sequence's portion and the query heads of one key/value head, a
// wave 16 rows.  Keys are walked in tiles of KT (64 or 32 keys, see AG_KT) that start at
// absolute multiples of KT.  A tile's keys and values are moved in 16-byte pieces, from the cache
// into registers a tile ahead and from there as float into LDS: keys as [key][d], values as
// [d][key], which is how the cache holds a page's values.  A wave computes S = Q K^T for its 16 rows
// in blocks of 16 keys, the softmax of the tile per row (row maximum and sum by butterflies over
// the 16 lanes that hold a row), rescales what it has summed so far (online softmax), passes P
// through LDS into operand layout and adds P V.  Every sum runs in an order fixed by absolute key
// positions, by the row, and by which of three forms the launch takes: rows of prompt portions (a
// wave per 16 rows, a tile's keys in order); a step in which no sequence brings more than one
// token, unsplit (the four waves share the rows and take a block of 16 keys of each tile each,
// put together at the end in the order of the waves); and that step with the keys split into runs
// at absolute positions, added by the merge kernel in ascending order.  The form follows from the
// step (its longest query, whether it only decodes) and from the engine's longest context, never
// from the context of one sequence.  Within a form the result for a position depends neither on
// how the sequence was cut into steps nor on what else is in the batch, to the bit, and a step
// replayed from a graph takes the form of its eager twin; between forms (a token decoded alone,
// or beside another request's prompt portion) results agree within float rounding.
//
// Operand layout of the 16x16x4 product D = A B + C: lane l gives A[l % 16][l / 16] and
// B[l / 16][l % 16]; it holds D[4 (l / 16) + v][l % 16] in register v.  The four k of one product
// need not be neighbours: here lane group g = l / 16 feeds k = 16 kk + 4 g + v to the v-th of four
// products, for A and B alike, so that each lane's four operands are one 16-byte read.
#pragma once
#include "common.h"

#define AG_THREADS 256
#define AG_ROWS 64
#define AG_WROWS 16   // rows per wave

#define AG_MAXC 8     // 16-byte pieces of a tile's keys (and of its values) a thread moves
// keys per tile for head size D: 64 up to a head size of 128 where the waves share the keys of a tile (KW),
// 64 up to a head size of 64 otherwise; else 32, which keeps a work-group's LDS and the registers of its
// pieces on their way small enough for two work-groups to share a CU
#define AG_KT(D, KW) (((D) <= 64 || ((KW) && (D) <= 128)) ? 64 : 32)

template <typename T>
__device__ __forceinline__ float ag_load(const T* p) { return tl_to_float(*p); }

// A 16-byte piece of the cache as floats: four of them, or eight bfloat16.
template <typename T> struct AgPiece;
template <> struct AgPiece<float> {
    static constexpr int E = 4;
    static __device__ __forceinline__ void unpack(const uint4& raw, float* f) {
        f[0] = __uint_as_float(raw.x);
        f[1] = __uint_as_float(raw.y);
        f[2] = __uint_as_float(raw.z);
        f[3] = __uint_as_float(raw.w);
    }
};
template <> struct AgPiece<bf16_t> {
    static constexpr int E = 8;
    static __device__ __forceinline__ void unpack(const uint4& raw, float* f) {
        const uint32_t w[4] = {raw.x, raw.y, raw.z, raw.w};
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            f[2 * i] = __uint_as_float(w[i] << 16);
            f[2 * i + 1] = __uint_as_float(w[i] & 0xffff0000u);
        }
    }
};

typedef float ag_f32x4 __attribute__((ext_vector_type(4)));

// All lanes of a group of 16 get the same bits: every step adds a value to its mirror image.
__device__ __forceinline__ float ag_row16_max(float v) {
#pragma unroll
    for (int off = 8; off > 0; off >>= 1) v = fmaxf(v, __shfl_xor(v, off, TL_WAVE));
    return v;
}
__device__ __forceinline__ float ag_row16_sum(float v) {
#pragma unroll
    for (int off = 8; off > 0; off >>= 1) v += __shfl_xor(v, off, TL_WAVE);
    return v;
}

// LDS: Ks [KT][d + 4] | Vt [d][KT + 4] | Ps [4 waves][16][KT + 4] | row_pos [64] | row_lo [64]
// KW ("keys over waves"): for steps of so few tokens that a work-group's rows fit one wave (at
// most 16 (token, head) pairs: a decoded token and its group of query heads).  All four waves then
// take the same 16 rows and one block of 16 keys of each tile each, instead of three of them
// standing by; a wave keeps its own running maximum, sum and accumulator over its blocks, and the
// four are put together through LDS at the end, in the order of the waves.
template <typename T, int DB, bool KW>    // DB: blocks of 16 head dimensions (d / 16), 1..16
__global__ __launch_bounds__(AG_THREADS) void attn_generic_kernel(
    const T* __restrict__ q, int q_stride, const T* __restrict__ k_cache, const T* __restrict__ v_cache,
    const int32_t* __restrict__ tables, int NB, const int32_t* __restrict__ q_start, const int32_t* __restrict__ pos,
    T* __restrict__ out, int out_stride, int tiles_per_seq, int QT, int GC, int nq, int nkv, int bs, int bs_shift,
    int window, float scale, int nsplit, int split_keys, float* __restrict__ ws_o, float* __restrict__ ws_ml) {
    constexpr int d = DB * 16;
    constexpr int KT = AG_KT(d, KW);
    extern __shared__ float smem[];
    constexpr int ks_ld = d + 4;
    constexpr int vt_ld = KT + 4, ps_ld = KT + 4;
    // the page that holds a key and the key's place in it: a shift and a mask for pages of a power of two
    // of tokens (bs_shift >= 0), which spares the loader two divisions per piece
    auto page_of = [&](int key) { return bs_shift >= 0 ? key >> bs_shift : key / bs; };
    auto in_page = [&](int key) { return bs_shift >= 0 ? key & (bs - 1) : key % bs; };
    float* Ks = smem;
    float* Vt = Ks + KT * ks_ld;
    float* Ps = Vt + d * vt_ld;
    int* row_pos = reinterpret_cast<int*>(Ps + 4 * AG_WROWS * ps_ld);
    int* row_lo = row_pos + AG_ROWS;

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int li = lane & 15, lg = lane >> 4;             // position in the group of 16, and the group
    const int s = blockIdx.x / tiles_per_seq, ti = blockIdx.x - s * tiles_per_seq;
    const int kvh = blockIdx.y;
    const int G = nq / nkv;
    const int chunk = blockIdx.z / nsplit, sp = blockIdx.z - chunk * nsplit;
    const int g0 = chunk * GC;                            // first query head of this chunk within the group
    const int gc = (G - g0 < GC) ? G - g0 : GC;
    const int t_first = q_start[s] + ti * QT, t_end = q_start[s + 1];
    if (t_first >= t_end) return;
    const int nt = (t_end - t_first < QT) ? t_end - t_first : QT;
    const int32_t* table = tables + (size_t)s * NB;

    // rows: r = i * GC + g for token i of the tile and head g of the chunk; others are padding
    if (tid < AG_ROWS) {
        const int i = tid / GC, g = tid - i * GC;
        int p = -1, lo = 0;
        if (i < nt && g < gc) {
            p = pos[t_first + i];
            lo = (window > 0 && p - window + 1 > 0) ? p - window + 1 : 0;
        }
        row_pos[tid] = p;
        row_lo[tid] = lo;
    }
    __syncthreads();

    // the keys any row of the tile sees, [k_lo, k_hi), and those the rows of this wave see
    int k_lo = 0x7fffffff, k_hi = 0, w_lo = 0x7fffffff, w_hi = 0;
    for (int r = 0; r < AG_ROWS; ++r) {
        const int p = row_pos[r];
        if (p < 0) continue;
        const int lo = row_lo[r];
        k_lo = (lo < k_lo) ? lo : k_lo;
        k_hi = (p + 1 > k_hi) ? p + 1 : k_hi;
        if (r / AG_WROWS == (KW ? 0 : wave)) {
            w_lo = (lo < w_lo) ? lo : w_lo;
            w_hi = (p + 1 > w_hi) ? p + 1 : w_hi;
        }
    }

    // A operand of S = Q K^T: this lane's row is li of the wave's 16; scaled queries, kept in registers
    ag_f32x4 qa[DB];
    {
        const int row = (KW ? 0 : wave * AG_WROWS) + li;
        const int i = row / GC, g = row - i * GC;
        const bool real = row_pos[row] >= 0;
        const T* qrow = q + (size_t)(t_first + (real ? i : 0)) * q_stride + (size_t)(kvh * G + g0 + (real ? g : 0)) * d;
#pragma unroll
        for (int kk = 0; kk < DB; ++kk) {
#pragma unroll
            for (int v = 0; v < 4; ++v) qa[kk][v] = real ? ag_load(qrow + 16 * kk + 4 * lg + v) * scale : 0.f;
        }
    }
    // the rows this lane holds of S and of the output: 4 lg + v
    int my_pos[4], my_lo[4];
    float m[4], l[4];
    ag_f32x4 acc[DB];
#pragma unroll
    for (int v = 0; v < 4; ++v) {
        my_pos[v] = row_pos[(KW ? 0 : wave * AG_WROWS) + 4 * lg + v];
        my_lo[v] = row_lo[(KW ? 0 : wave * AG_WROWS) + 4 * lg + v];
        m[v] = -INFINITY;
        l[v] = 0.f;
    }
#pragma unroll
    for (int db = 0; db < DB; ++db) acc[db] = (ag_f32x4){0.f, 0.f, 0.f, 0.f};
    float* Pw = Ps + wave * AG_WROWS * ps_ld;

    // A tile's keys and values travel in 16-byte pieces: from the cache into registers (issued a tile
    // ahead, so the loads are in flight while the tile before is computed), from there as float into LDS.
    // Keys: a piece is E consecutive head dimensions of one key.  Values: E consecutive keys of one
    // head dimension (one page holds them contiguously; needs a page size that is a multiple of E,
    // otherwise values are fetched one by one).
    constexpr int E = AgPiece<T>::E;
    constexpr int cpr = d / E;                             // pieces per key
    constexpr int vpc = KT / E;                            // pieces per head dimension
    constexpr int pieces = KT * cpr;                       // == d * vpc, at most AG_MAXC * AG_THREADS
    const bool v_pieces = (bs % E) == 0;
    uint4 kreg[AG_MAXC], vreg[AG_MAXC];

    // No branch in here: every piece is loaded from a valid address (indices clamped into the range
    // the tile's rows see; what lies outside is zeroed on the way into LDS), so all page lookups are
    // issued together and all cache loads after one wait.
    auto fetch = [&](int k0) {
        int krow[AG_MAXC], vpage[AG_MAXC];
#pragma unroll
        for (int it = 0; it < AG_MAXC; ++it) {
            int qi = tid + it * AG_THREADS;
            qi = (qi < pieces) ? qi : pieces - 1;
            int key = k0 + qi / cpr;
            key = (key < k_hi) ? key : k_hi - 1;
            krow[it] = table[page_of(key)] * bs + in_page(key);
            const int c = qi / vpc;
            int vkey = k0 + (qi - c * vpc) * E;
            vkey = (vkey < k_hi) ? vkey : ((k_hi - 1) / E) * E;
            vpage[it] = table[page_of(vkey)];
        }
#pragma unroll
        for (int it = 0; it < AG_MAXC; ++it) {
            int qi = tid + it * AG_THREADS;
            qi = (qi < pieces) ? qi : pieces - 1;
            const int j = qi / cpr, cc = qi - j * cpr;
            kreg[it] = *reinterpret_cast<const uint4*>(k_cache + ((size_t)krow[it] * nkv + kvh) * d + cc * E);
            if (v_pieces) {
                const int c = qi / vpc;
                int vkey = k0 + (qi - c * vpc) * E;
                vkey = (vkey < k_hi) ? vkey : ((k_hi - 1) / E) * E;
                vreg[it] = *reinterpret_cast<const uint4*>(v_cache + (((size_t)vpage[it] * nkv + kvh) * d + c) * bs + in_page(vkey));
            }
        }
    };
    auto to_lds = [&](int k0) {
#pragma unroll
        for (int it = 0; it < AG_MAXC; ++it) {
            const int qi = tid + it * AG_THREADS;
            if (qi >= pieces) continue;
            float f[E];
            const int j = qi / cpr, cc = qi - j * cpr;
            AgPiece<T>::unpack(kreg[it], f);
            const bool key_seen = k0 + j < k_hi;
#pragma unroll
            for (int e = 0; e < E; e += 4)
                *reinterpret_cast<float4*>(Ks + j * ks_ld + cc * E + e) =
                    key_seen ? make_float4(f[e], f[e + 1], f[e + 2], f[e + 3]) : make_float4(0.f, 0.f, 0.f, 0.f);
            if (v_pieces) {
                const int c = qi / vpc, j0 = (qi - c * vpc) * E;
                AgPiece<T>::unpack(vreg[it], f);
#pragma unroll
                for (int e = 0; e < E; ++e) f[e] = (k0 + j0 + e < k_hi) ? f[e] : 0.f;
#pragma unroll
                for (int e = 0; e < E; e += 4)
                    *reinterpret_cast<float4*>(Vt + c * vt_ld + j0 + e) = make_float4(f[e], f[e + 1], f[e + 2], f[e + 3]);
            }
        }
        if (!v_pieces) {
            for (int idx = tid; idx < KT * d; idx += AG_THREADS) {
                const int c = idx / KT, j = idx - c * KT;
                const int key = k0 + j;
                float v = 0.f;
                if (key < k_hi) {
                    const int page = table[page_of(key)];
                    v = ag_load(v_cache + (((size_t)page * nkv + kvh) * d + c) * bs + in_page(key));
                }
                Vt[c * vt_ld + j] = v;
            }
        }
    };

    // With split keys this work-group walks the tiles of split sp only: keys [sp * split_keys,
    // (sp + 1) * split_keys), a multiple of KT at absolute positions, so that the same keys are summed
    // together whatever the context length and the number of splits of the launch.
    int k_first = (k_lo / KT) * KT, k_end = k_hi;
    if (nsplit > 1) {
        k_first = (k_first > sp * split_keys) ? k_first : sp * split_keys;
        k_end = (k_end < (sp + 1) * split_keys) ? k_end : (sp + 1) * split_keys;
    }
    constexpr int key_blocks = KT / 16;
    if (k_first < k_end) fetch(k_first);
    for (int k0 = k_first; k0 < k_end; k0 += KT) {
        to_lds(k0);
        __syncthreads();
        if (k0 + KT < k_end) fetch(k0 + KT);

        // a tile none of the wave's rows sees is skipped; KW: a wave without a key block of its own stands by
        if (k0 < w_hi && k0 + KT > w_lo && (!KW || wave < key_blocks)) {
            // ---- S = Q K^T: per block of 16 keys, 4 DB products; lane holds rows 4 lg + v, key li ----
            ag_f32x4 sblk[4];
#pragma unroll
            for (int jb = 0; jb < (KW ? 1 : 4); ++jb) {          // KW: sblk[0] is key block `wave`
                sblk[jb] = (ag_f32x4){0.f, 0.f, 0.f, 0.f};
                if (KW || jb < key_blocks) {
                    const float* kr = Ks + ((KW ? wave : jb) * 16 + li) * ks_ld + 4 * lg;
#pragma unroll
                    for (int kk = 0; kk < DB; ++kk) {
                        const float4 kb = *reinterpret_cast<const float4*>(kr + 16 * kk);
                        sblk[jb] = __builtin_amdgcn_mfma_f32_16x16x4f32(qa[kk][0], kb.x, sblk[jb], 0, 0, 0);
                        sblk[jb] = __builtin_amdgcn_mfma_f32_16x16x4f32(qa[kk][1], kb.y, sblk[jb], 0, 0, 0);
                        sblk[jb] = __builtin_amdgcn_mfma_f32_16x16x4f32(qa[kk][2], kb.z, sblk[jb], 0, 0, 0);
                        sblk[jb] = __builtin_amdgcn_mfma_f32_16x16x4f32(qa[kk][3], kb.w, sblk[jb], 0, 0, 0);
                    }
                }
            }
            // ---- softmax over the tile, per row; rescale what was summed so far ----------------------
#pragma unroll
            for (int v = 0; v < 4; ++v) {
                float sv[4], mx = -INFINITY;
#pragma unroll
                for (int jb = 0; jb < 4; ++jb) {
                    if (KW && jb > 0) {
                        sv[jb] = -INFINITY;
                        continue;
                    }
                    const int key = k0 + (KW ? wave : jb) * 16 + li;
                    const bool seen = (KW || jb < key_blocks) && my_pos[v] >= 0 && key <= my_pos[v] && key >= my_lo[v];
                    sv[jb] = seen ? sblk[jb][v] : -INFINITY;
                    mx = fmaxf(mx, sv[jb]);
                }
                const float m_new = fmaxf(m[v], ag_row16_max(mx));
                float alpha = 1.f, psum = 0.f;
                if (m_new > -INFINITY) {                   // else: the row sees no key yet
                    alpha = expf(m[v] - m_new);            // exp(-inf) = 0 for the first tile the row sees
#pragma unroll
                    for (int jb = 0; jb < 4; ++jb) {
                        sv[jb] = (sv[jb] > -INFINITY) ? expf(sv[jb] - m_new) : 0.f;
                        psum += sv[jb];
                    }
                } else {
#pragma unroll
                    for (int jb = 0; jb < 4; ++jb) sv[jb] = 0.f;
                }
                l[v] = l[v] * alpha + ag_row16_sum(psum);
                m[v] = m_new;
#pragma unroll
                for (int db = 0; db < DB; ++db) acc[db][v] *= alpha;
#pragma unroll
                for (int jb = 0; jb < (KW ? 1 : 4); ++jb)
                    if (KW || jb < key_blocks) Pw[(4 * lg + v) * ps_ld + (KW ? wave : jb) * 16 + li] = sv[jb];
            }
            // Pw is written and read by this wave only; LDS operations of a wave complete in order
            __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
            __builtin_amdgcn_wave_barrier();
            __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
            // ---- O += P V: A = P (row li, keys 16 kk + 4 lg + v), B = values (keys likewise, dimension li) ----
#pragma unroll
            for (int kq = 0; kq < (KW ? 1 : 4); ++kq) {
                const int kk = KW ? wave : kq;
                if (KW || kk < key_blocks) {
                    const float4 pa = *reinterpret_cast<const float4*>(Pw + li * ps_ld + 16 * kk + 4 * lg);
#pragma unroll
                    for (int db = 0; db < DB; ++db) {
                        const float4 vb = *reinterpret_cast<const float4*>(Vt + (db * 16 + li) * vt_ld + 16 * kk + 4 * lg);
                        acc[db] = __builtin_amdgcn_mfma_f32_16x16x4f32(pa.x, vb.x, acc[db], 0, 0, 0);
                        acc[db] = __builtin_amdgcn_mfma_f32_16x16x4f32(pa.y, vb.y, acc[db], 0, 0, 0);
                        acc[db] = __builtin_amdgcn_mfma_f32_16x16x4f32(pa.z, vb.z, acc[db], 0, 0, 0);
                        acc[db] = __builtin_amdgcn_mfma_f32_16x16x4f32(pa.w, vb.w, acc[db], 0, 0, 0);
                    }
                }
            }
        }
        __syncthreads();                                   // the tile is used up: the next one may be loaded
    }

    if (KW) {
        // The waves' results for the same 16 rows -> LDS (the tiles are used up), then wave 0 adds them in
        // the order of the waves: M = max m_w, l = sum l_w e^(m_w - M), acc = sum acc_w e^(m_w - M).
        float* cacc = smem;                                  // [wave][row][d]: 4 * 16 * d floats, within Ks and Vt
        float* cml = Ps;                                     // [wave][row][2]
        constexpr int NW = key_blocks < 4 ? key_blocks : 4;  // waves that had a key block
        if (wave < NW) {
#pragma unroll
            for (int v = 0; v < 4; ++v) {
                const int row = 4 * lg + v;
#pragma unroll
                for (int db = 0; db < DB; ++db) cacc[(wave * AG_WROWS + row) * d + db * 16 + li] = acc[db][v];
                if (li == 0) {
                    cml[(wave * AG_WROWS + row) * 2] = m[v];
                    cml[(wave * AG_WROWS + row) * 2 + 1] = l[v];
                }
            }
        }
        __syncthreads();
        if (wave != 0) return;
#pragma unroll
        for (int v = 0; v < 4; ++v) {
            const int row = 4 * lg + v;
            float M = -INFINITY;
#pragma unroll
            for (int w = 0; w < NW; ++w) M = fmaxf(M, cml[(w * AG_WROWS + row) * 2]);
            float lsum = 0.f;
#pragma unroll
            for (int db = 0; db < DB; ++db) acc[db][v] = 0.f;
#pragma unroll
            for (int w = 0; w < NW; ++w) {
                const float mw = cml[(w * AG_WROWS + row) * 2];
                const float f = (mw > -INFINITY) ? expf(mw - M) : 0.f;   // a wave that saw no key of the row: nothing
                lsum += f * cml[(w * AG_WROWS + row) * 2 + 1];
#pragma unroll
                for (int db = 0; db < DB; ++db) acc[db][v] += f * cacc[(w * AG_WROWS + row) * d + db * 16 + li];
            }
            m[v] = M;
            l[v] = lsum;
        }
    }
    // this lane holds output rows 4 lg + v at head dimensions 16 db + li
    if (nsplit > 1) {
        // the split's sums as they are, with their maximum and denominator (a split that holds no key
        // of a row leaves -inf, 0 and zeros); attn_generic_merge_kernel puts the splits together
#pragma unroll
        for (int v = 0; v < 4; ++v) {
            if (my_pos[v] < 0) continue;
            const int row = wave * AG_WROWS + 4 * lg + v;
            const int i = row / GC, g = row - i * GC;
            const size_t part = ((size_t)(t_first + i) * nq + (kvh * G + g0 + g)) * nsplit + sp;
#pragma unroll
            for (int db = 0; db < DB; ++db) ws_o[part * d + db * 16 + li] = acc[db][v];
            if (li == 0) {
                ws_ml[part * 2] = m[v];
                ws_ml[part * 2 + 1] = l[v];
            }
        }
        return;
    }
#pragma unroll
    for (int v = 0; v < 4; ++v) {
        if (my_pos[v] < 0) continue;
        const int row = wave * AG_WROWS + 4 * lg + v;
        const int i = row / GC, g = row - i * GC;
        const float inv = (l[v] > 0.f) ? 1.f / l[v] : 0.f;
        T* orow = out + (size_t)(t_first + i) * out_stride + (size_t)(kvh * G + g0 + g) * d;
#pragma unroll
        for (int db = 0; db < DB; ++db) orow[db * 16 + li] = tl_from_float<T>(acc[db][v] * inv);
    }
}

// out[t, h, :] = sum_s w_s acc_s / sum_s w_s l_s with w_s = exp(m_s - max m), over the splits in
// ascending order (a split without keys of the row has l_s = 0, sums of zero and the weight 0).
// One work-group per (row, head).  First a thread per split: its maximum and denominator, the
// largest maximum over the group, its weight; then a thread per head dimension adds the splits'
// sums, eight loads in flight at a time.  Nothing waits for a load that another load depends on.
#define AG_MAX_SPLITS 1024
__device__ __forceinline__ float ag_group_max(float v, float* red) {   // red: one float per wave
    for (int off = 32; off > 0; off >>= 1) v = fmaxf(v, __shfl_xor(v, off, TL_WAVE));
    if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = v;
    __syncthreads();
    float r = red[0];
    for (int w = 1; w < (int)(blockDim.x >> 6); ++w) r = fmaxf(r, red[w]);
    return r;
}
template <typename T>
__global__ __launch_bounds__(256) void attn_generic_merge_kernel(const float* __restrict__ ws_o,
                                                                 const float* __restrict__ ws_ml, T* __restrict__ out,
                                                                 int out_stride, int nq, int d, int nsplit) {
    __shared__ float wgt[AG_MAX_SPLITS], wl[AG_MAX_SPLITS], red[4];
    const int t = blockIdx.x, h = blockIdx.y, tid = threadIdx.x;
    const size_t base = ((size_t)t * nq + h) * nsplit;
    const float2* ml = reinterpret_cast<const float2*>(ws_ml) + base;
    float2 mine[AG_MAX_SPLITS / 256];
    float mx = -INFINITY;
#pragma unroll
    for (int i = 0; i < AG_MAX_SPLITS / 256; ++i) {
        const int sp = tid + i * 256;
        mine[i] = sp < nsplit ? ml[sp] : make_float2(-INFINITY, 0.f);
        if (mine[i].y > 0.f) mx = fmaxf(mx, mine[i].x);
    }
    const float M = ag_group_max(mx, red);
#pragma unroll
    for (int i = 0; i < AG_MAX_SPLITS / 256; ++i) {
        const int sp = tid + i * 256;
        if (sp < nsplit) {
            const float w = mine[i].y > 0.f ? expf(mine[i].x - M) : 0.f;
            wgt[sp] = w;
            wl[sp] = w * mine[i].y;
        }
    }
    __syncthreads();
    if (tid >= d) return;
    float den = 0.f;
    for (int sp = 0; sp < nsplit; ++sp) den += wl[sp];
    const float* acc = ws_o + base * d + tid;
    float num = 0.f;
    for (int s0 = 0; s0 < nsplit; s0 += 8) {
        float a[8];
#pragma unroll
        for (int j = 0; j < 8; ++j) a[j] = acc[(size_t)(s0 + j < nsplit ? s0 + j : nsplit - 1) * d];
#pragma unroll
        for (int j = 0; j < 8; ++j)
            if (s0 + j < nsplit) num += wgt[s0 + j] * a[j];
    }
    out[(size_t)t * out_stride + (size_t)h * d + tid] = tl_from_float<T>(den > 0.f ? num / den : 0.f);
}

static size_t ag_lds_bytes(int d, int KT) {
    return sizeof(float) * ((size_t)KT * (d + 4) + (size_t)d * (KT + 4) + 4 * AG_WROWS * (KT + 4)) + sizeof(int) * (2 * AG_ROWS);
}

// What the launches of one storage type need; filled in by tl_attention_generic.
struct AgLaunch {
    const void *q, *k_cache, *v_cache;
    const int32_t *tables, *q_start, *pos;
    void* out;
    float *ws_o, *ws_ml;
    int q_stride, NB, out_stride, T, tiles_per_seq, QT, GC, nq, nkv, d, bs, bs_shift, window, nsplit, split_keys;
    float scale;
    bool keys_over_waves;
    dim3 grid;
    size_t smem;
    hipStream_t stream;
};

// The kernel for head size 16 DB with keys over waves or not, then the merge of the splits: every
// instantiation of one storage type.  Each storage type has a source file of its own that instantiates
// this (attention_generic.hip: float, attention_generic_bf16.hip: bfloat16), so that the two halves of
// the instantiations compile side by side.
template <typename TT>
static void ag_launch_all(const AgLaunch& a) {
    const dim3 block(AG_THREADS);
#define AG_LAUNCH_KW(DB, KWV)                                                                                         \
    hipLaunchKernelGGL((attn_generic_kernel<TT, DB, KWV>), a.grid, block, a.smem, a.stream, (const TT*)a.q,           \
                       a.q_stride, (const TT*)a.k_cache, (const TT*)a.v_cache, a.tables, a.NB, a.q_start, a.pos,      \
                       (TT*)a.out, a.out_stride, a.tiles_per_seq, a.QT, a.GC, a.nq, a.nkv, a.bs, a.bs_shift, a.window, \
                       a.scale, a.nsplit, a.split_keys, a.ws_o, a.ws_ml)
#define AG_CASE(DB)                                                                                                   \
    case DB:                                                                                                          \
        if (a.keys_over_waves) AG_LAUNCH_KW(DB, true); else AG_LAUNCH_KW(DB, false);                                  \
        break;
    switch (a.d / 16) {
        AG_CASE(1) AG_CASE(2) AG_CASE(3) AG_CASE(4) AG_CASE(5) AG_CASE(6) AG_CASE(7) AG_CASE(8)
        AG_CASE(9) AG_CASE(10) AG_CASE(11) AG_CASE(12) AG_CASE(13) AG_CASE(14) AG_CASE(15) AG_CASE(16)
    }
#undef AG_CASE
#undef AG_LAUNCH_KW
    if (a.nsplit > 1)
        hipLaunchKernelGGL(attn_generic_merge_kernel<TT>, dim3(a.T, a.nq), dim3(256), 0, a.stream, a.ws_o, a.ws_ml,
                           (TT*)a.out, a.out_stride, a.nq, a.d, a.nsplit);
}
