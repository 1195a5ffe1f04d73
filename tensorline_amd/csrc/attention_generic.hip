// The entry point of the any-shape attention (attention_generic_kernel.h) and its float instantiations;
// the bfloat16 ones are compiled in attention_generic_bf16.hip.
#include "attention_generic_kernel.h"

void tl_attention_generic_bf16(const AgLaunch& a);

// q_start: int32 [S + 1], the first row of each sequence in the flat batch (rows of a sequence are
// consecutive); max_query_len: the most tokens one sequence brings to this step.  nsplit > 1 cuts
// the keys into runs of split_keys (a multiple of 64) at absolute positions, one work-group each,
// and a second kernel merges them: for steps of few tokens with long contexts, which would
// otherwise be walked by one work-group per sequence and key/value head.  nsplit * split_keys must
// cover the longest context; ws holds T * nq * nsplit * (d + 2) floats.
extern "C" int tl_attention_generic(const void* q, int q_stride, const void* k_cache, const void* v_cache,
                                    const int32_t* tables, int NB, const int32_t* q_start, const int32_t* pos,
                                    void* out, int out_stride, int dtype, int T, int S, int max_query_len, int nq, int nkv,
                                    int d, int bs, int window, float scale, int nsplit, int split_keys, float* ws,
                                    hipStream_t stream) {
    TL_CHECK_ARG(T >= 0 && S >= 0 && nq > 0 && nkv > 0 && d > 0 && bs > 0 && NB > 0,
                 "tl_attention_generic: bad sizes T=%d S=%d nq=%d nkv=%d d=%d page=%d NB=%d", T, S, nq, nkv, d, bs, NB);
    TL_CHECK_ARG(nq % nkv == 0, "tl_attention_generic: %d query heads are not a multiple of %d key/value heads", nq, nkv);
    TL_CHECK_ARG(d <= 256 && d % 16 == 0, "tl_attention_generic: head size %d must be a multiple of 16 and at most 256", d);
    TL_CHECK_ARG(nkv <= 65535, "tl_attention_generic: too many key/value heads %d", nkv);
    TL_CHECK_ARG(q_stride >= nq * d && out_stride >= nq * d, "tl_attention_generic: row strides too small");
    TL_CHECK_ARG(max_query_len >= 1 || T == 0, "tl_attention_generic: max_query_len %d", max_query_len);
    if (T == 0 || S == 0) return 0;
    const int G = nq / nkv;
    const int GC = (G < AG_ROWS) ? G : AG_ROWS;           // query heads per work-group
    const int QT = AG_ROWS / GC;                          // tokens per work-group
    const int chunks = tl_ceil_div(G, GC);
    TL_CHECK_ARG(nsplit >= 1 && nsplit <= AG_MAX_SPLITS && (long long)chunks * nsplit <= 65535,
                 "tl_attention_generic: %d chunks of query heads x %d key splits are more than a launch takes", chunks, nsplit);
    TL_CHECK_ARG(nsplit == 1 || (ws && split_keys > 0 && split_keys % 64 == 0),
                 "tl_attention_generic: split keys need a workspace and a split length that is a multiple of 64 (%d)", split_keys);
    float* ws_o = ws;
    float* ws_ml = ws ? ws + (size_t)T * nq * nsplit * d : nullptr;
    const int tiles_per_seq = tl_ceil_div(max_query_len, QT);
    const long long groups = (long long)S * tiles_per_seq;
    TL_CHECK_ARG(groups <= 0x7fffffffLL, "tl_attention_generic: too many work-groups");
    // a work-group's rows fit one wave: the waves share the keys of a tile instead (at most one token
    // per work-group then, so that tokens are not held back by the 16-row limit: QT stays as it is)
    const bool keys_over_waves = max_query_len * GC <= AG_WROWS && max_query_len <= QT;
    const int KT = AG_KT(d, keys_over_waves);
    const size_t smem = ag_lds_bytes(d, KT);
    int bs_shift = -1;
    if ((bs & (bs - 1)) == 0)
        for (bs_shift = 0; (1 << bs_shift) < bs;) ++bs_shift;
    TL_CHECK_ARG(smem <= 160 * 1024, "tl_attention_generic: head size %d needs %zu bytes of LDS", d, smem);
    TL_CHECK_ARG(KT * d / 4 <= AG_MAXC * AG_THREADS, "tl_attention_generic: a tile of head size %d has too many pieces", d);
    AgLaunch a;
    a.q = q; a.k_cache = k_cache; a.v_cache = v_cache; a.tables = tables; a.q_start = q_start; a.pos = pos; a.out = out;
    a.ws_o = ws_o; a.ws_ml = ws_ml; a.q_stride = q_stride; a.NB = NB; a.out_stride = out_stride; a.T = T;
    a.tiles_per_seq = tiles_per_seq; a.QT = QT; a.GC = GC; a.nq = nq; a.nkv = nkv; a.d = d; a.bs = bs; a.bs_shift = bs_shift;
    a.window = window; a.nsplit = nsplit; a.split_keys = split_keys; a.scale = scale; a.keys_over_waves = keys_over_waves;
    a.grid = dim3((unsigned)groups, nkv, chunks * nsplit);
    a.smem = smem; a.stream = stream;
    if (dtype == TL_F32)
        ag_launch_all<float>(a);
    else if (dtype == TL_BF16)
        tl_attention_generic_bf16(a);
    else
        return tl_fail("tl_attention_generic: unknown dtype %d", dtype);
    TL_CHECK_LAUNCH("tl_attention_generic");
    return 0;
}
