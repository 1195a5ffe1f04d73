"""The host-side choices of kernels and launch shapes (tensorline_amd/ops/kernels.py): pure functions of
the step's facts and the matrices' shapes, checked here without a GPU.  They decide speed, never a
result beyond rounding; what they must keep is stated per test."""
from tensorline_amd.engine.batch import StepFacts
from tensorline_amd.ops import kernels as K


def test_key_splits_follow_the_batch_and_the_context_and_never_exceed_what_the_merge_takes():
    for seqs in (1, 2, 8, 9, 64, 65, 300):
        for kv in (1, 4, 8):
            last = None
            for ctx in (1, 63, 64, 65, 4096, 4097, 8192, 8193, 32768, 70001, 1 << 20):
                length, n = K._key_splits(seqs, kv, ctx)
                if length == 0:
                    assert n == 1                                   # a large batch fills the GPU unsplit
                    continue
                assert length % 32 == 0 and n == max(1, -(-ctx // length)) and n <= K.MAX_KEY_SPLITS
                assert last is None or length >= last               # longer contexts never get shorter runs
                last = length
    # the runs double where the graphs' context buckets do, and stop at LONG_SPLIT_KEYS until the merge's limit is reached
    assert [K._key_splits(8, 4, c)[0] for c in (4096, 4097, 8193, 16385, 32768, 65536)] == [128, 256, 512, 1024, 1024, 1024]
    assert K._key_splits(1, 4, 4096)[0] == 64 and K._key_splits(64, 4, 4096)[0] == 512
    # fitted to the engine's longest context, a short step cuts as the graph captured for the longest one does
    assert K._fit_key_splits(64, 100, fit_context=1 << 20)[0] == K._fit_key_splits(64, 1 << 20)[0]


def test_one_token_sequences_of_a_step():
    mixed = StepFacts(max_context=900, max_query_len=300, decode_only=False, num_seqs=5, q_lens=[300, 1, 1, 7], starts=[600, 40, 0, 3])
    assert K.one_token_sequences(mixed) == [1, 2, 4]                # the padding sequence too
    decode = StepFacts(max_context=900, max_query_len=1, decode_only=True, num_seqs=3, q_lens=[1, 1, 1], starts=[5, 6, 7])
    assert K.one_token_sequences(decode) == []


def test_one_token_sequences_get_a_launch_of_their_own_only_behind_long_contexts():
    def facts(portion, single_ctx, n_single=8):
        return StepFacts(max_context=max(portion, single_ctx), max_query_len=portion, decode_only=False, num_seqs=1 + n_single,
                         q_lens=[portion] + [1] * n_single, starts=[0] + [single_ctx - 1] * n_single)
    singles = list(range(1, 9))
    assert K._singles_get_own_launch(facts(64, 32768), singles, 28, 4, 128, 0)
    assert K._singles_get_own_launch(facts(2040, 32768), singles, 28, 4, 128, 0)
    assert not K._singles_get_own_launch(facts(64, 1000), singles, 28, 4, 128, 0)
    assert not K._singles_get_own_launch(facts(64, 32768), singles, 28, 4, 128, 512)      # a window bounds their walk


def test_prompt_kernels_by_the_shape_of_the_step():
    # 32 columns per wave: thousands of keys per column and columns enough for 128 work-groups of 256
    assert K._tile32_waves([2048], [30720], 28) == 8
    assert K._tile32_waves([2048], [4096], 28) == 8
    assert K._tile32_waves([2048], [0], 28) == 0                    # a fresh prompt: too few keys per column
    assert K._tile32_waves([300], [30720], 28) == 0                 # too few columns
    assert K._tile32_waves([1, 1, 2048], [9, 9, 30720], 28) == 8    # one-token sequences do not count
    assert K._tile32_waves([1, 1], [5, 6], 28) == 0
    # two chains of tiles: at most one work-group per CU and a walk of 16 tiles or more
    assert K._tile16_chains(56, 4, None, 5120) == 2                 # 1,024 tokens behind 4,096 at 28 / 4 heads
    assert K._tile16_chains(112, 4, None, 2048) == 1                # a fresh prompt of 2,048: 448 work-groups
    assert K._tile16_chains(4, 4, None, 300) == 1                   # short walks
    assert K._tile16_chains(112, 4, "mfma-tile16x2") == 2 and K._tile16_chains(1, 1, "mfma-tile16", 1 << 20) == 1


def test_few_row_products_of_long_k_and_an_unfull_last_round_go_to_the_kernel_that_shares_k():
    assert K._few_rows_go_to_rows64(5120, 13824) and K._few_rows_go_to_rows64(5120, 27648)   # the 14B and 32B down projections
    assert not K._few_rows_go_to_rows64(5120, 5120)                 # K too short to pay for a second kernel
    assert not K._few_rows_go_to_rows64(3584, 18944)                # 224 tiles: one round
    assert not K._few_rows_go_to_rows64(152064, 3584)               # many rounds: the last one hardly matters


def test_head_sizes_the_kernels_take():
    assert [d for d in range(1, 300) if K.attention_takes_head_dim(d)] == list(range(16, 257, 16))
