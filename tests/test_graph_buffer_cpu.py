"""The replayed decode step's host buffer: bringing it up to date in place gives what packing the
step again gives, and is not done when it would be wrong (host data only, no GPU)."""
import numpy as np
import pytest
import torch

from tensorline_amd.cache.manager import CacheManager
from tensorline_amd.engine.batch import StepEntry
from tensorline_amd.engine.graphs import GraphRunner, _Captured
from tensorline_amd.parts.spec import keys_and_values, ScheduleEntry


class _Model:
    vocab_size = 1000
    device = "cpu"
    schedule = [ScheduleEntry(0)]


def _setup(window=0, page=4, max_blocks=8):
    cache = CacheManager([keys_and_values(1, 8, window)], [ScheduleEntry(0)], [None], page_size=page, num_blocks=40,
                         max_requests=4, dtype=torch.float32, device="cpu", allocate_storage=False)
    runner = GraphRunner(_Model(), cache, max_batch=4, max_blocks_per_seq=max_blocks)
    return cache, runner


def _cap(runner, entries, B=4):
    packed = runner.pack(entries, pad_seqs=B, pad_nb=[runner.max_blocks])
    host = torch.from_numpy(packed.data.copy())
    cap = _Captured(None, None, host, None, packed)
    cap.rids = tuple(e.rid for e in entries)
    cap.admissions = tuple(runner.cache.admission(r) for r in cap.rids)
    cap.starts = np.array([e.start for e in entries], np.int64)
    return cap


def test_in_place_update_equals_packing_again():
    cache, runner = _setup()
    lens = {"a": 3, "b": 7, "c": 4}
    for rid, n in lens.items():
        cache.add_request(rid)
        assert cache.grow(rid, n + 1)
    entries = [StepEntry(rid, [5], n, [0]) for rid, n in lens.items()]
    cap = _cap(runner, entries)
    rng = np.random.default_rng(0)
    for step in range(1, 14):                                 # crosses several page boundaries
        entries = []
        for rid in lens:
            lens[rid] += 1
            assert cache.grow(rid, lens[rid] + 1)
            entries.append(StepEntry(rid, [int(rng.integers(0, 1000))], lens[rid], [0]))
        assert runner._advance(cap, entries)
        want = runner.pack(entries, pad_seqs=4, pad_nb=[runner.max_blocks]).data
        np.testing.assert_array_equal(cap.host.numpy(), want)


def test_in_place_update_declines_when_the_buffer_is_stale():
    cache, runner = _setup()
    for rid in "ab":
        cache.add_request(rid)
        cache.grow(rid, 6)
    entries = [StepEntry("a", [1], 5, [0]), StepEntry("b", [2], 5, [0])]
    cap = _cap(runner, entries)
    before = cap.host.numpy().copy()
    nxt = [StepEntry("a", [1], 6, [0]), StepEntry("b", [2], 6, [0])]
    cache.grow("a", 7), cache.grow("b", 7)
    assert not runner._advance(cap, nxt[::-1])                # other order of rows
    assert not runner._advance(cap, nxt[:1])                  # fewer requests
    assert not runner._advance(cap, [StepEntry("a", [1], 7, [0]), nxt[1]])   # a request moved two tokens
    cache.release("a")                                        # given back and admitted again: other pages
    cache.add_request("a")
    cache.grow("a", 7)
    assert not runner._advance(cap, nxt)
    np.testing.assert_array_equal(cap.host.numpy(), before)   # declining touches nothing
    with pytest.raises(ValueError, match="token id"):
        cap2 = _cap(runner, entries)
        runner._advance(cap2, [StepEntry("a", [1000], 6, [0]), nxt[1]])


def test_in_place_update_is_off_for_windowed_caches():
    cache, runner = _setup(window=6)
    cache.add_request("a")
    cache.grow("a", 6)
    cap = _cap(runner, [StepEntry("a", [1], 5, [0])])
    cache.grow("a", 7)
    assert not runner._advance(cap, [StepEntry("a", [1], 6, [0])])


def test_key_splits_follow_the_batch_and_the_context_bucket():
    """A graph is captured for a context bucket, an eager step sees the real context: both must cut
    the keys into the same runs.  The length of a split follows the batch and doubles with the
    context where the buckets do (4,096, 8,192, ...), up to 1,024 keys; beyond that, and for split
    lengths the caller forces, it is fitted to the engine's longest context so that no launch has
    more splits than the merge takes."""
    from tensorline_amd.ops.kernels import LONG_SPLIT_KEYS, MAX_KEY_SPLITS, _fit_key_splits, _key_splits
    assert _key_splits(1, 4, 3000) == (64, 47)
    assert _key_splits(1, 4, 4096) == (64, 64) and _key_splits(1, 4, 4097) == (128, 33)
    assert _key_splits(1, 4, 5000) == _key_splits(1, 4, 5000, fit_context=8192) == (128, 40)
    assert _key_splits(1, 4, 8192)[0] == _key_splits(1, 4, 4200)[0] == 128        # a live context and its bucket cut alike
    assert _key_splits(8, 4, 32768) == (1024, 32) and _key_splits(8, 4, 32784)[0] == LONG_SPLIT_KEYS
    assert _key_splits(64, 4, 32768) == (1024, 32)                                # 512 by the batch, capped
    assert _key_splits(1, 4, 10 ** 6)[0] == LONG_SPLIT_KEYS
    long = 64 * MAX_KEY_SPLITS * 2                        # a forced length: twice what 1,024 splits of 64 keys cover
    assert _fit_key_splits(64, long, long) == (128, MAX_KEY_SPLITS) and _fit_key_splits(64, 3000, long) == (128, 24)
    assert _fit_key_splits(64, 3000) == (64, 47)          # without the hint only the step's own context counts
    assert _fit_key_splits(0, 10 ** 6, 10 ** 7) == (0, 1)
