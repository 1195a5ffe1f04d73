"""The cache manager on host data: pages per group, tables, windows, state slots, prefix sharing.
No page is lost, held twice or freed twice, under random orders of requests."""
import random

import pytest
import torch
from hypothesis import given, settings, strategies as st

from tensorline_amd.cache.allocator import PagePool, page_key
from tensorline_amd.cache.manager import CacheManager
from tensorline_amd.parts.spec import keys_and_values, ScheduleEntry, StateNeed


def test_allocator_refcount_lru_and_eviction():
    # the sequence of the reference's own test (tests/test_prefix_cache.py:8-22)
    a = PagePool(4)
    x = a.take(2)
    h0 = page_key(None, [1, 2])
    a.publish(x[0], h0)
    a.give_back(x)
    assert a.num_free == 4 and a.num_cached == 1          # freed but still cached
    assert a.revive(h0) == x[0] and a.num_free == 3       # revived from the free list
    assert a.revive(h0) == x[0]                           # shared: two references
    a.give_back([x[0]])
    assert a.num_free == 3                                # still referenced once
    a.give_back([x[0]])
    assert a.num_free == 4
    a.take(4)                                         # memory pressure evicts it
    assert a.num_cached == 0 and a.revive(h0) is None


def test_allocator_details():
    assert page_key(page_key(None, [1]), [2]) != page_key(page_key(None, [9]), [2])   # chained over the prefix
    a = PagePool(3)
    assert a.take(4) is None and a.num_free == 3      # all or nothing
    x = a.take(3)
    a.give_back([x[1]])
    with pytest.raises(AssertionError, match="double free"):
        a.give_back([x[1]])
    a.give_back([x[0], x[2]])                                  # reversed: the tail page is handed out first
    assert a.take(1) == [x[1]] and a.take(1) == [x[2]]
    b = PagePool(2)
    y = b.take(1)
    b.publish(y[0], 5, contents=(None, (1, 2)))
    assert b.revive(5, contents=(None, (9, 9))) is None    # same hash, other tokens: no hit
    assert b.revive(5, contents=(None, (1, 2))) == y[0]
    b.check({y[0]: 2})


@settings(max_examples=60, deadline=None)
@given(st.lists(st.tuples(st.sampled_from(["take", "give", "publish", "revive"]), st.integers(0, 7)), max_size=80))
def test_pool_hands_out_in_the_order_of_return_whatever_leaves_the_middle_of_the_queue(ops):
    """The pool against a plain list as the queue: same pages in the same order, a published page
    found while it waits and gone once it is handed out for something else."""
    n = 6
    pool, queue, holders, key_of = PagePool(n), list(range(n)), [0] * n, {}
    held: list[int] = []
    for op, x in ops:
        if op == "take":
            k = x % 4
            got = pool.take(k)
            if k > len(queue):
                assert got is None
            else:
                want, queue = queue[:k], queue[k:]
                assert got == want
                for p in want:
                    holders[p] = 1
                    key_of = {key: q for key, q in key_of.items() if q != p}
                held += want
        elif op == "give" and held:
            p = held.pop(x % len(held))
            pool.give_back([p])
            holders[p] -= 1
            if holders[p] == 0:
                queue.append(p)
        elif op == "publish" and held:
            p = held[x % len(held)]
            if x not in key_of and p not in key_of.values():
                key_of[x] = p
            pool.publish(p, x)
        elif op == "revive":
            got = pool.revive(x)
            assert got == key_of.get(x)
            if got is not None:
                if holders[got] == 0:
                    queue.remove(got)
                holders[got] += 1
                held.append(got)
        pool.check({p: c for p, c in enumerate(holders) if c})
        assert pool.num_free == len(queue) and pool.num_cached == len(key_of)


def manager(needs, schedule=None, states=None, **kw):
    schedule = schedule or [ScheduleEntry(i) for i in range(len(needs))]
    states = states or [None] * len(needs)
    args = dict(page_size=4, num_blocks=16, max_requests=4, dtype=torch.float32, device="cpu")
    args.update(kw)
    return CacheManager(needs, schedule, states, **args)


def test_groups_tables_and_storage():
    full, win = keys_and_values(2, 8), keys_and_values(2, 8, window=6)
    m = manager([full, win, full, None], states=[None, None, None, StateNeed((5,))])
    assert len(m.groups) == 2 and m.group_of_entry == [0, 1, 0, None]
    assert m.groups[0].entries == [0, 2] and m.groups[1].entries == [1]
    k, v = m.storage(2)["k"], m.storage(2)["v"]
    assert tuple(k.shape) == (17, 4, 2, 8) and tuple(v.shape) == (17, 2, 8, 4)     # one scratch page; V transposed
    assert m.storage(3) == {} and tuple(m.state[3].shape) == (5, 5)
    per_page = CacheManager.bytes_per_page([full, win, full, None], [ScheduleEntry(i) for i in range(4)], 4, 2)
    assert per_page == 3 * 2 * 4 * 2 * 8 * 2
    assert m.add_request("a") is not None
    assert m.grow("a", 9) and m.table("a", 0) == m.table("a", 0)[:3] and len(m.table("a", 1)) == 3
    assert m.num_free(0) == 13 and m.num_free(1) == 13
    assert m.grow("a", 9) and m.num_free(0) == 13                                  # nothing more to take
    m.check()
    m.release("a")
    assert m.all_free()


def test_window_pages_are_given_back_and_used_again():
    m = manager([keys_and_values(1, 8), keys_and_values(1, 8, window=6)], num_blocks=6)
    m.add_request("a")
    computed = 0
    for n in (5, 4, 3, 7, 1, 1, 1):
        assert m.grow("a", computed + n)
        computed += n
        m.trim("a", computed)
        m.check()
        tab = m.table("a", 1)
        first_needed = computed - 6 + 1
        for lp, blk in enumerate(tab):
            assert (blk == -1) == ((lp + 1) * 4 <= first_needed), (lp, computed)    # exactly the pages the window passed
        assert all(b >= 0 for b in m.table("a", 0))                                 # the full group keeps everything
    assert computed == 22 and len(m.table("a", 0)) == 6
    assert m.num_free(1) >= 3            # 22 tokens in 6 pages of 4: the windowed group never holds more than 3 at rest
    assert m.can_ever_hold(200, step_tokens=4) is False and manager([keys_and_values(1, 8, window=6)], num_blocks=6).can_ever_hold(200, 4)
    m.release("a")
    assert m.all_free()


def test_shared_cache_entry_and_bad_schedules():
    need = keys_and_values(2, 8)
    m = manager([need, need], schedule=[ScheduleEntry(0), ScheduleEntry(0, cache_from=0)])
    assert m.group_of_entry == [0, 0] and m.storage(1)["k"] is m.storage(0)["k"] and not m.owns_storage(1)
    with pytest.raises(ValueError, match="something else per token"):
        manager([need, keys_and_values(1, 8)], schedule=[ScheduleEntry(0), ScheduleEntry(0, cache_from=0)])
    with pytest.raises(ValueError, match="further back"):
        manager([keys_and_values(2, 8, window=4), need], schedule=[ScheduleEntry(0), ScheduleEntry(0, cache_from=0)])


def test_state_slots():
    m = manager([None], states=[StateNeed((3,))], max_requests=2)
    s0, s1 = m.add_request("a"), m.add_request("b")
    assert {s0, s1} == {0, 1} and m.add_request("c") is None and m.scratch_slot == 2
    m.state[0][s0].fill_(7.0)
    m.release("a")
    assert m.add_request("c") == s0 and torch.all(m.state[0][s0] == 0)              # handed out again from zero
    with pytest.raises(KeyError):
        m.add_request("c")
    m.check()


def test_prefix_sharing_through_the_manager():
    m = manager([keys_and_values(1, 8)], prefix_caching=True)
    toks = list(range(11))
    m.add_request("a")
    assert m.match_prefix("a", toks) == 0 and m.grow("a", 11)
    m.publish("a", toks, 11)                                                        # two full pages are published
    m.add_request("b")
    assert m.match_prefix("b", toks[:8] + [99, 98]) == 8
    assert m.table("b")[:2] == m.table("a")[:2]
    m.check()
    m.add_request("c")
    assert m.match_prefix("c", toks[:8]) == 4                                       # fully cached: the last page is recomputed
    m.release("a"); m.release("b"); m.release("c")
    assert m.all_free() and m.groups[0].allocator.num_cached == 2                   # free, and still there for the next request
    m.add_request("d")
    assert m.match_prefix("d", toks) == 8
    m.release("d")
    # windows or state switch it off
    assert not manager([keys_and_values(1, 8, window=4)], prefix_caching=True).prefix_caching
    assert not manager([keys_and_values(1, 8), None], states=[None, StateNeed((2,))], prefix_caching=True).prefix_caching


@settings(max_examples=60, deadline=None)
@given(seed=st.integers(0, 10 ** 6), window=st.sampled_from([0, 5, 9]), prefix=st.booleans())
def test_random_orders_keep_every_page_accounted_for(seed, window, prefix):
    rng = random.Random(seed)
    needs = [keys_and_values(1, 8), keys_and_values(1, 8, window=window)] if window else [keys_and_values(1, 8)]
    m = manager(needs, num_blocks=12, max_requests=3, prefix_caching=prefix, allocate_storage=False)
    live: dict[int, int] = {}
    toks = {}
    next_id = 0
    for _ in range(80):
        op = rng.random()
        if op < 0.25 and len(live) < 3:
            assert m.add_request(next_id) is not None
            toks[next_id] = [rng.randrange(3) for _ in range(40)]
            live[next_id] = m.match_prefix(next_id, toks[next_id][:rng.randrange(1, 30)])
            next_id += 1
        elif op < 0.8 and live:
            rid = rng.choice(list(live))
            n = rng.randrange(1, 9)
            before = [list(m.table(rid, g)) for g in range(len(m.groups))]
            free_before = [m.num_free(g) for g in range(len(m.groups))]
            if live[rid] + n <= 40 and m.grow(rid, live[rid] + n):
                live[rid] += n
                m.publish(rid, toks[rid], live[rid])
                m.trim(rid, live[rid])
            else:                                               # a failed grow changes nothing
                assert [list(m.table(rid, g)) for g in range(len(m.groups))] == before
                assert [m.num_free(g) for g in range(len(m.groups))] == free_before
        elif live:
            rid = rng.choice(list(live))
            m.release(rid)
            del live[rid]
        m.check()
    for rid in list(live):
        m.release(rid)
    m.check()
    assert m.all_free()


def test_a_mixer_may_declare_any_planes_and_the_manager_only_lays_them_out():
    """Not keys and values: one compressed vector per token kept in the cache's dtype and a float32
    score per token and head, the latter with a page's tokens innermost.  The manager allocates what
    is declared, counts its bytes, and groups entries by equal declarations."""
    from tensorline_amd.parts.spec import CacheNeed, CachePlane
    latent = CacheNeed((CachePlane("latent", (24,)), CachePlane("gate", (3,), token_axis="last", dtype="float32")))
    kv = keys_and_values(2, 8)
    m = manager([latent, kv, latent], dtype=torch.bfloat16, page_size=4, num_blocks=5)
    assert m.group_of_entry == [0, 1, 0] and len(m.groups) == 2
    planes = m.storage(2)
    assert set(planes) == {"latent", "gate"} and planes["latent"] is not m.storage(0)["latent"]
    assert tuple(planes["latent"].shape) == (6, 4, 24) and planes["latent"].dtype == torch.bfloat16
    assert tuple(planes["gate"].shape) == (6, 3, 4) and planes["gate"].dtype == torch.float32
    assert set(m.storage(1)) == {"k", "v"}
    sched = [ScheduleEntry(i) for i in range(3)]
    assert CacheManager.bytes_per_page([latent, kv, latent], sched, 4, 2) == 2 * 4 * (24 * 2 + 3 * 4) + 4 * 2 * (2 * 8) * 2
    with pytest.raises(ValueError):
        CacheNeed(())
    with pytest.raises(ValueError):
        CacheNeed((CachePlane("a", (2,)), CachePlane("a", (3,))))
    with pytest.raises(ValueError):
        CachePlane("a", (2,), token_axis="middle")
