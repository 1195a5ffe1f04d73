"""The scheduler's decisions and the engine loop, on the CPU with kernel stand-ins: generated
tokens must equal the plain implementation's one-request-at-a-time greedy tokens in every regime
of the reference's batching test (tests/test_batching.py:67-92)."""
import pytest
import torch

from tensorline_amd.cache.manager import CacheManager
from tensorline_amd.engine.engine import InferenceEngine
from tensorline_amd.engine.loading import load_model
from tensorline_amd.engine.scheduler import Request, RequestError, Scheduler
from tensorline_amd.parts.spec import keys_and_values, ScheduleEntry
from tensorline_amd.sampling.params import GenStats, SamplingParams
from tests import helpers, plain

NO_STOP = {-1}


@pytest.fixture(scope="module")
def tiny(tmp_path_factory):
    d = helpers.make_model_dir(tmp_path_factory, "A", seed=2)
    w, cfg = plain.load_folder(d)
    prompts = helpers.prompts_for("A", [1, 9, 3, 12, 2, 7, 2, 5], seed=1)
    want = {(i, mt): plain.greedy_generate(w, cfg, p, mt) for i, p in enumerate(prompts) for mt in (5, 17)}
    return d, prompts, want


def make_engine(d, num_blocks=256, block_size=16, prefix_caching=False, **kw):
    model, _ = load_model(d, "float32", "cpu")
    cache = CacheManager(model.cache_needs(), model.schedule, model.state_needs(), page_size=block_size,
                         num_blocks=num_blocks, max_requests=kw.get("max_num_seqs", 64), dtype=torch.float32,
                         device="cpu", prefix_caching=prefix_caching)
    return InferenceEngine(model, cache, **kw)


@pytest.mark.parametrize("kw", [
    dict(),
    dict(max_batched_tokens=4),                 # chunked prefill
    dict(num_blocks=12, block_size=4),          # preemption and recompute
    dict(max_num_seqs=2),                       # queueing
    dict(prefix_caching=True, block_size=4, max_num_seqs=3),    # shared prefixes change no token
], ids=["plain", "chunked-prefill", "preemption", "seq-limit", "prefix-cache"])
def test_batched_matches_one_at_a_time(tiny, kw, cpu_kernels):
    d, prompts, want = tiny
    eng = make_engine(d, **kw)
    jobs = [(i, mt) for i in range(len(prompts)) for mt in (5, 17)]
    reqs = [eng.add_request(prompts[i], SamplingParams(mt, stop_token_ids=NO_STOP)) for i, mt in jobs]
    steps = 0
    while eng.has_work():
        eng.step()
        eng.cache.check()
        steps += 1
        assert steps < 2000
    for (i, mt), r in zip(jobs, reqs):
        assert r.output_tokens == want[(i, mt)], (i, mt)
        assert r.stats.completion_tokens == mt and r.stats.finish_reason == "length"
    assert eng.cache.all_free()                                   # no page leaked
    assert not eng.scheduler.running and not eng.scheduler.waiting
    if "num_blocks" in kw:
        assert eng.scheduler.preemptions > 0
    if kw == {}:
        assert eng.scheduler.max_running_seen > 1                 # really batched
    if kw.get("max_num_seqs"):
        assert eng.scheduler.max_running_seen <= kw["max_num_seqs"]
    if kw.get("prefix_caching"):
        assert eng.scheduler.prefix_hit_tokens > 0                # each prompt is submitted twice


def test_stop_token_is_not_emitted(tiny, cpu_kernels):
    d, prompts, want = tiny
    full = want[(1, 17)]
    stop = full[6]
    first = full.index(stop)
    eng = make_engine(d)
    r = eng.add_request(prompts[1], SamplingParams(17, stop_token_ids={stop}))
    eng.run_until_done()
    assert r.output_tokens == full[:first] and r.stats.finish_reason == "stop"
    assert r.stats.completion_tokens == first and eng.cache.all_free()


def test_oversized_request_errors_not_hangs(tiny, cpu_kernels):
    d, prompts, _ = tiny
    eng = make_engine(d, num_blocks=2, block_size=4)
    with pytest.raises(RequestError):
        eng.add_request(list(range(10)), SamplingParams(4, stop_token_ids=NO_STOP))
    # fits at first, outgrows the pool while decoding: it preempts itself and then fails, no hang
    r = eng.add_request([1, 2, 3, 4, 5], SamplingParams(8, stop_token_ids=NO_STOP))
    for _ in range(50):
        if not eng.has_work():
            break
        eng.step()
    assert r.done and isinstance(r.error, RequestError) and eng.cache.all_free()
    with pytest.raises(ValueError):
        make_engine(d, max_model_len=8).add_request(list(range(8)))


@pytest.mark.parametrize("budget, prompt_len, max_tokens", [(48, 60, 128), (16, 40, 100), (7, 62, 9)])
def test_request_that_outgrows_the_pool_with_a_small_budget_errors(tiny, cpu_kernels, budget, prompt_len, max_tokens):
    """The prompt fits, prompt plus generated tokens do not, and the token budget is smaller than
    either: the first portion of a re-admission always fits, so only the request's whole length
    tells that it can never run.  It must end with an error after a bounded number of steps."""
    d, prompts, _ = tiny
    eng = make_engine(d, num_blocks=8, block_size=8, max_batched_tokens=budget)
    bystander = eng.add_request([1, 2, 3], SamplingParams(4, stop_token_ids=NO_STOP))
    r = eng.add_request([t % 512 for t in range(prompt_len)], SamplingParams(max_tokens, stop_token_ids=NO_STOP))
    steps = 0
    while eng.has_work():
        eng.step()
        eng.cache.check()
        steps += 1
        assert steps <= prompt_len + 64 + 10, "the request is admitted and preempted again and again"
    assert r.done and isinstance(r.error, RequestError) and "does not fit" in str(r.error)
    assert len(r.tokens) <= 64 + 1                                # it got as far as the pool allows: 64 cached, one sampled
    assert bystander.stats.finish_reason == "length" and bystander.error is None
    assert eng.cache.all_free() and eng.counters()["requests_finished"].get("error") == 1


def test_abort_frees_pages(tiny, cpu_kernels):
    d, prompts, _ = tiny
    eng = make_engine(d, block_size=4)
    a = eng.add_request(prompts[3], SamplingParams(500, stop_token_ids=NO_STOP))
    b = eng.add_request(prompts[1], SamplingParams(6, stop_token_ids=NO_STOP))
    for _ in range(3):
        eng.step()
    eng.abort(a)
    assert a.done and a.stats.finish_reason == "abort"
    eng.run_until_done()
    assert b.stats.finish_reason == "length" and eng.cache.all_free()
    eng.abort(a)                                                   # a second abort is a no-op


@pytest.mark.parametrize("bad,word", [(dict(max_tokens=0), "max_tokens"), (dict(max_tokens=2.5), "max_tokens"),
                                      (dict(temperature=float("nan")), "temperature"), (dict(top_p=0.0), "top_p"),
                                      (dict(top_p=-0.1), "top_p"), (dict(top_p=float("nan")), "top_p")])
def test_options_without_a_sampling_rule_are_refused_when_added(tiny, cpu_kernels, bad, word):
    d, prompts, _ = tiny
    eng = make_engine(d)
    with pytest.raises(ValueError, match=word):
        eng.add_request(prompts[1], SamplingParams(**bad))
    assert not eng.has_work() and eng.cache.all_free()
    eng.add_request(prompts[1], SamplingParams(max_tokens=1, temperature=-1.0, top_p=1.5))    # greedy; keeps every token
    eng.run_until_done()


def test_temperature_sampling_is_seeded_and_batch_independent(tiny, cpu_kernels):
    d, prompts, _ = tiny
    sp = lambda seed: SamplingParams(12, temperature=0.9, top_p=0.8, stop_token_ids=NO_STOP, seed=seed)
    eng = make_engine(d)
    alone = eng.add_request(prompts[1], sp(5))
    eng.run_until_done()
    eng2 = make_engine(d, max_batched_tokens=5)
    others = [eng2.add_request(p, sp(100 + i)) for i, p in enumerate(prompts[2:6])]
    same = eng2.add_request(prompts[1], sp(5))
    other_seed = eng2.add_request(prompts[1], sp(6))
    eng2.run_until_done()
    assert same.output_tokens == alone.output_tokens
    assert other_seed.output_tokens != alone.output_tokens
    assert all(len(o.output_tokens) == 12 for o in others)


# ---- decisions on host data only -----------------------------------------------------------------
def host_cache(num_blocks, page=4, slots=8, window=0):
    return CacheManager([keys_and_values(1, 8, window)], [ScheduleEntry(0)], [None], page_size=page, num_blocks=num_blocks,
                        max_requests=slots, dtype=torch.float32, device="cpu", allocate_storage=False)


def new_req(i, n, max_tokens=4):
    return Request(i, n, list(range(n)), SamplingParams(max_tokens), set(), GenStats())


def test_plan_serves_running_first_and_cuts_under_budget():
    s = Scheduler(host_cache(64), max_num_seqs=4, max_batched_tokens=10, max_model_len=100)
    a, b = new_req(0, 14), new_req(1, 3)
    s.add(a)
    s.add(b)
    plan = s.schedule()
    assert [(r.rid, n) for r, n in plan] == [(0, 10)]            # a's first portion takes the budget
    s.computed(plan)
    plan = s.schedule()
    assert [(r.rid, n) for r, n in plan] == [(0, 4), (1, 3)]     # the rest of a, then b is admitted
    s.computed(plan)
    for r in (a, b):
        s.accept(r, 7)
    plan = s.schedule()
    assert [(r.rid, n) for r, n in plan] == [(0, 1), (1, 1)]     # both decode


def test_newest_is_preempted_when_pages_run_out():
    s = Scheduler(host_cache(4, page=4), max_num_seqs=4, max_batched_tokens=100, max_model_len=100)
    a, b = new_req(0, 8, 50), new_req(1, 7, 50)
    s.add(a)
    s.add(b)
    plan = s.schedule()
    assert [(r.rid, n) for r, n in plan] == [(0, 8), (1, 7)]
    s.computed(plan)
    s.accept(a, 1)
    s.accept(b, 1)
    plan = s.schedule()                                           # a needs a third page: b, the newest, goes
    assert [(r.rid, n) for r, n in plan] == [(0, 1)]
    assert s.preemptions == 1 and s.waiting[0] is b and b.num_computed == 0
    assert not s.cache.has_request(b.rid)
    s.computed(plan)
    s.cache.check()


def test_head_of_line_waits_and_is_admitted_later():
    s = Scheduler(host_cache(3, page=4), max_num_seqs=4, max_batched_tokens=100, max_model_len=100)
    a, b = new_req(0, 8, 1), new_req(1, 8, 1)
    s.add(a)
    s.add(b)
    plan = s.schedule()
    assert [(r.rid, n) for r, n in plan] == [(0, 8)] and list(s.waiting) == [b]
    s.computed(plan)
    s.accept(a, 3)                                                # max_tokens 1: a finishes, pages return
    assert a.done and s.cache.all_free()
    plan = s.schedule()
    assert [(r.rid, n) for r, n in plan] == [(1, 8)]


def test_distribution_buckets_and_quantiles():
    from tensorline_amd.engine.metrics import BATCH_BOUNDS, Distribution
    d = Distribution(BATCH_BOUNDS)
    assert d.as_dict()["count"] == 0 and d.quantile(0.5) == 0.0
    for v in [1, 1, 2, 3, 4, 64, 65, 500]:
        d.observe(v)
    b = d.as_dict()["buckets"]
    # a value on a bound belongs to the bucket that bound closes (the reference's bisect_left rule)
    assert (b["le_1"], b["le_2"], b["le_4"], b["le_8"], b["le_64"], b["le_128"], b["above"]) == (2, 1, 2, 0, 1, 1, 1)
    assert d.count == 8 and d.total == 640 and d.smallest == 1 and d.largest == 500
    assert 2 <= d.quantile(0.5) <= 4 and d.quantile(1.0) == 500 and d.quantile(0.0) == 1
    with pytest.raises(ValueError):
        Distribution((2, 1))


def test_engine_reports_distributions_of_latency_and_batch_size(tiny, cpu_kernels):
    d, prompts, want = tiny
    eng = make_engine(d, max_num_seqs=3)
    reqs = [eng.add_request(p, SamplingParams(5, stop_token_ids=NO_STOP)) for p in prompts[:6]]
    gone = eng.add_request(prompts[6], SamplingParams(50, stop_token_ids=NO_STOP))
    eng.step()
    eng.abort(gone)
    eng.run_until_done()
    c = eng.counters()
    assert c["tokens_generated"] == 6 * 5 and c["requests_finished"] == {"length": 6, "abort": 1}
    assert c["ttft_s"]["count"] == 6 and c["e2e_s"]["count"] == 6           # the aborted one gave no token
    assert c["e2e_s"]["min"] >= c["ttft_s"]["min"] > 0
    assert abs(c["e2e_s"]["sum"] - sum(r.stats.total_s for r in reqs)) < 1e-9
    bs = c["batch_size"]
    assert bs["count"] == c["steps"] and bs["max"] == 3 == c["max_running_seen"]
    assert sum(bs["buckets"].values()) == bs["count"] and bs["buckets"]["le_4"] > 0


def test_decode_steps_overlap_and_change_no_token(tiny, cpu_kernels):
    """Steady decoding queues step t + 1 before it reads step t's tokens (they are taken from the
    device): the tokens are those of the plain implementation with the overlap on and off, for
    every small token limit (the last token of a request is never run ahead of), and a request
    that a stop token ends while the next step is in flight costs its neighbours nothing."""
    d, prompts, want = tiny
    for overlap in (True, False):
        eng = make_engine(d, overlap=overlap)
        reqs = [eng.add_request(prompts[i], SamplingParams(17, stop_token_ids=NO_STOP)) for i in (1, 3, 5)]
        eng.run_until_done()
        assert [r.output_tokens for r in reqs] == [want[(i, 17)] for i in (1, 3, 5)]
        c = eng.counters()
        assert (c["overlapped_steps"] > 10) == overlap and c["tokens_generated"] == 3 * 17 and eng.cache.all_free()
    for limit in (1, 2, 3, 4):
        eng = make_engine(d)
        reqs = [eng.add_request(prompts[i], SamplingParams(limit + k, stop_token_ids=NO_STOP)) for k, i in enumerate((1, 3))]
        eng.run_until_done()
        assert [r.output_tokens for r in reqs] == [want[(1, 17)][:limit], want[(3, 17)][:limit + 1]]
        assert all(r.stats.finish_reason == "length" for r in reqs) and eng.cache.all_free()
    # a stop token in the middle: the request ends there, the other goes on to its limit
    full = want[(1, 17)]
    stop = full[6]
    eng = make_engine(d)
    a = eng.add_request(prompts[1], SamplingParams(17, stop_token_ids={stop}))
    b = eng.add_request(prompts[3], SamplingParams(17, stop_token_ids=NO_STOP))
    eng.run_until_done()
    assert a.output_tokens == full[:full.index(stop)] and a.stats.finish_reason == "stop"
    assert b.output_tokens == want[(3, 17)] and eng.counters()["overlapped_steps"] > 0 and eng.cache.all_free()
    # the longest length the engine allows ends a request as a token limit does
    eng = make_engine(d, max_model_len=len(prompts[3]) + 5)
    r = eng.add_request(prompts[3], SamplingParams(500, stop_token_ids=NO_STOP))
    eng.run_until_done()
    assert r.output_tokens == want[(3, 17)][:5] and r.stats.finish_reason == "length"


def test_abort_while_a_step_is_in_flight(tiny, cpu_kernels):
    d, prompts, want = tiny
    eng = make_engine(d)
    a = eng.add_request(prompts[1], SamplingParams(17, stop_token_ids=NO_STOP))
    b = eng.add_request(prompts[3], SamplingParams(17, stop_token_ids=NO_STOP))
    for _ in range(6):
        eng.step()
    assert eng._inflight is not None                      # a decode step is queued and unread
    eng.abort(a)
    eng.run_until_done()
    assert a.stats.finish_reason == "abort" and a.output_tokens == want[(1, 17)][:len(a.output_tokens)]
    assert b.output_tokens == want[(3, 17)] and eng.cache.all_free()
    assert eng.drain() == []
