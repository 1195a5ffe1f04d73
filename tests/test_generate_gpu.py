"""Generation through the entry point, graph replay, and the parts of a layer alone, on the GPU."""
import numpy as np
import pytest
import torch

from tests import helpers, plain

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
NO_STOP = {-1}
LIMIT = {"float32": 1e-5, "bfloat16": 2e-2}

# how each tiny configuration is driven: page size, prompt lengths, tokens to generate, a pool so
# small that requests are preempted, a token budget that cuts prompts into portions
DRIVE = {"A": dict(page=16, lengths=[1, 5, 17, 33, 70], max_tokens=16, tight_blocks=12, chunk=12),
         "B": dict(page=8, lengths=[1, 8, 31, 64, 100], max_tokens=24, tight_blocks=40, chunk=24)}


class Case:
    """A model folder of one tiny configuration with prompts and what the plain implementation
    generates for them greedily, one request at a time, and its logits at every generated token."""

    def __init__(self, name, tmp_path_factory):
        self.name, self.drive = name, DRIVE[name]
        self.page, self.max_tokens = self.drive["page"], self.drive["max_tokens"]
        self.dir = helpers.make_model_dir(tmp_path_factory, name, seed=21)
        self.w, self.cfg = plain.load_folder(self.dir)
        self.prompts = helpers.prompts_for(name, self.drive["lengths"], seed=2)
        self.want = [plain.greedy_generate(self.w, self.cfg, p, self.max_tokens) for p in self.prompts]
        self.want_logits = []
        for p, out in zip(self.prompts, self.want):
            lg = plain.model_forward(self.w, self.cfg, p + out)
            self.want_logits.append(lg[len(p) - 1:len(p) - 1 + len(out)].numpy())

    def llm(self, dtype="float32", **opts):
        from tensorline_amd import LLM
        return LLM(self.dir, dtype=dtype, device=DEV, **{"num_blocks": 1024 // self.page, "block_size": self.page, **opts})

    def regimes(self):
        d = self.drive
        return {"eager": dict(graphs=False), "graphs": dict(graphs=True),
                "portions": dict(graphs=True, max_batched_tokens=d["chunk"]),
                "preemption": dict(graphs=False, num_blocks=d["tight_blocks"], prefix_caching=False),
                "preemption-shared-prefixes": dict(graphs=True, num_blocks=d["tight_blocks"], prefix_caching=True),
                "seq-limit": dict(graphs=True, max_num_seqs=2), "graphs-no-overlap": dict(graphs=True, overlap=False)}


@pytest.fixture(scope="module", params=["A", "B"])
def case(request, tmp_path_factory):
    return Case(request.param, tmp_path_factory)


@pytest.fixture(scope="module")
def folder_b(tmp_path_factory):
    d = helpers.make_model_dir(tmp_path_factory, "B", seed=21)
    w, cfg = plain.load_folder(d)
    return d, w, cfg


@pytest.fixture(scope="module")
def greedy_want(folder_b):
    d, w, cfg = folder_b
    prompts = helpers.prompts_for("B", [1, 8, 31, 64, 100], seed=2)
    return prompts, [plain.greedy_generate(w, cfg, p, 24) for p in prompts]


REGIMES = ["eager", "graphs", "portions", "preemption", "preemption-shared-prefixes", "seq-limit", "graphs-no-overlap"]


@pytest.mark.parametrize("regime", REGIMES)
def test_greedy_generation_matches_plain(case, regime):
    """32-bit tokens through the entry point equal the plain implementation's in every regime of
    the reference's batching test (tests/test_batching.py:67-85), on both tiny configurations."""
    from tensorline_amd import SamplingParams
    opts = case.regimes()[regime]
    llm = case.llm("float32", **opts)
    outs = llm.generate(case.prompts, SamplingParams(max_tokens=case.max_tokens, stop_token_ids=NO_STOP))
    assert [o.token_ids for o in outs] == case.want
    assert all(o.finish_reason == "length" and o.stats.completion_tokens == case.max_tokens for o in outs)
    assert llm.cache.all_free()
    llm.cache.check()
    c = llm.counters()
    if opts.get("graphs"):
        assert c["graph_replays"] > 0
    if "num_blocks" in opts:
        assert c["preemptions"] > 0
    if "max_num_seqs" in opts:
        assert c["max_running_seen"] == 2


@pytest.mark.parametrize("regime", REGIMES)
def test_bfloat16_logits_through_the_scheduler_match_plain(case, regime):
    """bfloat16 under the scheduler, in every regime: the plain implementation's tokens are forced
    on every request, so each step sees the contexts the plain run saw, and the logits the sampler
    is shown must be the plain ones within the bfloat16 limit at every generated position.  The
    forced tokens come back on the device, so steady decoding runs as it does in serving: a step
    queued behind the one in flight, its token ids taken from the device (graph replay, bfloat16)."""
    from tensorline_amd import SamplingParams
    opts = case.regimes()[regime]
    llm = case.llm("bfloat16", **opts)
    forced = helpers.ForcedSampler({100 + i: out for i, out in enumerate(case.want)})
    llm.engine.sampler = forced
    params = [SamplingParams(max_tokens=case.max_tokens, stop_token_ids=NO_STOP, seed=100 + i) for i in range(len(case.prompts))]
    outs = llm.generate(case.prompts, params)
    assert [o.token_ids for o in outs] == case.want and llm.cache.all_free()
    worst = 0.0
    for i, want in enumerate(case.want_logits):
        scale = float(np.abs(want).max())
        for k in range(case.max_tokens):
            err = float(np.abs(forced.logits[(100 + i, k)] - want[k]).max()) / scale
            assert np.isfinite(err) and err < LIMIT["bfloat16"], f"request {i} generated token {k}: relative error {err:.3e}"
            worst = max(worst, err)
    print(f"config {case.name} {regime} bfloat16 through the scheduler: worst relative error {worst:.3e}")
    c = llm.counters()
    if "num_blocks" in opts:
        assert c["preemptions"] > 0
    if opts.get("graphs"):
        assert c["graph_replays"] > 0
    if regime in ("eager", "graphs", "seq-limit"):
        assert c["overlapped_steps"] > 0, "no decode step was queued behind the one in flight"
    if opts.get("overlap") is False:
        assert c["overlapped_steps"] == 0


@pytest.mark.parametrize("block_size", [16, 32, 64, 128])
def test_generation_with_other_page_sizes(folder_b, greedy_want, block_size):
    """Pages larger than the kernels' key blocks and tiles: 32-bit tokens equal the plain ones, and
    bfloat16 logits, with the plain tokens forced, stay within the bfloat16 limit."""
    from tensorline_amd import LLM, SamplingParams
    d, w, cfg = folder_b
    prompts, want = greedy_want
    sp = SamplingParams(max_tokens=24, stop_token_ids=NO_STOP)
    llm = LLM(d, dtype="float32", device=DEV, num_blocks=2048 // block_size, block_size=block_size, max_batched_tokens=48)
    assert [o.token_ids for o in llm.generate(prompts, sp)] == want
    llm = LLM(d, dtype="bfloat16", device=DEV, num_blocks=2048 // block_size, block_size=block_size, max_batched_tokens=48)
    forced = helpers.ForcedSampler({i: out for i, out in enumerate(want)})
    llm.engine.sampler = forced
    outs = llm.generate(prompts, [SamplingParams(max_tokens=24, stop_token_ids=NO_STOP, seed=i) for i in range(len(prompts))])
    assert [o.token_ids for o in outs] == want
    for i, (p, out) in enumerate(zip(prompts, want)):
        lg = plain.model_forward(w, cfg, p + out)[len(p) - 1:len(p) - 1 + len(out)].numpy()
        for k in range(len(out)):
            assert float(np.abs(forced.logits[(i, k)] - lg[k]).max()) / float(np.abs(lg).max()) < LIMIT["bfloat16"], (i, k)


def test_bfloat16_generation_same_with_and_without_graphs(folder_b, greedy_want):
    from tensorline_amd import LLM, SamplingParams
    d, w, cfg = folder_b
    prompts, want = greedy_want
    got = {}
    for graphs in (False, True):
        llm = LLM(d, dtype="bfloat16", device=DEV, num_blocks=128, block_size=8, graphs=graphs)
        got[graphs] = [o.token_ids for o in llm.generate(prompts, SamplingParams(max_tokens=24, stop_token_ids=NO_STOP))]
    assert got[True] == got[False]


# ---- shared prefixes (the reference's tests/test_prefix_cache.py:42-74, on the GPU) ----------------
def _shared_prompts(case, n, tail=3, seed=5):
    rng = np.random.default_rng(seed)
    V = case.cfg["vocab_size"]
    shared = rng.integers(0, V, 5 * case.page + 3).tolist()           # five full pages and a bit
    return shared, [shared + rng.integers(0, V, tail + i).tolist() for i in range(n)]


def test_shared_prefix_hits_and_matches_uncached(case):
    from tensorline_amd import SamplingParams
    shared, prompts = _shared_prompts(case, 5)
    sp = SamplingParams(max_tokens=12, stop_token_ids=NO_STOP)
    want = [plain.greedy_generate(case.w, case.cfg, p, 12) for p in prompts]
    llm = case.llm("float32", prefix_caching=True)
    first = llm.generate([prompts[0]], sp)[0]                         # warms the cache
    assert first.token_ids == want[0] and first.stats.cached_tokens == 0
    outs = llm.generate(prompts[1:], sp)
    assert [o.token_ids for o in outs] == want[1:]
    full_shared = len(shared) // case.page * case.page
    assert all(o.stats.cached_tokens >= full_shared for o in outs)
    c = llm.counters()
    assert c["prefix_hit_tokens"] >= 4 * full_shared
    assert llm.cache.all_free() and llm.cache.groups[0].allocator.num_cached > 0    # free, and still findable
    llm.cache.check()


def test_identical_prompt_fully_cached_recomputes_its_last_page(case):
    from tensorline_amd import SamplingParams
    rng = np.random.default_rng(8)
    prompt = rng.integers(0, case.cfg["vocab_size"], 4 * case.page).tolist()     # ends exactly on a page edge
    want = plain.greedy_generate(case.w, case.cfg, prompt, 10)
    want_logits = plain.model_forward(case.w, case.cfg, prompt + want)[len(prompt) - 1:len(prompt) + 9].numpy()
    for dtype in ("float32", "bfloat16"):
        llm = case.llm(dtype, prefix_caching=True)
        forced = helpers.ForcedSampler({1: want, 2: want})
        llm.engine.sampler = forced
        a = llm.generate([prompt], SamplingParams(max_tokens=10, stop_token_ids=NO_STOP, seed=1))[0]
        b = llm.generate([prompt], SamplingParams(max_tokens=10, stop_token_ids=NO_STOP, seed=2))[0]
        assert a.stats.cached_tokens == 0 and b.stats.cached_tokens == 3 * case.page
        assert 0 < b.stats.cached_tokens < b.stats.prompt_tokens     # the last page is computed again for its logits
        for seed in (1, 2):                                          # computed from cached keys or from scratch: the plain logits
            for k in range(10):
                err = float(np.abs(forced.logits[(seed, k)] - want_logits[k]).max()) / float(np.abs(want_logits).max())
                assert err < LIMIT[dtype], (dtype, seed, k, err)
        assert llm.cache.all_free()


def test_preemption_with_shared_prefixes_matches_plain(case):
    from tensorline_amd import SamplingParams
    shared, prompts = _shared_prompts(case, 6, tail=2, seed=6)
    n_new = 2 * case.page + 4                                        # every request grows by more than two pages
    want = [plain.greedy_generate(case.w, case.cfg, p, n_new) for p in prompts]
    prompt_pages = -(-len(prompts[-1]) // case.page)
    # three prompts fit with one page to spare: all three then want more pages, and the newest gives way
    llm = case.llm("float32", prefix_caching=True, num_blocks=3 * prompt_pages + 1)
    outs = llm.generate(prompts, SamplingParams(max_tokens=n_new, stop_token_ids=NO_STOP))
    assert [o.token_ids for o in outs] == want
    c = llm.counters()
    assert c["preemptions"] > 0 and c["prefix_hit_tokens"] > 0
    assert llm.cache.all_free()
    llm.cache.check()


# ---- ways a request ends ---------------------------------------------------------------------------
def test_stop_token_and_length_limits_end_requests(case):
    """On the GPU, with graphs: a stop token ends a request and is neither kept nor counted; the
    model's longest length ends it with "length"; a request ending frees its pages while others go on."""
    from tensorline_amd import SamplingParams
    full = case.want[2]
    stop = full[5]
    first = full.index(stop)
    llm = case.llm("float32", graphs=True, max_model_len=len(case.prompts[3]) + 7)
    outs = llm.generate([case.prompts[2], case.prompts[3], case.prompts[1]],
                        [SamplingParams(max_tokens=case.max_tokens, stop_token_ids={stop}),
                         SamplingParams(max_tokens=500, stop_token_ids=NO_STOP),
                         SamplingParams(max_tokens=3, stop_token_ids=NO_STOP)])
    assert outs[0].token_ids == full[:first] and outs[0].finish_reason == "stop"
    assert outs[0].stats.completion_tokens == first
    # prompt + generated may not pass max_model_len: 7 more tokens, whatever max_tokens says
    assert outs[1].token_ids == case.want[3][:7] and outs[1].finish_reason == "length"
    assert outs[2].token_ids == case.want[1][:3] and outs[2].finish_reason == "length"
    with pytest.raises(ValueError, match="max_model_len"):
        llm.generate([case.prompts[4] + case.prompts[4]], SamplingParams(max_tokens=2))
    assert llm.cache.all_free()
    assert llm.counters()["requests_finished"] == {"stop": 1, "length": 2}


def test_seeded_sampling_survives_preemption_and_batching(folder_b, greedy_want):
    """A request's sampled tokens depend on its seed and its logits only: the same in a roomy pool, in a
    pool so small that requests are preempted and recomputed, and alone (32-bit, so that rounding between
    different cuttings stays far below the probabilities' spacing)."""
    from tensorline_amd import LLM, SamplingParams
    d, w, cfg = folder_b
    prompts, _ = greedy_want
    params = [SamplingParams(max_tokens=24, temperature=0.8, top_p=0.9, stop_token_ids=NO_STOP, seed=50 + i)
              for i in range(len(prompts))]
    roomy = LLM(d, dtype="float32", device=DEV, num_blocks=128, block_size=8)
    a = [o.token_ids for o in roomy.generate(prompts, params)]
    tight = LLM(d, dtype="float32", device=DEV, num_blocks=40, block_size=8, prefix_caching=False, graphs=False)
    b = [o.token_ids for o in tight.generate(prompts, params)]
    assert tight.counters()["preemptions"] > 0 and tight.cache.all_free()
    assert a == b
    alone = [roomy.generate([p], sp)[0].token_ids for p, sp in zip(prompts[:2], params[:2])]
    assert alone == a[:2]
    assert len({tuple(x) for x in a}) == len(a)


def test_stream_and_abort(folder_b, greedy_want):
    from tensorline_amd import LLM, GenStats, SamplingParams
    d, w, cfg = folder_b
    prompts, want = greedy_want
    llm = LLM(d, dtype="float32", device=DEV, num_blocks=64, block_size=8)
    st = GenStats()
    got = list(llm.stream(prompts[2], SamplingParams(max_tokens=24, stop_token_ids=NO_STOP), st))
    assert got == want[2] and st.finish_reason == "length" and st.ttft_s > 0
    st = GenStats()
    gen = llm.stream(prompts[3], SamplingParams(max_tokens=500, stop_token_ids=NO_STOP), st)
    assert [next(gen), next(gen)] == want[3][:2]
    gen.close()                                     # the consumer leaves: the request is aborted
    assert st.finish_reason == "abort" and llm.cache.all_free()


def test_graph_decode_matches_eager_and_isolates_padding(folder_b):
    """20 decode steps across a page edge, batch 3 in a bucket of 4 (one padding row): logits equal
    the eager step's, a page no sequence owns stays untouched (tests/test_cuda_graphs.py:20-45)."""
    from tensorline_amd.cache.manager import CacheManager
    from tensorline_amd.engine.batch import StepEntry
    from tensorline_amd.engine.graphs import GraphRunner
    from tensorline_amd.engine.loading import load_model
    from tensorline_amd.engine.runner import ModelRunner
    d, w, cfg = folder_b
    model, _ = load_model(d, "bfloat16", DEV)
    mk = lambda: CacheManager(model.cache_needs(), model.schedule, model.state_needs(), page_size=8, num_blocks=32,
                              max_requests=8, dtype=model.dtype, device=DEV)
    ce, cg = mk(), mk()
    eager, graph = ModelRunner(model, ce), GraphRunner(model, cg, max_batch=8, max_blocks_per_seq=8)
    seqs = helpers.prompts_for("B", [2, 13, 21], seed=4)
    bystander = 31
    for c in (ce, cg):
        for i, s in enumerate(seqs):
            c.add_request(i)
        c.groups[0].allocator.take(5)             # shift the ids so tables are not 0, 1, 2, ...
        for i, s in enumerate(seqs):
            assert c.grow(i, len(s) + 21)
        assert all(bystander not in c.table(i) for i in range(3))
        c.storage(0)["k"][bystander].fill_(7.0)
    first = [StepEntry(i, s, 0, [len(s) - 1]) for i, s in enumerate(seqs)]
    le, lg = eager.step(first), graph.step(first)      # not pure decode: both run eagerly
    torch.testing.assert_close(le, lg, atol=0, rtol=0)
    seqs = [list(s) for s in seqs]
    for step in range(20):
        nxt = lg.argmax(-1).tolist()
        for s, t in zip(seqs, nxt):
            s.append(t)
        entries = [StepEntry(i, [s[-1]], len(s) - 1, [0]) for i, s in enumerate(seqs)]
        le, lg = eager.step(entries).clone(), graph.step(entries).clone()
        assert lg.argmax(-1).tolist() == le.argmax(-1).tolist(), step
        torch.testing.assert_close(lg, le, atol=1e-5, rtol=1e-5)
    assert graph.graph_replays == 20 and len(graph.graphs) == 1
    assert torch.all(cg.storage(0)["k"][bystander] == 7.0)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["A", "B"])
def test_replayed_step_and_its_eager_twin_give_the_same_bits(name, dtype, tmp_path):
    """Up to 16 rows a decode step replayed from a graph (padded batch, context rounded up to the
    graph's bucket) and the same step run eagerly by a runner that knows the same longest context
    give the same logits to the bit, with the MFMA attention kernels (B in bfloat16) and with the
    any-shape ones (A: head size 16; B in 32-bit), whose keys go through the merge kernel in the
    graph although these contexts would fit one run."""
    from tensorline_amd.cache.manager import CacheManager
    from tensorline_amd.engine.batch import StepEntry
    from tensorline_amd.engine.graphs import GraphRunner
    from tensorline_amd.engine.loading import load_model
    from tensorline_amd.engine.runner import ModelRunner
    d = helpers.make_model_dir(tmp_path, name, seed=8)
    model, _ = load_model(d, dtype, DEV)
    page = DRIVE[name]["page"]
    mk = lambda: CacheManager(model.cache_needs(), model.schedule, model.state_needs(), page_size=page, num_blocks=160,
                              max_requests=8, dtype=model.dtype, device=DEV)
    ce, cg = mk(), mk()
    eager, graph = ModelRunner(model, ce), GraphRunner(model, cg, max_batch=8, max_blocks_per_seq=512 // page)
    eager.fit_context = graph.fit_context
    seqs = [list(p) for p in helpers.prompts_for(name, [2, 13, 40, 7, 90], seed=4)]
    for c in (ce, cg):
        for i, s in enumerate(seqs):
            c.add_request(i)
            assert c.grow(i, len(s) + 13)
    first = [StepEntry(i, s, 0, [len(s) - 1]) for i, s in enumerate(seqs)]
    le, lg = eager.step(first).clone(), graph.step(first).clone()
    assert torch.equal(le, lg)
    for step in range(12):
        for s, t in zip(seqs, lg.argmax(-1).tolist()):
            s.append(t)
        entries = [StepEntry(i, [s[-1]], len(s) - 1, [0]) for i, s in enumerate(seqs)]
        le, lg = eager.step(entries).clone(), graph.step(entries).clone()
        assert torch.equal(le, lg), (step, float((le - lg).abs().max()))
    assert graph.graph_replays == 12


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("rows, bucket", [(19, 32), (41, 64), (70, 128)])
def test_graph_replay_of_wide_buckets_matches_plain(case, rows, bucket, dtype):
    """Graphs of 32 and of 64 rows (the 17-to-64-row kernels inside a captured graph) and of 128 (the
    library's products and the separate norm kernels of steps above 64 rows), with padding rows: 12 decode steps whose logits are the plain implementation's at every row and step, on
    scattered pages, and a page no sequence owns stays as it was (tests/test_cuda_graphs.py:20-45
    at the buckets its batch of three never reaches)."""
    from tensorline_amd.cache.manager import CacheManager
    from tensorline_amd.engine.batch import StepEntry
    from tensorline_amd.engine.graphs import GraphRunner
    from tensorline_amd.engine.loading import load_model
    steps = 12
    model, _ = load_model(case.dir, dtype, DEV)
    # rows are copies of the case's prompts (the plain logits of each are known), in changing order
    source = [(3 * r + r // 5) % len(case.prompts) for r in range(rows)]
    page = case.page
    per_seq = max(-(-(len(p) + steps) // page) for p in case.prompts)
    cache = CacheManager(model.cache_needs(), model.schedule, model.state_needs(), page_size=page,
                         num_blocks=(rows + 1) * per_seq + 9, max_requests=128, dtype=model.dtype, device=DEV)
    runner = GraphRunner(model, cache, max_batch=128, max_blocks_per_seq=per_seq)
    held = cache.groups[0].allocator.take(7)                  # so that tables do not start at page 0
    bystander = held[3]
    cache.storage(0)["k"][bystander].fill_(7.0)
    cache.storage(len(model.schedule) - 1)["v"][bystander].fill_(-3.0)
    for r in range(rows):
        cache.add_request(r)
    order = sorted(range(rows), key=lambda r: (r * 7) % rows)   # pages of neighbours in the batch are not neighbours
    for r in order:
        assert cache.grow(r, len(case.prompts[source[r]]) + steps)
    seqs = [list(case.prompts[source[r]]) for r in range(rows)]
    for r0 in range(0, rows, 8):                              # prompts, eight to a step: eager
        runner.step([StepEntry(r, seqs[r], 0, []) for r in range(r0, min(r0 + 8, rows))])
    cache.add_request(rows)                                   # one more request, whose prompt runs eagerly between replays
    assert cache.grow(rows, len(case.prompts[0]))
    scale = [float(np.abs(case.want_logits[i]).max()) for i in range(len(case.prompts))]
    worst = 0.0
    for k in range(1, steps):
        # the plain run's own tokens: step k feeds generated token k-1 and gives the logits for token k
        for r in range(rows):
            seqs[r].append(case.want[source[r]][k - 1])
        entries = [StepEntry(r, [seqs[r][-1]], len(seqs[r]) - 1, [0]) for r in range(rows)]
        logits = runner.step(entries).cpu().numpy()
        if k % 3 == 0:
            # the program's own eager work between two replays (library products and what they leave in
            # workspaces included): the replays after it must be as right as the first
            last = runner.step([StepEntry(rows, case.prompts[0], 0, [len(case.prompts[0]) - 1])]).cpu().numpy()[0]
            assert float(np.abs(last - case.want_logits[0][0]).max()) / scale[0] < LIMIT[dtype]
        for r in range(rows):
            want = case.want_logits[source[r]][k]
            err = float(np.abs(logits[r] - want).max()) / scale[source[r]]
            assert err < LIMIT[dtype], f"row {r} step {k}: relative error {err:.3e}"
            worst = max(worst, err)
    print(f"config {case.name} graph of {bucket} rows, {rows} live, {dtype}: worst relative error {worst:.3e}")
    assert runner.graph_replays == steps - 1 and [b for b, c in runner.graphs] == [bucket]
    assert torch.all(cache.storage(0)["k"][bystander] == 7.0)
    assert torch.all(cache.storage(len(model.schedule) - 1)["v"][bystander] == -3.0)


def test_decoding_across_a_context_bucket_switches_graphs_and_keeps_the_logits(folder_b):
    """Graphs are captured per batch bucket and per context bucket (4,096 keys, then the engine's
    limit): a request decoding from 4,090 to 4,110 tokens replays two graphs, and its logits are
    those of the eager step to the bit and the plain implementation's within the bfloat16 limit."""
    from tensorline_amd.cache.manager import CacheManager
    from tensorline_amd.engine.batch import StepEntry
    from tensorline_amd.engine.graphs import GraphRunner
    from tensorline_amd.engine.loading import load_model
    from tensorline_amd.engine.runner import ModelRunner
    d, w, cfg = folder_b
    model, _ = load_model(d, "bfloat16", DEV)
    limit_tokens, page = 4200, 8
    toks = helpers.prompts_for("B", [4111], seed=12)[0]
    want = plain.model_forward(w, cfg, toks)[4089:].numpy()
    mk = lambda: CacheManager(model.cache_needs(), model.schedule, model.state_needs(), page_size=page,
                              num_blocks=limit_tokens // page + 4, max_requests=2, dtype=model.dtype, device=DEV)
    ce, cg = mk(), mk()
    eager, graph = ModelRunner(model, ce), GraphRunner(model, cg, max_batch=2, max_blocks_per_seq=limit_tokens // page)
    eager.fit_context = graph.fit_context
    assert graph.context_buckets == [4096, limit_tokens]
    for c, r in ((ce, eager), (cg, graph)):
        c.add_request("a")
        assert c.grow("a", len(toks))
        for start in range(0, 4090, 1024):                      # the prompt in portions: eager either way
            n = min(1024, 4090 - start)
            r.step([StepEntry("a", toks[start:start + n], start, [])])
    for pos in range(4090, len(toks)):
        entry = [StepEntry("a", [toks[pos]], pos, [0])]
        le, lg = eager.step(entry).clone(), graph.step(entry).clone()
        torch.testing.assert_close(lg, le, atol=0, rtol=0)
        err = float(np.abs(lg[0].cpu().numpy() - want[pos - 4089]).max()) / float(np.abs(want).max())
        assert err < LIMIT["bfloat16"], (pos, err)
    assert sorted(graph.graphs) == [(1, 4096), (1, limit_tokens)] and graph.graph_replays == len(toks) - 4090


def test_parts_alone(folder_b):
    """Each part of a layer alone against the plain implementation: norm, attention over a prompt
    (cache, RoPE and projections together), feed-forward."""
    from tensorline_amd.cache.manager import CacheManager
    from tensorline_amd.engine.batch import StepEntry
    from tensorline_amd.engine.loading import load_model
    from tensorline_amd.engine.runner import ModelRunner
    d, w, cfg = folder_b
    model, mc = load_model(d, "float32", DEV)
    block = model.blocks[1]
    T, H = 37, mc.hidden_size
    torch.manual_seed(0)
    h = torch.randn(T, H, device=DEV)
    p = "model.layers.1."
    # norm
    x = h.clone()
    got = block.mixer_norm.forward(x, None)
    torch.testing.assert_close(got.cpu(), plain.rmsnorm(h.cpu(), w[p + "input_layernorm.weight"], mc.rms_norm_eps),
                               atol=1e-5, rtol=1e-5)
    # feed-forward
    got = block.feed_forward.forward(h, None)
    want = plain.swiglu(h.cpu(), w[p + "mlp.gate_proj.weight"], w[p + "mlp.up_proj.weight"], w[p + "mlp.down_proj.weight"])
    torch.testing.assert_close(got.cpu(), want, atol=1e-5, rtol=1e-4)
    # attention: a whole prompt, then the same prompt cut in two portions
    cache = CacheManager(model.cache_needs(), model.schedule, model.state_needs(), page_size=8, num_blocks=16,
                         max_requests=2, dtype=torch.float32, device=DEV)
    runner = ModelRunner(model, cache)
    want = plain.attention_block(h.cpu(), w, p + "self_attn.", torch.arange(T), mc.num_attention_heads,
                                 mc.num_key_value_heads, mc.head_dim, mc.rope_theta)
    for cuts in ([T], [20, 17]):
        cache.add_request("a")
        cache.grow("a", T)
        outs, start = [], 0
        for n in cuts:
            packed = runner.pack([StepEntry("a", [0] * n, start, [])])
            ctx, views = runner.context(packed, runner._upload(packed.data))
            outs.append(block.mixer.forward(h[start:start + n].contiguous(), ctx, views[1]))
            start += n
        torch.testing.assert_close(torch.cat(outs).cpu(), want, atol=1e-5, rtol=1e-4)
        cache.release("a")


def test_decode_steps_hand_norms_to_the_products(folder_b, monkeypatch):
    """bfloat16 steps of up to 64 rows run one norm kernel only (the first layer's first norm): the other
    norms ride on the products around them.  The logits agree with the same step run with a norm
    kernel for every norm, whether all rows or some are wanted."""
    from tensorline_amd.cache.manager import CacheManager
    from tensorline_amd.engine.batch import StepEntry
    from tensorline_amd.engine.loading import load_model
    from tensorline_amd.engine.runner import ModelRunner
    from tensorline_amd.ops import kernels
    d, w, cfg = folder_b
    model, mc = load_model(d, "bfloat16", DEV)
    cache = CacheManager(model.cache_needs(), model.schedule, model.state_needs(), page_size=8, num_blocks=32,
                         max_requests=4, dtype=torch.bfloat16, device=DEV)
    runner = ModelRunner(model, cache)
    calls = []
    real = kernels.add_rmsnorm
    monkeypatch.setattr(kernels, "add_rmsnorm", lambda *a, **k: (calls.append(1), real(*a, **k))[1])
    for lengths in ([9, 5, 2], [30, 21, 9]):                 # 16 rows: the few-row kernels; 60: the mid-row ones
        prompts = helpers.prompts_for("B", lengths, seed=4)
        for i, p in enumerate(prompts):
            cache.add_request(i)
            cache.grow(i, len(p))
        for want_all in (True, False):
            entries = [StepEntry(i, p, 0, list(range(len(p))) if want_all else [len(p) - 1])
                       for i, p in enumerate(prompts)]
            calls.clear()
            got = runner.step(entries)
            assert len(calls) == 1
            with monkeypatch.context() as m:
                m.setattr(kernels, "can_defer_norm", lambda rows, dtype: False)
                calls.clear()
                ref = runner.step(entries)
                assert len(calls) == 2 * mc.num_hidden_layers + 1
            torch.testing.assert_close(got, ref, atol=2e-2, rtol=2e-2)
            assert (got.argmax(-1) == ref.argmax(-1)).float().mean() > 0.8
        for i in range(len(prompts)):
            cache.release(i)


def test_toy_mixer_with_state_registers_and_steps(tmp_path):
    """A mixer defined here, with per-request state of fixed size, is registered, built into a model
    beside the framework's own parts and stepped, without a change to the framework's files."""
    from tensorline_amd.cache.manager import CacheManager
    from tensorline_amd.engine.batch import StepEntry
    from tensorline_amd.engine.runner import ModelRunner
    from tensorline_amd.models.decoder import DecoderModel
    from tensorline_amd.parts.base import Part
    from tensorline_amd.parts.registry import register_mixer
    from tensorline_amd.parts.spec import LayerSpec, ModelSpec, PartSpec, ScheduleEntry, StateNeed, TensorDecl
    from tensorline_amd.weights.loader import load_from_getter
    from tensorline_amd.weights.random_init import random_tensor

    @register_mixer("toy_running_mean", replace=True)
    class RunningMean(Part):
        """out[t] = (decay * state + h[t]) W^T, state <- decay * state + h[t]: a causal running sum
        kept per request between steps."""

        def __init__(self, hidden_size, prefix, dtype, device, decay: float):
            super().__init__(hidden_size, prefix, dtype, device)
            self.decay = decay
            self.w = None

        def tensors(self):
            return {self.prefix + "mix.weight": TensorDecl((self.hidden_size, self.hidden_size), "normal", 0.05, "float32")}

        def load(self, get):
            self.w = get(self.prefix + "mix.weight")

        def cache_need(self):
            return None

        def state_need(self):
            return StateNeed((self.hidden_size,), "float32")

        def forward(self, h, ctx, cache):
            out = torch.empty(h.shape[0], self.hidden_size, dtype=torch.float32, device=h.device)
            for s in range(ctx.num_seqs):
                r0, r1 = ctx.host_q_start[s], ctx.host_q_start[s + 1]
                st = cache.state[ctx.host_state_slots[s]]
                for r in range(r0, r1):
                    st.mul_(self.decay).add_(h[r].float())
                    out[r] = st @ self.w.T
            return out

    H, V = 32, 50
    norm = lambda name: PartSpec("rmsnorm", {"eps": 1e-6, "name": name})
    attn = PartSpec("attention", {"num_heads": 2, "num_kv_heads": 1, "head_dim": 16, "qkv_bias": True,
                                  "position": PartSpec("rope", {"theta": 100.0})}, prefix="self_attn.")
    ffn = PartSpec("swiglu", {"intermediate_size": 48}, prefix="mlp.")
    layers = (
        LayerSpec("l0.", PartSpec("toy_running_mean", {"decay": 0.9}, prefix="toy."), ffn, norm("n1"), norm("n2")),
        LayerSpec("l1.", attn, ffn, norm("n1"), norm("n2")),
    )
    # the attention layer runs twice (a cache for each run); the toy layer runs between them
    spec = ModelSpec(H, V, PartSpec("token_embedding", {"name": "emb"}), layers, norm("nf"),
                     PartSpec("lm_head", {"name": "head", "tied": False}),
                     schedule=(ScheduleEntry(1), ScheduleEntry(0), ScheduleEntry(1)))
    model = DecoderModel(spec, torch.float32, DEV)
    assert [n is not None for n in model.state_needs()] == [False, True, False]
    load_from_getter(model, lambda name, decl: random_tensor(name, decl, 3, "cpu"), DEV)
    mk = lambda: CacheManager(model.cache_needs(), model.schedule, model.state_needs(), page_size=4, num_blocks=16,
                              max_requests=3, dtype=torch.float32, device=DEV)
    toks = [3, 1, 4, 1, 5, 9, 2, 6, 5, 3, 5]
    c1 = mk()
    c1.add_request("w")
    c1.grow("w", len(toks))
    whole = ModelRunner(model, c1).step([StepEntry("w", toks, 0, list(range(len(toks))))])
    # the same model written out plainly: attention layer, toy layer, attention layer again (its
    # weights a second time), each followed by its feed-forward; the toy is a decayed running sum
    w = {name: random_tensor(name, decl, 3, "cpu") for name, decl in model.tensor_decls().items()}
    T, pos = len(toks), torch.arange(len(toks))
    x = w["emb"][torch.tensor(toks)]
    for p in ("l1.", "l0.", "l1."):
        h = plain.rmsnorm(x, w[p + "n1"], 1e-6)
        if p == "l0.":
            state, rows = torch.zeros(H), []
            for t in range(T):
                state = 0.9 * state + h[t]
                rows.append(state)
            x = x + torch.stack(rows) @ w["l0.toy.mix.weight"].T
        else:
            x = x + plain.attention_block(h, w, p + "self_attn.", pos, 2, 1, 16, 100.0)
        h = plain.rmsnorm(x, w[p + "n2"], 1e-6)
        x = x + plain.swiglu(h, w[p + "mlp.gate_proj.weight"], w[p + "mlp.up_proj.weight"], w[p + "mlp.down_proj.weight"])
    expected = plain.rmsnorm(x, w["nf"], 1e-6) @ w["head"].T
    torch.testing.assert_close(whole.cpu(), expected, atol=2e-5, rtol=1e-4)
    # cut into portions, beside another request: same logits, state carried in the request's slot
    c2 = mk()
    r2 = ModelRunner(model, c2)
    c2.add_request("other")
    c2.add_request("w")
    c2.grow("other", 6)
    got, start = [], 0
    for n in (4, 1, 2, 4):
        c2.grow("w", start + n)
        entries = [StepEntry("w", toks[start:start + n], start, list(range(n)))]
        if start == 0:
            entries.insert(0, StepEntry("other", [7, 7, 7, 7, 7, 7], 0, [5]))
        out = r2.step(entries)
        got.append(out[-n:])
        start += n
    torch.testing.assert_close(torch.cat(got), whole, atol=1e-5, rtol=1e-4)
    # a slot handed out again starts from zero state
    c2.release("w")
    c2.add_request("again")
    c2.grow("again", len(toks))
    again = r2.step([StepEntry("again", toks, 0, list(range(len(toks))))])
    torch.testing.assert_close(again, whole, atol=1e-5, rtol=1e-4)


def test_command_line_generate(case):
    import json
    import os
    import subprocess
    import sys
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    cmd = [sys.executable, os.path.join(root, "bin", "tensorline"), "generate", "--model", case.dir, "--dtype", "float32",
           "--num-blocks", "64", "--block-size", str(case.page), "--max-tokens", str(case.max_tokens), "--stop-token-id", "-1"]
    for p in case.prompts[1:3]:
        cmd += ["--prompt-ids", " ".join(map(str, p))]
    proc = subprocess.run(cmd, capture_output=True, text=True, timeout=300)
    assert proc.returncode == 0, proc.stderr[-2000:]
    recs = [json.loads(l) for l in proc.stdout.splitlines() if l.startswith("{")]
    assert [r["token_ids"] for r in recs] == case.want[1:3]
    assert all(r["finish_reason"] == "length" and r["completion_tokens"] == case.max_tokens for r in recs)
    counters = json.loads([l for l in proc.stderr.splitlines() if l.startswith('{"counters"')][-1])["counters"]
    assert counters["tokens_generated"] == 2 * case.max_tokens and counters["ttft_s"]["count"] == 2


def test_library_tuning_keeps_results(folder_b):
    """Letting the library choose its kernels by measurement changes which kernel runs, not what a
    prompt portion computes."""
    from tensorline_amd import LLM, SamplingParams
    d, w, cfg = folder_b
    prompt = helpers.prompts_for("B", [150], seed=9)
    sp = SamplingParams(max_tokens=6, stop_token_ids=NO_STOP)
    plainly = LLM(d, dtype="bfloat16", device=DEV, num_blocks=64, block_size=8, max_batched_tokens=128)
    want = plainly.generate(prompt, sp)[0].token_ids
    # with more sequences than the engine's own kernels take rows, the graphs' row counts above that are searched too
    tuned = LLM(d, dtype="bfloat16", device=DEV, num_blocks=64, block_size=8, max_batched_tokens=128, tune_library=True,
                max_num_seqs=96)
    try:
        assert tuned.engine.runner.batch_buckets[-1] == 96 and tuned.model.tune_library(128) >= 1
        assert tuned.generate(prompt, sp)[0].token_ids == want
    finally:
        torch.cuda.tunable.enable(False)
