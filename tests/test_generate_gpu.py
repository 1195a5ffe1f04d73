"""Generation through the entry point, graph replay, and the parts of a layer alone, on the GPU."""
import pytest
import torch

from tests import helpers, plain

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
NO_STOP = {-1}


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


@pytest.mark.parametrize("opts", [
    dict(graphs=False), dict(graphs=True), dict(graphs=True, max_batched_tokens=24),
    dict(graphs=False, num_blocks=40, block_size=8, prefix_caching=False), dict(graphs=True, max_num_seqs=2),
], ids=["eager", "graphs", "chunk24", "preemption", "seq-limit"])
def test_greedy_generation_matches_plain(folder_b, greedy_want, opts):
    from tensorline_amd import LLM, SamplingParams
    d, w, cfg = folder_b
    prompts, want = greedy_want
    llm = LLM(d, dtype="float32", device=DEV, **{"num_blocks": 128, "block_size": 8, **opts})
    outs = llm.generate(prompts, SamplingParams(max_tokens=24, stop_token_ids=NO_STOP))
    assert [o.token_ids for o in outs] == want
    assert all(o.finish_reason == "length" and o.stats.completion_tokens == 24 for o in outs)
    assert llm.cache.all_free()
    c = llm.counters()
    if opts.get("graphs"):
        assert c["graph_replays"] > 0
    if "num_blocks" in opts:
        assert c["preemptions"] > 0


@pytest.mark.parametrize("block_size", [16, 32, 64, 128])
def test_greedy_generation_with_other_page_sizes(folder_b, greedy_want, block_size):
    """Pages larger than the kernels' key blocks and tiles: 32-bit tokens equal the plain ones, and
    bfloat16 agrees with 32-bit on most tokens."""
    from tensorline_amd import LLM, SamplingParams
    d, w, cfg = folder_b
    prompts, want = greedy_want
    sp = SamplingParams(max_tokens=24, stop_token_ids=NO_STOP)
    llm = LLM(d, dtype="float32", device=DEV, num_blocks=2048 // block_size, block_size=block_size, max_batched_tokens=48)
    assert [o.token_ids for o in llm.generate(prompts, sp)] == want
    llm = LLM(d, dtype="bfloat16", device=DEV, num_blocks=2048 // block_size, block_size=block_size, max_batched_tokens=48)
    got = [o.token_ids for o in llm.generate(prompts, sp)]
    same = sum(a == b for g, x in zip(got, want) for a, b in zip(g, x))
    assert same >= 0.6 * sum(len(x) for x in want)


def test_bfloat16_generation_same_with_and_without_graphs(folder_b, greedy_want):
    from tensorline_amd import LLM, SamplingParams
    d, w, cfg = folder_b
    prompts, want = greedy_want
    got = {}
    for graphs in (False, True):
        llm = LLM(d, dtype="bfloat16", device=DEV, num_blocks=128, block_size=8, graphs=graphs)
        got[graphs] = [o.token_ids for o in llm.generate(prompts, SamplingParams(max_tokens=24, stop_token_ids=NO_STOP))]
    assert got[True] == got[False]
    # rounding may flip an arg-max between near-equal logits; most tokens still agree with 32-bit
    same = sum(a == b for g, x in zip(got[True], want) for a, b in zip(g, x))
    assert same >= 0.6 * sum(len(x) for x in want)


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
    assert whole.shape == (len(toks), V) and torch.isfinite(whole).all()
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


def test_command_line_generate(folder_b, greedy_want):
    import json
    import os
    import subprocess
    import sys
    d, w, cfg = folder_b
    prompts, want = greedy_want
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    cmd = [sys.executable, os.path.join(root, "bin", "tensorline"), "generate", "--model", d, "--dtype", "float32",
           "--num-blocks", "64", "--block-size", "8", "--max-tokens", "24", "--stop-token-id", "-1"]
    for p in prompts[1:3]:
        cmd += ["--prompt-ids", " ".join(map(str, p))]
    proc = subprocess.run(cmd, capture_output=True, text=True, timeout=300)
    assert proc.returncode == 0, proc.stderr[-2000:]
    recs = [json.loads(l) for l in proc.stdout.splitlines() if l.startswith("{")]
    assert [r["token_ids"] for r in recs] == want[1:3]
    assert all(r["finish_reason"] == "length" and r["completion_tokens"] == 24 for r in recs)


def test_library_tuning_keeps_results(folder_b):
    """Letting the library choose its kernels by measurement changes which kernel runs, not what a
    prompt portion computes."""
    from tensorline_amd import LLM, SamplingParams
    d, w, cfg = folder_b
    prompt = helpers.prompts_for("B", [150], seed=9)
    sp = SamplingParams(max_tokens=6, stop_token_ids=NO_STOP)
    plainly = LLM(d, dtype="bfloat16", device=DEV, num_blocks=64, block_size=8, max_batched_tokens=128)
    want = plainly.generate(prompt, sp)[0].token_ids
    tuned = LLM(d, dtype="bfloat16", device=DEV, num_blocks=64, block_size=8, max_batched_tokens=128, tune_library=True)
    try:
        assert tuned.model.tune_library(128) >= 1
        assert tuned.generate(prompt, sp)[0].token_ids == want
    finally:
        torch.cuda.tunable.enable(False)
