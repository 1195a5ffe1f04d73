"""Replay on the GPU: every way of cutting requests into steps gives the plain implementation's
logits, in 32-bit and in bfloat16."""
import json
import os
import subprocess
import sys

import numpy as np
import pytest

from tests import helpers, plain

pytestmark = pytest.mark.gpu

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
LENGTHS = {"A": [5, 17, 33, 70, 130], "B": [1, 8, 31, 64, 100, 300], "C": [2, 40, 65, 257], "D": [3, 64, 97, 600]}
# error of the logits relative to the largest logit of the request
LIMIT = {"float32": 1e-5, "bfloat16": 2e-2}


@pytest.fixture(scope="module", params=["A", "B", "C", "D"])
def setup(request, tmp_path_factory):
    name = request.param
    d = helpers.make_model_dir(tmp_path_factory, name, seed=5)
    w, cfg = plain.load_folder(d)
    reqs = {f"r{i}": p for i, p in enumerate(helpers.prompts_for(name, LENGTHS[name], seed=9))}
    return name, d, reqs, helpers.plain_logits(w, cfg, reqs)


def _compare(got, want, reqs, limit):
    assert set(got) == set(want)
    worst = 0.0
    for rid, toks in reqs.items():
        scale = max(float(np.abs(want[(rid, i)]).max()) for i in range(len(toks)))
        for i in range(len(toks)):
            err = float(np.abs(got[(rid, i)] - want[(rid, i)]).max()) / scale
            assert np.isfinite(err) and err < limit, f"request {rid} position {i}: relative error {err:.3e} >= {limit}"
            worst = max(worst, err)
    return worst


CUTS = {"whole": helpers.steps_whole, "decode": helpers.steps_prefill_then_decode,
        "portions": helpers.steps_portions, "mixed": helpers.steps_mixed}


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("cut", list(CUTS))
def test_cuttings_match_plain(setup, cut, dtype):
    from tensorline_amd.engine.loading import load_model
    from tensorline_amd.engine.replay import TraceSession
    name, d, reqs, want = setup
    steps = CUTS[cut](reqs)
    model, _ = load_model(d, dtype, "cuda:0")
    # the pool is as small as the trace allows, so pages are used again
    session = TraceSession(model, helpers.max_live_tokens(steps), page_size=helpers.PAGE[name])
    pages = helpers.watch_pages(session.cache)
    got = helpers.collect_logits(session.step, steps)
    worst = _compare(got, want, reqs, LIMIT[dtype])
    print(f"config {name} {cut} {dtype}: worst relative error {worst:.3e}, {helpers.reused(pages)} pages used again")
    assert session.cache.all_free()
    session.cache.check()
    if cut == "mixed":             # the point of the small pool: later requests compute on pages earlier ones left
        assert helpers.reused(pages) >= 4, "no page was handed out twice: the pool is too large to test reuse"


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_decode_tail_replayed_from_graphs_matches_plain(setup, dtype):
    """The cut that decodes the last 32 tokens one by one, with every pure decode step replayed
    from a HIP graph as in serving (prompt portions still run eagerly): same logits."""
    from tensorline_amd.engine.loading import load_model
    from tensorline_amd.engine.replay import TraceSession
    name, d, reqs, want = setup
    steps = helpers.steps_prefill_then_decode(reqs)
    model, _ = load_model(d, dtype, "cuda:0")
    session = TraceSession(model, helpers.max_live_tokens(steps), page_size=helpers.PAGE[name], max_requests=4, graphs=True)
    got = helpers.collect_logits(session.step, steps)
    _compare(got, want, reqs, LIMIT[dtype])
    # every token after a request's first step is a decode step, and every decode step replays
    assert session.runner.graph_replays == sum(len(t) - max(1, len(t) - 32) for t in reqs.values())
    assert session.cache.all_free()


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_first_tokens_and_long_decode(setup, dtype):
    """A request that starts with one token and is decoded from there for a long time."""
    from tensorline_amd.engine.loading import load_model
    from tensorline_amd.engine.replay import TraceSession
    name, d, reqs, want = setup
    rid = max(reqs, key=lambda r: len(reqs[r]))
    one = {rid: reqs[rid]}
    steps = helpers.steps_prefill_then_decode(one, tail=len(reqs[rid]) - 1)
    model, _ = load_model(d, dtype, "cuda:0")
    session = TraceSession(model, helpers.max_live_tokens(steps), page_size=helpers.PAGE[name])
    got = helpers.collect_logits(session.step, steps)
    _compare(got, {k: v for k, v in want.items() if k[0] == rid}, one, LIMIT[dtype])


def test_mixed_steps_with_one_token_sequences_on_a_launch_of_their_own(setup, monkeypatch):
    """Steps that hold prompt portions beside decoded tokens give the latter's attention to a
    separate launch with split keys once their contexts are long; here whenever keys are split, so
    that the tiny configurations take that way, with few pages, against the plain implementation."""
    from tensorline_amd.engine.loading import load_model
    from tensorline_amd.engine.replay import TraceSession
    from tensorline_amd.ops import kernels
    name, d, reqs, want = setup
    monkeypatch.setattr(kernels, "_singles_get_own_launch", lambda *a: True)
    routed = []
    call = kernels._call

    def counting(fn, *args):
        if fn == "tl_attention_mfma" and args[-4].value:       # the list of one-token sequences
            routed.append(args[-3])
        return call(fn, *args)
    monkeypatch.setattr(kernels, "_call", counting)
    steps = helpers.steps_mixed(reqs)
    model, cfg = load_model(d, "bfloat16", "cuda:0")
    session = TraceSession(model, helpers.max_live_tokens(steps), page_size=helpers.PAGE[name])
    got = helpers.collect_logits(session.step, steps)
    _compare(got, want, reqs, LIMIT["bfloat16"])
    assert session.cache.all_free()
    if cfg.head_dim in (32, 64, 128):                 # other head sizes run the any-shape kernel
        assert routed and max(routed) >= 1, "no step gave its one-token sequences a launch of their own"


def test_wide_feed_forward_whose_product_comes_in_shares(tmp_path, monkeypatch):
    """A feed-forward so wide (8,192) that many-row steps compute the down projection in shares of
    K, which the next norm adds: whole prompts and portions against the plain implementation, and a
    step of few rows (no shares) beside them."""
    from tensorline_amd.config import Qwen2Config
    from tensorline_amd.engine.loading import load_model
    from tensorline_amd.engine.replay import TraceSession
    from tensorline_amd.weights import write_random_model
    cfg_dict = dict(architectures=["Qwen2ForCausalLM"], vocab_size=300, hidden_size=96, intermediate_size=8192,
                    num_hidden_layers=2, num_attention_heads=3, num_key_value_heads=1, head_dim=32,
                    rope_theta=10000.0, rms_norm_eps=1e-6, tie_word_embeddings=False, max_position_embeddings=512)
    d = write_random_model(Qwen2Config.from_dict(cfg_dict), str(tmp_path / "wide"), seed=2)
    w, cfg = plain.load_folder(d)
    import random
    rng = random.Random(1)
    reqs = {f"r{i}": [rng.randrange(300) for _ in range(n)] for i, n in enumerate([150, 9, 260])}
    want = helpers.plain_logits(w, cfg, reqs)
    model, _ = load_model(d, "bfloat16", "cuda:0")
    from tensorline_amd.ops import kernels
    made = []

    class CountedShareSum(kernels.ShareSum):
        def __init__(self, parts):
            super().__init__(parts)
            made.append(parts.shape[0])
    monkeypatch.setattr(kernels, "ShareSum", CountedShareSum)
    for steps in (helpers.steps_whole(reqs), helpers.steps_portions(reqs, sizes=(100, 70, 3, 90))):
        session = TraceSession(model, helpers.max_live_tokens(steps), page_size=16)
        got = helpers.collect_logits(session.step, steps)
        _compare(got, want, reqs, LIMIT["bfloat16"])
        assert session.cache.all_free()
    assert made and min(made) > 1, "no step computed the down projection in shares"


def test_trace_run_program(setup, tmp_path):
    """bin/trace_run as a user calls it: JSON lines in, <step>.f32 files and 'done' lines out."""
    name, d, reqs, want = setup
    if name != "B":
        pytest.skip("one configuration is enough for the program itself")
    steps = helpers.steps_mixed(reqs, seed=4)
    lines = [json.dumps({"step": i, **st}) for i, st in enumerate(steps)]
    out = tmp_path / "out"
    proc = subprocess.run(
        [sys.executable, os.path.join(ROOT, "bin", "trace_run"), "--model", d, "--dtype", "float32", "--out", str(out),
         "--max-tokens", str(helpers.max_live_tokens(steps)), "--block-size", str(helpers.PAGE[name])],
        input="\n".join(lines) + "\n", capture_output=True, text=True, timeout=600)
    assert proc.returncode == 0, proc.stderr[-2000:]
    assert [l for l in proc.stdout.splitlines() if l.startswith("done")] == [f"done {i}" for i in range(len(steps))]
    V = helpers.CONFIGS[name]["vocab_size"]
    files = {}

    def run_step(entries, end, _i=[0]):
        i = _i[0]
        _i[0] += 1
        path = out / f"{i}.f32"
        n = sum(len(e["want"]) for e in entries)
        if n == 0:
            assert not path.exists()
            return None
        return np.fromfile(path, dtype="<f4").reshape(n, V)

    got = helpers.collect_logits(run_step, steps)
    _compare(got, want, reqs, LIMIT["float32"])


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["A", "B"])
def test_massive_hidden_channels_keep_the_tolerance(name, dtype, tmp_path):
    """Trained checkpoints have a few hidden channels tens of times larger than the rest, fed by the
    embedding and by single rows of the down projections; random weights have none.  With two such
    channels (x60 and x-40 in the embedding, a down-projection row x20, a norm gain x8) the residual
    stream, the norms' sums of squares and the products that carry them must still give the plain
    logits within the usual limits, whole and with the last tokens decoded one by one."""
    import torch
    from safetensors.torch import load_file, save_file
    from tensorline_amd.engine.loading import load_model
    from tensorline_amd.engine.replay import TraceSession
    d = helpers.make_model_dir(tmp_path, name, seed=3)
    path = os.path.join(d, "model.safetensors")
    t = load_file(path)
    for k in list(t):
        if k.endswith("embed_tokens.weight"):
            t[k] = t[k].clone()
            t[k][:, 3] *= 60
            t[k][:, 17] *= -40
        if k.endswith("down_proj.weight"):
            t[k] = t[k].clone()
            t[k][3] *= 20
        if k.endswith("input_layernorm.weight"):
            t[k] = t[k].clone()
            t[k][17] *= 8
    save_file(t, path, metadata={"format": "pt"})
    w, cfg = plain.load_folder(d)
    assert float(w["model.embed_tokens.weight"][:, 3].abs().max()) > 20 * float(w["model.embed_tokens.weight"][:, 4].abs().max())
    reqs = {f"r{i}": p for i, p in enumerate(helpers.prompts_for(name, [3, 70, 129, 40], seed=5))}
    want = helpers.plain_logits(w, cfg, reqs)
    for cut in ("whole", "decode"):
        steps = CUTS[cut](reqs)
        model, _ = load_model(d, dtype, "cuda:0")
        session = TraceSession(model, helpers.max_live_tokens(steps), page_size=helpers.PAGE[name])
        worst = _compare(helpers.collect_logits(session.step, steps), want, reqs, LIMIT[dtype])
        print(f"config {name} with massive channels, {cut}, {dtype}: worst relative error {worst:.3e}")


LONG_TOKENS, LONG_PORTION, LONG_TAIL = 8192 + 33, 2048, 64


@pytest.fixture(scope="module", params=["B", "D"])
def long_case(request, tmp_path_factory):
    """One request of 8,225 tokens.  With weights as random as the others' every key would weigh about
    1/8000 and a run of keys left out or taken twice would hide in the tolerance, so the query and key
    projections are four times as large: the scores spread over a few units and a fraction of the keys,
    anywhere among the thousands, carries each position's sum.  (Six times as large, and the rounding
    of the bfloat16 scores alone, 2^-9 of a score of ten, takes the logits to the bfloat16 limit.)"""
    import torch
    from safetensors.torch import load_file, save_file
    name = request.param
    d = helpers.make_model_dir(tmp_path_factory, name, seed=31)
    path = os.path.join(d, "model.safetensors")
    t = load_file(path)
    for k in list(t):
        if k.endswith(("q_proj.weight", "k_proj.weight")):
            t[k] = (t[k].to(torch.float32) * 4).to(t[k].dtype)
    save_file(t, path, metadata={"format": "pt"})
    w, cfg = plain.load_folder(d)
    toks = helpers.prompts_for(name, [LONG_TOKENS], seed=13)[0]
    with torch.inference_mode():
        logits = plain.model_forward(w, cfg, toks)
    first_decoded = LONG_TOKENS - LONG_TAIL
    kept = sorted({min(s + LONG_PORTION, first_decoded) - 1 for s in range(0, first_decoded, LONG_PORTION)}
                  | set(range(first_decoded, LONG_TOKENS)))
    return name, d, toks, {p: logits[p].numpy().copy() for p in kept}


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_long_context_in_portions_then_decoded_across_a_graph_bucket_matches_plain(long_case, dtype):
    """A context of more than 8,192 tokens as a whole model against the plain implementation: the
    prompt in portions of 2,048 (prompt attention behind thousands of cached keys), the last 64
    tokens decoded one by one from graphs, across the edge between the context buckets of 8,192 and
    of the pool's size, where decode attention's key splits change their length."""
    from tensorline_amd.engine.loading import load_model
    from tensorline_amd.engine.replay import TraceSession
    name, d, toks, want = long_case
    first_decoded = LONG_TOKENS - LONG_TAIL
    steps = []
    for s in range(0, first_decoded, LONG_PORTION):
        n = min(LONG_PORTION, first_decoded - s)
        steps.append({"entries": [{"id": "long", "tokens": toks[s:s + n], "want": [n - 1]}], "end": []})
    for p in range(first_decoded, LONG_TOKENS):
        steps.append({"entries": [{"id": "long", "tokens": [toks[p]], "want": [0]}], "end": ["long"] if p == LONG_TOKENS - 1 else []})
    model, _ = load_model(d, dtype, "cuda:0")
    session = TraceSession(model, helpers.max_live_tokens(steps), page_size=helpers.PAGE[name], max_requests=2, graphs=True)
    got = helpers.collect_logits(session.step, steps)
    assert {p for _, p in got} == set(want)
    scale = max(float(np.abs(row).max()) for row in want.values())
    worst = 0.0
    for (_, p), row in got.items():
        err = float(np.abs(row - want[p]).max()) / scale
        assert np.isfinite(err) and err < LIMIT[dtype], f"position {p}: relative error {err:.3e} >= {LIMIT[dtype]}"
        worst = max(worst, err)
    print(f"config {name}, {LONG_TOKENS} tokens, {dtype}: worst relative error {worst:.3e}")
    assert session.runner.graph_replays == LONG_TAIL
    assert {c for _, c in session.runner.graphs} == {8192, session.runner.fit_context}, "both context buckets were to replay"
    assert session.cache.all_free()


def test_a_decoded_token_alone_and_beside_a_prompt_portion_agree_within_rounding(tmp_path):
    """What is promised about batch mates in 32-bit: a token decoded in a step of its own and the
    same token decoded beside another request's prompt portion are summed in different orders (the
    attention kernel and the products choose their form from the step), so their logits are not
    the same bits, but they differ by rounding only: both within the 32-bit limit of the plain
    logits, and of each other."""
    from tensorline_amd.engine.loading import load_model
    from tensorline_amd.engine.replay import TraceSession
    for name in ("A", "B"):
        d = helpers.make_model_dir(tmp_path / name, name, seed=8)
        w, cfg = plain.load_folder(d)
        a, b = helpers.prompts_for(name, [300, 45], seed=14)
        want = plain.model_forward(w, cfg, a)[-1].numpy()
        model, _ = load_model(d, "float32", "cuda:0")
        rows = []
        for beside in (False, True):
            session = TraceSession(model, 512, page_size=helpers.PAGE[name])
            session.step([{"id": "a", "tokens": a[:-1], "want": []}])
            entries = [{"id": "a", "tokens": a[-1:], "want": [0]}]
            if beside:
                entries.insert(0, {"id": "b", "tokens": b, "want": []})
            rows.append(session.step(entries, ["a", "b"] if beside else ["a"])[0])
        scale = float(np.abs(want).max())
        for row in rows:
            assert float(np.abs(row - want).max()) / scale < LIMIT["float32"]
        assert float(np.abs(rows[0] - rows[1]).max()) / scale < LIMIT["float32"]


def test_long_portions_run_on_the_kernel_of_32_columns_per_wave_and_match_plain(tmp_path, monkeypatch):
    """A model with 16 query heads of 64 and a request of 8,200 tokens in portions of 2,048: from the
    third portion on (2,048 tokens behind 4,096 and more) prompt attention is given to the kernel
    with 32 columns per wave and work-groups of 256 columns; the logits at the end of every portion
    and at the decoded tokens are the plain ones.  Query and key projections are four times as
    large as random ones, so that a few keys among the thousands carry each sum."""
    import torch
    from safetensors.torch import load_file, save_file
    from tensorline_amd.config import Qwen2Config
    from tensorline_amd.engine.loading import load_model
    from tensorline_amd.engine.replay import TraceSession
    from tensorline_amd.ops import kernels
    from tensorline_amd.weights import write_random_model
    cfg_dict = dict(architectures=["Qwen2ForCausalLM"], vocab_size=500, hidden_size=256, intermediate_size=384,
                    num_hidden_layers=2, num_attention_heads=16, num_key_value_heads=4, head_dim=64, rope_theta=1e6,
                    rms_norm_eps=1e-6, tie_word_embeddings=False, max_position_embeddings=8192)
    d = write_random_model(Qwen2Config.from_dict(cfg_dict), str(tmp_path / "m"), seed=41)
    path = os.path.join(d, "model.safetensors")
    t = load_file(path)
    for k in list(t):
        if k.endswith(("q_proj.weight", "k_proj.weight")):
            t[k] = (t[k].to(torch.float32) * 4).to(t[k].dtype)
    save_file(t, path, metadata={"format": "pt"})
    w, cfg = plain.load_folder(d)
    total, portion, tail = 8200, 2048, 8
    toks = [(7 * i * i + 3 * i + 1) % 500 for i in range(total)]
    with torch.inference_mode():
        logits = plain.model_forward(w, cfg, toks)
    called = []
    call = kernels._call
    monkeypatch.setattr(kernels, "_call", lambda name, *a: (called.append(name), call(name, *a))[1])
    first_decoded = total - tail
    steps = []
    for s in range(0, first_decoded, portion):
        n = min(portion, first_decoded - s)
        steps.append({"entries": [{"id": "r", "tokens": toks[s:s + n], "want": [0, n // 2, n - 1]}], "end": []})
    for p in range(first_decoded, total):
        steps.append({"entries": [{"id": "r", "tokens": [toks[p]], "want": [0]}], "end": ["r"] if p == total - 1 else []})
    model, _ = load_model(d, "bfloat16", "cuda:0")
    session = TraceSession(model, helpers.max_live_tokens(steps), page_size=16)
    got = helpers.collect_logits(session.step, steps)
    assert called.count("tl_attention_tile32") == 2 * 2, "two layers, the third and the fourth portion"
    scale = float(logits.abs().max())
    worst = max(float(np.abs(row - logits[p].numpy()).max()) / scale for (_, p), row in got.items())
    print(f"16 heads of 64, {total} tokens in portions of {portion}, bfloat16: worst relative error {worst:.3e}")
    assert worst < LIMIT["bfloat16"]
