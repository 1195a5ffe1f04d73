"""Seeded random configurations of the architecture, each with its own random weights, requests
and way of cutting them into steps, against the plain implementation, in 32-bit and in bfloat16.
The two fixed configurations of the other tests pin known traps; these walk the sizes between
them: head sizes in steps of 16 (most of which only the any-shape kernels take), groups of 1 to 7
query heads, widths and vocabularies that are no power of two, tied and untied heads, pages of 8
to 64 tokens, and contexts long enough that one-token steps split their keys."""
import os
import random
import tempfile

import numpy as np
import pytest

from tests import helpers, plain

pytestmark = pytest.mark.gpu
LIMIT = {"float32": 1e-5, "bfloat16": 2e-2}
CUTS = {"whole": helpers.steps_whole, "decode": helpers.steps_prefill_then_decode, "portions": helpers.steps_portions,
        "mixed": helpers.steps_mixed}


def _case(seed: int):
    rng = random.Random(9000 + seed)
    d = rng.choice([16, 32, 48, 64, 80, 96, 112, 128])
    nkv = rng.choice([1, 2, 3, 4])
    nq = nkv * rng.choice([1, 2, 3, 5, 7])
    cfg = dict(architectures=["Qwen2ForCausalLM"], vocab_size=rng.choice([97, 300, 512, 777, 1000, 2051]),
               hidden_size=rng.choice([40, 64, 72, 120, 136, 192, 200, 256]),
               intermediate_size=rng.choice([48, 88, 176, 200, 368, 520]), num_hidden_layers=rng.choice([1, 2, 3]),
               num_attention_heads=nq, num_key_value_heads=nkv, head_dim=d, rope_theta=rng.choice([1e4, 5e4, 1e6]),
               rms_norm_eps=rng.choice([1e-6, 1e-5, 3e-6]), tie_word_embeddings=rng.random() < 0.4,
               max_position_embeddings=1024)
    page = rng.choice([8, 16, 32, 64])
    lengths = [rng.choice([1, 2, 7, 31, 33, 64, 65, 100, 130, 257, 300, 530]) for _ in range(rng.choice([2, 3, 4, 5]))]
    cut = rng.choice(sorted(CUTS))
    return cfg, page, lengths, cut, rng


def _compare(cfg_dict, page, lengths, cut, rng, seed, what):
    from tensorline_amd.config import Qwen2Config
    from tensorline_amd.engine.loading import load_model
    from tensorline_amd.engine.replay import TraceSession
    from tensorline_amd.weights import write_random_model
    with tempfile.TemporaryDirectory() as tmp:
        folder = write_random_model(Qwen2Config.from_dict(cfg_dict), os.path.join(tmp, "m"), seed=seed)
        w, cfg = plain.load_folder(folder)
        reqs = {f"r{i}": [rng.randrange(cfg_dict["vocab_size"]) for _ in range(n)] for i, n in enumerate(lengths)}
        want = helpers.plain_logits(w, cfg, reqs)
        steps = CUTS[cut](reqs)
        for dtype in ("float32", "bfloat16"):
            model, _ = load_model(folder, dtype, "cuda:0")
            session = TraceSession(model, helpers.max_live_tokens(steps, round_to=max(64, page)), page_size=page)
            got = helpers.collect_logits(session.step, steps)
            for rid, toks in reqs.items():
                scale = max(float(np.abs(want[(rid, i)]).max()) for i in range(len(toks)))
                for i in range(len(toks)):
                    err = float(np.abs(got[(rid, i)] - want[(rid, i)]).max()) / scale
                    assert np.isfinite(err) and err < LIMIT[dtype], (what, dtype, rid, i, err)
            assert session.cache.all_free(), what


@pytest.mark.parametrize("seed", range(24))
def test_random_configuration_matches_plain(seed):
    cfg_dict, page, lengths, cut, rng = _case(seed)
    _compare(cfg_dict, page, lengths, cut, rng, seed, f"seed {seed}: {cfg_dict} page={page} lengths={lengths} cut={cut}")


@pytest.mark.parametrize("hidden,inter,vocab,d", [(50, 90, 97, 16), (7, 9, 11, 16), (100, 25, 33, 48), (1, 1, 2, 16),
                                                  (136, 88, 300, 160), (72, 176, 777, 256),
                                                  (64, 96, 200, 8), (96, 64, 301, 40), (128, 176, 500, 72), (80, 112, 150, 120)])
@pytest.mark.parametrize("cut", sorted(CUTS))
def test_odd_widths_and_large_heads_match_plain(hidden, inter, vocab, d, cut):
    """Widths that are no multiple of 8 (rows of the weights are not 16-byte aligned, so no streaming
    kernel takes them), down to a width of one, head sizes above 128, and head sizes between the
    kernels' steps of 16 (8, 40, 72, 120: served with zeros added to every head) through the whole model."""
    rng = random.Random(hidden * 1000 + d)
    nkv = rng.choice([1, 2, 3])
    cfg_dict = dict(architectures=["Qwen2ForCausalLM"], vocab_size=vocab, hidden_size=hidden, intermediate_size=inter,
                    num_hidden_layers=2, num_attention_heads=nkv * rng.choice([1, 2, 3]), num_key_value_heads=nkv, head_dim=d,
                    rope_theta=1e4, rms_norm_eps=1e-6, tie_word_embeddings=hidden % 4 == 0, max_position_embeddings=1024)
    page, lengths = rng.choice([8, 16, 32]), [rng.choice([2, 33, 65, 130]) for _ in range(3)]
    _compare(cfg_dict, page, lengths, cut, rng, hidden, f"{cfg_dict} page={page} lengths={lengths} cut={cut}")


@pytest.mark.parametrize("seed", range(12))
def test_random_trace_with_many_live_requests(seed):
    """Up to 70 live requests of a random configuration: prompts in random portions, a few requests
    to a step, then steps in which a random subset decodes one token each, so that batches of every
    size come up (graph buckets from 1 to 128 rows when graphs are on), until all have ended; every
    wanted logit against the plain implementation."""
    from tensorline_amd.config import Qwen2Config
    from tensorline_amd.engine.loading import load_model
    from tensorline_amd.engine.replay import TraceSession
    from tensorline_amd.weights import write_random_model
    rng = random.Random(7000 + seed)
    nkv = rng.choice([1, 2, 4])
    vocab, page = rng.choice([97, 300, 1000]), rng.choice([8, 16, 32])
    cfg_dict = dict(architectures=["Qwen2ForCausalLM"], vocab_size=vocab, hidden_size=rng.choice([40, 64, 136]),
                    intermediate_size=rng.choice([48, 176]), num_hidden_layers=rng.choice([1, 2]),
                    num_attention_heads=nkv * rng.choice([1, 2, 7]), num_key_value_heads=nkv, head_dim=rng.choice([16, 32, 48, 64, 128]),
                    rope_theta=1e4, rms_norm_eps=1e-6, tie_word_embeddings=rng.random() < 0.5, max_position_embeddings=1024)
    live_most = [2, 5, 17, 33, 70][seed % 5]
    graphs, dtype, tail = seed % 3 != 2, ("float32", "bfloat16")[seed % 2], 12
    what = f"seed {seed}: {cfg_dict} page={page} requests={live_most} graphs={graphs} {dtype}"
    with tempfile.TemporaryDirectory() as tmp:
        folder = write_random_model(Qwen2Config.from_dict(cfg_dict), os.path.join(tmp, "m"), seed=seed)
        w, cfg = plain.load_folder(folder)
        reqs = {f"r{i}": [rng.randrange(vocab) for _ in range(rng.choice([3, 10, 40, 70]) + tail)] for i in range(live_most)}
        want = helpers.plain_logits(w, cfg, reqs)
        done = {rid: 0 for rid in reqs}
        steps, pending = [], list(reqs)
        while pending:
            entries = []
            for rid in rng.sample(pending, min(len(pending), rng.choice([1, 3, 8]))):
                n = min(len(reqs[rid]) - tail - done[rid], rng.choice([2, 7, 30, 100]))
                entries.append({"id": rid, "tokens": reqs[rid][done[rid]:done[rid] + n], "want": [n - 1]})
                done[rid] += n
                if done[rid] == len(reqs[rid]) - tail:
                    pending.remove(rid)
            steps.append({"entries": entries, "end": []})
        live = list(reqs)
        while live:
            chosen = rng.sample(live, rng.randint(1, len(live)))
            steps.append({"entries": [{"id": rid, "tokens": [reqs[rid][done[rid]]], "want": [0]} for rid in chosen], "end": []})
            for rid in chosen:
                done[rid] += 1
                if done[rid] == len(reqs[rid]):
                    live.remove(rid)
                    steps[-1]["end"].append(rid)
        model, _ = load_model(folder, dtype, "cuda:0")
        session = TraceSession(model, sum(-(-len(t) // 64) * 64 for t in reqs.values()), page_size=page,
                               max_requests=live_most, graphs=graphs)
        at = {rid: 0 for rid in reqs}
        scale = {rid: max(float(np.abs(want[(rid, i)]).max()) for i in range(len(toks))) for rid, toks in reqs.items()}
        for number, st in enumerate(steps):
            out = session.step(st["entries"], st["end"])
            row = 0
            for e in st["entries"]:
                for place in e["want"]:
                    ref = want[(e["id"], at[e["id"]] + place)]
                    err = float(np.abs(out[row] - ref).max()) / scale[e["id"]]
                    assert np.isfinite(err) and err < LIMIT[dtype], (what, number, e["id"], err)
                    row += 1
                at[e["id"]] += len(e["tokens"])
        assert session.cache.all_free(), what
        if graphs:
            assert session.runner.graph_replays > 0 and max(b for b, c in session.runner.graphs) >= min(live_most, 16), what
