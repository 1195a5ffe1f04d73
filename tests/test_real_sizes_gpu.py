"""Models with the layer sizes of Qwen2.5-7B (hidden 3584, 28 query and 4 key/value heads of 128,
feed-forward 18944, vocabulary 152064; 2 of its 28 layers), of Qwen2.5-14B (hidden 5120, 40 and 8
heads, feed-forward 13824; 1 of its 48 layers) and of Qwen2.5-32B (the same with a feed-forward of
27648; 1 of its 64 layers) against the plain implementation: the branches that only real sizes
take (the wide head, products cut into shares of K, groups of seven and of five query heads, 224
and 320 column tiles for 256 CUs, hundreds of column groups in prompt attention, the 17-to-64-row
kernels and graph buckets above 16 rows) as a whole model, in 32-bit and in bfloat16 (analogue of
the reference's tests/test_batching.py:48-64 at sizes its own tests never reach).  The 7B sizes
run every way of cutting; the two wider shapes run whole prompts, prompt then decoding, and 8 and
40 rows decoding from graphs."""
import random

import numpy as np
import pytest
import torch

from tests import helpers, plain

pytestmark = pytest.mark.gpu

SHAPE_7B = dict(
    architectures=["Qwen2ForCausalLM"], vocab_size=152064, hidden_size=3584, intermediate_size=18944,
    num_hidden_layers=2, num_attention_heads=28, num_key_value_heads=4, head_dim=128, rope_theta=1000000.0,
    rms_norm_eps=1e-6, tie_word_embeddings=False, max_position_embeddings=32768)
SHAPE_14B = dict(SHAPE_7B, hidden_size=5120, intermediate_size=13824, num_hidden_layers=1, num_attention_heads=40,
                 num_key_value_heads=8, rms_norm_eps=1e-5)
SHAPE_32B = dict(SHAPE_14B, intermediate_size=27648, rms_norm_eps=1e-6)
SHAPES = {"7b-2-of-28-layers": SHAPE_7B, "14b-1-of-48-layers": SHAPE_14B, "32b-1-of-64-layers": SHAPE_32B}
S7, S14, S32 = SHAPES
LENGTHS = {"tiny": 3, "short": 70, "mid": 200, "long": 2100}
LIMIT = {"float32": 1e-5, "bfloat16": 2e-2}
PAGE = 16


def kept_positions(n: int) -> list[int]:
    """Where logits are compared: the first tokens, both sides of page and tile edges, a sparse
    sweep, and the last 40 (all of them for short requests)."""
    if n <= 256:
        return list(range(n))
    keep = {0, 1, 2, 15, 16, 17, 63, 64, 65, 127, 128, 1023, 1024, 2047, 2048}
    keep |= set(range(0, n, 97)) | set(range(n - 40, n))
    return sorted(p for p in keep if p < n)


def build_oracle(shape: str, folder: str):
    """The model folder of a shape, requests, and the plain implementation's logits at the kept positions."""
    from tensorline_amd.config import Qwen2Config
    from tensorline_amd.weights import write_random_model
    print(f"real sizes: writing and running the plain model of {shape}", flush=True)
    d = write_random_model(Qwen2Config.from_dict(SHAPES[shape]), folder, seed=17)
    w, cfg = plain.load_folder(d)
    rng = random.Random(23)
    reqs = {name: [rng.randrange(cfg["vocab_size"]) for _ in range(n)] for name, n in LENGTHS.items()}
    want = {}
    with torch.inference_mode():
        for name, toks in reqs.items():
            logits = plain.model_forward(w, cfg, toks)
            for p in kept_positions(len(toks)):
                want[(name, p)] = logits[p].numpy().copy()
            del logits
    del w
    return d, reqs, want, {}


@pytest.fixture(scope="module")
def oracles(tmp_path_factory):
    """``oracles(shape)``: built at the first call for a shape and kept until the module's tests are
    through, whatever order they run in (three folders of a few gigabytes, six models on the GPU)."""
    import shutil
    built = {}

    def get(shape):
        if shape not in built:
            built[shape] = build_oracle(shape, str(tmp_path_factory.mktemp("real_sizes")))
        return built[shape]
    yield get
    for d, _, _, models in built.values():
        models.clear()
        shutil.rmtree(d, ignore_errors=True)
    torch.cuda.empty_cache()


def model_of(oracle, dtype: str):
    """The engine's model of the shape in one dtype, loaded once."""
    from tensorline_amd.engine.loading import load_model
    models = oracle[3]
    if dtype not in models:
        models[dtype] = load_model(oracle[0], dtype, "cuda:0")[0]
    return models[dtype]


def only_kept(steps, source_of=lambda rid: rid):
    """The same steps, asking only for the logits at the kept positions of each request."""
    done: dict[str, int] = {}
    out = []
    for st in steps:
        entries = []
        for e in st["entries"]:
            base = done.get(e["id"], 0)
            keep = set(kept_positions(LENGTHS[source_of(e["id"])]))
            entries.append({"id": e["id"], "tokens": e["tokens"], "want": [w for w in e["want"] if base + w in keep]})
            done[e["id"]] = base + len(e["tokens"])
        out.append({"entries": entries, "end": st["end"]})
    return out


def compare(got, want, source_of=lambda rid: rid, limit=1e-5):
    scale = {}
    for (name, p), row in want.items():
        scale[name] = max(scale.get(name, 0.0), float(np.abs(row).max()))
    worst = 0.0
    for (rid, p), row in got.items():
        name = source_of(rid)
        err = float(np.abs(row - want[(name, p)]).max()) / scale[name]
        assert np.isfinite(err) and err < limit, f"request {rid} position {p}: relative error {err:.3e} >= {limit}"
        worst = max(worst, err)
    return worst


CUTS = {"whole": helpers.steps_whole, "decode": helpers.steps_prefill_then_decode,
        "portions": lambda reqs: helpers.steps_portions(reqs, sizes=(700, 130, 2, 64, 513, 17, 300, 3)),
        "mixed": lambda reqs: helpers.steps_mixed(reqs, seed=3, tail=12)}


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("shape, cut", [(S7, c) for c in CUTS] + [(s, c) for s in (S14, S32) for c in ("whole", "decode")])
def test_cuttings_match_plain_at_real_layer_sizes(oracles, shape, cut, dtype):
    from tensorline_amd.engine.replay import TraceSession
    d, reqs, want, _ = oracle = oracles(shape)
    model = model_of(oracle, dtype)
    steps = only_kept(CUTS[cut](reqs))
    session = TraceSession(model, helpers.max_live_tokens(steps), page_size=PAGE)
    got = helpers.collect_logits(session.step, steps)
    assert set(got) == set(want)
    worst = compare(got, want, limit=LIMIT[dtype])
    print(f"real layer sizes, {cut} {dtype}: worst relative error {worst:.3e}")
    assert session.cache.all_free()


def batch_decode_steps(copies: dict[str, list[int]], tail: int, budget: int = 2048):
    """Every request's tokens but the last ``tail`` as whole prompts, several to a step under a
    token budget; then ``tail`` steps in which every request decodes one token."""
    steps, entries, used = [], [], 0
    for rid, toks in copies.items():
        n = len(toks) - tail
        if entries and used + n > budget:
            steps.append({"entries": entries, "end": []})
            entries, used = [], 0
        entries.append({"id": rid, "tokens": toks[:n], "want": list(range(n))})
        used += n
    steps.append({"entries": entries, "end": []})
    for i in range(tail, 0, -1):
        steps.append({"entries": [{"id": rid, "tokens": [toks[len(toks) - i]], "want": [0]} for rid, toks in copies.items()],
                      "end": list(copies) if i == 1 else []})
    return steps


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize(
    "shape, rows, graphs",
    [(S7, 8, False), (S7, 8, True), (S7, 40, False), (S7, 40, True), (S7, 72, True)]
    + [(s, rows, True) for s in (S14, S32) for rows in (8, 40)])
def test_decoding_many_rows_at_real_layer_sizes(oracles, shape, rows, graphs, dtype):
    """The last 32 tokens of 8, 40 and 72 requests decoded together: the few-row and the
    17-to-64-row kernels of the bfloat16 path, eagerly and replayed from the graphs of the buckets
    of 8 and of 40 rows, and the library's products (the down projection's K in shares) inside the
    graph of 128 rows."""
    from tensorline_amd.engine.replay import TraceSession
    d, reqs, want, _ = oracle = oracles(shape)
    model = model_of(oracle, dtype)
    names = ["short", "mid", "long", "short", "mid"] if rows == 8 else ["short", "mid"]
    source = {f"c{i}": ("long" if rows >= 40 and i in (7, 31) else names[i % len(names)]) for i in range(rows)}
    copies = {rid: reqs[name] for rid, name in source.items()}
    steps = only_kept(batch_decode_steps(copies, tail=32), source.get)
    # room for 64 requests: 40 rows then replay the graph of 64 rows, 24 of them padding
    session = TraceSession(model, helpers.max_live_tokens(steps), page_size=PAGE,
                           max_requests=128 if rows > 64 else 64 if rows > 16 else 8, graphs=graphs)
    got = helpers.collect_logits(session.step, steps)
    assert {(source[rid], p) for rid, p in got} == {k for k in want if k[0] in set(source.values())}
    worst = compare(got, want, source.get, LIMIT[dtype])
    print(f"real layer sizes, {rows} rows decoding, graphs={graphs}, {dtype}: worst relative error {worst:.3e}")
    if graphs:
        assert session.runner.graph_replays == 32
        widest = max(b for b, c in session.runner.graphs)
        assert widest >= rows and (rows <= 16 or widest > 16)
    assert session.cache.all_free()


def test_tuned_library_products_match_plain(oracles):
    """With the library's kernels for a full prompt portion chosen by measurement, as the benchmark
    and serving run them, whole prompts in bfloat16 still give the plain logits: the chosen kernels
    are compared with the plain implementation, not with the engine's untuned self."""
    from tensorline_amd.engine.loading import load_model
    from tensorline_amd.engine.replay import TraceSession
    d, reqs, want, _ = oracles(S7)
    model, _ = load_model(d, "bfloat16", "cuda:0")
    searched = model.tune_library(len(reqs["long"]))       # the row count of the step that is compared
    assert searched >= 4, "q/k/v, o, gate/up and down were to be searched"
    steps = only_kept(helpers.steps_whole({"long": reqs["long"], "mid": reqs["mid"]}))
    session = TraceSession(model, helpers.max_live_tokens(steps), page_size=PAGE)
    got = helpers.collect_logits(session.step, steps)
    worst = compare(got, want, limit=LIMIT["bfloat16"])
    print(f"7B layer sizes, tuned library products, whole prompts, bfloat16: worst relative error {worst:.3e}")
    assert session.cache.all_free()
