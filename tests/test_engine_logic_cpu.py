"""The engine's batch and cache logic against the plain implementation, on the CPU with kernel
stand-ins: every way of cutting must give the plain implementation's logits."""
import numpy as np
import pytest

from tensorline_amd.engine.loading import load_model
from tensorline_amd.engine.replay import TraceSession
from tests import helpers, plain


@pytest.fixture(scope="module", params=["A", "B", "C"])
def setup(request, tmp_path_factory):
    name = request.param
    d = helpers.make_model_dir(tmp_path_factory, name, seed=3)
    w, cfg = plain.load_folder(d)
    lengths = {"A": [5, 17, 33, 70], "B": [1, 8, 31, 64, 100], "C": [2, 40, 65]}[name]
    reqs = {f"r{i}": p for i, p in enumerate(helpers.prompts_for(name, lengths, seed=7))}
    return name, d, reqs, helpers.plain_logits(w, cfg, reqs)


@pytest.mark.parametrize("cut", ["whole", "decode", "portions", "mixed"])
def test_cuttings_match_plain(setup, cut, cpu_kernels):
    name, d, reqs, want = setup
    steps = {"whole": helpers.steps_whole, "decode": helpers.steps_prefill_then_decode,
             "portions": helpers.steps_portions, "mixed": helpers.steps_mixed}[cut](reqs)
    model, _ = load_model(d, "float32", "cpu")
    session = TraceSession(model, helpers.max_live_tokens(steps), page_size=helpers.PAGE[name])
    got = helpers.collect_logits(session.step, steps)
    assert set(got) == set(want)
    for key in want:
        np.testing.assert_allclose(got[key], want[key], atol=2e-5, rtol=1e-4, err_msg=str(key))
    assert session.cache.all_free()
    session.cache.check()


def test_more_live_requests_than_the_default_when_asked_for(setup, cpu_kernels):
    """The number of requests live at a time is the caller's to give: ten at once with room for
    twelve, and a clear error where the room is too small."""
    from tensorline_amd.engine.replay import TraceError
    name, d, reqs, want = setup
    if name != "A":
        pytest.skip("one configuration is enough")
    model, _ = load_model(d, "float32", "cpu")
    toks = reqs["r1"]
    ids = [f"x{i}" for i in range(10)]
    session = TraceSession(model, 64 * len(ids), page_size=16, max_requests=12)
    got = session.step([{"id": i, "tokens": toks, "want": [len(toks) - 1]} for i in ids], end=ids[:5])
    for row in got:
        np.testing.assert_allclose(row, want[("r1", len(toks) - 1)], atol=2e-5, rtol=1e-4)
    assert len(session.cache.live_requests()) == 5
    small = TraceSession(model, 64 * len(ids), page_size=16, max_requests=4)
    with pytest.raises(TraceError, match="max-requests"):
        small.step([{"id": i, "tokens": toks, "want": []} for i in ids])
    # what a step may not bring: a token id outside the vocabulary, no tokens, a request twice, a place outside its tokens
    fresh = TraceSession(model, 128, page_size=16)
    for bad, word in (([{"id": "a", "tokens": [model.vocab_size], "want": []}], "token id"),
                      ([{"id": "a", "tokens": [-1], "want": []}], "token id"),
                      ([{"id": "a", "tokens": [], "want": []}], "no tokens"),
                      ([{"id": "a", "tokens": [1], "want": []}, {"id": "a", "tokens": [2], "want": []}], "twice")):
        with pytest.raises(TraceError, match=word):
            fresh.step(bad)
    with pytest.raises(ValueError, match="outside its 2 tokens"):
        fresh.step([{"id": "b", "tokens": [1, 2], "want": [2]}])
