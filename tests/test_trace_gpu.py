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
    got = helpers.collect_logits(session.step, steps)
    worst = _compare(got, want, reqs, LIMIT[dtype])
    print(f"config {name} {cut} {dtype}: worst relative error {worst:.3e}")
    assert session.cache.all_free()
    session.cache.check()


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
