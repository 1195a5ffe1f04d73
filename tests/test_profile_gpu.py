"""The per-class kernel timer behind ``bench.py --profile`` (reference: the breakdown reported by
hand in README.md:80-86,248-259), on a tiny model."""
import pytest
import torch

from tests import helpers

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("dtype", ["bfloat16", "float32"])
def test_kernel_timer_books_every_launch_of_a_decode_step(tmp_path, dtype):
    """One eager decode step of three requests under ``KernelTimer``: every class of kernel has time
    and launches, the launches are those of the step (counted at the same door by a second, plain
    counter on a twin step), nothing stays patched afterwards, and the tokens are those of an
    unobserved engine."""
    from tensorline_amd import LLM, SamplingParams
    from tensorline_amd.ops import kernels
    from tensorline_amd.ops.profile import CLASSES, KernelTimer, kernel_class
    d = helpers.make_model_dir(tmp_path, "B", seed=4)
    prompts = helpers.prompts_for("B", [5, 19, 40], seed=6)
    sp = SamplingParams(max_tokens=6, stop_token_ids={-1})
    want = [o.token_ids for o in LLM(d, dtype=dtype, device="cuda:0", num_blocks=64, block_size=8, graphs=False).generate(prompts, sp)]

    llm = LLM(d, dtype=dtype, device="cuda:0", num_blocks=64, block_size=8, graphs=False, overlap=False)
    eng = llm.engine
    reqs = [eng.add_request(p, sp) for p in prompts]
    while any(r.num_generated < 2 for r in reqs):           # prompts done, every request decodes
        eng.step()
    call, library = kernels._call, kernels._library_linear
    counted = []
    kernels._call = lambda name, *a: (counted.append(name), call(name, *a))[1]
    try:
        eng.step()                                           # the twin step, counted without events
    finally:
        kernels._call = call
    timer = KernelTimer()
    with timer.measuring():
        eng.step()
    assert kernels._call is call and kernels._library_linear is library
    eng.run_until_done()
    assert [r.tokens[r.prompt_len:] for r in reqs] == want

    out = timer.summary()
    assert set(out["ms"]) == set(CLASSES) == set(out["launches"])
    for cls in CLASSES:
        assert out["ms"][cls] > 0 and out["launches"][cls] > 0, f"class {cls}: {out}"
        assert out["launches"][cls] == sum(kernel_class(n) == cls for n in counted)
    layers = 3
    assert out["launches"]["attention"] == layers and out["launches"]["sampling"] == 1
    assert out["launches"]["products"] >= 4 * layers + 1     # q/k/v, o, gate/up, down per layer, and the head
    assert abs(out["kernels_ms"] - sum(out["ms"].values())) < 1e-3 and out["host_ms"] > 0
    assert sum(out["top"].values()) <= out["kernels_ms"] + 1e-3
    torch.cuda.synchronize()
