#!/usr/bin/env python3
"""Decode and prefill throughput of the engine at the Qwen2.5-7B shape on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--batch 8] [--context 4096]

A step is one decode step of the whole batch through the engine loop (schedule, one graph replay
of the model, sampling, accept).  Weights are random (generated on the GPU from a seed), prompts
are token ids uniform over the vocabulary.  One JSON line is printed: decoded tokens per second
at the default batch, the prefill of one 2,048-token prompt, the decode step's share of the HBM
roofline, and under ``points`` decode throughput at batch 1 and 64 at the same context
(``decode_b*``) and the decode phase of the workload the shape is quoted with, 2,048-token
prompts and 256 generated tokens each, at batch 1, 8 and 64 (``gen_b*``), each with its time per
step, its mean context and its share of the HBM roofline.  ``fp32`` holds the cost of the true
32-bit path at the same layer sizes with fewer layers (both numbers are named), ``sizes`` batch 8
decoding and the same prefill at the 14B and 32B shapes (all layers) and, for the default shape,
batch 8 decoding at a context of 32,768 and a prompt portion behind 30,720 cached tokens.  The fractions
are of the published peaks; ``machine`` holds what this GPU reaches on a plain copy and on a
large library product, and the ``frac_of_measured_*`` fields are the same figures relative to
those.  ``--profile`` adds the time of one eagerly run decode step by class of kernel.
"""
from __future__ import annotations

import argparse
import gc
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

# MI355X published peaks
HBM_GBPS = 8000.0
PEAK_FLOPS = {"bfloat16": 2.5e15, "float32": 157.3e12}

# layer sizes of the Qwen2.5 shapes; the default run is the 7B one
SHAPE_7B = dict(vocab_size=152064, hidden_size=3584, intermediate_size=18944, num_hidden_layers=28,
                num_attention_heads=28, num_key_value_heads=4, head_dim=128, rope_theta=1000000.0,
                rms_norm_eps=1e-6, tie_word_embeddings=False, max_position_embeddings=32768)
SHAPE_14B = dict(SHAPE_7B, hidden_size=5120, intermediate_size=13824, num_hidden_layers=48, num_attention_heads=40,
                 num_key_value_heads=8, rms_norm_eps=1e-5)
SHAPE_32B = dict(SHAPE_7B, hidden_size=5120, intermediate_size=27648, num_hidden_layers=64, num_attention_heads=40,
                 num_key_value_heads=8)
SHAPES = {"7b": SHAPE_7B, "14b": SHAPE_14B, "32b": SHAPE_32B}


def make_config(layers: int | None, shape: str = "7b", positions: int = 0):
    from tensorline_amd.config import Qwen2Config
    d = dict(SHAPES[shape], architectures=["Qwen2ForCausalLM"])
    if layers:
        d["num_hidden_layers"] = layers
    if positions:
        d["max_position_embeddings"] = positions
    return Qwen2Config.from_dict(d)


def layer_matrix_params(cfg) -> int:
    H, I = cfg.hidden_size, cfg.intermediate_size
    return (cfg.q_size + 2 * cfg.kv_size) * H + cfg.q_size * H + 3 * H * I


def decode_bytes(cfg, batch: int, context: int, elem: int = 2) -> float:
    """Bytes a decode step has to read: every weight it uses once, and the cache of the live requests."""
    L, H, V = cfg.num_hidden_layers, cfg.hidden_size, cfg.vocab_size
    weights = (L * layer_matrix_params(cfg) + V * H) * elem
    weights += L * (cfg.q_size + 2 * cfg.kv_size) * 4 + (2 * L + 1) * H * 4          # biases and norm weights
    weights += batch * H * elem                                                        # embedding rows
    kv = batch * context * 2 * cfg.kv_size * elem * L
    return float(weights + kv)


def prefill_flops(cfg, tokens: int, rows: int = 1) -> float:
    L, V, H = cfg.num_hidden_layers, cfg.vocab_size, cfg.hidden_size
    linear = 2.0 * tokens * L * layer_matrix_params(cfg)
    attn = 4.0 * cfg.num_attention_heads * cfg.head_dim * (tokens * (tokens + 1) / 2) * L
    head = 2.0 * rows * V * H
    return linear + attn + head


def random_prompts(n: int, length: int, vocab: int, seed: int):
    import numpy as np
    rng = np.random.default_rng(seed)
    return [rng.integers(0, vocab, size=length).tolist() for _ in range(n)]


def sync():
    import torch
    torch.cuda.synchronize()


def bench_decode(llm, batch: int, context: int, steps: int, warmup: int, seed: int) -> dict:
    """Fill ``batch`` sequences, then time ``steps`` decode steps in which every sequence decodes one
    token.  Prompts are prefilled in portions under the engine's token budget; sequences admitted
    early decode while the later ones are still being prefilled (continuous batching), so prompts
    are shortened by the number of prefill steps: no sequence passes ``context`` tokens before the
    last timed step, and none finishes before it."""
    from tensorline_amd import SamplingParams
    cfg = llm.model_config
    eng = llm.engine
    budget = eng.scheduler.max_batched_tokens
    prompt_len = context - (warmup + steps) - 1
    prefill_steps = -(-batch * prompt_len // budget) + 1
    prompt_len -= prefill_steps if batch > 1 else 0
    assert prompt_len >= 1
    reqs = [eng.add_request(p, SamplingParams(max_tokens=10 ** 9, stop_token_ids={-1}))
            for p in random_prompts(batch, prompt_len, cfg.vocab_size, seed)]
    t0 = time.perf_counter()
    while any(r.num_computed < r.prompt_len for r in reqs):          # prefill, in portions
        eng.step()
    sync()
    fill_s = time.perf_counter() - t0
    for _ in range(warmup):
        eng.step()
    eng.drain()                                                      # nothing in flight when the clock starts
    sync()
    assert all(not r.done for r in reqs) and len(eng.scheduler.running) == batch and not eng.scheduler.waiting
    import torch
    c0 = eng.counters()
    lens0 = [len(r.tokens) for r in reqs]
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    t0 = time.perf_counter()
    e0.record()
    for _ in range(steps):
        eng.step()
    eng.drain()                                                      # and nothing when it stops: K steps queued, K read
    e1.record()
    sync()
    dt = time.perf_counter() - t0
    c1 = eng.counters()
    lens1 = [len(r.tokens) for r in reqs]
    assert c1["tokens_generated"] - c0["tokens_generated"] == batch * steps, "a timed step did not decode every sequence"
    assert all(b - a == steps for a, b in zip(lens0, lens1)) and max(lens1) <= context + 1
    assert c1["preemptions"] == c0["preemptions"], "a sequence was preempted inside the timed steps"
    mean_ctx = (sum(lens0) + sum(lens1)) / (2.0 * batch)
    out = {"tok_s": batch * steps / dt, "ms_per_step": dt / steps * 1e3, "fill_s": fill_s, "mean_context": mean_ctx,
           "graph_replays": c1["graph_replays"] - c0["graph_replays"], "ms_per_step_events": e0.elapsed_time(e1) / steps}
    for r in reqs:
        eng.abort(r)
    assert llm.cache.all_free()
    return out


def bench_decode_at_context(llm, batch: int, context: int, steps: int, warmup: int, seed: int) -> dict:
    """Decode steps of ``batch`` sequences at a long context without the prefill that would put them
    there (a million tokens for 64 sequences at 16,384): every sequence is given pages for ``context``
    tokens of a cache filled with random values, and the step function (the graphs' runner, as in
    serving) decodes ``warmup + steps`` tokens for each, the engine's greedy pick read after every
    step.  What a step reads and computes is what it would after a real prompt; the scheduler and the
    overlap of its host work with the step before are not part of this measurement."""
    import torch

    from tensorline_amd.engine.batch import StepEntry
    from tensorline_amd.ops import kernels
    cfg, cache, runner = llm.model_config, llm.cache, llm.engine.runner
    g = torch.Generator(device="cuda:0").manual_seed(seed)
    for i in range(len(llm.model.schedule)):
        if cache.owns_storage(i):
            for plane in cache.storage(i).values():
                plane.normal_(0.0, 0.5, generator=g)
    first = context - (warmup + steps)
    rids = [("long", i) for i in range(batch)]
    for rid in rids:
        cache.add_request(rid)
        assert cache.grow(rid, context), "the pool is too small for this point"
    tokens = [p[0] for p in random_prompts(batch, 1, cfg.vocab_size, seed)]
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    t0 = 0.0
    for s in range(warmup + steps):
        if s == warmup:
            sync()
            t0 = time.perf_counter()
            e0.record()
        logits = runner.step([StepEntry(rid, [tok], first + s, [0]) for rid, tok in zip(rids, tokens)])
        tokens = kernels.argmax(logits).tolist()
    e1.record()
    sync()
    dt = time.perf_counter() - t0
    for rid in rids:
        cache.release(rid)
    assert cache.all_free()
    return {"tok_s": batch * steps / dt, "ms_per_step": dt / steps * 1e3, "ms_per_step_events": e0.elapsed_time(e1) / steps,
            "mean_context": first + warmup + (steps + 1) / 2.0, "fill_s": 0.0, "graph_replays": 0}


def bench_generate(llm, batch: int, prompt_len: int, new_tokens: int, seed: int) -> dict:
    """The decode phase of the workload the shape is quoted with: ``batch`` requests, each a prompt of
    ``prompt_len`` random tokens and ``new_tokens`` generated ones.  Prompts are prefilled under the
    engine's token budget (requests admitted early decode meanwhile); the timed steps are those
    from the moment every prompt is cached until the first request ends, so each of them decodes
    one token for every one of the ``batch`` requests."""
    import torch

    from tensorline_amd import SamplingParams
    cfg, eng = llm.model_config, llm.engine
    reqs = [eng.add_request(p, SamplingParams(max_tokens=new_tokens, stop_token_ids={-1}))
            for p in random_prompts(batch, prompt_len, cfg.vocab_size, seed)]
    while any(r.num_computed < r.prompt_len for r in reqs):
        eng.step()
    eng.drain()
    sync()                                                  # every request has its first token; all decode from here
    assert all(not r.done for r in reqs) and len(eng.scheduler.running) == batch
    steps = new_tokens - max(r.num_generated for r in reqs)
    lens0 = [len(r.tokens) for r in reqs]
    g0 = eng.tokens_generated
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    t0 = time.perf_counter()
    e0.record()
    for _ in range(steps):
        eng.step()
    eng.drain()
    e1.record()
    sync()
    dt = time.perf_counter() - t0
    lens1 = [len(r.tokens) for r in reqs]
    assert eng.tokens_generated - g0 == batch * steps and all(b - a == steps for a, b in zip(lens0, lens1))
    eng.run_until_done()
    assert all(r.done and r.num_generated == new_tokens for r in reqs) and llm.cache.all_free()
    return {"tok_s": batch * steps / dt, "ms_per_step": dt / steps * 1e3, "steps": steps,
            "mean_context": (sum(lens0) + sum(lens1)) / (2.0 * batch), "ms_per_step_events": e0.elapsed_time(e1) / steps}


def profile_decode_step(llm, batch: int, context: int, seed: int) -> dict:
    """One decode step of ``batch`` sequences at about ``context`` tokens run eagerly, timed by class
    of kernel with events around every launch (tensorline_amd/ops/profile.py)."""
    from tensorline_amd import SamplingParams
    from tensorline_amd.engine.runner import ModelRunner
    from tensorline_amd.ops.profile import KernelTimer
    cfg, eng = llm.model_config, llm.engine
    prompt_len = context - 16 - (-(-batch * context // eng.scheduler.max_batched_tokens) if batch > 1 else 0)
    reqs = [eng.add_request(p, SamplingParams(max_tokens=10 ** 9, stop_token_ids={-1}))
            for p in random_prompts(batch, prompt_len, cfg.vocab_size, seed)]
    while any(r.num_computed < r.prompt_len for r in reqs):
        eng.step()
    eng.drain()
    graph_runner, eager, overlap = eng.runner, ModelRunner(llm.model, llm.cache), eng.overlap
    eager.fit_context = graph_runner.fit_context
    eng.runner, eng.overlap = eager, False                   # one step at a time, read before the next
    try:
        for _ in range(3):
            eng.step()
        timer = KernelTimer()
        with timer.measuring():
            eng.step()
    finally:
        eng.runner, eng.overlap = graph_runner, overlap
    for r in reqs:
        eng.abort(r)
    return timer.summary()


def bench_prefill(llm, tokens: int, reps: int, seed: int) -> dict:
    """One prompt of ``tokens`` tokens in one step, logits for its last position."""
    from tensorline_amd.engine.batch import StepEntry
    from tensorline_amd.ops import kernels
    cfg = llm.model_config
    cache, runner = llm.cache, llm.engine.runner
    prompt = random_prompts(1, tokens, cfg.vocab_size, seed)[0]
    times = []
    for i in range(reps + 1):
        rid = ("prefill", i)
        cache.add_request(rid)
        assert cache.grow(rid, tokens)
        sync()
        t0 = time.perf_counter()
        logits = runner.step([StepEntry(rid, prompt, 0, [tokens - 1])])
        kernels.argmax(logits).tolist()                                # the engine's greedy pick, as in a decode step
        sync()
        times.append(time.perf_counter() - t0)
        cache.release(rid)
    best = min(times[1:])                                              # the first run warms up
    return {"s": best, "tok_s": tokens / best}


def prefill_portion_flops(cfg, tokens: int, context: int) -> float:
    """A portion of ``tokens`` tokens behind ``context`` cached ones, logits for its last position."""
    L, V, H = cfg.num_hidden_layers, cfg.vocab_size, cfg.hidden_size
    linear = 2.0 * tokens * L * layer_matrix_params(cfg)
    attn = 4.0 * cfg.num_attention_heads * cfg.head_dim * (tokens * context + tokens * (tokens + 1) / 2) * L
    return linear + attn + 2.0 * V * H


def bench_prefill_portion(llm, context: int, tokens: int, reps: int, seed: int) -> dict:
    """A prompt portion of ``tokens`` tokens in one step behind ``context`` tokens that earlier steps
    cached (in portions of the same size), logits for its last position."""
    from tensorline_amd.engine.batch import StepEntry
    from tensorline_amd.ops import kernels
    cfg, cache, runner = llm.model_config, llm.cache, llm.engine.runner
    prompt = random_prompts(1, context + tokens, cfg.vocab_size, seed)[0]
    rid = ("portion", 0)
    cache.add_request(rid)
    assert cache.grow(rid, context + tokens)
    for start in range(0, context, tokens):
        n = min(tokens, context - start)
        runner.step([StepEntry(rid, prompt[start:start + n], start, [])])
    times = []
    for _ in range(reps + 1):                                          # the same portion again: it overwrites its own keys
        sync()
        t0 = time.perf_counter()
        logits = runner.step([StepEntry(rid, prompt[context:], context, [tokens - 1])])
        kernels.argmax(logits).tolist()
        sync()
        times.append(time.perf_counter() - t0)
    cache.release(rid)
    best = min(times[1:])
    return {"s": best, "tok_s": tokens / best}


def measure_machine(dtype) -> dict:
    """What this GPU reaches on two plain jobs, beside the published peaks: a device-to-device
    copy of 2 GiB (bytes read plus bytes written per second) and a square library product of
    8,192 rows in the benchmark's dtype (float32: the library's true 32-bit kernels)."""
    import torch
    src = torch.empty(1 << 30, dtype=torch.int16, device="cuda:0").fill_(1)
    dst = torch.empty_like(src)
    n = 8192
    a = torch.randn(n, n, dtype=dtype, device="cuda:0")
    b = torch.randn(n, n, dtype=dtype, device="cuda:0")

    def best_ms(fn, reps):
        fn()
        best = float("inf")
        for _ in range(reps):
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record()
            fn()
            e1.record()
            e1.synchronize()
            best = min(best, e0.elapsed_time(e1))
        return best
    copy_ms = best_ms(lambda: dst.copy_(src), 5)
    mm_ms = best_ms(lambda: torch.mm(a, b.t()), 5)
    return {"copy_GBps": round(2 * src.numel() * 2 / copy_ms / 1e6, 1),
            "gemm_TFLOPs": round(2 * n ** 3 / mm_ms / 1e9, 1)}


def run_workload(llm, requests: int, prompt_min: int, prompt_max: int, output_tokens: int, temperature: float,
                 seed: int) -> dict:
    """``requests`` prompts of uniform random length in [prompt_min, prompt_max] given to the scheduler
    at once (continuous batching, prompts in portions), ``output_tokens`` generated for each, greedy or
    seeded temperature sampling; the clock runs from the call to the last token."""
    import numpy as np
    import torch

    from tensorline_amd import SamplingParams
    cfg = llm.model_config
    rng = np.random.default_rng(seed)
    lengths = rng.integers(prompt_min, prompt_max + 1, size=requests)
    prompts = [rng.integers(0, cfg.vocab_size, size=int(n)).tolist() for n in lengths]
    params = [SamplingParams(max_tokens=output_tokens, temperature=temperature, top_p=1.0,
                             stop_token_ids={-1}, seed=seed + i) for i in range(requests)]
    c0 = llm.counters()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    outs = llm.generate(prompts, params)
    torch.cuda.synchronize()
    dt = time.perf_counter() - t0
    c = llm.counters()
    gen = sum(len(o.token_ids) for o in outs)
    assert all(len(o.token_ids) == output_tokens for o in outs) and llm.cache.all_free()
    ttft = sorted(o.stats.ttft_s for o in outs)
    steps = c["steps"] - c0["steps"]
    # what the run cannot do without: every step reads the weights once, every prompt token and every
    # generated token is multiplied with them once (attention left out: a lower bound on both)
    weight_bytes = decode_bytes(cfg, 0, 0, 2 if llm.model.dtype == torch.bfloat16 else 4)
    flops = 2.0 * (int(lengths.sum()) + gen) * cfg.num_hidden_layers * layer_matrix_params(cfg)
    return {"tok_s": gen / dt, "total_s": dt, "steps": steps, "prompt_tokens": int(lengths.sum()), "generated": gen,
            "ttft_p50_s": ttft[len(ttft) // 2], "ttft_max_s": ttft[-1],
            "preemptions": c["preemptions"] - c0["preemptions"], "graph_replays": c["graph_replays"] - c0["graph_replays"],
            "weight_reads_GBps": steps * weight_bytes / dt / 1e9, "product_flops_per_s": flops / dt}


def bench_workload(args) -> int:
    """A serving-style run: many concurrent requests through the scheduler (continuous batching,
    chunked prefill), as in the 14B and 32B workloads: ``--requests`` prompts of uniform random
    length in [--prompt-min, --prompt-max], ``--output-tokens`` each, greedy or seeded temperature
    sampling.  Prints one JSON line: generated tokens per second over the whole run."""
    from tensorline_amd import LLM
    cfg = make_config(args.layers, args.shape)
    max_len = args.prompt_max + args.output_tokens + 16
    page = 16
    llm = LLM(config=cfg, seed=args.seed, dtype=args.dtype, device="cuda:0", block_size=page,
              num_blocks=args.num_blocks or None, kv_mem_fraction=0.8, max_num_seqs=args.requests,
              max_batched_tokens=2048, max_model_len=max_len, graphs=not args.no_graphs, prefix_caching=False,
              tune_library=not args.no_tune)
    w = run_workload(llm, args.requests, args.prompt_min, args.prompt_max, args.output_tokens, args.temperature, args.seed)
    print(json.dumps({
        "metric": f"generated tok/s, {args.requests} concurrent requests (Qwen2.5-{args.shape.upper()} shape)",
        "value": round(w["tok_s"], 1), "unit": "tok/s", "n_gpus": 1, "steps": w["steps"], "warmup": 0,
        "ms_per_step": round(w["total_s"] / max(w["steps"], 1) * 1e3, 3), "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": "bf16" if args.dtype in ("bfloat16", "bf16") else "fp32",
        "data": "synthetic: random weights from a seed, token ids uniform over the vocabulary",
        "config": {"model": f"Qwen2.5-{args.shape.upper()} shape", "global_batch": args.requests, "seq_len": max_len,
                   "parallelism": "single GPU", "layers": cfg.num_hidden_layers,
                   "layers_of_shape": SHAPES[args.shape]["num_hidden_layers"], "prompt_min": args.prompt_min,
                   "prompt_max": args.prompt_max, "output_tokens": args.output_tokens, "prompt_tokens": w["prompt_tokens"],
                   "temperature": args.temperature, "chunk": 2048, "kv_pages": llm.cache.num_blocks, "page_size": page,
                   "preemptions": w["preemptions"], "graph_replays": w["graph_replays"],
                   "ttft_p50_s": round(w["ttft_p50_s"], 3), "ttft_max_s": round(w["ttft_max_s"], 3),
                   "total_s": round(w["total_s"], 2)}}))
    return 0


def main() -> int:
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=64)
    ap.add_argument("--warmup", type=int, default=8)
    ap.add_argument("--batch", type=int, default=8)
    ap.add_argument("--context", type=int, default=4096)
    ap.add_argument("--layers", type=int, default=0, help="fewer layers than the shape has (0: all)")
    ap.add_argument("--dtype", default="bfloat16")
    ap.add_argument("--prefill-tokens", type=int, default=2048)
    ap.add_argument("--prefill-behind", type=int, default=0,
                    help="measure the prefill as a portion behind this many cached tokens (0: a fresh prompt)")
    ap.add_argument("--no-points", action="store_true", help="skip the batch 1 and 64 decode points")
    ap.add_argument("--no-graphs", action="store_true")
    ap.add_argument("--no-overlap", action="store_true", help="read every decode step's tokens before queueing the next")
    ap.add_argument("--no-fp32", action="store_true", help="skip the 32-bit point")
    ap.add_argument("--no-sizes", action="store_true", help="skip the 14B and 32B shapes and the 32k contexts")
    ap.add_argument("--fp32-layers", type=int, default=4, help="layers of the model the 32-bit point runs")
    ap.add_argument("--profile", action="store_true", help="add the time of one eager decode step by class of kernel")
    ap.add_argument("--no-tune", action="store_true", help="keep the library's heuristic choice of kernels for prompt portions")
    ap.add_argument("--seed", type=int, default=0)
    ap.add_argument("--shape", default="7b", choices=sorted(SHAPES), help="layer sizes (default: the 7B shape)")
    ap.add_argument("--workload", action="store_true", help="serving-style run instead of the step benchmark")
    ap.add_argument("--requests", type=int, default=32)
    ap.add_argument("--prompt-min", type=int, default=256)
    ap.add_argument("--prompt-max", type=int, default=4096)
    ap.add_argument("--output-tokens", type=int, default=512)
    ap.add_argument("--temperature", type=float, default=0.7)
    ap.add_argument("--num-blocks", type=int, default=0, help="KV pages for --workload (0: 80%% of free memory)")
    args = ap.parse_args()
    if args.gpus != 1:
        print(f"bench.py: this engine runs on one GPU; --gpus {args.gpus} is not supported")
        return 2
    if args.workload:
        return bench_workload(args)

    import torch

    from tensorline_amd import LLM
    cfg = make_config(args.layers, args.shape)
    full_layers = SHAPES[args.shape]["num_hidden_layers"]
    max_batch = max(args.batch, 1 if args.no_points else 64)
    max_len = max(args.context, args.prefill_behind + args.prefill_tokens) + 16
    page = 16
    llm = LLM(config=cfg, seed=args.seed, dtype=args.dtype, device="cuda:0", block_size=page,
              num_blocks=max_batch * (-(-max_len // page)) + 8, max_num_seqs=max_batch, max_batched_tokens=2048,
              max_model_len=max_len, graphs=not args.no_graphs, graph_warmup_tokens=0, prefix_caching=False,
              tune_library=not args.no_tune, overlap=not args.no_overlap)
    elem = 2 if args.dtype in ("bfloat16", "bf16") else 4
    dtype_key = "bfloat16" if elem == 2 else "float32"

    def with_roofline(run: dict, batch: int, model_cfg=cfg, elem_size=elem) -> dict:
        """tok/s, ms per step (wall clock and events), mean context and the share of the HBM peak of a decode run."""
        gbps = decode_bytes(model_cfg, batch, int(run["mean_context"]), elem_size) / (run["ms_per_step"] / 1e3) / 1e9
        return {"tok_s": round(run["tok_s"], 1), "ms": round(run["ms_per_step"], 4), "ms_events": round(run["ms_per_step_events"], 4),
                "ctx": round(run["mean_context"], 1), "GBps": round(gbps, 1), "hbm_frac": round(gbps / HBM_GBPS, 4)}

    main_run = bench_decode(llm, args.batch, args.context, args.steps, args.warmup, args.seed + 1)
    if args.prefill_behind > 0:
        pre = bench_prefill_portion(llm, args.prefill_behind, args.prefill_tokens, 3, args.seed + 2)
    else:
        pre = bench_prefill(llm, args.prefill_tokens, 3, args.seed + 2)
    points = {}
    if not args.no_points:
        for b in (1, 64):
            k = max(8, args.steps // 2)
            r = with_roofline(bench_decode(llm, b, args.context, k, 4, args.seed + 3 + b), b)
            points[f"decode_b{b}"] = r["tok_s"]
            points.update({f"decode_b{b}_{key}": r[key] for key in ("ms", "ctx", "hbm_frac")})
        # the workload the shape is quoted with: 2,048-token prompts, 256 generated tokens each
        for b in (1, 8, 64):
            r = with_roofline(bench_generate(llm, b, 2048, 256, args.seed + 100 + b), b)
            points[f"gen_b{b}"] = r["tok_s"]
            points.update({f"gen_b{b}_{key}": r[key] for key in ("ms", "ms_events", "ctx", "hbm_frac")})
    profile = profile_decode_step(llm, args.batch, args.context, args.seed + 7) if args.profile else None

    machine = measure_machine(torch.bfloat16 if elem == 2 else torch.float32)
    fp32 = None
    if elem == 2 and not args.no_points and not args.no_fp32:
        # the true 32-bit path at the same layer sizes, fewer layers: what the equality checks cost
        llm = None
        gc.collect()
        torch.cuda.empty_cache()
        cfg32 = make_config(args.fp32_layers, args.shape)
        llm32 = LLM(config=cfg32, seed=args.seed, dtype="float32", device="cuda:0", block_size=page,
                    num_blocks=8 * (-(-max_len // page)) + 8, max_num_seqs=8, max_batched_tokens=2048,
                    max_model_len=max_len, graphs=not args.no_graphs, graph_warmup_tokens=0, prefix_caching=False)
        pre32 = bench_prefill(llm32, args.prefill_tokens, 2, args.seed + 2)
        dec32 = with_roofline(bench_decode(llm32, 8, 2304, 8, 2, args.seed + 9), 8, cfg32, 4)
        fp32 = {"layers": cfg32.num_hidden_layers, "layers_of_shape": full_layers,
                "prefill_tok_s": round(pre32["tok_s"], 1), "prefill_ms": round(pre32["s"] * 1e3, 3),
                "prefill_frac": round(prefill_flops(cfg32, args.prefill_tokens) / pre32["s"] / PEAK_FLOPS["float32"], 4),
                "decode_b8_tok_s": dec32["tok_s"], "decode_b8_ms": dec32["ms"], "decode_b8_ctx": dec32["ctx"],
                "decode_b8_hbm_frac": dec32["hbm_frac"]}
        del llm32
    sizes = None
    if elem == 2 and not args.no_points and not args.no_sizes and args.shape == "7b" and not args.layers:
        # further sizes and contexts, all layers of each shape: batch 8 decoding at the same context and the
        # same prefill for the 14B and 32B shapes; for the default shape batch 8 decoding at a context of
        # 32,768 and a prompt portion behind 30,720 cached tokens
        llm = None
        gc.collect()
        torch.cuda.empty_cache()
        sizes = {}

        def other(shape: str, context: int, batch: int, steps: int, seqs: int = 0, length: int = 0, positions: int = 0,
                  pages: int = 0):
            """A model of all the layers of ``shape`` with room for ``seqs`` sequences of ``length`` tokens (or
            ``pages`` pages), and its decode point at ``batch`` sequences of ``context`` tokens (none for batch 0)."""
            c = make_config(0, shape, positions)
            seqs, length = max(seqs, batch), max(length, context + 16)
            m = LLM(config=c, seed=args.seed, dtype=args.dtype, device="cuda:0", block_size=page,
                    num_blocks=pages or seqs * (-(-length // page)) + 8, max_num_seqs=seqs, max_batched_tokens=2048,
                    max_model_len=length, graphs=not args.no_graphs, graph_warmup_tokens=0, prefix_caching=False,
                    tune_library=not args.no_tune, overlap=not args.no_overlap)
            if batch == 0:
                return c, m, {"layers": c.num_hidden_layers}
            dec = with_roofline(bench_decode(m, batch, context, steps, 4, args.seed + 11), batch, c)
            return c, m, {"layers": c.num_hidden_layers, f"decode_b{batch}_tok_s": dec["tok_s"], f"decode_b{batch}_ms": dec["ms"],
                          f"decode_b{batch}_ctx": dec["ctx"], f"decode_b{batch}_hbm_frac": dec["hbm_frac"]}

        def portion(m, c, behind: int, tag: str) -> dict:
            p = bench_prefill_portion(m, behind, args.prefill_tokens, 2, args.seed + 2)
            return {f"{tag}_behind": behind, f"{tag}_tokens": args.prefill_tokens, f"{tag}_tok_s": round(p["tok_s"], 1),
                    f"{tag}_ms": round(p["s"] * 1e3, 3),
                    f"{tag}_frac": round(prefill_portion_flops(c, args.prefill_tokens, behind) / p["s"] / PEAK_FLOPS[dtype_key], 4)}

        # the workloads the two wider shapes are quoted with: 32 requests with prompts of 256 to 4,096 tokens and
        # 512 tokens each sampled at temperature 0.7; 64 requests of 1,024 + 256 tokens, greedy
        workloads = {"14b": dict(requests=32, prompt_min=256, prompt_max=4096, output_tokens=512, temperature=0.7),
                     "32b": dict(requests=64, prompt_min=1024, prompt_max=1024, output_tokens=256, temperature=0.0)}
        for shape, wl in workloads.items():
            c, m, out = other(shape, args.context, 8, 16, seqs=wl["requests"], length=wl["prompt_max"] + wl["output_tokens"] + 16)
            p2 = bench_prefill(m, args.prefill_tokens, 2, args.seed + 2)
            out.update({"prefill_tok_s": round(p2["tok_s"], 1), "prefill_ms": round(p2["s"] * 1e3, 3),
                        "prefill_frac": round(prefill_flops(c, args.prefill_tokens) / p2["s"] / PEAK_FLOPS[dtype_key], 4)})
            w = run_workload(m, seed=args.seed, **wl)
            out.update({"workload_tok_s": round(w["tok_s"], 1), "workload_requests": wl["requests"],
                        "workload_prompt_tokens": w["prompt_tokens"], "workload_generated": w["generated"],
                        "workload_temperature": wl["temperature"], "workload_s": round(w["total_s"], 2),
                        "workload_steps": w["steps"], "workload_ttft_p50_s": round(w["ttft_p50_s"], 3),
                        "workload_preemptions": w["preemptions"],
                        # lower bounds: the weights once per step, the products of every token; attention left out
                        "workload_hbm_frac_weights": round(w["weight_reads_GBps"] / HBM_GBPS, 4),
                        "workload_mfma_frac_products": round(w["product_flops_per_s"] / PEAK_FLOPS[dtype_key], 4)})
            sizes[shape] = out
            del m
            gc.collect()
            torch.cuda.empty_cache()
        c, m, out = other("7b", 32768, 8, 16)
        out.update(portion(m, c, 32768 - args.prefill_tokens, "portion"))
        out.update(portion(m, c, 8192, "portion_8k"))
        out.update(portion(m, c, 16384, "portion_16k"))
        sizes["7b_32k"] = out
        del m
        gc.collect()
        torch.cuda.empty_cache()
        # batch 64 at 16,384 tokens and batch 8 at 65,536 (positions beyond the shape's 32,768 allowed for this
        # point): the cache is filled with random values instead of by a million tokens of prefill
        points_long = ((64, 16384), (8, 65536))
        c, m, out = other("7b", 0, 0, 0, seqs=64, length=65536 + 16, positions=131072,
                          pages=max(b * (-(-(n + 16) // page)) for b, n in points_long) + 8)
        out.update({"max_position_embeddings": 131072, "cache": "random values, no prefill"})
        for batch, context in points_long:
            d = with_roofline(bench_decode_at_context(m, batch, context, 12, 4, args.seed + 13), batch, c)
            out.update({f"decode_b{batch}_ctx{context}_{key}": d[key] for key in ("tok_s", "ms", "ms_events", "hbm_frac")})
        sizes["7b_long"] = out
        del m
        gc.collect()
        torch.cuda.empty_cache()
    step_s = main_run["ms_per_step"] / 1e3
    achieved = decode_bytes(cfg, args.batch, int(main_run["mean_context"]), elem) / step_s / 1e9
    flops = (prefill_portion_flops(cfg, args.prefill_tokens, args.prefill_behind) if args.prefill_behind > 0
             else prefill_flops(cfg, args.prefill_tokens))
    line = {
        "metric": f"decode tok/s @ batch {args.batch}, context {args.context} (Qwen2.5-{args.shape.upper()} shape)",
        "value": round(main_run["tok_s"], 1),
        "unit": "tok/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(main_run["ms_per_step"], 4),
        "ms_per_step_gpu_events": round(main_run["ms_per_step_events"], 4),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "bf16" if elem == 2 else "fp32",
        "data": "synthetic: random weights from a seed, token ids uniform over the vocabulary",
        "config": {
            "model": f"Qwen2.5-{args.shape.upper()} shape", "global_batch": args.batch, "seq_len": args.context,
            "parallelism": "single GPU", "layers": cfg.num_hidden_layers, "layers_of_shape": full_layers,
            "hidden_size": cfg.hidden_size, "intermediate_size": cfg.intermediate_size,
            "num_attention_heads": cfg.num_attention_heads, "num_key_value_heads": cfg.num_key_value_heads,
            "head_dim": cfg.head_dim, "vocab_size": cfg.vocab_size, "page_size": page,
            "prefill_tokens": args.prefill_tokens, "graphs": not args.no_graphs, "library_tuning": not args.no_tune, "sampling": "greedy",
            "overlap": not args.no_overlap,
            "decode_graph_replays": main_run["graph_replays"], "mean_context": round(main_run["mean_context"], 1),
        },
        "prefill": {"value": round(pre["tok_s"], 1), "tokens": args.prefill_tokens, "behind": args.prefill_behind,
                    "ms": round(pre["s"] * 1e3, 3),
                    "frac": round(flops / pre["s"] / PEAK_FLOPS[dtype_key], 4),
                    "frac_of_measured_gemm": round(flops / pre["s"] / (machine["gemm_TFLOPs"] * 1e12), 4)},
        "roofline": {"bound": "hbm", "achieved": round(achieved, 1), "peak": HBM_GBPS, "unit": "GB/s",
                     "frac": round(achieved / HBM_GBPS, 4),
                     "frac_of_measured_copy": round(achieved / machine["copy_GBps"], 4)},
        "points": points,
        "machine": machine,
    }
    if fp32 is not None:
        line["fp32"] = fp32
    if sizes is not None:
        line["sizes"] = sizes
    if profile is not None:
        line["profile"] = profile
    print(json.dumps(line))
    torch.cuda.synchronize()
    return 0


if __name__ == "__main__":
    sys.exit(main())
