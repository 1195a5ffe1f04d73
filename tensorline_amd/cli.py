"""Command line: ``tensorline generate | replay | random-model | bench``.

Options keep the names and meanings of the reference's launcher where it has them
(tensorline/server.py:256-283): ``--model`` (default from ``TL_MODEL``), ``--device``, ``--dtype``,
``--max-num-seqs``, ``--max-batched-tokens``, ``--num-blocks``, ``--no-cuda-graphs``,
``--graph-warmup-tokens``, ``--no-prefix-caching``, ``--no-overlap``, ``--kv-cache-gb``.  Its server, engine choice,
speculation, overlap, quantisation and multi-model options have no counterpart here.  Added: the
constructor-only options of the reference (``--block-size``, ``--max-model-len``) and the request
options (``--max-tokens``, ``--temperature``, ``--top-p``, ``--seed``).
"""
from __future__ import annotations

import argparse
import json
import os
import sys


def _engine_options(ap: argparse.ArgumentParser) -> None:
    ap.add_argument("--model", default=os.getenv("TL_MODEL"), help="folder with config.json and model.safetensors")
    ap.add_argument("--device", default="cuda:0")
    ap.add_argument("--dtype", default="bfloat16", help="bfloat16 | float32")
    ap.add_argument("--max-num-seqs", type=int, default=64)
    ap.add_argument("--max-batched-tokens", type=int, default=2048)
    ap.add_argument("--num-blocks", type=int, default=None, help="KV pages (default: fit 60%% of free memory)")
    ap.add_argument("--kv-cache-gb", type=float, default=None, help="KV cache size (default: 60%% of free memory)")
    ap.add_argument("--block-size", type=int, default=16, help="tokens per KV page")
    ap.add_argument("--max-model-len", type=int, default=4096)
    ap.add_argument("--no-cuda-graphs", "--no-graphs", dest="no_graphs", action="store_true",
                    help="run decode steps eagerly instead of replaying a HIP graph")
    ap.add_argument("--graph-warmup-tokens", type=int, default=512,
                    help="capture the decode graphs before serving (0 = at first use)")
    ap.add_argument("--no-prefix-caching", action="store_true", help="never reuse KV pages across requests")
    ap.add_argument("--no-overlap", action="store_true", help="read every decode step's tokens before queueing the next step")
    ap.add_argument("--tune-library", action="store_true",
                    help="at start-up, let the library pick its kernels for full prompt portions by measurement")


def _make_llm(a):
    from tensorline_amd import LLM
    if not a.model:
        raise SystemExit("--model (or TL_MODEL) is required: a folder with config.json and model.safetensors")
    return LLM(a.model, device=a.device, dtype=a.dtype, max_num_seqs=a.max_num_seqs,
               max_batched_tokens=a.max_batched_tokens, num_blocks=a.num_blocks, kv_cache_gb=a.kv_cache_gb,
               block_size=a.block_size, max_model_len=a.max_model_len, graphs=not a.no_graphs,
               graph_warmup_tokens=a.graph_warmup_tokens, prefix_caching=not a.no_prefix_caching, overlap=not a.no_overlap,
               tune_library=a.tune_library)


def cmd_generate(a) -> int:
    from tensorline_amd import SamplingParams
    llm = _make_llm(a)
    prompts: list = []
    for p in a.prompt_ids or []:
        prompts.append([int(t) for t in p.replace(",", " ").split()])
    prompts += a.prompt or []
    if not prompts:
        raise SystemExit("give --prompt-ids '1 2 3' (token ids) or --prompt 'text' (needs tokenizer.json), one per request")
    stops = set(a.stop_token_id or [])
    params = SamplingParams(max_tokens=a.max_tokens, temperature=a.temperature, top_p=a.top_p,
                            stop_token_ids=stops, seed=a.seed)
    for prompt, out in zip(prompts, llm.generate(prompts, params)):
        rec = {"prompt": prompt, "token_ids": out.token_ids, "finish_reason": out.finish_reason,
               "prompt_tokens": out.stats.prompt_tokens, "completion_tokens": out.stats.completion_tokens,
               "cached_tokens": out.stats.cached_tokens, "ttft_s": round(out.stats.ttft_s, 4),
               "total_s": round(out.stats.total_s, 4)}
        if out.text is not None:
            rec["text"] = out.text
        print(json.dumps(rec), flush=True)
    print(json.dumps({"counters": llm.counters()}), file=sys.stderr)
    return 0


def cmd_random_model(a) -> int:
    from tensorline_amd.config.registry import architecture_name, get_architecture
    from tensorline_amd.weights import write_random_model
    with open(a.config, "r", encoding="utf-8") as f:
        raw = json.load(f)
    arch = get_architecture(architecture_name(raw))
    write_random_model(arch.config_cls.from_dict(raw), a.out, seed=a.seed, store_dtype=a.store_dtype)
    print(a.out)
    return 0


def cmd_replay(a, rest) -> int:
    from tensorline_amd.engine.replay import main as replay_main
    return replay_main(rest)


def cmd_bench(a, rest) -> int:
    import runpy
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    sys.argv = [os.path.join(root, "bench.py")] + rest
    runpy.run_path(sys.argv[0], run_name="__main__")
    return 0


def main(argv=None) -> int:
    argv = list(sys.argv[1:] if argv is None else argv)
    ap = argparse.ArgumentParser("tensorline", description="one-GPU inference engine for AMD MI355X")
    sub = ap.add_subparsers(dest="cmd", required=True)
    g = sub.add_parser("generate", help="generate tokens for one or more prompts")
    _engine_options(g)
    g.add_argument("--prompt-ids", action="append", help="a prompt as token ids, e.g. '5 17 3' (repeatable)")
    g.add_argument("--prompt", action="append", help="a prompt as text (repeatable; needs tokenizer.json)")
    g.add_argument("--max-tokens", type=int, default=128)
    g.add_argument("--temperature", type=float, default=0.0, help="0 = greedy")
    g.add_argument("--top-p", type=float, default=1.0)
    g.add_argument("--seed", type=int, default=None, help="seed of the request's random draws")
    g.add_argument("--stop-token-id", type=int, action="append", help="stop token (default: the model's eos; -1: never)")
    r = sub.add_parser("random-model", help="write a model folder with random weights from a config.json and a seed")
    r.add_argument("--config", required=True, help="a config.json (its 'architectures' picks the model)")
    r.add_argument("--out", required=True)
    r.add_argument("--seed", type=int, default=0)
    r.add_argument("--store-dtype", default="bfloat16", choices=["bfloat16", "float32"])
    sub.add_parser("replay", help="replay a token trace and write logits (options of bin/trace_run)", add_help=False)
    sub.add_parser("bench", help="run bench.py (its options follow)", add_help=False)
    if argv and argv[0] in ("replay", "bench"):
        return {"replay": cmd_replay, "bench": cmd_bench}[argv[0]](None, argv[1:])
    a = ap.parse_args(argv)
    return {"generate": cmd_generate, "random-model": cmd_random_model}[a.cmd](a)


if __name__ == "__main__":
    sys.exit(main())
