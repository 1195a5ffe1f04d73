"""Shared by the tests: the tiny configurations, model folders, and ways of cutting requests."""
from __future__ import annotations

import random

import numpy as np
import torch

from tensorline_amd.config import Qwen2Config
from tensorline_amd.weights import write_random_model

# Two tiny configurations that differ in every size and option.
TINY_A = dict(architectures=["Qwen2ForCausalLM"], vocab_size=512, hidden_size=64, intermediate_size=176,
              num_hidden_layers=2, num_attention_heads=4, num_key_value_heads=2, head_dim=16,
              rope_theta=10000.0, rms_norm_eps=1e-6, tie_word_embeddings=True, max_position_embeddings=256)
TINY_B = dict(architectures=["Qwen2ForCausalLM"], vocab_size=1000, hidden_size=192, intermediate_size=512,
              num_hidden_layers=3, num_attention_heads=6, num_key_value_heads=2, head_dim=32,
              rope_theta=1000000.0, rms_norm_eps=1e-5, tie_word_embeddings=False, max_position_embeddings=512)
# A third one whose head size is not hidden/heads and whose group is 5 (neither a power of two).
TINY_C = dict(architectures=["Qwen2ForCausalLM"], vocab_size=777, hidden_size=120, intermediate_size=200,
              num_hidden_layers=2, num_attention_heads=5, num_key_value_heads=1, head_dim=48,
              rope_theta=50000.0, rms_norm_eps=3e-6, tie_word_embeddings=False, max_position_embeddings=1024)
# One with the head size of the large models (128), heads wider than the hidden size, group 3.
TINY_D = dict(architectures=["Qwen2ForCausalLM"], vocab_size=2000, hidden_size=256, intermediate_size=368,
              num_hidden_layers=2, num_attention_heads=6, num_key_value_heads=2, head_dim=128,
              rope_theta=1000000.0, rms_norm_eps=1e-6, tie_word_embeddings=False, max_position_embeddings=2048)
CONFIGS = {"A": TINY_A, "B": TINY_B, "C": TINY_C, "D": TINY_D}
PAGE = {"A": 16, "B": 8, "C": 16, "D": 16}


def make_model_dir(tmp_path_factory_or_dir, name: str, seed: int = 0) -> str:
    cfg = Qwen2Config.from_dict(CONFIGS[name])
    base = tmp_path_factory_or_dir
    out = str(base.mktemp(f"model_{name}") if hasattr(base, "mktemp") else base)
    return write_random_model(cfg, out, seed=seed)


def prompts_for(name: str, lengths, seed: int = 0) -> list[list[int]]:
    rng = random.Random(seed)
    V = CONFIGS[name]["vocab_size"]
    return [[rng.randrange(V) for _ in range(n)] for n in lengths]


# ---- ways of cutting a set of requests into steps --------------------------------------------
def steps_whole(reqs: dict[str, list[int]]):
    """Each request alone and whole, logits at every position."""
    steps = []
    for rid, toks in reqs.items():
        steps.append({"entries": [{"id": rid, "tokens": toks, "want": list(range(len(toks)))}], "end": [rid]})
    return steps


def steps_prefill_then_decode(reqs: dict[str, list[int]], tail: int = 32):
    """Most of a request in one step, the last ``tail`` tokens one by one."""
    steps = []
    for rid, toks in reqs.items():
        n = max(1, len(toks) - tail)
        steps.append({"entries": [{"id": rid, "tokens": toks[:n], "want": list(range(n))}], "end": []})
        for i in range(n, len(toks)):
            steps.append({"entries": [{"id": rid, "tokens": [toks[i]], "want": [0]}],
                          "end": [rid] if i == len(toks) - 1 else []})
        if n == len(toks):
            steps[-1]["end"] = [rid]
    return steps


def steps_portions(reqs: dict[str, list[int]], sizes=(24, 7, 2, 13, 2, 5, 31, 3)):
    """Portions of changing size, down to two tokens."""
    steps = []
    for rid, toks in reqs.items():
        i, k = 0, 0
        while i < len(toks):
            n = min(sizes[k % len(sizes)], len(toks) - i)
            steps.append({"entries": [{"id": rid, "tokens": toks[i:i + n], "want": list(range(n))}],
                          "end": [rid] if i + n == len(toks) else []})
            i += n
            k += 1
    return steps


def steps_mixed(reqs: dict[str, list[int]], seed: int = 0, max_live: int = 4, tail: int = 8):
    """Up to ``max_live`` requests live: portions of some beside single tokens of others.  A
    request goes through portions of random size, then its last ``tail`` tokens one by one; it may
    sit a step out.  A new request starts as soon as one ends."""
    rng = random.Random(seed)
    waiting = list(reqs.items())
    live: dict[str, int] = {}
    steps = []
    while waiting or live:
        while waiting and len(live) < max_live:
            rid, _ = waiting.pop(0)
            live[rid] = 0
        entries, end = [], []
        for rid in list(live):
            toks, done = reqs[rid], live[rid]
            if len(live) > 1 and rng.random() < 0.2:
                continue                                  # left out of this step
            left = len(toks) - done
            n = 1 if left <= tail else min(left - tail, rng.choice([2, 3, 5, 8, 13, 21]))
            entries.append({"id": rid, "tokens": toks[done:done + n], "want": list(range(n))})
            live[rid] = done + n
            if live[rid] == len(toks):
                end.append(rid)
                del live[rid]
        if entries:
            steps.append({"entries": entries, "end": end})
    return steps


def collect_logits(run_step, steps) -> dict[tuple[str, int], np.ndarray]:
    """Run ``steps`` through ``run_step(entries, end) -> logits|None``; logits by (request, position)."""
    out: dict[tuple[str, int], np.ndarray] = {}
    done: dict[str, int] = {}
    for st in steps:
        logits = run_step(st["entries"], st["end"])
        r = 0
        for e in st["entries"]:
            base = done.get(e["id"], 0)
            for w in e["want"]:
                out[(e["id"], base + w)] = np.asarray(logits[r])
                r += 1
            done[e["id"]] = base + len(e["tokens"])
        assert (logits is None and r == 0) or r == len(logits)
    return out


def max_live_tokens(steps, round_to: int = 64) -> int:
    """The most tokens live requests hold at any time, each rounded up to ``round_to``."""
    held: dict[str, int] = {}
    worst = 0
    for st in steps:
        for e in st["entries"]:
            held[e["id"]] = held.get(e["id"], 0) + len(e["tokens"])
        worst = max(worst, sum(-(-n // round_to) * round_to for n in held.values()))
        for rid in st["end"]:
            held.pop(rid, None)
    return worst


def plain_logits(weights, cfg, reqs):
    from tests import plain
    out = {}
    for rid, toks in reqs.items():
        lg = plain.model_forward(weights, cfg, toks)
        for i in range(len(toks)):
            out[(rid, i)] = lg[i].to(torch.float32).numpy()
    return out


# ---- looking into the engine from a test -------------------------------------------------------
class ForcedSampler:
    """Stands in for the engine's sampler: whatever the logits say, a request continues with the
    tokens given for it (a request is known by its seed), and the logits it was shown are kept.
    With the plain implementation's own tokens forced, a bfloat16 run sees the contexts the
    plain run saw at every position, so its logits can be compared one by one; a token picked
    from near-equal logits cannot send the rest of the comparison elsewhere.

    It has both of the sampler's forms.  ``sample_device`` awaits nothing: it keeps a copy of the
    logits on the device (a replayed graph writes the next step's over them) and returns the forced
    tokens as an int32 tensor on the device, so the engine leaves decode steps in flight and takes
    the next step's token ids from the device, as it does in serving."""

    def __init__(self, forced: dict[int, list[int]]):
        self.forced = forced
        self._rows: dict[tuple[int, int], np.ndarray] = {}        # (seed, index of the generated token) -> row
        self._kept: list = []                                      # (logits on the device, seeds, indices), not read yet

    @property
    def logits(self) -> dict[tuple[int, int], np.ndarray]:
        for dev, seeds, indices in self._kept:
            for row, seed, index in zip(dev.cpu().numpy(), seeds, indices):
                self._rows[(seed, index)] = row
        self._kept.clear()
        return self._rows

    def sample_device(self, logits, temperatures, top_ps, seeds, indices):
        self._kept.append((logits.detach().to(torch.float32, copy=True), list(seeds), list(indices)))
        # a row past a request's last forced token is one the engine throws away (the step queued ahead of a stop)
        toks = torch.tensor([self.forced[s][i] if i < len(self.forced[s]) else 0 for s, i in zip(seeds, indices)],
                            dtype=torch.int32)
        return toks.to(logits.device)

    def sample(self, logits, temperatures, top_ps, seeds, indices):
        return self.sample_device(logits, temperatures, top_ps, seeds, indices).tolist()


def watch_pages(cache) -> dict:
    """Count how often each page of each group is handed out from now on; ``reused(counts)`` then
    says how many pages went to a second holder after the first gave them back."""
    counts: dict[tuple[int, int], int] = {}
    for gi, g in enumerate(cache.groups):
        take = g.allocator.take

        def counting(n, _take=take, _gi=gi):
            got = _take(n)
            for p in got or []:
                counts[(_gi, p)] = counts.get((_gi, p), 0) + 1
            return got
        g.allocator.take = counting
    return counts


def reused(counts: dict) -> int:
    return sum(1 for c in counts.values() if c > 1)
