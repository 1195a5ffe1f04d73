"""The plain implementation: a slow, whole-sequence forward pass of the dense Qwen2.5 decoder.

No cache, no batching, no kernels; one function per part; shares no code with
``tensorline_amd``.  Written from the formulas of the reference (cited per function) and pinned
by ``tests/test_plain.py``.  Everything runs in the dtype of the tensors given (float32 by
default, float64 for error budgets).
"""
from __future__ import annotations

import json
import math
import os

import torch


# ---- parts ---------------------------------------------------------------------------------
def rmsnorm(x: torch.Tensor, weight: torch.Tensor, eps: float) -> torch.Tensor:
    """out = x * rsqrt(mean(x^2) + eps) * w   (reference: tensorline/fused.py:29-32)."""
    var = x.pow(2).mean(dim=-1, keepdim=True)
    return x * torch.rsqrt(var + eps) * weight


def rope_angles(positions: torch.Tensor, rotary_dim: int, theta: float, dtype=torch.float32) -> torch.Tensor:
    """angle[t, i] = pos[t] * theta^(-2i/rotary_dim), i < rotary_dim/2.  The frequency is computed
    in float64 and rounded to float32 once; the product is taken in float32, as an engine working
    in 32-bit does (the reference takes cos/sin tables from its model library, paged.py:241-242;
    their layout cat(cos, cos) is fixed by tests/test_quant.py:116-118)."""
    i = torch.arange(0, rotary_dim, 2, dtype=torch.float64)
    inv_freq = (float(theta) ** (-i / rotary_dim)).to(torch.float32)
    ang = positions.to(torch.float32)[:, None] * inv_freq[None, :]
    return ang.to(dtype)


def rotate_half(x: torch.Tensor) -> torch.Tensor:
    """cat(-x2, x1) over the last dim (reference: tensorline/fused.py:83-85)."""
    half = x.shape[-1] // 2
    return torch.cat((-x[..., half:], x[..., :half]), dim=-1)


def rope(x: torch.Tensor, positions: torch.Tensor, theta: float, rotary_dim: int | None = None) -> torch.Tensor:
    """x: [T, heads, d].  out = x*cos + rotate_half(x)*sin with cos = cat(cos a, cos a)
    (reference: tensorline/fused.py:72-78; kernel form fused.py:47-51)."""
    d = x.shape[-1]
    rd = d if rotary_dim is None else rotary_dim
    ang = rope_angles(positions, rd, theta, x.dtype)
    cos = torch.cat((ang.cos(), ang.cos()), dim=-1)[:, None, :]
    sin = torch.cat((ang.sin(), ang.sin()), dim=-1)[:, None, :]
    xr, xp = x[..., :rd], x[..., rd:]
    return torch.cat((xr * cos + rotate_half(xr) * sin, xp), dim=-1)


def causal_attention(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, scale: float, window: int = 0,
                     q_offset: int = 0) -> torch.Tensor:
    """q: [n, nq, d]; k, v: [ctx, nkv, d]; query i sits at position q_offset + i and sees keys
    j <= q_offset + i (reference: mask m[i, j] = j <= start + i, tensorline/paged.py:237), and with a
    window only j > q_offset + i - window.  Query head h uses key/value head h // (nq // nkv)
    (paged.py:153-157).  softmax(q k^T * scale + mask) v, in the input dtype."""
    n, nq, d = q.shape
    ctx, nkv, _ = k.shape
    g = nq // nkv
    out = torch.empty_like(q)
    qi = torch.arange(n)[:, None] + q_offset
    kj = torch.arange(ctx)[None, :]
    allowed = kj <= qi
    if window > 0:
        allowed &= kj > qi - window
    for h in range(nq):
        kh, vh = k[:, h // g, :], v[:, h // g, :]
        s = (q[:, h, :] @ kh.T) * scale
        s = s.masked_fill(~allowed, float("-inf"))
        out[:, h, :] = torch.softmax(s, dim=-1) @ vh
    return out


def swiglu(h: torch.Tensor, w_gate: torch.Tensor, w_up: torch.Tensor, w_down: torch.Tensor) -> torch.Tensor:
    """down(silu(gate(h)) * up(h)), silu(z) = z * sigmoid(z), no biases.  The reference calls the
    checkpoint's module (tensorline/paged.py:276); names and shapes of the three projections:
    tensorline/manager.py:52-54."""
    g = h @ w_gate.T
    u = h @ w_up.T
    return (g * torch.sigmoid(g) * u) @ w_down.T


def attention_block(h, w, prefix, positions, nq, nkv, d, theta, window=0):
    """q/k/v projections with bias, RoPE on q and k, causal GQA attention, output projection
    (reference order: tensorline/paged.py:248-275; y = x W^T + b, tensorline/quant.py:3)."""
    T = h.shape[0]
    q = (h @ w[prefix + "q_proj.weight"].T + w[prefix + "q_proj.bias"]).view(T, nq, d)
    k = (h @ w[prefix + "k_proj.weight"].T + w[prefix + "k_proj.bias"]).view(T, nkv, d)
    v = (h @ w[prefix + "v_proj.weight"].T + w[prefix + "v_proj.bias"]).view(T, nkv, d)
    q, k = rope(q, positions, theta), rope(k, positions, theta)
    o = causal_attention(q, k, v, d ** -0.5, window=window)
    return o.reshape(T, nq * d) @ w[prefix + "o_proj.weight"].T


# ---- whole model ---------------------------------------------------------------------------
def model_forward(w: dict[str, torch.Tensor], cfg: dict, ids: list[int]) -> torch.Tensor:
    """Logits [len(ids), vocab] of one whole sequence.  Residual order of the reference
    (tensorline/paged.py:243-247,275-276,286): x = E[ids]; per layer x += attn(norm1(x));
    x += mlp(norm2(x)); logits = norm_f(x) W_head^T, W_head = E when tied (manager.py:65)."""
    nq = cfg["num_attention_heads"]
    nkv = cfg.get("num_key_value_heads", nq)
    d = cfg.get("head_dim") or cfg["hidden_size"] // nq
    eps, theta = cfg.get("rms_norm_eps", 1e-6), cfg.get("rope_theta", 10000.0)
    positions = torch.arange(len(ids))
    x = w["model.embed_tokens.weight"][torch.tensor(ids)]
    for i in range(cfg["num_hidden_layers"]):
        p = f"model.layers.{i}."
        h = rmsnorm(x, w[p + "input_layernorm.weight"], eps)
        x = x + attention_block(h, w, p + "self_attn.", positions, nq, nkv, d, theta)
        h = rmsnorm(x, w[p + "post_attention_layernorm.weight"], eps)
        x = x + swiglu(h, w[p + "mlp.gate_proj.weight"], w[p + "mlp.up_proj.weight"], w[p + "mlp.down_proj.weight"])
    h = rmsnorm(x, w["model.norm.weight"], eps)
    head = w["model.embed_tokens.weight"] if cfg.get("tie_word_embeddings", False) else w["lm_head.weight"]
    return h @ head.T


def greedy_generate(w, cfg, prompt: list[int], max_tokens: int, stop: set[int] = frozenset()) -> list[int]:
    """One request at a time, whole sequence recomputed per token (the reference's naive engine
    loop, tensorline/engine.py:98-114: argmax of the last logits; a stop token ends the request and
    is not emitted)."""
    seq, out = list(prompt), []
    for _ in range(max_tokens):
        tok = int(model_forward(w, cfg, seq)[-1].argmax())
        if tok in stop:
            break
        seq.append(tok)
        out.append(tok)
    return out


def load_folder(model_dir: str, dtype=torch.float32) -> tuple[dict[str, torch.Tensor], dict]:
    """config.json as a dict and every tensor of model.safetensors in ``dtype``."""
    from safetensors.torch import load_file
    with open(os.path.join(model_dir, "config.json")) as f:
        cfg = json.load(f)
    w = {k: v.to(dtype) for k, v in load_file(os.path.join(model_dir, "model.safetensors")).items()}
    return w, cfg


# ---- sampling ------------------------------------------------------------------------------
def top_p_keep(probs: torch.Tensor, top_p: float) -> torch.Tensor:
    """Boolean mask of the tokens kept: sort descending, keep where the mass before the token is
    < top_p (reference: tensorline/engine.py:46-49; the top token always survives)."""
    sorted_p, idx = torch.sort(probs, descending=True, stable=True)
    keep_sorted = torch.cumsum(sorted_p, dim=-1) - sorted_p < top_p
    keep = torch.zeros_like(probs, dtype=torch.bool)
    keep[idx[keep_sorted]] = True
    return keep


def sample_with_uniform(logits: torch.Tensor, temperature: float, top_p: float, u: float) -> int:
    """The reference's sample() (tensorline/engine.py:42-51) with the random draw made explicit:
    the token is the first, in index order, whose running kept probability exceeds u * kept mass."""
    if temperature <= 0:
        return int(torch.argmax(logits))
    probs = torch.softmax(logits.double() / temperature, dim=-1)
    if top_p < 1.0:
        probs = probs * top_p_keep(probs, top_p)
    cum = torch.cumsum(probs, dim=-1)
    target = u * float(cum[-1])
    return int(torch.searchsorted(cum, torch.tensor(target, dtype=cum.dtype), right=True).clamp(max=len(probs) - 1))


def softmax_reference(x: torch.Tensor) -> torch.Tensor:
    m = x.max(dim=-1, keepdim=True).values
    e = torch.exp(x - m)
    return e / e.sum(dim=-1, keepdim=True)


def expected_inv_sqrt(d: int) -> float:
    return 1.0 / math.sqrt(d)
