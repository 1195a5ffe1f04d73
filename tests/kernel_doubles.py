"""Stand-ins for the HIP kernels, in torch on the CPU, for tests of the engine's *logic* (batch
flattening, page tables, cutting, scheduling) where no GPU is present.  They have the signatures
of ``tensorline_amd.ops.kernels`` and are installed by the ``cpu_kernels`` fixture; the product
has no such path and refuses to run without a GPU.
"""
from __future__ import annotations

import torch


def require_gpu(device):
    return torch.device(device)


def embed(ids, table, out=None):
    x = table[ids.long()].to(torch.float32)
    if out is not None:
        out.copy_(x)
        return out
    return x


def add_rmsnorm(x, residual, weight, eps, out_dtype, rows=None, out=None):
    if rows is None:
        if residual is not None:
            x.add_(residual.to(torch.float32))
        v = x
    else:
        v = x[rows.long()]
        if residual is not None:
            v = v + residual[rows.long()].to(torch.float32)
    r = v * torch.rsqrt(v.pow(2).mean(-1, keepdim=True) + eps) * weight
    return r.to(out_dtype)


def qkv_rope_store(*args, **kw):
    return None


def shuffle_weight(weight):
    return None


def linear(a, weight, bias=None, out_dtype=None, out=None, shuffled=None, sink=None, keep_shares=False):
    assert sink is None, "the stand-ins make no shuffled copies, so no part defers a norm"
    y = a.to(torch.float32) @ weight.to(torch.float32).T
    if bias is not None:
        y = y + bias
    return y.to(out_dtype or a.dtype)


def rope_store(qkv, pos, inv_freq, num_heads, num_kv_heads, head_dim, k_cache, v_cache, slots, bias=None):
    T = qkv.shape[0]
    d = head_dim
    if bias is not None:
        qkv.copy_((qkv.to(torch.float32) + bias).to(qkv.dtype))
    heads = qkv.view(T, num_heads + 2 * num_kv_heads, d)
    rot_heads = heads[:, :num_heads + num_kv_heads].to(torch.float32)
    if inv_freq is not None and inv_freq.numel():
        half = inv_freq.numel()
        ang = pos.to(torch.float32)[:, None] * inv_freq[None, :]
        cs, sn = ang.cos()[:, None, :], ang.sin()[:, None, :]
        a, b = rot_heads[..., :half].clone(), rot_heads[..., half:2 * half].clone()
        rot_heads[..., :half] = a * cs - b * sn
        rot_heads[..., half:2 * half] = b * cs + a * sn
    rot_heads = rot_heads.to(qkv.dtype)
    heads[:, :num_heads] = rot_heads[:, :num_heads]
    if k_cache is not None:
        ok = slots >= 0
        bs = k_cache.shape[1]
        kc = k_cache.view(-1, num_kv_heads, d)
        kc[slots[ok].long()] = rot_heads[ok][:, num_heads:]
        sl = slots[ok].long()
        v_cache[sl // bs, :, :, sl % bs] = heads[ok][:, num_heads + num_kv_heads:]      # [pages, nkv, d, page]


def paged_attention(q, k_cache, v_cache, tables, seq_of_token, pos, num_heads, num_kv_heads, head_dim, scale,
                    window=0, out=None, q_start=None, ctx_start=None, plan=None, path=None, split_keys=None,
                    single_seqs=None, route_singles=None):
    T, d, bs = q.shape[0], head_dim, k_cache.shape[1]
    g = num_heads // num_kv_heads
    o = torch.empty(T, num_heads * d, dtype=q.dtype)
    kc = k_cache.view(-1, num_kv_heads, d)
    vc = v_cache.permute(0, 3, 1, 2).reshape(-1, num_kv_heads, d)                      # back to [slot, nkv, d]
    for t in range(T):
        s, p = int(seq_of_token[t]), int(pos[t])
        lo = max(0, p - window + 1) if window > 0 else 0
        keys = torch.arange(lo, p + 1)
        rows = tables[s][keys // bs].long() * bs + keys % bs
        K, V = kc[rows].to(torch.float32), vc[rows].to(torch.float32)          # [n, nkv, d]
        qt = q[t, :num_heads * d].view(num_heads, d).to(torch.float32)
        for h in range(num_heads):
            sc = (K[:, h // g] @ qt[h]) * scale
            o[t, h * d:(h + 1) * d] = (torch.softmax(sc, -1) @ V[:, h // g]).to(q.dtype)
    return o


def silu_mul(gate_up, out=None):
    I = gate_up.shape[1] // 2
    g, u = gate_up[:, :I].to(torch.float32), gate_up[:, I:].to(torch.float32)
    return (g * torch.sigmoid(g) * u).to(gate_up.dtype)


def swiglu_gate_up(h, gate_up_weight, shuffled=None):
    return silu_mul(linear(h, gate_up_weight))


def argmax(logits, out=None):
    return logits.argmax(-1).to(torch.int32)


def sample(logits, temperature, top_p, uniform, out=None, any_top_p=None, any_greedy=True):
    res = torch.empty(logits.shape[0], dtype=torch.int32)
    for r in range(logits.shape[0]):
        t = float(temperature[r])
        if t <= 0:
            res[r] = int(logits[r].argmax())
            continue
        w = torch.exp((logits[r] - logits[r].max()) / t)
        tp = float(top_p[r])
        if tp < 1.0:
            sw, idx = torch.sort(w, descending=True, stable=True)
            keep = torch.cumsum(sw, 0) - sw < tp * w.sum()
            mask = torch.zeros_like(w, dtype=torch.bool)
            mask[idx[keep]] = True
            w = w * mask
        cum = torch.cumsum(w, 0)
        res[r] = int(torch.searchsorted(cum, float(uniform[r]) * cum[-1], right=True).clamp(max=len(w) - 1))
    return res


ALL = ["require_gpu", "embed", "add_rmsnorm", "linear", "rope_store", "paged_attention", "silu_mul", "swiglu_gate_up", "shuffle_weight", "qkv_rope_store", "argmax",
       "sample"]


def install(monkeypatch) -> None:
    from tensorline_amd.ops import kernels
    for name in ALL:
        monkeypatch.setattr(kernels, name, globals()[name])
