"""Pins for the plain implementation (tests/plain.py) beside the reference's text: library routines
it must reduce to, special cases, invariants, and the vectors the reference's own tests hold.  Each
is chosen so that a plausible mistake (a wrong sign or pairing, a norm in the wrong place) fails it."""
import math

import pytest
import torch
import torch.nn.functional as F

from tests import plain

torch.manual_seed(0)


# ---- RMSNorm ---------------------------------------------------------------------------------
def test_rmsnorm_is_the_library_routine():
    x, w = torch.randn(5, 896), torch.empty(896).uniform_(0.5, 1.5)      # sizes of tests/test_quant.py:100-106
    torch.testing.assert_close(plain.rmsnorm(x, w, 1e-6), F.rms_norm(x, (896,), w, 1e-6))


def test_rmsnorm_invariants():
    x = torch.randn(3, 64, dtype=torch.float64)
    one = torch.ones(64, dtype=torch.float64)
    y = plain.rmsnorm(x, one, 0.0)
    torch.testing.assert_close(y.pow(2).mean(-1), torch.ones(3, dtype=torch.float64))      # unit RMS, not unit variance
    torch.testing.assert_close(plain.rmsnorm(7.5 * x, one, 0.0), y)                          # scale invariance
    assert not torch.allclose(y.mean(-1), torch.zeros(3, dtype=torch.float64))             # no mean is subtracted


# ---- RoPE ------------------------------------------------------------------------------------
def test_rope_matches_the_reference_vector_form():
    # the reference's own check: x*cos + rotate_half(x)*sin with cos = cat(cos a, cos a) (tests/test_quant.py:114-123)
    T = 5
    q = torch.randn(T, 14, 64)
    pos = torch.arange(3, 3 + T)
    ang = plain.rope_angles(pos, 64, 1e6)
    cos, sin = torch.cat([ang.cos(), ang.cos()], -1), torch.cat([ang.sin(), ang.sin()], -1)
    x1, x2 = q.chunk(2, dim=-1)
    want = q * cos[:, None] + torch.cat((-x2, x1), dim=-1) * sin[:, None]
    torch.testing.assert_close(plain.rope(q, pos, 1e6), want)


def test_rope_is_a_complex_rotation_on_the_half_split_layout():
    # (a + ib) * e^{i theta} with a = x[i], b = x[i + d/2]: fixes the pairing and the sign
    d, theta = 32, 10000.0
    x = torch.randn(7, 3, d, dtype=torch.float64)
    pos = torch.tensor([0, 1, 2, 50, 51, 1000, 4095])
    freq = theta ** (-torch.arange(0, d, 2, dtype=torch.float64) / d)
    ang = (pos[:, None].float() * freq[None, :].float()).double()      # the angle itself is a float32 product
    z = torch.complex(x[..., : d // 2], x[..., d // 2:]) * torch.polar(torch.ones_like(ang), ang)[:, None, :]
    want = torch.cat([z.real, z.imag], dim=-1)
    torch.testing.assert_close(plain.rope(x, pos, theta), want, atol=1e-9, rtol=1e-9)


def test_rope_invariants():
    x = torch.randn(4, 2, 16, dtype=torch.float64)
    torch.testing.assert_close(plain.rope(x, torch.zeros(4, dtype=torch.long), 1e4), x)     # position 0: identity
    y = plain.rope(x, torch.tensor([5, 9, 100, 7]), 1e4)
    pair_norm = lambda t: t[..., :8] ** 2 + t[..., 8:] ** 2
    torch.testing.assert_close(pair_norm(y), pair_norm(x))                                  # each pair keeps its length
    # <R(q, m), R(k, n)> depends on m - n only
    q, k = torch.randn(1, 1, 16, dtype=torch.float64), torch.randn(1, 1, 16, dtype=torch.float64)
    dot = lambda m, n: (plain.rope(q, torch.tensor([m]), 1e4) * plain.rope(k, torch.tensor([n]), 1e4)).sum()
    torch.testing.assert_close(dot(17, 5), dot(112, 100), atol=1e-5, rtol=1e-5)   # angles are float32 products
    assert abs(dot(17, 5) - dot(17, 6)) > 1e-6
    # partial rotation leaves the tail alone
    z = plain.rope(x, torch.tensor([5, 9, 100, 7]), 1e4, rotary_dim=8)
    torch.testing.assert_close(z[..., 8:], x[..., 8:])


def test_rope_angles_frequency_table():
    ang = plain.rope_angles(torch.tensor([1]), 8, 10000.0, torch.float64)
    torch.testing.assert_close(ang[0], torch.tensor([1.0, 0.1, 0.01, 0.001], dtype=torch.float64), rtol=1e-6, atol=0)


# ---- attention -------------------------------------------------------------------------------
@pytest.mark.parametrize("nq,nkv", [(4, 4), (6, 2), (7, 1)])
def test_attention_is_the_library_routine(nq, nkv):
    n, d = 19, 16
    q, k, v = torch.randn(n, nq, d), torch.randn(n, nkv, d), torch.randn(n, nkv, d)
    g = nq // nkv
    want = F.scaled_dot_product_attention(q.transpose(0, 1)[None], k.repeat_interleave(g, 1).transpose(0, 1)[None],
                                          v.repeat_interleave(g, 1).transpose(0, 1)[None], is_causal=True,
                                          scale=d ** -0.5)[0].transpose(0, 1)
    torch.testing.assert_close(plain.causal_attention(q, k, v, d ** -0.5), want, atol=1e-5, rtol=1e-5)


def test_attention_special_cases():
    d = 8
    q, k, v = torch.randn(1, 2, d), torch.randn(1, 1, d), torch.randn(1, 1, d)
    torch.testing.assert_close(plain.causal_attention(q, k, v, 1.0)[0, 0], v[0, 0])          # one key: o = v
    k, v = torch.randn(6, 1, d), torch.randn(6, 1, d)
    o = plain.causal_attention(torch.zeros(6, 2, d), k, v, 1.0)
    torch.testing.assert_close(o[3, 1], v[:4, 0].mean(0))                                    # q = 0: mean of visible values
    # a chunk of queries against a longer context: query i sits at q_offset + i (tensorline/paged.py:237)
    q = torch.randn(6, 2, d)
    full = plain.causal_attention(q, k, v, 0.3)
    part = plain.causal_attention(q[4:], k, v, 0.3, q_offset=4)
    torch.testing.assert_close(part, full[4:])
    # window: only the last `window` keys count
    w = plain.causal_attention(q, k, v, 0.3, window=2)
    torch.testing.assert_close(w[5], plain.causal_attention(q[5:], k[4:], v[4:], 0.3, q_offset=1)[0])
    torch.testing.assert_close(plain.causal_attention(q, k, v, 0.3, window=100), full)


def test_softmax_rows_sum_to_one_and_reference_decode_form():
    # the reference's decode test: gather pages, mask beyond the length (tests/test_paged_attn.py:11-19)
    d, n = 16, 37
    q, k, v = torch.randn(1, 4, d), torch.randn(n, 2, d), torch.randn(n, 2, d)
    o = plain.causal_attention(q, k, v, d ** -0.5, q_offset=n - 1)
    s = torch.einsum("hd,nhd->hn", q[0], k.repeat_interleave(2, 1)) * d ** -0.5
    p = plain.softmax_reference(s)
    torch.testing.assert_close(p.sum(-1), torch.ones(4))
    torch.testing.assert_close(o[0], torch.einsum("hn,nhd->hd", p, v.repeat_interleave(2, 1)), atol=1e-5, rtol=1e-5)


# ---- feed-forward ----------------------------------------------------------------------------
def test_swiglu():
    h, wg, wu, wd = torch.randn(3, 8), torch.randn(12, 8), torch.randn(12, 8), torch.randn(8, 12)
    want = F.linear(F.silu(F.linear(h, wg)) * F.linear(h, wu), wd)
    torch.testing.assert_close(plain.swiglu(h, wg, wu, wd), want)
    assert torch.all(plain.swiglu(h, torch.zeros_like(wg), wu, wd) == 0)                     # silu(0) = 0
    assert not torch.allclose(plain.swiglu(h, wg, wu, wd), plain.swiglu(h, wu, wg, wd))     # gate and up are not symmetric


# ---- whole model -----------------------------------------------------------------------------
def _tiny(tied):
    from tensorline_amd.config import Qwen2Config
    from tensorline_amd.models.decoder import DecoderModel
    from tensorline_amd.models.qwen2 import qwen2_spec
    from tensorline_amd.weights.random_init import random_tensor
    cfg = dict(vocab_size=50, hidden_size=24, intermediate_size=40, num_hidden_layers=2, num_attention_heads=3,
               num_key_value_heads=1, head_dim=16, rope_theta=100.0, rms_norm_eps=1e-5, tie_word_embeddings=tied)
    model = DecoderModel(qwen2_spec(Qwen2Config.from_dict(dict(cfg, architectures=["Qwen2ForCausalLM"]))), torch.float32, "cpu")
    w = {n: random_tensor(n, d, 1).double() for n, d in model.tensor_decls().items()}
    return w, cfg


def test_model_is_causal_and_uses_the_tied_head():
    w, cfg = _tiny(tied=True)
    ids = [3, 14, 15, 9, 2, 6]
    full = plain.model_forward(w, cfg, ids)
    torch.testing.assert_close(plain.model_forward(w, cfg, ids[:4]), full[:4])               # later tokens change nothing
    w2 = dict(w, **{"lm_head.weight": w["model.embed_tokens.weight"]})
    torch.testing.assert_close(plain.model_forward(w2, dict(cfg, tie_word_embeddings=False), ids), full)
    w3 = dict(w2, **{"lm_head.weight": torch.randn(50, 24, dtype=torch.float64)})
    assert not torch.allclose(plain.model_forward(w3, dict(cfg, tie_word_embeddings=False), ids), full)


def test_model_layer_composition_by_hand():
    # one layer, written out: x + attn(norm1(x)), then + mlp(norm2(.)), final norm, head
    w, cfg = _tiny(tied=False)
    cfg = dict(cfg, num_hidden_layers=1)
    ids = [1, 2, 3]
    x = w["model.embed_tokens.weight"][ids]
    p = "model.layers.0."
    a = plain.attention_block(plain.rmsnorm(x, w[p + "input_layernorm.weight"], 1e-5), w, p + "self_attn.",
                              torch.arange(3), 3, 1, 16, 100.0)
    x = x + a
    x = x + plain.swiglu(plain.rmsnorm(x, w[p + "post_attention_layernorm.weight"], 1e-5), w[p + "mlp.gate_proj.weight"],
                         w[p + "mlp.up_proj.weight"], w[p + "mlp.down_proj.weight"])
    want = plain.rmsnorm(x, w["model.norm.weight"], 1e-5) @ w["lm_head.weight"].T
    torch.testing.assert_close(plain.model_forward(w, cfg, ids), want)


def test_attention_block_depends_on_distances_only():
    w, cfg = _tiny(tied=False)
    h = torch.randn(5, 24, dtype=torch.float64)
    p = "model.layers.0.self_attn."
    a = plain.attention_block(h, w, p, torch.arange(5), 3, 1, 16, 100.0)
    b = plain.attention_block(h, w, p, torch.arange(5) + 300, 3, 1, 16, 100.0)
    torch.testing.assert_close(a, b, atol=1e-5, rtol=1e-5)         # float32 angles at position ~300 cost a little


# ---- sampling --------------------------------------------------------------------------------
def test_top_p_keep_rule_hand_vectors():
    p = torch.tensor([0.2, 0.5, 0.3])
    assert plain.top_p_keep(p, 0.5).tolist() == [False, True, False]          # mass before the top token is 0 < 0.5
    assert plain.top_p_keep(p, 0.51).tolist() == [False, True, True]
    assert plain.top_p_keep(p, 0.81).tolist() == [True, True, True]
    # the same rule as the reference's three lines (tensorline/engine.py:47-49)
    probs = torch.softmax(torch.randn(40), -1)
    sp, idx = torch.sort(probs, descending=True)
    keep = torch.cumsum(sp, -1) - sp < 0.7
    assert sorted(idx[keep].tolist()) == torch.nonzero(plain.top_p_keep(probs, 0.7)).flatten().tolist()


def test_sample_with_uniform():
    lg = torch.log(torch.tensor([0.5, 0.3, 0.2]))
    assert plain.sample_with_uniform(lg, 0.0, 1.0, 0.9) == 0                   # temperature 0: arg-max
    assert [plain.sample_with_uniform(lg, 1.0, 1.0, u) for u in (0.0, 0.49, 0.51, 0.79, 0.81, 0.999)] == [0, 0, 1, 1, 2, 2]
    assert plain.sample_with_uniform(lg, 1.0, 0.5, 0.999) == 0                 # top-p 0.5 keeps the top token only
    assert plain.sample_with_uniform(lg, 1e-3, 1.0, 0.999) == 0                # temperature -> 0+: arg-max
    n = 20000
    draws = torch.tensor([plain.sample_with_uniform(lg, 2.0, 1.0, (i + 0.5) / n) for i in range(0, n, 7)])
    freq = torch.bincount(draws, minlength=3).double() / len(draws)
    torch.testing.assert_close(freq, torch.softmax(lg.double() / 2.0, -1), atol=5e-3, rtol=0)


def test_greedy_generate_stops_without_emitting_the_stop_token():
    w, cfg = _tiny(tied=True)
    full = plain.greedy_generate(w, cfg, [1, 2, 3], 6)
    assert len(full) == 6
    cut = plain.greedy_generate(w, cfg, [1, 2, 3], 6, stop={full[2]})
    assert cut == full[:full.index(full[2])]
    assert math.isfinite(float(plain.model_forward(w, cfg, [1, 2, 3]).sum()))
