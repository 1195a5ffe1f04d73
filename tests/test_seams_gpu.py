"""The seams of the framework, each shown with a toy part defined here and registered from the test:
a mixer that caches something that is neither keys nor values (a plane of its own in the paged
cache), a block that knows nothing of the norm hand-off between two blocks that do, an embedding
with a scale and a head with a bias and a cap.  The model they form is nobody's; it is stepped by
the framework's own cache manager and step function, whole, in portions and mixed, and compared
with a plain whole-sequence computation written here."""
import numpy as np
import pytest
import torch

from tests import helpers, plain

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
H, V, LATENT = 48, 70, 10
SCALE, CAP = 1.7, 3.0


def _register_toys():
    from tensorline_amd.ops import kernels
    from tensorline_amd.parts.base import Part
    from tensorline_amd.parts.registry import (build_part, register_block, register_embedding, register_head,
                                               register_mixer)
    from tensorline_amd.parts.spec import CacheNeed, CachePlane, TensorDecl

    @register_mixer("toy_latent_mean", replace=True)
    class LatentMean(Part):
        """Caches z[t] = h[t] Wz^T (one short vector per token, always float32) and returns the mean
        of the cached vectors up to each token, times Wo^T."""

        def __init__(self, hidden_size, prefix, dtype, device, latent: int):
            super().__init__(hidden_size, prefix, dtype, device)
            self.latent = latent

        def tensors(self):
            return {self.prefix + "wz": TensorDecl((self.latent, self.hidden_size), "normal", 0.2, "float32"),
                    self.prefix + "wo": TensorDecl((self.hidden_size, self.latent), "normal", 0.2, "float32")}

        def load(self, get):
            self.wz, self.wo = get(self.prefix + "wz"), get(self.prefix + "wo")

        def cache_need(self):
            return CacheNeed((CachePlane("latent", (self.latent,), dtype="float32"),))

        def forward(self, h, ctx, cache):
            store = cache.planes["latent"]                        # [pages, page, latent]
            page = store.shape[1]
            store.view(-1, self.latent)[cache.slots.long()] = h.float() @ self.wz.T
            out = torch.empty(h.shape[0], self.hidden_size, dtype=torch.float32, device=h.device)
            tables = cache.tables.cpu()
            for s in range(ctx.num_seqs):
                r0, r1, start = ctx.host_q_start[s], ctx.host_q_start[s + 1], ctx.host_ctx_start[s]
                upto = start + r1 - r0
                pages = tables[s, :-(-upto // page)].long().to(h.device)
                z = store[pages].reshape(-1, self.latent)[:upto]
                mean = z.cumsum(0) / torch.arange(1, upto + 1, device=h.device)[:, None]
                out[r0:r1] = mean[start:] @ self.wo.T
            return out

    @register_block("toy_add_at_once", replace=True)
    class AddAtOnce:
        """norm, mixer, add; norm, feed-forward, add: nothing is left to the next block, and nothing
        but a tensor is taken from the one before (it has no ``intake``)."""

        def __init__(self, spec, hidden_size, dtype, device):
            common = dict(hidden_size=hidden_size, dtype=dtype, device=device)
            self.n1 = build_part("norm", spec.mixer_norm, layer_prefix=spec.prefix, **common)
            self.mixer = build_part("mixer", spec.mixer, layer_prefix=spec.prefix, **common)
            self.n2 = build_part("norm", spec.feed_forward_norm, layer_prefix=spec.prefix, **common)
            self.ffn = build_part("feed_forward", spec.feed_forward, layer_prefix=spec.prefix, **common)

        def parts(self):
            return [self.n1, self.mixer, self.n2, self.ffn]

        def cache_need(self):
            return self.mixer.cache_need()

        def state_need(self):
            return None

        def forward(self, x, carry, ctx, cache):
            assert carry is None or isinstance(carry, torch.Tensor), "a block without intake gets tensors only"
            h = self.n1.forward(x, carry)
            h = self.n2.forward(x, self.mixer.forward(h, ctx, cache))
            x.add_(self.ffn.forward(h, ctx).float())
            return None

    @register_embedding("toy_scaled_embedding", replace=True)
    class ScaledEmbedding(Part):
        def __init__(self, hidden_size, prefix, dtype, device, vocab_size, name, scale):
            super().__init__(hidden_size, prefix, dtype, device)
            self.vocab_size, self.name, self.scale = vocab_size, name, scale

        def tensors(self):
            return {self.name: TensorDecl((self.vocab_size, self.hidden_size), "normal", 0.5, "compute")}

        def load(self, get):
            self.table = get(self.name)

        def weight_tensors(self):
            return [self.table]

        def forward(self, ids):
            return kernels.embed(ids, self.table).mul_(self.scale)

    @register_head("toy_capped_head", replace=True)
    class CappedHead(Part):
        def __init__(self, hidden_size, prefix, dtype, device, vocab_size, name, cap):
            super().__init__(hidden_size, prefix, dtype, device)
            self.vocab_size, self.name, self.cap = vocab_size, name, cap

        def tensors(self):
            return {self.name + ".weight": TensorDecl((self.vocab_size, self.hidden_size), "normal", 0.3, "compute"),
                    self.name + ".bias": TensorDecl((self.vocab_size,), "normal", 0.5, "float32")}

        def load(self, get, embedding=None):
            self.weight, self.bias = get(self.name + ".weight"), get(self.name + ".bias")

        def weight_tensors(self):
            return [self.weight, self.bias]

        def forward(self, h):
            logits = kernels.linear(h, self.weight, self.bias, out_dtype=torch.float32)
            return self.cap * torch.tanh(logits / self.cap)


def _spec():
    from tensorline_amd.parts.spec import LayerSpec, ModelSpec, PartSpec
    norm = lambda name: PartSpec("rmsnorm", {"eps": 1e-6, "name": name})
    attn = PartSpec("attention", {"num_heads": 3, "num_kv_heads": 1, "head_dim": 16, "qkv_bias": True,
                                  "position": PartSpec("rope", {"theta": 100.0})}, prefix="a.")
    ffn = PartSpec("swiglu", {"intermediate_size": 64}, prefix="mlp.")
    layers = (LayerSpec("l0.", attn, ffn, norm("n1"), norm("n2")),
              LayerSpec("l1.", PartSpec("toy_latent_mean", {"latent": LATENT}, prefix="mix."), ffn, norm("n1"), norm("n2"),
                        block="toy_add_at_once"),
              LayerSpec("l2.", attn, ffn, norm("n1"), norm("n2")))
    return ModelSpec(H, V, PartSpec("toy_scaled_embedding", {"name": "emb", "scale": SCALE}), layers, norm("nf"),
                     PartSpec("toy_capped_head", {"name": "out", "cap": CAP}))


def _plain_forward(w, ids):
    T = len(ids)
    pos = torch.arange(T)
    x = w["emb"][torch.tensor(ids)] * SCALE
    for i in range(3):
        p = f"l{i}."
        h = plain.rmsnorm(x, w[p + "n1"], 1e-6)
        if i == 1:
            z = h @ w[p + "mix.wz"].T
            x = x + (z.cumsum(0) / torch.arange(1, T + 1)[:, None]) @ w[p + "mix.wo"].T
        else:
            x = x + plain.attention_block(h, w, p + "a.", pos, 3, 1, 16, 100.0)
        h = plain.rmsnorm(x, w[p + "n2"], 1e-6)
        x = x + plain.swiglu(h, w[p + "mlp.gate_proj.weight"], w[p + "mlp.up_proj.weight"], w[p + "mlp.down_proj.weight"])
    logits = plain.rmsnorm(x, w["nf"], 1e-6) @ w["out.weight"].T + w["out.bias"]
    return CAP * torch.tanh(logits / CAP)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_toy_parts_at_every_seam_match_a_plain_computation(dtype):
    from tensorline_amd.engine.replay import TraceSession
    from tensorline_amd.models.decoder import DecoderModel
    from tensorline_amd.weights.loader import load_from_getter
    from tensorline_amd.weights.random_init import random_tensor
    _register_toys()
    tdt = {"float32": torch.float32, "bfloat16": torch.bfloat16}[dtype]
    model = DecoderModel(_spec(), tdt, DEV)
    decls = model.tensor_decls()
    assert {"emb", "out.weight", "out.bias", "l1.mix.wz", "l0.a.q_proj.bias"} <= set(decls)
    w = {n: random_tensor(n, d, 8, "cpu") for n, d in decls.items()}
    if dtype == "bfloat16":                                      # what the engine keeps in bfloat16, the oracle sees rounded
        w = {n: (t.to(torch.bfloat16).float() if decls[n].storage == "compute" else t) for n, t in w.items()}
    load_from_getter(model, lambda name, decl: w[name], DEV)
    needs = model.cache_needs()
    assert [p.name for p in needs[1].planes] == ["latent"] and [p.name for p in needs[0].planes] == ["k", "v"]
    reqs = {f"r{i}": [int(t) for t in np.random.default_rng(i).integers(0, V, n)] for i, n in enumerate([37, 5, 90, 18])}
    want = {(rid, i): lg.numpy() for rid, toks in reqs.items() for i, lg in enumerate(_plain_forward(w, toks))}
    limit = {"float32": 1e-5, "bfloat16": 2e-2}[dtype]
    for cut in (helpers.steps_whole, helpers.steps_portions, helpers.steps_mixed):
        steps = cut(reqs)
        session = TraceSession(model, helpers.max_live_tokens(steps), page_size=8)
        assert len(session.cache.groups) == 2                    # keys and values; the toy's plane
        assert session.cache.storage(1)["latent"].dtype == torch.float32
        got = helpers.collect_logits(session.step, steps)
        for rid, toks in reqs.items():
            scale = max(float(np.abs(want[(rid, i)]).max()) for i in range(len(toks)))
            for i in range(len(toks)):
                err = float(np.abs(got[(rid, i)] - want[(rid, i)]).max()) / scale
                assert err < limit, (cut.__name__, rid, i, err)
        assert session.cache.all_free()


def test_a_block_between_two_that_hand_norms_over_gets_and_gives_tensors_only(monkeypatch):
    """In few-row bfloat16 steps the framework's blocks pass norms to each other as objects; a
    block in between that knows nothing of that must never see one.  (The toy block asserts it; here
    the hand-off is also seen to happen where both sides know it: block 2 to the final norm.)"""
    from tensorline_amd.models.decoder import DecoderModel
    from tensorline_amd.parts.spec import Intake
    _register_toys()
    model = DecoderModel(_spec(), torch.bfloat16, DEV)
    from tensorline_amd.weights.loader import load_from_getter
    from tensorline_amd.weights.random_init import random_tensor
    load_from_getter(model, lambda name, decl: random_tensor(name, decl, 8, "cpu"), DEV)
    after = model._negotiate()
    assert after[1] is None                                      # the toy block takes no `after=`
    assert after[0] == Intake()                                  # so the block before it is asked for a tensor
    assert after[2].normed_rows_for is None                      # the toy head takes no normed rows
    assert after[2].share_sums                                   # but the final norm adds products left in shares
