"""Configuration, registry and weight loading: defaults, validation, and one error that lists
everything wrong with a checkpoint."""
import json
import os

import pytest
import torch
from safetensors.torch import load_file, save_file

from tensorline_amd.config import (ConfigError, EngineConfig, Qwen2Config, get_architecture, known_architectures,
                                   load_model_config)
from tensorline_amd.engine.loading import load_model
from tensorline_amd.weights import WeightError, write_random_model
from tests import helpers

BASE = dict(architectures=["Qwen2ForCausalLM"], vocab_size=100, hidden_size=48, intermediate_size=64,
            num_hidden_layers=2, num_attention_heads=6)


def test_defaults_and_derived_sizes():
    c = Qwen2Config.from_dict(BASE)
    assert (c.num_key_value_heads, c.head_dim, c.group_size) == (6, 8, 1)
    assert (c.rms_norm_eps, c.rope_theta, c.tie_word_embeddings) == (1e-6, 10000.0, False)
    c = Qwen2Config.from_dict(dict(BASE, num_key_value_heads=2, head_dim=16, rms_norm_eps=1e-5, rope_theta=1e6,
                                   tie_word_embeddings=True, eos_token_id=[7, 9]))
    assert (c.group_size, c.q_size, c.kv_size, c.eos_token_id) == (3, 96, 32, (7, 9))
    assert Qwen2Config.from_dict(c.to_dict()) == c                       # config.json round trip


@pytest.mark.parametrize("patch,word", [
    ({"hidden_size": None}, "hidden_size"), ({"vocab_size": -1}, "vocab_size"), ({"num_hidden_layers": 1.5}, "integer"),
    ({"num_key_value_heads": 4}, "multiple"), ({"head_dim": 7}, "even"), ({"hidden_act": "gelu"}, "hidden_act"),
    ({"use_sliding_window": True}, "use_sliding_window"), ({"rope_scaling": {"type": "yarn"}}, "rope_scaling"),
    ({"num_attention_heads": 5}, "head_dim"), ({"rope_theta": 0}, "rope_theta"),
])
def test_bad_configs_are_refused_with_the_reason(patch, word):
    with pytest.raises(ConfigError, match=word):
        Qwen2Config.from_dict({k: v for k, v in dict(BASE, **patch).items() if v is not None})


def test_registry(tmp_path):
    assert "Qwen2ForCausalLM" in known_architectures()
    with pytest.raises(ConfigError, match="known: .*Qwen2ForCausalLM"):
        get_architecture("LlamaForCausalLM")
    with open(tmp_path / "config.json", "w") as f:
        json.dump(dict(BASE, architectures=["NopeForCausalLM"]), f)
    with pytest.raises(ConfigError, match="NopeForCausalLM"):
        load_model_config(tmp_path)
    with open(tmp_path / "config.json", "w") as f:
        json.dump({k: v for k, v in BASE.items() if k != "architectures"}, f)
    with pytest.raises(ConfigError, match="architectures"):
        load_model_config(tmp_path)
    with pytest.raises(ConfigError, match="config.json"):
        load_model_config(tmp_path / "missing")
    spec = get_architecture("Qwen2ForCausalLM").build_spec(Qwen2Config.from_dict(BASE))
    assert len(spec.layers) == 2 and spec.layers[1].mixer.params["num_heads"] == 6


@pytest.mark.parametrize("head_dim", [272, 300])
def test_head_sizes_no_kernel_serves_are_refused_when_the_model_is_built(head_dim):
    """The configuration allows any even head size; the attention part refuses, before any weight is
    read, those the kernels do not take, instead of failing in the first step.  Sizes between the
    kernels' steps of 16 are served at the next step, with zeros added to every head at loading."""
    from tensorline_amd.models.decoder import DecoderModel
    arch = get_architecture("Qwen2ForCausalLM")
    spec = arch.build_spec(Qwen2Config.from_dict(dict(BASE, head_dim=head_dim)))
    with pytest.raises(ValueError, match=f"head size of {head_dim}"):
        DecoderModel(spec, torch.float32, "cpu")
    for d, served_at in ((48, 48), (8, 16), (40, 48), (250, 256)):
        model = DecoderModel(arch.build_spec(Qwen2Config.from_dict(dict(BASE, head_dim=d))), torch.float32, "cpu")
        mixer = model.blocks[0].mixer
        assert (mixer.head_dim, mixer.kernel_dim) == (d, served_at)
        assert model.cache_needs()[0].planes[0].shape[-1] == served_at       # the cache is laid out for the kernels' size


def test_engine_config_names():
    e = EngineConfig(dtype="bf16")
    assert (e.dtype, e.block_size, e.max_num_seqs, e.max_batched_tokens, e.max_model_len) == ("bfloat16", 16, 64, 2048, 4096)
    assert EngineConfig(dtype="torch.float32").dtype == "float32"
    with pytest.raises(ValueError):
        EngineConfig(dtype="float16")


# ---- weights -----------------------------------------------------------------------------------
@pytest.fixture()
def folder(tmp_path):
    cfg = Qwen2Config.from_dict(helpers.TINY_B)
    return write_random_model(cfg, str(tmp_path / "m"), seed=3), cfg


def test_random_model_round_trip(folder):
    d, cfg = folder
    files = sorted(os.listdir(d))
    assert files == ["config.json", "model.safetensors"]
    raw = load_file(os.path.join(d, "model.safetensors"))
    assert all(t.dtype == torch.bfloat16 for t in raw.values())
    model, c2 = load_model(d, "float32", "cpu")
    assert c2 == cfg
    # by name, fused in file order, identical values
    attn = model.blocks[1].mixer
    want = torch.cat([raw[f"model.layers.1.self_attn.{n}_proj.weight"] for n in "qkv"]).float()
    assert torch.equal(attn.qkv.weight, want) and attn.qkv.weight.dtype == torch.float32
    assert torch.equal(model.head.linear.weight, raw["lm_head.weight"].float())
    assert torch.equal(model.final_norm.weight, raw["model.norm.weight"].float())
    # the same seed gives the same model, another seed another
    d2 = write_random_model(cfg, d + "2", seed=3)
    d3 = write_random_model(cfg, d + "3", seed=4)
    again, other = load_file(os.path.join(d2, "model.safetensors")), load_file(os.path.join(d3, "model.safetensors"))
    assert all(torch.equal(raw[k], again[k]) for k in raw) and not torch.equal(raw["lm_head.weight"], other["lm_head.weight"])
    # the initialisation scheme: N(0, 0.02) matrices and biases, 1 + N(0, 0.1) norm weights
    assert abs(float(raw["lm_head.weight"].float().std()) - 0.02) < 2e-3
    nw = raw["model.layers.0.input_layernorm.weight"].float()
    assert abs(float(nw.mean()) - 1.0) < 0.05 and 0.05 < float(nw.std()) < 0.15


def test_checkpoint_tensor_names_and_shapes_are_those_of_the_reference_modules(tmp_path):
    """The names a random model folder holds and the loader asks for, written out here: the module
    paths the reference walks (paged.py:172-188: ``inner.embed_tokens``, ``layer.input_layernorm``,
    ``attn.q_proj`` .. ``o_proj``, ``layer.post_attention_layernorm``, ``mlp.gate_proj`` ..
    ``down_proj``, ``inner.norm``, ``hf.lm_head``; manager.py:52-53 for the projections' shapes), with
    ``.weight`` and, for q/k/v, ``.bias``.  Neither side of this comparison comes from the product."""
    cfg = Qwen2Config.from_dict(dict(architectures=["Qwen2ForCausalLM"], vocab_size=99, hidden_size=40, intermediate_size=56,
                                     num_hidden_layers=2, num_attention_heads=6, num_key_value_heads=2, head_dim=16,
                                     tie_word_embeddings=False))
    d = write_random_model(cfg, str(tmp_path / "m"), seed=1)
    got = {name: tuple(t.shape) for name, t in load_file(os.path.join(d, "model.safetensors")).items()}
    h, i, v, q, kv = 40, 56, 99, 6 * 16, 2 * 16
    want = {"model.embed_tokens.weight": (v, h), "model.norm.weight": (h,), "lm_head.weight": (v, h)}
    for layer in range(2):
        p = f"model.layers.{layer}."
        want.update({p + "input_layernorm.weight": (h,), p + "post_attention_layernorm.weight": (h,),
                     p + "self_attn.q_proj.weight": (q, h), p + "self_attn.q_proj.bias": (q,),
                     p + "self_attn.k_proj.weight": (kv, h), p + "self_attn.k_proj.bias": (kv,),
                     p + "self_attn.v_proj.weight": (kv, h), p + "self_attn.v_proj.bias": (kv,),
                     p + "self_attn.o_proj.weight": (h, q),
                     p + "mlp.gate_proj.weight": (i, h), p + "mlp.up_proj.weight": (i, h), p + "mlp.down_proj.weight": (h, i)})
    assert got == want


def test_storage_dtypes(folder):
    d, _ = folder
    model, _ = load_model(d, "bfloat16", "cpu")
    attn = model.blocks[0].mixer
    assert attn.qkv.weight.dtype == torch.bfloat16 and model.embedding.table.dtype == torch.bfloat16
    assert attn.qkv.bias.dtype == torch.float32 and model.final_norm.weight.dtype == torch.float32
    assert attn.qkv.shuffled is not None and attn.qkv.shuffled.shape[-3:] == (4, 16, 8)
    # a tensor stored in 32-bit that the model keeps in 32-bit stays exact
    raw = load_file(os.path.join(d, "model.safetensors"))
    exact = torch.full_like(raw["model.norm.weight"], 1.0).float() + 1e-4
    raw["model.norm.weight"] = exact
    save_file(raw, os.path.join(d, "model.safetensors"))
    model, _ = load_model(d, "bfloat16", "cpu")
    assert torch.equal(model.final_norm.weight, exact)


def test_one_error_lists_missing_unexpected_and_wrong_shapes(folder):
    d, _ = folder
    path = os.path.join(d, "model.safetensors")
    raw = load_file(path)
    del raw["model.layers.0.mlp.up_proj.weight"]
    del raw["model.layers.2.self_attn.q_proj.bias"]
    raw["model.layers.0.mlp.extra.weight"] = torch.zeros(2, 2)
    raw["model.layers.1.self_attn.k_proj.weight"] = torch.zeros(64, 191, dtype=torch.bfloat16)
    save_file(raw, path)
    with pytest.raises(WeightError) as e:
        load_model(d, "float32", "cpu")
    err = e.value
    assert err.missing == ["model.layers.0.mlp.up_proj.weight", "model.layers.2.self_attn.q_proj.bias"]
    assert err.unexpected == ["model.layers.0.mlp.extra.weight"]
    assert len(err.wrong_shape) == 1 and "k_proj.weight" in err.wrong_shape[0] and "[64, 192]" in err.wrong_shape[0]
    msg = str(err)
    assert "missing tensors (2)" in msg and "unexpected tensors (1)" in msg and "wrong shapes (1)" in msg


def test_wrong_dtypes_are_an_error_and_extra_tensors_alone_a_warning(folder):
    d, _ = folder
    path = os.path.join(d, "model.safetensors")
    good = load_file(path)
    raw = dict(good)
    raw["rotary.inv_freq"] = torch.zeros(4)                                  # something the model does not know
    save_file(raw, path)
    with pytest.warns(UserWarning, match="rotary.inv_freq"):
        model, _ = load_model(d, "float32", "cpu")
    assert torch.equal(model.embedding.table, good["model.embed_tokens.weight"].float())
    # integer and 64-bit tensors under the names of float weights: one error names each, and the extra tensor too
    raw["model.layers.1.mlp.down_proj.weight"] = torch.zeros_like(good["model.layers.1.mlp.down_proj.weight"], dtype=torch.int64)
    raw["model.norm.weight"] = good["model.norm.weight"].double()
    raw["model.layers.0.self_attn.v_proj.bias"] = good["model.layers.0.self_attn.v_proj.bias"].to(torch.int8)
    save_file(raw, path)
    with pytest.raises(WeightError) as e:
        load_model(d, "bfloat16", "cpu")
    err = e.value
    assert sorted(w.split(":")[0] for w in err.wrong_dtype) == [
        "model.layers.0.self_attn.v_proj.bias", "model.layers.1.mlp.down_proj.weight", "model.norm.weight"]
    assert "I64" in str(err) and "F64" in str(err) and "I8" in str(err) and "wrong dtypes (3)" in str(err)
    assert err.unexpected == ["rotary.inv_freq"] and not err.missing and not err.wrong_shape
    # half precision is a float dtype: accepted
    raw = dict(good)
    raw["model.norm.weight"] = good["model.norm.weight"].half()
    save_file(raw, path)
    load_model(d, "float32", "cpu")
    save_file(good, path)


def test_tied_head(tmp_path):
    cfg = Qwen2Config.from_dict(helpers.TINY_A)
    d = write_random_model(cfg, str(tmp_path / "tied"), seed=1)
    path = os.path.join(d, "model.safetensors")
    raw = load_file(path)
    assert "lm_head.weight" not in raw
    model, _ = load_model(d, "float32", "cpu")
    assert model.head.linear.weight is model.embedding.table                           # shared, not copied
    one = sum(t.numel() * t.element_size() for t in [model.embedding.table])
    assert model.weight_bytes() < 2 * one + 10 ** 6
    raw["lm_head.weight"] = raw["model.embed_tokens.weight"].clone()         # stored too, and equal: accepted
    save_file(raw, path)
    load_model(d, "float32", "cpu")
    raw["lm_head.weight"] = raw["lm_head.weight"] * 2                        # stored too, and different: refused
    save_file(raw, path)
    with pytest.raises(WeightError, match="tied"):
        load_model(d, "float32", "cpu")
    # untied and missing: listed as missing
    cfg_b = Qwen2Config.from_dict(helpers.TINY_B)
    d2 = write_random_model(cfg_b, str(tmp_path / "untied"), seed=1)
    raw = load_file(os.path.join(d2, "model.safetensors"))
    del raw["lm_head.weight"]
    save_file(raw, os.path.join(d2, "model.safetensors"))
    with pytest.raises(WeightError) as e:
        load_model(d2, "float32", "cpu")
    assert e.value.missing == ["lm_head.weight"]


def test_sharded_checkpoint(folder):
    d, _ = folder
    raw = load_file(os.path.join(d, "model.safetensors"))
    names = sorted(raw)
    a, b = names[: len(names) // 2], names[len(names) // 2:]
    save_file({n: raw[n] for n in a}, os.path.join(d, "model-00001-of-00002.safetensors"))
    save_file({n: raw[n] for n in b}, os.path.join(d, "model-00002-of-00002.safetensors"))
    os.unlink(os.path.join(d, "model.safetensors"))
    with open(os.path.join(d, "model.safetensors.index.json"), "w") as f:
        json.dump({"weight_map": {**{n: "model-00001-of-00002.safetensors" for n in a},
                                  **{n: "model-00002-of-00002.safetensors" for n in b}}}, f)
    model, _ = load_model(d, "float32", "cpu")
    assert torch.equal(model.embedding.table, raw["model.embed_tokens.weight"].float())


def test_engine_refuses_to_run_without_a_gpu(folder):
    if torch.cuda.is_available():
        pytest.skip("a GPU is visible")
    from tensorline_amd import LLM
    from tensorline_amd.ops.kernels import KernelError
    with pytest.raises(KernelError):
        LLM(folder[0], device="cpu")
    with pytest.raises(KernelError):
        LLM(folder[0], device="cuda:0")
