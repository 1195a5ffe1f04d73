"""``Qwen2ForCausalLM``: how its configuration turns into layers.

Every layer is the same here: attention with q/k/v bias and rotate-half RoPE, SwiGLU, RMSNorm
before each, in pre-norm order.  Tensor names are those of the attribute paths the reference
walks (tensorline/paged.py:112,172-188; projection names tensorline/quant.py:25).
"""
from __future__ import annotations

from tensorline_amd.config.model_config import Qwen2Config
from tensorline_amd.config.registry import Architecture, register_architecture
from tensorline_amd.parts.spec import LayerSpec, ModelSpec, PartSpec


def qwen2_spec(cfg: Qwen2Config) -> ModelSpec:
    position = PartSpec("rope", {"theta": cfg.rope_theta})
    layers = []
    for i in range(cfg.num_hidden_layers):
        layers.append(LayerSpec(
            prefix=f"model.layers.{i}.",
            mixer=PartSpec("attention", {
                "num_heads": cfg.num_attention_heads, "num_kv_heads": cfg.num_key_value_heads,
                "head_dim": cfg.head_dim, "qkv_bias": cfg.attention_bias, "position": position,
            }, prefix="self_attn."),
            feed_forward=PartSpec("swiglu", {"intermediate_size": cfg.intermediate_size}, prefix="mlp."),
            mixer_norm=PartSpec("rmsnorm", {"eps": cfg.rms_norm_eps, "name": "input_layernorm.weight"}),
            feed_forward_norm=PartSpec("rmsnorm", {"eps": cfg.rms_norm_eps, "name": "post_attention_layernorm.weight"}),
            block="prenorm",
        ))
    spec = ModelSpec(
        hidden_size=cfg.hidden_size,
        vocab_size=cfg.vocab_size,
        embedding=PartSpec("token_embedding", {"name": "model.embed_tokens.weight"}),
        layers=tuple(layers),
        final_norm=PartSpec("rmsnorm", {"eps": cfg.rms_norm_eps, "name": "model.norm.weight"}),
        head=PartSpec("lm_head", {"name": "lm_head.weight", "tied": cfg.tie_word_embeddings}),
        max_position=cfg.max_position_embeddings,
        eos_token_ids=tuple(cfg.eos_token_id),
    )
    spec.validate()
    return spec


QWEN2 = register_architecture(Architecture("Qwen2ForCausalLM", Qwen2Config, qwen2_spec), replace=True)
