"""Qwen2 dense decoder: typed configuration -> ModelSpec.

Tensor names are the reference's (/root/reference/src/models/layer_key_prefix.cpp:77-87,
/root/reference/src/models/embedding.cpp:30): model.embed_tokens.weight,
model.layers.{i}.self_attn.{q,k,v,o}_proj.{weight,bias}, model.layers.{i}.input_layernorm.weight,
model.layers.{i}.post_attention_layernorm.weight, model.layers.{i}.mlp.{gate,up,down}_proj.weight,
model.norm.weight, and lm_head.weight when the output is not tied.
"""
from __future__ import annotations

from ..config.qwen2 import Qwen2Config
from ..config.registry import Architecture, register_architecture
from ..parts.spec import LayerSpec, ModelSpec, PartSpec, RunSpec


def qwen2_spec(cfg: Qwen2Config) -> ModelSpec:
    layers = []
    for i in range(cfg.num_hidden_layers):
        p = f"model.layers.{i}."
        layers.append(
            LayerSpec(
                block="pre_norm",
                mixer=PartSpec(
                    "gq_attention",
                    dict(
                        n_heads=cfg.num_attention_heads,
                        n_kv_heads=cfg.num_key_value_heads,
                        head_dim=cfg.head_dim,
                        qkv_bias=cfg.attention_bias,
                        out_bias=False,
                        window=cfg.layer_window(i),
                        position=PartSpec("rope_half_split", dict(theta=cfg.rope_theta)),
                    ),
                    prefix=p + "self_attn.",
                ),
                feed_forward=PartSpec(
                    "swiglu",
                    dict(intermediate_size=cfg.intermediate_size, activation=cfg.hidden_act),
                    prefix=p + "mlp.",
                ),
                norms={
                    "mixer": PartSpec("rmsnorm", dict(eps=cfg.rms_norm_eps), prefix=p + "input_layernorm."),
                    "feed_forward": PartSpec("rmsnorm", dict(eps=cfg.rms_norm_eps), prefix=p + "post_attention_layernorm."),
                },
            )
        )
    return ModelSpec(
        hidden_size=cfg.hidden_size,
        vocab_size=cfg.vocab_size,
        max_position=cfg.max_position_embeddings,
        embedding=PartSpec("token_embedding", {}, prefix="model.embed_tokens."),
        layers=tuple(layers),
        run_order=tuple(RunSpec(layer=i, cache=i) for i in range(cfg.num_hidden_layers)),
        final_norm=PartSpec("rmsnorm", dict(eps=cfg.rms_norm_eps), prefix="model.norm."),
        output_head=PartSpec("linear_head", dict(tied=cfg.tie_word_embeddings), prefix="lm_head."),
        # a tied checkpoint may still carry a copy of the output matrix; the reference
        # leaves it unconsumed with a warning (src/models/model_param_validation.cpp:198-218)
        ignorable_tensors=("lm_head.weight",) if cfg.tie_word_embeddings else (),
        bos_token_id=cfg.bos_token_id,
        eos_token_id=cfg.eos_token_id,
    )


QWEN2 = register_architecture(
    Architecture(name="Qwen2ForCausalLM", config_class=Qwen2Config, build_spec=qwen2_spec, model_types=("qwen2",)),
    replace=True,
)
