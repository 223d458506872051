"""Configuration and registry (no GPU)."""
import json

import pytest

from conftest import TINY_A, TINY_B, TINY_C
from easy_gpt.cpp_amd.config import (
    Architecture, ConfigError, Qwen2Config, UnknownArchitectureError, load_model_config, register_architecture,
    registered_architectures, resolve_architecture, unregister_architecture,
)


def test_reads_every_size_from_keys():
    a = Qwen2Config.from_dict(TINY_A)
    assert (a.num_hidden_layers, a.hidden_size, a.num_attention_heads, a.num_key_value_heads) == (2, 64, 4, 2)
    assert a.head_dim == 16 and a.intermediate_size == 176 and a.vocab_size == 512
    assert a.rope_theta == 10000.0 and a.rms_norm_eps == 1e-6 and a.tie_word_embeddings is True
    assert a.max_position_embeddings == 128 and a.eos_token_id == 2 and a.bos_token_id == 1
    b = Qwen2Config.from_dict(TINY_B)
    assert b.head_dim == 32 and b.hidden_size == 96 and b.num_attention_heads == 3   # head_dim key wins over H/nq
    assert b.rms_norm_eps == 1e-5 and b.tie_word_embeddings is False and b.rope_theta == 1e6


def test_head_dim_defaults_to_hidden_over_heads():
    d = dict(TINY_A)
    assert "head_dim" not in d
    assert Qwen2Config.from_dict(d).head_dim == 64 // 4
    d["num_attention_heads"] = 3
    d["num_key_value_heads"] = 3
    with pytest.raises(ConfigError, match="hidden_size"):
        Qwen2Config.from_dict(d)


@pytest.mark.parametrize("key", ["hidden_size", "num_hidden_layers", "num_attention_heads", "vocab_size",
                                 "intermediate_size", "rope_theta", "max_position_embeddings"])
def test_missing_required_key_is_named(key):
    d = dict(TINY_A)
    del d[key]
    with pytest.raises(ConfigError, match=key):
        Qwen2Config.from_dict(d)


def test_wrong_types_and_ranges_are_named():
    for key, bad in [("hidden_size", "64"), ("num_hidden_layers", 0), ("rope_theta", -1.0),
                     ("tie_word_embeddings", "yes"), ("rms_norm_eps", 0), ("vocab_size", 1.5)]:
        d = dict(TINY_A)
        d[key] = bad
        with pytest.raises(ConfigError, match=key):
            Qwen2Config.from_dict(d)


def test_consistency_checks():
    d = dict(TINY_A, num_key_value_heads=3)
    with pytest.raises(ConfigError, match="multiple"):
        Qwen2Config.from_dict(d)
    d = dict(TINY_A, head_dim=15)
    with pytest.raises(ConfigError, match="even"):
        Qwen2Config.from_dict(d)
    d = dict(TINY_A, hidden_act="gelu")
    with pytest.raises(ConfigError, match="hidden_act"):
        Qwen2Config.from_dict(d)
    d = dict(TINY_A, use_sliding_window=True)
    with pytest.raises(ConfigError, match="sliding_window"):
        Qwen2Config.from_dict(d)


def test_window_per_layer():
    c = Qwen2Config.from_dict(TINY_C)
    assert [c.layer_window(i) for i in range(3)] == [None, 24, 24]
    a = Qwen2Config.from_dict(TINY_A)
    assert [a.layer_window(i) for i in range(2)] == [None, None]


def test_registry_vectors_of_the_reference():
    # /root/reference/test/layer_key_prefix_test.cpp:23-47
    arch = resolve_architecture({"architectures": ["Qwen2ForCausalLM"], "model_type": "qwen2"})
    assert arch.name == "Qwen2ForCausalLM"
    assert resolve_architecture({"model_type": "qwen2"}).name == "Qwen2ForCausalLM"
    with pytest.raises(UnknownArchitectureError) as e:
        resolve_architecture({"architectures": ["UnknownArchForCausalLM"], "model_type": "unknown"})
    assert "UnknownArchForCausalLM" in str(e.value) and "unknown" in str(e.value)
    assert "Qwen2ForCausalLM" in registered_architectures()


def test_tensor_names_of_the_reference():
    # model.layers.3 prefix as in /root/reference/test/layer_key_prefix_test.cpp:23-35
    from easy_gpt.cpp_amd.parts import build_model

    d = dict(TINY_A, num_hidden_layers=4)
    arch = resolve_architecture(d)
    model = build_model(arch.build_spec(arch.config_class.from_dict(d)))
    names = {s.name for s in model.param_specs()}
    for n in ["model.embed_tokens.weight", "model.norm.weight", "model.layers.3.self_attn.q_proj.weight",
              "model.layers.3.self_attn.k_proj.bias", "model.layers.3.self_attn.o_proj.weight",
              "model.layers.3.input_layernorm.weight", "model.layers.3.post_attention_layernorm.weight",
              "model.layers.3.mlp.gate_proj.weight", "model.layers.3.mlp.up_proj.weight",
              "model.layers.3.mlp.down_proj.weight"]:
        assert n in names
    assert "lm_head.weight" not in names           # tied
    assert "model.layers.3.self_attn.o_proj.bias" not in names
    d["tie_word_embeddings"] = False
    model = build_model(arch.build_spec(arch.config_class.from_dict(d)))
    assert "lm_head.weight" in {s.name for s in model.param_specs()}


def test_register_another_architecture(tmp_path):
    class C:
        @classmethod
        def from_dict(cls, d, where="config.json"):
            return cls()

    arch = Architecture(name="ToyArch", config_class=C, build_spec=lambda c: None, model_types=("toy",))
    register_architecture(arch)
    try:
        with pytest.raises(ValueError):
            register_architecture(arch)
        assert resolve_architecture({"architectures": ["ToyArch"]}) is arch
        assert resolve_architecture({"model_type": "TOY"}) is arch
        (tmp_path / "config.json").write_text(json.dumps({"architectures": ["ToyArch"]}))
        a, cfg = load_model_config(str(tmp_path))
        assert a is arch and isinstance(cfg, C)
    finally:
        unregister_architecture("ToyArch")
    with pytest.raises(UnknownArchitectureError):
        resolve_architecture({"architectures": ["ToyArch"]})


def test_missing_config_file(tmp_path):
    with pytest.raises(ConfigError, match="not found"):
        load_model_config(str(tmp_path))


def test_a_published_config_reads_and_scaled_rotation_is_refused():
    # the keys a published Qwen2.5 config.json carries (values of the 0.5B model), unknown ones included
    d = {"architectures": ["Qwen2ForCausalLM"], "attention_dropout": 0.0, "bos_token_id": 151643, "eos_token_id": 151645,
         "hidden_act": "silu", "hidden_size": 896, "initializer_range": 0.02, "intermediate_size": 4864,
         "max_position_embeddings": 32768, "max_window_layers": 21, "model_type": "qwen2", "num_attention_heads": 14,
         "num_hidden_layers": 24, "num_key_value_heads": 2, "rms_norm_eps": 1e-06, "rope_theta": 1000000.0,
         "sliding_window": 32768, "tie_word_embeddings": True, "torch_dtype": "bfloat16", "use_cache": True,
         "use_sliding_window": False, "vocab_size": 151936, "rope_scaling": None}
    cfg = Qwen2Config.from_dict(d)
    assert cfg.head_dim == 64 and cfg.attention_bias and all(cfg.layer_window(i) is None for i in range(24))
    d["rope_scaling"] = {"type": "yarn", "factor": 4.0}
    with pytest.raises(ConfigError, match="rope_scaling"):
        Qwen2Config.from_dict(d)
