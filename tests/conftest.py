import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)
sys.path.insert(0, os.path.dirname(os.path.abspath(__file__)))


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs an MI355X (run with -m gpu)")


# ----------------------------------------------------------------------------- tiny configurations
# Two tiny Qwen2 configurations that differ in every size and option.
TINY_A = {
    "architectures": ["Qwen2ForCausalLM"], "model_type": "qwen2",
    "num_hidden_layers": 2, "hidden_size": 64, "num_attention_heads": 4, "num_key_value_heads": 2,
    "intermediate_size": 176, "vocab_size": 512, "rope_theta": 10000.0, "rms_norm_eps": 1e-6,
    "tie_word_embeddings": True, "max_position_embeddings": 128, "hidden_act": "silu",
    "use_sliding_window": False, "bos_token_id": 1, "eos_token_id": 2, "torch_dtype": "float32",
}
TINY_B = {
    "architectures": ["Qwen2ForCausalLM"], "model_type": "qwen2",
    "num_hidden_layers": 3, "hidden_size": 96, "num_attention_heads": 3, "num_key_value_heads": 1,
    "head_dim": 32, "intermediate_size": 256, "vocab_size": 1000, "rope_theta": 1000000.0,
    "rms_norm_eps": 1e-5, "tie_word_embeddings": False, "max_position_embeddings": 256, "hidden_act": "silu",
    "use_sliding_window": False, "bos_token_id": 0, "eos_token_id": 7, "torch_dtype": "float32",
}
# A third one with odd sizes, a head size that is no power of two and windowed upper layers.
TINY_C = {
    "architectures": ["Qwen2ForCausalLM"], "model_type": "qwen2",
    "num_hidden_layers": 3, "hidden_size": 120, "num_attention_heads": 6, "num_key_value_heads": 3,
    "head_dim": 48, "intermediate_size": 200, "vocab_size": 777, "rope_theta": 50000.0,
    "rms_norm_eps": 3e-6, "tie_word_embeddings": True, "max_position_embeddings": 512, "hidden_act": "silu",
    "use_sliding_window": True, "sliding_window": 24, "max_window_layers": 1,
    "bos_token_id": 3, "eos_token_id": 4, "torch_dtype": "float32",
}
# A fourth one with the head size of the benchmark models (64), for which bfloat16 attention runs on the
# matrix cores; query width 6 * 64 differs from the model width.
TINY_D = {
    "architectures": ["Qwen2ForCausalLM"], "model_type": "qwen2",
    "num_hidden_layers": 2, "hidden_size": 192, "num_attention_heads": 6, "num_key_value_heads": 2,
    "head_dim": 64, "intermediate_size": 328, "vocab_size": 650, "rope_theta": 1000000.0,
    "rms_norm_eps": 1e-6, "tie_word_embeddings": True, "max_position_embeddings": 640, "hidden_act": "silu",
    "use_sliding_window": True, "sliding_window": 40, "max_window_layers": 1,
    "bos_token_id": 5, "eos_token_id": 6, "torch_dtype": "bfloat16",
}
# A fifth one with the other head size of the matrix-core attention kernels (128), four query heads on one
# kv head, a width that is no multiple of the head size, a separate output matrix.
TINY_E = {
    "architectures": ["Qwen2ForCausalLM"], "model_type": "qwen2",
    "num_hidden_layers": 2, "hidden_size": 160, "num_attention_heads": 4, "num_key_value_heads": 1,
    "head_dim": 128, "intermediate_size": 264, "vocab_size": 901, "rope_theta": 300000.0,
    "rms_norm_eps": 2e-6, "tie_word_embeddings": False, "max_position_embeddings": 384, "hidden_act": "silu",
    "use_sliding_window": False, "bos_token_id": 8, "eos_token_id": 9, "torch_dtype": "bfloat16",
}
TINY = {"A": (TINY_A, 0), "B": (TINY_B, 1), "C": (TINY_C, 2), "D": (TINY_D, 3), "E": (TINY_E, 4)}


@pytest.fixture(scope="session")
def tiny_models(tmp_path_factory):
    """name -> model folder with random float32 weights, written once per session into a temporary folder."""
    from easy_gpt.cpp_amd.weights import write_random_model

    out = {}
    for name, (cfg, seed) in TINY.items():
        d = tmp_path_factory.mktemp(f"tiny_{name}")
        write_random_model(str(d), cfg, seed)
        out[name] = str(d)
    return out
