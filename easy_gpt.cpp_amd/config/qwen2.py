"""Typed configuration of the Qwen2 dense decoder, read from its config.json keys.

The reference reads num_hidden_layers, num_attention_heads, num_key_value_heads,
hidden_size, vocab_size, max_position_embeddings, bos/eos_token_id, rope_theta,
model_type and architectures[0] (/root/reference/src/config.cpp:16-31) and fixes
the rest in code (eps 1e-6 at src/models/norm.cpp:41, head_dim = hidden/heads at
src/models/self_attn.cpp:174, always-tied output at src/models/gpt_model.cpp:328).
Here every one of those constants is a key: rms_norm_eps, head_dim,
intermediate_size, tie_word_embeddings, hidden_act and the sliding-window keys.
"""
from __future__ import annotations

import dataclasses
from dataclasses import dataclass
from typing import Any, Mapping

from .base import ConfigError, KeyReader


@dataclass(frozen=True)
class Qwen2Config:
    architecture: str
    model_type: str
    vocab_size: int
    hidden_size: int
    num_hidden_layers: int
    num_attention_heads: int
    num_key_value_heads: int
    head_dim: int
    intermediate_size: int
    max_position_embeddings: int
    rope_theta: float
    rms_norm_eps: float
    tie_word_embeddings: bool
    attention_bias: bool
    hidden_act: str
    use_sliding_window: bool
    sliding_window: int | None
    max_window_layers: int
    bos_token_id: int
    eos_token_id: int
    torch_dtype: str

    # ------------------------------------------------------------------ reading
    @classmethod
    def from_dict(cls, data: Mapping[str, Any], where: str = "config.json") -> "Qwen2Config":
        r = KeyReader(data, where)
        archs = data.get("architectures")
        architecture = archs[0] if isinstance(archs, list) and archs and isinstance(archs[0], str) else ""
        model_type = r.string("model_type", "")
        hidden = r.integer("hidden_size", minimum=1)
        heads = r.integer("num_attention_heads", minimum=1)
        kv_heads = r.integer("num_key_value_heads", heads, minimum=1)
        head_dim = r.integer("head_dim", None, minimum=1)
        if head_dim is None:
            if hidden % heads != 0:
                raise ConfigError(
                    f"{where}: hidden_size ({hidden}) is not a multiple of num_attention_heads ({heads}) "
                    "and no 'head_dim' key is given"
                )
            head_dim = hidden // heads
        layers = r.integer("num_hidden_layers", minimum=1)
        if data.get("rope_scaling") is not None:
            # the reference has plain rotary position encoding only (/root/reference/src/ops.cpp:392-458);
            # running a model that was trained with scaled angles without them would give wrong logits
            raise ConfigError(f"{where}: 'rope_scaling' ({data['rope_scaling']!r}) is not supported (only plain RoPE)")
        use_window = r.boolean("use_sliding_window", False)
        window = r.integer("sliding_window", None, minimum=1)
        cfg = cls(
            architecture=architecture,
            model_type=model_type,
            vocab_size=r.integer("vocab_size", minimum=1),
            hidden_size=hidden,
            num_hidden_layers=layers,
            num_attention_heads=heads,
            num_key_value_heads=kv_heads,
            head_dim=head_dim,
            intermediate_size=r.integer("intermediate_size", minimum=1),
            max_position_embeddings=r.integer("max_position_embeddings", minimum=1),
            rope_theta=r.number("rope_theta", positive=True),
            rms_norm_eps=r.number("rms_norm_eps", 1e-6, positive=True),
            tie_word_embeddings=r.boolean("tie_word_embeddings", False),
            attention_bias=r.boolean("attention_bias", True),
            hidden_act=r.string("hidden_act", "silu"),
            use_sliding_window=use_window,
            sliding_window=window,
            max_window_layers=r.integer("max_window_layers", layers, minimum=0),
            bos_token_id=r.token_id("bos_token_id"),
            eos_token_id=r.token_id("eos_token_id"),
            torch_dtype=r.string("torch_dtype", data.get("dtype") or "bfloat16"),
        )
        cfg.validate(where)
        return cfg

    def validate(self, where: str = "config.json") -> None:
        if self.num_attention_heads % self.num_key_value_heads != 0:
            raise ConfigError(
                f"{where}: num_attention_heads ({self.num_attention_heads}) must be a multiple of "
                f"num_key_value_heads ({self.num_key_value_heads})"
            )
        if self.head_dim % 2 != 0:
            raise ConfigError(f"{where}: head_dim ({self.head_dim}) must be even for rotary position encoding")
        if self.hidden_act != "silu":
            raise ConfigError(f"{where}: hidden_act '{self.hidden_act}' is not supported (only 'silu')")
        if self.use_sliding_window and self.sliding_window is None:
            raise ConfigError(f"{where}: use_sliding_window is true but 'sliding_window' is missing")

    # ------------------------------------------------------------------ derived
    def layer_window(self, layer: int) -> int | None:
        """Window of a layer's attention, or None for all keys.

        With use_sliding_window, the layers from max_window_layers on see only
        the last `sliding_window` keys (their own included).  The reference reads
        none of these keys and has no windowed attention, so this follows the
        meaning of Qwen2's config.json keys and has no counterpart there.
        """
        if self.use_sliding_window and layer >= self.max_window_layers:
            return self.sliding_window
        return None

    def to_dict(self) -> dict:
        d = dataclasses.asdict(self)
        arch = d.pop("architecture")
        d["architectures"] = [arch]
        return d
