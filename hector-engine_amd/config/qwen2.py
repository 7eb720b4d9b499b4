"""Typed configuration of the Qwen2 dense decoder, read from its config.json keys.

Defaults follow the reference's accessors where it has them: rms_norm_eps 1e-6
and rope_theta 10000 (src/hnf_loader.hpp:487-492, src/graph_builder.cpp:285);
head_dim falls back to hidden_size / num_attention_heads as in the reference's
own oracle (tools/quant_bench/ref_qwen3.py:91). The sliding-window keys are not
read by the reference on this path; layers with index >= max_window_layers use
the window when use_sliding_window is true.
"""
from __future__ import annotations

import dataclasses

from .base import ConfigError, ModelConfig, read_field, read_int_list, architecture_name


@dataclasses.dataclass
class Qwen2Config(ModelConfig):
    vocab_size: int = 0
    hidden_size: int = 0
    intermediate_size: int = 0
    num_hidden_layers: int = 0
    num_attention_heads: int = 0
    num_key_value_heads: int = 0
    head_dim: int = 0
    hidden_act: str = "silu"
    rms_norm_eps: float = 1e-6
    rope_theta: float = 10000.0
    max_position_embeddings: int = 0
    tie_word_embeddings: bool = False
    attention_bias: bool = True
    use_sliding_window: bool = False
    sliding_window: int | None = None
    max_window_layers: int | None = None
    torch_dtype: str = "bfloat16"
    bos_token_id: int | None = None
    eos_token_id: list[int] | None = None
    model_type: str = "qwen2"

    @classmethod
    def from_dict(cls, data: dict) -> "Qwen2Config":
        heads = read_field(data, "num_attention_heads", int)
        hidden = read_field(data, "hidden_size", int)
        if heads <= 0:
            raise ConfigError("config key 'num_attention_heads' must be positive")
        cfg = cls(
            architecture=architecture_name(data),
            model_type=read_field(data, "model_type", str, "qwen2"),
            vocab_size=read_field(data, "vocab_size", int),
            hidden_size=hidden,
            intermediate_size=read_field(data, "intermediate_size", int),
            num_hidden_layers=read_field(data, "num_hidden_layers", int),
            num_attention_heads=heads,
            num_key_value_heads=read_field(data, "num_key_value_heads", int, heads),
            head_dim=read_field(data, "head_dim", int, hidden // heads),
            hidden_act=read_field(data, "hidden_act", str, "silu"),
            rms_norm_eps=read_field(data, "rms_norm_eps", float, 1e-6),
            rope_theta=read_field(data, "rope_theta", float, 10000.0),
            max_position_embeddings=read_field(data, "max_position_embeddings", int),
            tie_word_embeddings=read_field(data, "tie_word_embeddings", bool, False),
            attention_bias=read_field(data, "attention_bias", bool, True),
            use_sliding_window=read_field(data, "use_sliding_window", bool, False),
            sliding_window=read_field(data, "sliding_window", int, None),
            max_window_layers=read_field(data, "max_window_layers", int, None),
            torch_dtype=read_field(data, "torch_dtype", str, "bfloat16"),
            bos_token_id=read_field(data, "bos_token_id", int, None),
            eos_token_id=read_int_list(data, "eos_token_id", None),
        )
        if data.get("rope_scaling") is not None:
            raise ConfigError("config key 'rope_scaling': only null is supported for this architecture")
        cfg.validate()
        return cfg

    def validate(self) -> None:
        for key in ("vocab_size", "hidden_size", "intermediate_size", "num_hidden_layers",
                    "num_attention_heads", "num_key_value_heads", "head_dim",
                    "max_position_embeddings"):
            if getattr(self, key) <= 0:
                raise ConfigError(f"config key '{key}' must be positive, got {getattr(self, key)}")
        if self.num_attention_heads % self.num_key_value_heads != 0:
            raise ConfigError(
                f"config key 'num_key_value_heads' ({self.num_key_value_heads}) must divide "
                f"'num_attention_heads' ({self.num_attention_heads})")
        if self.head_dim % 2 != 0:
            raise ConfigError(f"config key 'head_dim' must be even for the rotary encoding, got {self.head_dim}")
        if self.hidden_act not in ("silu", "swish"):
            raise ConfigError(f"config key 'hidden_act': unsupported activation '{self.hidden_act}'")
        if self.rms_norm_eps <= 0 or self.rope_theta <= 0:
            raise ConfigError("config keys 'rms_norm_eps' and 'rope_theta' must be positive")
        if self.use_sliding_window:
            if self.sliding_window is None or self.sliding_window <= 0:
                raise ConfigError("config key 'sliding_window' must be positive when 'use_sliding_window' is true")
            if self.max_window_layers is not None and self.max_window_layers < 0:
                raise ConfigError("config key 'max_window_layers' must not be negative")
        if self.torch_dtype not in ("bfloat16", "float32", "float16"):
            raise ConfigError(f"config key 'torch_dtype': unsupported '{self.torch_dtype}'")

    def layer_window(self, layer: int) -> int:
        """Window of a layer: 0 = every key is visible."""
        if not self.use_sliding_window or self.sliding_window is None:
            return 0
        first_windowed = self.num_hidden_layers if self.max_window_layers is None else self.max_window_layers
        return self.sliding_window if layer >= first_windowed else 0

    def to_dict(self) -> dict:
        d = {
            "architectures": [self.architecture],
            "model_type": self.model_type,
            "vocab_size": self.vocab_size,
            "hidden_size": self.hidden_size,
            "intermediate_size": self.intermediate_size,
            "num_hidden_layers": self.num_hidden_layers,
            "num_attention_heads": self.num_attention_heads,
            "num_key_value_heads": self.num_key_value_heads,
            "head_dim": self.head_dim,
            "hidden_act": self.hidden_act,
            "rms_norm_eps": self.rms_norm_eps,
            "rope_theta": self.rope_theta,
            "max_position_embeddings": self.max_position_embeddings,
            "tie_word_embeddings": self.tie_word_embeddings,
            "attention_bias": self.attention_bias,
            "use_sliding_window": self.use_sliding_window,
            "sliding_window": self.sliding_window,
            "max_window_layers": self.max_window_layers,
            "torch_dtype": self.torch_dtype,
            "bos_token_id": self.bos_token_id,
            "eos_token_id": (None if self.eos_token_id is None else
                             (self.eos_token_id[0] if len(self.eos_token_id) == 1 else self.eos_token_id)),
        }
        return d
