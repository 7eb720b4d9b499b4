"""Qwen2 dense decoder as data: which parts each layer has, with which sizes.

Structure as the reference's generic graph path runs it (src/graph_builder.cpp:
130-304 detection, :968-1039 and :1138-1444 emission): token embedding; per
layer a pre-norm block of RMSNorm -> attention (q/k/v with bias, no o bias,
grouped-query, rotary with half-split pairs) and RMSNorm -> gated SiLU MLP;
final RMSNorm; output head (own matrix, or the embedding when tied). Layers
with index >= max_window_layers attend through the sliding window when the
configuration switches it on.
"""
from __future__ import annotations

from ..config.qwen2 import Qwen2Config
from ..parts.base import LayerSpec, ModelSpec, PartSpec, ScheduleEntry
from ..registry import register_architecture


def qwen2_spec(cfg: Qwen2Config) -> ModelSpec:
    norm = PartSpec("rmsnorm", {"size": cfg.hidden_size, "eps": cfg.rms_norm_eps})
    rotary = PartSpec("rotary", {"head_dim": cfg.head_dim, "theta": cfg.rope_theta})
    layers = []
    for l in range(cfg.num_hidden_layers):
        mixer = PartSpec("attention", {
            "hidden_size": cfg.hidden_size,
            "num_heads": cfg.num_attention_heads,
            "num_kv_heads": cfg.num_key_value_heads,
            "head_dim": cfg.head_dim,
            "qkv_bias": cfg.attention_bias,
            "out_bias": False,
            "window": cfg.layer_window(l),
            "position": rotary,
        })
        ff = PartSpec("gated_mlp", {"hidden_size": cfg.hidden_size,
                                    "intermediate_size": cfg.intermediate_size,
                                    "activation": cfg.hidden_act})
        block = PartSpec("pre_norm", {
            "mixer_norm": norm, "mixer": mixer, "feed_forward_norm": norm, "feed_forward": ff,
            "names": {"mixer_norm": "input_layernorm", "mixer": "self_attn",
                      "feed_forward_norm": "post_attention_layernorm", "feed_forward": "mlp"},
        })
        layers.append(LayerSpec(f"model.layers.{l}.", block))
    head_params = {"vocab_size": cfg.vocab_size, "hidden_size": cfg.hidden_size}
    if cfg.tie_word_embeddings:
        head_params["tied_to"] = "model.embed_tokens.weight"
    return ModelSpec(
        hidden_size=cfg.hidden_size,
        vocab_size=cfg.vocab_size,
        embedding=PartSpec("token_embedding", {"vocab_size": cfg.vocab_size,
                                               "hidden_size": cfg.hidden_size}),
        embedding_prefix="model.embed_tokens.",
        layers=layers,
        schedule=[ScheduleEntry(l) for l in range(cfg.num_hidden_layers)],
        final_norm=norm,
        final_norm_prefix="model.norm.",
        head=PartSpec("linear_head", head_params),
        head_prefix="lm_head.",
        max_positions=cfg.max_position_embeddings,
        # a folder of a tied model may still hold the output matrix (it is not read)
        unused_tensors=frozenset({"lm_head.weight"}) if cfg.tie_word_embeddings else frozenset(),
    )


register_architecture("Qwen2ForCausalLM", Qwen2Config, qwen2_spec)
