"""Shared fixtures: two tiny Qwen2 configurations that differ in every size and
option, model folders with random weights made in a temporary folder, and the
plain implementation's view of the same folders."""
import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs an MI355X (run on the GPU box)")


def pytest_collection_modifyitems(config, items):
    import torch
    if torch.cuda.is_available():
        return
    skip = pytest.mark.skip(reason="no GPU in this environment")
    for item in items:
        if "gpu" in item.keywords:
            item.add_marker(skip)


# Tiny A: tied embeddings, no window, group of 2, head_dim 16, H*hd == D
TINY_A = {
    "architectures": ["Qwen2ForCausalLM"], "model_type": "qwen2",
    "num_hidden_layers": 2, "hidden_size": 64, "num_attention_heads": 4,
    "num_key_value_heads": 2, "head_dim": 16, "intermediate_size": 160, "vocab_size": 256,
    "rope_theta": 10000.0, "rms_norm_eps": 1e-6, "max_position_embeddings": 128,
    "tie_word_embeddings": True, "use_sliding_window": False, "hidden_act": "silu",
}
# Tiny B: untied, window 8 from layer 1, one kv head (group of 3), head_dim 32, other eps/theta
TINY_B = {
    "architectures": ["Qwen2ForCausalLM"], "model_type": "qwen2",
    "num_hidden_layers": 3, "hidden_size": 96, "num_attention_heads": 3,
    "num_key_value_heads": 1, "head_dim": 32, "intermediate_size": 224, "vocab_size": 384,
    "rope_theta": 1000000.0, "rms_norm_eps": 1e-5, "max_position_embeddings": 256,
    "tie_word_embeddings": False, "use_sliding_window": True, "sliding_window": 8,
    "max_window_layers": 1, "hidden_act": "silu",
}
# Tiny C: H*hd != D, vocabulary and widths that are no power of two, longer context
# (over 300 positions, so pages and split boundaries are crossed), window 70 on the last layer
TINY_C = {
    "architectures": ["Qwen2ForCausalLM"], "model_type": "qwen2",
    "num_hidden_layers": 2, "hidden_size": 80, "num_attention_heads": 6,
    "num_key_value_heads": 3, "head_dim": 48, "intermediate_size": 136, "vocab_size": 301,
    "rope_theta": 50000.0, "rms_norm_eps": 3e-6, "max_position_embeddings": 512,
    "tie_word_embeddings": False, "use_sliding_window": True, "sliding_window": 70,
    "max_window_layers": 1, "hidden_act": "silu",
}
# Tiny D: head_dim 64 (the one-launch one-token attention takes it), H*hd = 2 D, window 40 on the
# last layer, bias-free norm eps and theta of their own
TINY_D = {
    "architectures": ["Qwen2ForCausalLM"], "model_type": "qwen2",
    "num_hidden_layers": 2, "hidden_size": 128, "num_attention_heads": 4,
    "num_key_value_heads": 2, "head_dim": 64, "intermediate_size": 208, "vocab_size": 200,
    "rope_theta": 20000.0, "rms_norm_eps": 2e-6, "max_position_embeddings": 512,
    "tie_word_embeddings": True, "use_sliding_window": True, "sliding_window": 40,
    "max_window_layers": 1, "hidden_act": "silu",
}
TINY = {"A": (TINY_A, 0), "B": (TINY_B, 1), "C": (TINY_C, 2), "D": (TINY_D, 3)}


@pytest.fixture(scope="session")
def model_dirs(tmp_path_factory):
    """name -> folder with config.json and model.safetensors (bfloat16 values)."""
    import hector_engine_amd  # noqa: F401
    from hector_engine_amd.registry import config_from_dict
    from hector_engine_amd.weights import write_random_model
    out = {}
    for name, (cfg, seed) in TINY.items():
        folder = str(tmp_path_factory.mktemp(f"tiny_{name}"))
        write_random_model(config_from_dict(dict(cfg)), seed, folder, "bfloat16")
        out[name] = folder
    return out


@pytest.fixture(scope="session")
def plain_models(model_dirs):
    """name -> (config dict, weights in float64) as the plain implementation reads them."""
    from tests.plain import qwen2_plain as P
    return {name: P.read_model(folder) for name, folder in model_dirs.items()}
