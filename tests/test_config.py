"""Configuration and registry: typed reading of config.json keys, defaults,
validation errors that name the key, and the architecture registry."""
import json

import pytest

import hector_engine_amd  # noqa: F401
from hector_engine_amd.config import ConfigError, Qwen2Config
from hector_engine_amd.registry import (config_from_dict, load_config, model_spec,
                                        registered_architectures)
from tests.conftest import TINY_A, TINY_B


def test_reads_every_size_from_the_file():
    a, b = config_from_dict(dict(TINY_A)), config_from_dict(dict(TINY_B))
    assert isinstance(a, Qwen2Config)
    for key in ("num_hidden_layers", "hidden_size", "num_attention_heads", "num_key_value_heads",
                "head_dim", "intermediate_size", "vocab_size", "rope_theta", "rms_norm_eps",
                "max_position_embeddings", "tie_word_embeddings"):
        assert getattr(a, key) == TINY_A[key] and getattr(b, key) == TINY_B[key]
        assert TINY_A[key] != TINY_B[key]          # the two tiny configurations differ in every size


def test_defaults():
    d = {k: v for k, v in TINY_A.items() if k not in ("num_key_value_heads", "head_dim", "rms_norm_eps",
                                                      "rope_theta", "tie_word_embeddings", "hidden_act")}
    c = config_from_dict(d)
    assert c.num_key_value_heads == c.num_attention_heads
    assert c.head_dim == c.hidden_size // c.num_attention_heads
    assert c.rms_norm_eps == 1e-6 and c.rope_theta == 10000.0
    assert c.tie_word_embeddings is False and c.hidden_act == "silu"
    assert c.use_sliding_window is False and c.layer_window(0) == 0


def test_window_layers():
    c = config_from_dict(dict(TINY_B))
    assert [c.layer_window(l) for l in range(3)] == [0, 8, 8]
    d = dict(TINY_B, use_sliding_window=False)
    assert [config_from_dict(d).layer_window(l) for l in range(3)] == [0, 0, 0]
    d = dict(TINY_B, max_window_layers=None)
    assert [config_from_dict(d).layer_window(l) for l in range(3)] == [0, 0, 0]
    spec = model_spec(c)
    assert [ls.block.params["mixer"].params["window"] for ls in spec.layers] == [0, 8, 8]


@pytest.mark.parametrize("change,needle", [
    ({"hidden_size": None}, "hidden_size"),
    ({"vocab_size": 0}, "vocab_size"),
    ({"num_key_value_heads": 3}, "num_key_value_heads"),
    ({"head_dim": 15}, "head_dim"),
    ({"hidden_act": "gelu"}, "hidden_act"),
    ({"rope_scaling": {"type": "linear", "factor": 2.0}}, "rope_scaling"),
    ({"use_sliding_window": True, "sliding_window": None}, "sliding_window"),
    ({"num_hidden_layers": "two"}, "num_hidden_layers"),
    ({"rms_norm_eps": "small"}, "rms_norm_eps"),
    ({"architectures": []}, "architectures"),
])
def test_errors_name_the_key(change, needle):
    d = dict(TINY_A)
    d.update(change)
    d = {k: v for k, v in d.items() if v is not None or k in ("sliding_window",)}
    with pytest.raises(ConfigError, match=needle):
        config_from_dict(d)


def test_unknown_architecture_lists_registered():
    with pytest.raises(ConfigError, match="Qwen2ForCausalLM"):
        config_from_dict(dict(TINY_A, architectures=["NopeForCausalLM"]))
    assert "Qwen2ForCausalLM" in registered_architectures()


def test_round_trip_through_a_folder(tmp_path):
    c = config_from_dict(dict(TINY_B, eos_token_id=[5, 7], bos_token_id=1))
    c.save(str(tmp_path))
    again = load_config(str(tmp_path))
    assert again == c
    assert json.load(open(tmp_path / "config.json"))["eos_token_id"] == [5, 7]
    with pytest.raises(ConfigError, match="not found"):
        load_config(str(tmp_path / "missing"))


def test_int_and_bool_coercion():
    c = config_from_dict(dict(TINY_A, rope_theta=10000, tie_word_embeddings=1, eos_token_id=3))
    assert c.rope_theta == 10000.0 and c.tie_word_embeddings is True and c.eos_token_id == [3]


def test_stop_ids_come_from_generation_config_then_config(tmp_path):
    """An instruction-tuned folder lists its end-of-turn id in generation_config.json beside the
    end-of-text id of config.json: both end a sequence. Without that file, or without the key
    in it, config.json's id counts; with neither, nothing ends a sequence by itself."""
    from hector_engine_amd.config.base import ConfigError, stop_token_ids
    cfg = config_from_dict(dict(TINY_A, eos_token_id=151643 % 256))
    folder = tmp_path / "m"
    folder.mkdir()
    assert stop_token_ids(str(folder), cfg) == [151643 % 256]
    assert stop_token_ids(None, cfg) == [151643 % 256]
    (folder / "generation_config.json").write_text(json.dumps({"eos_token_id": [7, 9], "temperature": 0.7}))
    assert stop_token_ids(str(folder), cfg) == [7, 9]
    (folder / "generation_config.json").write_text(json.dumps({"eos_token_id": 11}))
    assert stop_token_ids(str(folder), cfg) == [11]
    (folder / "generation_config.json").write_text(json.dumps({"temperature": 0.7}))
    assert stop_token_ids(str(folder), cfg) == [151643 % 256]
    assert stop_token_ids(str(folder), config_from_dict(dict(TINY_A))) == []
    (folder / "generation_config.json").write_text("{not json")
    with pytest.raises(ConfigError, match="generation_config.json"):
        stop_token_ids(str(folder), cfg)
    (folder / "generation_config.json").write_text(json.dumps({"eos_token_id": "x"}))
    with pytest.raises(ConfigError, match="eos_token_id"):
        stop_token_ids(str(folder), cfg)
