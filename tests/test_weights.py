"""Weights: safetensors by name, one error for all mismatches, the precision
rule, and the random-weights mode."""
import json
import os
import struct

import pytest
import torch

import hector_engine_amd  # noqa: F401
from hector_engine_amd.parts.base import BuildEnv, TensorSpec
from hector_engine_amd.registry import build_model, config_from_dict
from hector_engine_amd.weights import (SafetensorsFile, WeightsError, check_against, load_tensors,
                                       run_dtype_of, write_random_model, write_safetensors)
from tests.conftest import TINY_A, TINY_B
from tests.plain import qwen2_plain as P

CPU = torch.device("cpu")


def specs_for(cfg_dict):
    return build_model(config_from_dict(dict(cfg_dict)), BuildEnv(CPU, torch.float32)).tensor_specs()


def test_round_trip_all_dtypes(tmp_path):
    t = {"a": torch.randn(3, 5), "b": torch.randn(7).to(torch.bfloat16), "c": torch.randn(2, 2).half(),
         "i": torch.arange(6, dtype=torch.int32).reshape(2, 3)}
    path = str(tmp_path / "x.safetensors")
    write_safetensors(path, t, {"k": "v"})
    f = SafetensorsFile(path)
    assert set(f.names()) == set(t)
    for k, v in t.items():
        assert f.shape(k) == tuple(v.shape) and f.stored_dtype(k) == v.dtype
        assert torch.equal(f.tensor(k), v)
    # the independent reader of the plain implementation sees the same values
    mine = P.read_safetensors(path)
    assert torch.equal(mine["b"], t["b"].float()) and torch.equal(mine["a"], t["a"])


def test_reads_what_the_safetensors_library_writes(tmp_path):
    st = pytest.importorskip("safetensors.torch")
    t = {"w": torch.randn(4, 6).to(torch.bfloat16), "g": torch.randn(6)}
    path = str(tmp_path / "lib.safetensors")
    st.save_file(t, path)
    f = SafetensorsFile(path)
    assert torch.equal(f.tensor("w"), t["w"]) and torch.equal(f.tensor("g"), t["g"])
    ours = str(tmp_path / "ours.safetensors")
    write_safetensors(ours, t)
    back = st.load_file(ours)
    assert torch.equal(back["w"], t["w"]) and torch.equal(back["g"], t["g"])


def test_one_error_lists_missing_unexpected_and_wrong_shapes():
    expected = {"a": TensorSpec((2, 3)), "b": TensorSpec((4,)), "c": TensorSpec((5,))}
    found = {"a": (3, 2), "c": (5,), "d": (1,), "e": (2,)}
    with pytest.raises(WeightsError) as err:
        check_against(expected, found)
    msg = str(err.value)
    assert "missing 1: b" in msg and "unexpected 2: d, e" in msg
    assert "a is [3, 2], expected [2, 3]" in msg
    check_against(expected, {"a": (2, 3), "b": (4,), "c": (5,), "x": (1,)}, allowed_extra={"x"})


def test_model_folder_errors(tmp_path):
    folder = str(tmp_path / "m")
    write_random_model(config_from_dict(dict(TINY_B)), 1, folder)
    specs = specs_for(TINY_B)
    tensors = load_tensors(folder, specs, torch.float32, CPU)
    assert set(tensors) == set(specs)
    # drop one tensor, add one, misshape one
    f = SafetensorsFile(os.path.join(folder, "model.safetensors"))
    t = {n: f.tensor(n).clone() for n in f.names()}
    del t["model.layers.1.self_attn.k_proj.bias"]
    t["model.layers.9.extra.weight"] = torch.zeros(2)
    t["model.norm.weight"] = torch.zeros(7).to(torch.bfloat16)
    bad = str(tmp_path / "bad")
    os.makedirs(bad)
    write_safetensors(os.path.join(bad, "model.safetensors"), t)
    with pytest.raises(WeightsError) as err:
        load_tensors(bad, specs, torch.float32, CPU)
    msg = str(err.value)
    assert "model.layers.1.self_attn.k_proj.bias" in msg and "model.layers.9.extra.weight" in msg
    assert "model.norm.weight is [7], expected [96]" in msg


def test_truncated_and_garbled_files(tmp_path):
    folder = str(tmp_path / "m")
    write_random_model(config_from_dict(dict(TINY_A)), 0, folder)
    path = os.path.join(folder, "model.safetensors")
    raw = open(path, "rb").read()
    cut = str(tmp_path / "cut.safetensors")
    open(cut, "wb").write(raw[:len(raw) - 100])
    with pytest.raises(WeightsError, match="truncated"):
        SafetensorsFile(cut)
    open(cut, "wb").write(struct.pack("<Q", 10 ** 9) + b"{}")
    with pytest.raises(WeightsError, match="header length"):
        SafetensorsFile(cut)
    open(cut, "wb").write(struct.pack("<Q", 4) + b"nope")
    with pytest.raises(WeightsError, match="not valid JSON"):
        SafetensorsFile(cut)
    empty = str(tmp_path / "empty")
    os.makedirs(empty)
    with pytest.raises(WeightsError, match="no .safetensors"):
        load_tensors(empty, {}, torch.float32, CPU)


def test_shards_and_index(tmp_path):
    folder = str(tmp_path / "m")
    write_random_model(config_from_dict(dict(TINY_A)), 0, folder)
    f = SafetensorsFile(os.path.join(folder, "model.safetensors"))
    names = sorted(f.names())
    half = len(names) // 2
    sharded = str(tmp_path / "s")
    os.makedirs(sharded)
    write_safetensors(os.path.join(sharded, "model-00001-of-00002.safetensors"), {n: f.tensor(n) for n in names[:half]})
    write_safetensors(os.path.join(sharded, "model-00002-of-00002.safetensors"), {n: f.tensor(n) for n in names[half:]})
    json.dump({"weight_map": {n: ("model-00001-of-00002.safetensors" if i < half else "model-00002-of-00002.safetensors")
                              for i, n in enumerate(names)}},
              open(os.path.join(sharded, "model.safetensors.index.json"), "w"))
    specs = specs_for(TINY_A)
    a = load_tensors(sharded, specs, torch.float32, CPU)
    b = load_tensors(folder, specs, torch.float32, CPU)
    assert all(torch.equal(a[n], b[n]) for n in specs)
    os.remove(os.path.join(sharded, "model-00002-of-00002.safetensors"))
    with pytest.raises(WeightsError, match="shards named by the index are missing"):
        load_tensors(sharded, specs, torch.float32, CPU)


def test_precision_rule(tmp_path):
    assert run_dtype_of(torch.bfloat16, torch.bfloat16, False) == torch.bfloat16
    assert run_dtype_of(torch.float16, torch.bfloat16, False) == torch.bfloat16
    assert run_dtype_of(torch.float32, torch.bfloat16, False) == torch.float32     # stored in 32-bit stays so
    assert run_dtype_of(torch.bfloat16, torch.float32, False) == torch.float32
    assert run_dtype_of(torch.int64, torch.bfloat16, True) == torch.int32
    path = str(tmp_path / "p")
    os.makedirs(path)
    write_safetensors(os.path.join(path, "model.safetensors"),
                      {"w": torch.randn(2, 2).to(torch.bfloat16), "g": torch.randn(2)})
    specs = {"w": TensorSpec((2, 2)), "g": TensorSpec((2,))}
    t = load_tensors(path, specs, torch.bfloat16, CPU)
    assert t["w"].dtype == torch.bfloat16 and t["g"].dtype == torch.float32
    t = load_tensors(path, specs, torch.float32, CPU)
    assert t["w"].dtype == torch.float32 and t["g"].dtype == torch.float32


def test_random_mode_is_reproducible_and_by_name(tmp_path):
    a, b, c = (str(tmp_path / n) for n in "abc")
    cfg = config_from_dict(dict(TINY_A))
    write_random_model(cfg, 0, a)
    write_random_model(config_from_dict(dict(TINY_A)), 0, b)
    write_random_model(config_from_dict(dict(TINY_A)), 1, c)
    fa, fb, fc = (SafetensorsFile(os.path.join(x, "model.safetensors")) for x in (a, b, c))
    assert set(fa.names()) == set(specs_for(TINY_A))
    assert "lm_head.weight" not in set(fa.names())                  # tied
    for n in fa.names():
        assert torch.equal(fa.tensor(n), fb.tensor(n))
        assert fa.stored_dtype(n) == torch.bfloat16
    assert not torch.equal(fa.tensor("model.norm.weight"), fc.tensor("model.norm.weight"))
    w = fa.tensor("model.layers.0.mlp.up_proj.weight").float()
    g = fa.tensor("model.layers.0.input_layernorm.weight").float()
    assert abs(w.std().item() - 0.02) < 0.002 and abs(g.mean().item() - 1.0) < 0.05
    assert json.load(open(os.path.join(a, "config.json")))["architectures"] == ["Qwen2ForCausalLM"]


def test_expected_names_are_the_hf_names():
    names = set(specs_for(TINY_B))
    assert "lm_head.weight" in names and "model.embed_tokens.weight" in names
    for l in range(3):
        for n in ("input_layernorm.weight", "post_attention_layernorm.weight", "self_attn.q_proj.weight",
                  "self_attn.q_proj.bias", "self_attn.k_proj.weight", "self_attn.k_proj.bias",
                  "self_attn.v_proj.weight", "self_attn.v_proj.bias", "self_attn.o_proj.weight",
                  "mlp.gate_proj.weight", "mlp.up_proj.weight", "mlp.down_proj.weight"):
            assert f"model.layers.{l}.{n}" in names
    assert not any("o_proj.bias" in n for n in names)
    assert len(names) == 3 * 12 + 3


def test_init_rules_are_a_registry():
    """The random mode fills a tensor by the rule registered for the kind its TensorSpec names: the
    built-in kinds, a rule registered from outside, and an unknown kind as an error that lists them."""
    from hector_engine_amd.parts.base import TensorSpec
    from hector_engine_amd.weights import register_init
    from hector_engine_amd.weights.random_init import random_tensor
    z = random_tensor("t", TensorSpec((3, 5), ("zeros",)), 0, torch.float32, CPU)
    c = random_tensor("t", TensorSpec((3, 5), ("constant", 0.5)), 0, torch.bfloat16, CPU)
    assert torch.equal(z, torch.zeros(3, 5)) and torch.equal(c, torch.full((3, 5), 0.5, dtype=torch.bfloat16))
    with pytest.raises(ValueError, match="unknown init.*registered kinds.*normal"):
        random_tensor("t", TensorSpec((4,), ("test_wide", 3.0)), 0, torch.float32, CPU)
    register_init("test_wide", lambda init: (float(init[1]), 2.0))
    w = random_tensor("t", TensorSpec((4000,), ("test_wide", 3.0)), 0, torch.float32, CPU)
    assert abs(w.mean().item() - 3.0) < 0.15 and abs(w.std().item() - 2.0) < 0.15
    g = random_tensor("t", TensorSpec((4000,), ("gain", 1.0, 0.1)), 0, torch.float32, CPU)
    n = random_tensor("t", TensorSpec((4000,), ("normal", 0.1)), 0, torch.float32, CPU)
    assert torch.allclose(g, 1.0 + n, atol=0.01)          # the same draws, another mean (bfloat16 values)
