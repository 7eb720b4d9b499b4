"""Weight preparation on the GPU: the seeded random tensors of the device kernel against the
host's lines (the same bits), the conversion kernel against torch, and that an engine filled on
the device from a configuration and a seed is the model of the folder written from them."""
import warnings

import numpy as np
import pytest
import torch

from tests.conftest import TINY_B, TINY_C
from tests.helpers import rand_ids

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def ops():
    import hector_engine_amd  # noqa: F401
    from hector_engine_amd.kernels import lib, ops as _ops
    lib.load()
    return _ops


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("n", [1, 3, 4, 1001, 70001])
def test_random_fill_is_the_hosts_element_by_element(ops, dtype, n):
    from hector_engine_amd.weights.random_init import normal_values, quantile_table, tensor_key
    key = tensor_key(7, f"some.tensor.{n}")
    table = torch.from_numpy(quantile_table()).cuda()
    for mean, std in ((0.0, 0.02), (1.0, 0.1)):
        out = torch.empty(n, dtype=dtype, device="cuda")
        ops.fill_random(out, key, table, mean, std)
        want = normal_values(key, n, mean, std)
        assert np.array_equal(out.float().cpu().numpy(), want)
    # a prefix of a longer tensor with the same key is the same: values depend on (key, index) only
    assert np.array_equal(normal_values(key, n + 5, 0.0, 0.02)[:n], normal_values(key, n, 0.0, 0.02))
    if n > 1000:       # and they are what they claim to be
        v = normal_values(key, n, 1.0, 0.1).astype(np.float64)
        assert abs(v.mean() - 1.0) < 0.01 and abs(v.std() - 0.1) < 0.01
        assert tensor_key(7, "a") != tensor_key(8, "a") != tensor_key(7, "b")


def test_random_integer_tables(ops):
    from hector_engine_amd.weights.random_init import integer_values
    out = torch.empty(5000, dtype=torch.int32, device="cuda")
    ops.fill_random_integers(out, 12345, 7)
    want = integer_values(12345, 5000, 7)
    assert np.array_equal(out.cpu().numpy(), want)
    assert want.min() == 0 and want.max() == 6 and len(set(want.tolist())) == 7


@pytest.mark.parametrize("src", [torch.float32, torch.bfloat16, torch.float16])
@pytest.mark.parametrize("dst", [torch.float32, torch.bfloat16])
def test_cast_equals_torch(ops, src, dst):
    g = torch.Generator().manual_seed(3)
    x = (torch.randn(100003, generator=g) * 3).to(src)
    special = torch.tensor([0.0, -0.0, 1e-7, -1e-7, 6e-5, 65504.0, float("inf"), -float("inf"), 1.00390625, 1.01171875])
    x = torch.cat([x, special.to(src)])
    out = torch.empty(x.shape, dtype=dst, device="cuda")
    ops.cast(out, x.cuda())
    assert torch.equal(out.cpu(), x.to(dst))         # exact: widening, or rounding to nearest even
    nan = torch.tensor([float("nan")]).to(src).cuda()
    out = torch.empty(1, dtype=dst, device="cuda")
    ops.cast(out, nan)
    assert torch.isnan(out).all()


@pytest.mark.parametrize("cfg,seed", [(TINY_B, 11), (TINY_C, 12)])
def test_engine_from_a_seed_is_the_folders_model(tmp_path, cfg, seed):
    """Engine(config, seed) fills its tensors on the device; write_random_model(config, seed) on
    the host (forced here): the same logits, bit for bit, in 32-bit."""
    import hector_engine_amd as he
    from hector_engine_amd.engine.engine import StepEntry
    from hector_engine_amd.registry import config_from_dict
    config = config_from_dict(dict(cfg))
    folder = str(tmp_path)
    he.write_random_model(config, seed, folder, "bfloat16", device="cpu")
    ids = rand_ids(cfg["vocab_size"], 50, seed)
    outs = []
    for source in (dict(model_dir=folder), dict(config=config_from_dict(dict(cfg)), seed=seed)):
        eng = he.Engine(dtype="float32", max_tokens=256, **source)
        s = eng.acquire()
        outs.append(eng.step([StepEntry(s, ids, list(range(50)))]).clone())
        eng.release(s)
    assert torch.equal(outs[0], outs[1])
    assert outs[0].abs().max() > 0


def test_a_stored_output_matrix_of_a_tied_model_is_named_and_not_used(tmp_path):
    import hector_engine_amd as he
    from hector_engine_amd.registry import config_from_dict
    from hector_engine_amd.weights import WeightsError, write_safetensors
    from tests.conftest import TINY_A
    folder = str(tmp_path)
    he.write_random_model(config_from_dict(dict(TINY_A)), 1, folder)
    extra = str(tmp_path / "extra.safetensors")
    write_safetensors(extra, {"lm_head.weight": torch.ones(256, 64, dtype=torch.bfloat16)})
    with pytest.warns(UserWarning, match="lm_head.weight"):
        he.Engine(folder, dtype="float32", max_tokens=128)
    # an untied model does not allow it to be missing, nor a tied one any other stray tensor
    write_safetensors(extra, {"lm_head.bias": torch.ones(256, dtype=torch.bfloat16)})
    with pytest.raises(WeightsError, match="unexpected 1: lm_head.bias"):
        he.Engine(folder, dtype="float32", max_tokens=128)


def test_max_seq_len_is_bounded_by_the_configurations_positions(model_dirs):
    import hector_engine_amd as he
    eng = he.Engine(model_dirs["A"], dtype="float32", max_tokens=1024)
    assert eng.max_seq_len == 128                    # max_position_embeddings of this configuration
    with pytest.raises(ValueError, match="128 positions"):
        he.Engine(model_dirs["A"], dtype="float32", max_tokens=1024, max_seq_len=192)
    with warnings.catch_warnings():
        warnings.simplefilter("error")
        eng = he.Engine(model_dirs["A"], dtype="float32", max_tokens=1024, max_seq_len=192, beyond_max_positions=True)
    assert eng.max_seq_len == 192
