"""Random weights from a configuration and a seed: in memory (on the device they are made by
a kernel), or written as a model folder (config.json, model.safetensors). Matrices and biases
are N(0, 0.02), norm gains 1 + N(0, 0.1).

The generator is counter-based, keyed by (seed, tensor name, element index): a tensor's values do
not depend on which other tensors exist, and the host lines below and the device kernel
(csrc/fill_cast.hip) give the same bits, so a folder written here and an engine filled on the
device from the same configuration and seed hold the same model. Element i of a tensor with key
k takes 16 bits of mix64(k + (i // 4 + 1) * 0x9E3779B97F4A7C15) (the splitmix64 finaliser), looks
them up in a table of 65536 quantiles of the standard normal distribution, multiplies by the
standard deviation and adds the mean (each rounded to float32), and rounds to bfloat16: the values
are bfloat16 values whatever precision the model then runs in."""
from __future__ import annotations

import hashlib
import os

import numpy as np
import torch

from ..parts.base import TensorSpec
from .safetensors_io import write_safetensors

_GOLDEN = np.uint64(0x9E3779B97F4A7C15)
_CHUNK_WORDS = 1 << 22
_quantiles: np.ndarray | None = None
_quantiles_on: dict = {}


def tensor_key(seed: int, name: str) -> int:
    digest = hashlib.sha256(f"{seed}:{name}".encode()).digest()
    return int.from_bytes(digest[:8], "little")


def quantile_table() -> np.ndarray:
    """float32 [65536]: the standard normal quantile of (k + 1/2) / 65536."""
    global _quantiles
    if _quantiles is None:
        p = (torch.arange(65536, dtype=torch.float64) + 0.5) / 65536
        _quantiles = torch.special.ndtri(p).to(torch.float32).numpy()
    return _quantiles


def _quantiles_device(device) -> torch.Tensor:
    key = str(device)
    if key not in _quantiles_on:
        _quantiles_on[key] = torch.from_numpy(quantile_table()).to(device)
    return _quantiles_on[key]


def _mix64(z: np.ndarray) -> np.ndarray:
    z = z ^ (z >> np.uint64(30))
    z = z * np.uint64(0xBF58476D1CE4E5B9)
    z = z ^ (z >> np.uint64(27))
    z = z * np.uint64(0x94D049BB133111EB)
    return z ^ (z >> np.uint64(31))


def _words(key: int, first: int, count: int) -> np.ndarray:
    j = np.arange(first + 1, first + count + 1, dtype=np.uint64)
    with np.errstate(over="ignore"):
        return _mix64(np.uint64(key) + j * _GOLDEN)


def _normal_chunk(out: np.ndarray, key: int, n: int, w0: int, count: int, mean32, std32) -> None:
    w = _words(key, w0, count)
    idx = np.stack([(w >> np.uint64(16 * e)) & np.uint64(0xffff) for e in range(4)], axis=1).reshape(-1)
    v = quantile_table()[idx.astype(np.int64)] * std32 + mean32          # two float32 roundings
    u = v.view(np.uint32)
    u = (u + np.uint32(0x7fff) + ((u >> np.uint32(16)) & np.uint32(1))) & np.uint32(0xffff0000)
    lo = 4 * w0
    out[lo:lo + 4 * count] = u.view(np.float32)[:n - lo]


def normal_values(key: int, n: int, mean: float, std: float) -> np.ndarray:
    """float32 [n] of bfloat16 values, as the device kernel he_fill_random makes them."""
    quantile_table()
    out = np.empty(n, dtype=np.float32)
    mean32, std32 = np.float32(mean), np.float32(std)
    words = (n + 3) // 4
    chunks = [(w0, min(_CHUNK_WORDS, words - w0)) for w0 in range(0, words, _CHUNK_WORDS)]
    if len(chunks) <= 1:
        for w0, count in chunks:
            _normal_chunk(out, key, n, w0, count, mean32, std32)
        return out
    import concurrent.futures
    with concurrent.futures.ThreadPoolExecutor(min(8, os.cpu_count() or 1)) as pool:   # numpy releases the GIL
        list(pool.map(lambda c: _normal_chunk(out, key, n, c[0], c[1], mean32, std32), chunks))
    return out


def integer_values(key: int, n: int, high: int) -> np.ndarray:
    w = _words(key, 0, n)
    return (((w >> np.uint64(32)) * np.uint64(high)) >> np.uint64(32)).astype(np.int32)


# How a TensorSpec's `init` becomes values: kind -> rule(init) -> (mean, std) of the normal
# values the tensor is filled with (std 0: the constant `mean`). A part with another kind of
# initial values registers its rule; nothing else changes.
_init_rules: dict = {}


def register_init(kind: str, rule=None):
    """Registers rule(init: tuple) -> (mean, std) for TensorSpec.init tuples that start with
    `kind`; usable as a decorator."""
    def deco(f):
        _init_rules[kind] = f
        return f
    return deco(rule) if rule is not None else deco


register_init("normal", lambda init: (0.0, float(init[1])))
register_init("gain", lambda init: (float(init[1]), float(init[2])))
register_init("zeros", lambda init: (0.0, 0.0))
register_init("constant", lambda init: (float(init[1]), 0.0))


def init_moments(name: str, init: tuple) -> tuple[float, float]:
    try:
        rule = _init_rules[init[0]]
    except (KeyError, IndexError):
        raise ValueError(f"tensor '{name}': unknown init {init}; registered kinds: {sorted(_init_rules)}") from None
    return rule(init)


def random_tensor(name: str, spec: TensorSpec, seed: int, dtype: torch.dtype, device) -> torch.Tensor:
    device = torch.device(device)
    key = tensor_key(seed, name)
    shape = tuple(spec.shape)
    n = int(np.prod(shape, dtype=np.int64)) if shape else 1
    on_gpu = device.type == "cuda"
    if on_gpu:
        from ..kernels import ops
    if spec.integer:
        high = int(spec.init[1]) if len(spec.init) > 1 else 2
        if on_gpu:
            out = torch.empty(shape, dtype=torch.int32, device=device)
            ops.fill_random_integers(out, key, high)
            return out
        return torch.from_numpy(integer_values(key, n, high)).reshape(shape)
    mean, std = init_moments(name, spec.init)
    if std == 0.0:
        return torch.full(shape, mean, dtype=dtype, device=device)
    if on_gpu:
        out = torch.empty(shape, dtype=dtype, device=device)
        ops.fill_random(out, key, _quantiles_device(device), mean, std)
        return out
    return torch.from_numpy(normal_values(key, n, mean, std)).reshape(shape).to(dtype)


def random_tensors(expected: dict[str, TensorSpec], seed: int, dtype: torch.dtype,
                   device) -> dict[str, torch.Tensor]:
    return {name: random_tensor(name, spec, seed, dtype, device) for name, spec in expected.items()}


def write_random_model(config, seed: int, model_dir: str, dtype: str = "bfloat16", device=None) -> str:
    """Writes config.json and model.safetensors for `config` (an architecture's typed
    configuration); returns the folder. device: where the values are made (default: the GPU's
    kernel when there is a GPU, else the host's lines; the values are the same)."""
    from ..registry import build_model  # local: the registry imports the parts
    from ..parts.base import BuildEnv

    st_dtype = {"bfloat16": torch.bfloat16, "float32": torch.float32}[dtype]
    cpu = torch.device("cpu")
    if device is None:
        device = torch.device("cuda") if torch.cuda.is_available() else cpu
    model = build_model(config, BuildEnv(cpu, st_dtype))
    tensors = {name: random_tensor(name, spec, seed, st_dtype, device).cpu()
               for name, spec in model.tensor_specs().items()}
    os.makedirs(model_dir, exist_ok=True)
    config.torch_dtype = dtype
    config.save(model_dir)
    write_safetensors(os.path.join(model_dir, "model.safetensors"), tensors,
                      {"format": "pt", "seed": seed})
    return model_dir
