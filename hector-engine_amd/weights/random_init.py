"""Random weights from a configuration and a seed: in memory, or written as a
model folder (config.json, model.safetensors). Matrices and biases are
N(0, 0.02), norm gains 1 + N(0, 0.1); each tensor has a generator of its own
seeded from (seed, tensor name), so a tensor's values do not depend on which
other tensors exist."""
from __future__ import annotations

import hashlib
import os

import torch

from ..parts.base import TensorSpec
from .safetensors_io import write_safetensors


def _tensor_seed(seed: int, name: str) -> int:
    digest = hashlib.sha256(f"{seed}:{name}".encode()).digest()
    return int.from_bytes(digest[:8], "little") & ((1 << 63) - 1)


def random_tensor(name: str, spec: TensorSpec, seed: int, dtype: torch.dtype, device) -> torch.Tensor:
    gen = torch.Generator(device=device)
    gen.manual_seed(_tensor_seed(seed, name))
    shape = tuple(spec.shape)
    if spec.integer:
        high = int(spec.init[1]) if len(spec.init) > 1 else 2
        return torch.randint(0, high, shape, generator=gen, device=device, dtype=torch.int32)
    kind = spec.init[0]
    if kind == "zeros":
        return torch.zeros(shape, dtype=dtype, device=device)
    # always drawn in float32 and rounded to bfloat16 first, so that the values do not
    # depend on the precision the model is then run in
    t = torch.empty(shape, dtype=torch.float32, device=device).normal_(0.0, 1.0, generator=gen)
    if kind == "normal":
        t.mul_(spec.init[1])
    elif kind == "gain":
        t.mul_(spec.init[2]).add_(spec.init[1])
    else:
        raise ValueError(f"tensor '{name}': unknown init {spec.init}")
    return t.to(torch.bfloat16).to(dtype)


def random_tensors(expected: dict[str, TensorSpec], seed: int, dtype: torch.dtype,
                   device) -> dict[str, torch.Tensor]:
    return {name: random_tensor(name, spec, seed, dtype, device) for name, spec in expected.items()}


def write_random_model(config, seed: int, model_dir: str, dtype: str = "bfloat16") -> str:
    """Writes config.json and model.safetensors for `config` (an architecture's
    typed configuration); returns the folder."""
    from ..registry import build_model  # local: the registry imports the parts
    from ..parts.base import BuildEnv

    st_dtype = {"bfloat16": torch.bfloat16, "float32": torch.float32}[dtype]
    cpu = torch.device("cpu")
    model = build_model(config, BuildEnv(cpu, st_dtype))
    tensors = random_tensors(model.tensor_specs(), seed, st_dtype, cpu)
    os.makedirs(model_dir, exist_ok=True)
    config.torch_dtype = dtype
    config.save(model_dir)
    write_safetensors(os.path.join(model_dir, "model.safetensors"), tensors,
                      {"format": "pt", "seed": seed})
    return model_dir
