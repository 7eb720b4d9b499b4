"""Fills a model's tensors by name from a model folder.

The expected names and shapes come from the model's parts. All mismatches are
gathered into one error that lists missing tensors, unexpected tensors and wrong
shapes (the reference lists missing weights the same way:
src/graph_builder.cpp:1462-1516). Precision rule: under bfloat16, 16-bit tensors
are kept as bfloat16 and a tensor stored in 32-bit stays 32-bit; under float32
everything becomes float32; integer tables are kept as int32.
"""
from __future__ import annotations

import warnings

import torch

from ..parts.base import TensorSpec
from .safetensors_io import SafetensorsFile, WeightsError, open_model_files


def run_dtype_of(stored: torch.dtype, run: torch.dtype, integer: bool) -> torch.dtype:
    if integer or not stored.is_floating_point:
        return torch.int32
    if run == torch.float32 or stored == torch.float32:
        return torch.float32
    return torch.bfloat16


def check_against(expected: dict[str, TensorSpec], found: dict[str, tuple],
                  allowed_extra: set[str] = frozenset()) -> None:
    """Raises one WeightsError naming every missing, unexpected and misshapen tensor."""
    missing = sorted(n for n in expected if n not in found)
    unexpected = sorted(n for n in found if n not in expected and n not in allowed_extra)
    wrong = sorted((n, tuple(expected[n].shape), tuple(found[n])) for n in expected
                   if n in found and tuple(found[n]) != tuple(expected[n].shape))
    if not (missing or unexpected or wrong):
        return
    lines = ["the model folder's tensors do not match the configuration:"]
    if missing:
        lines.append(f"  missing {len(missing)}: " + ", ".join(missing))
    if unexpected:
        lines.append(f"  unexpected {len(unexpected)}: " + ", ".join(unexpected))
    if wrong:
        lines.append(f"  wrong shape {len(wrong)}: " + ", ".join(
            f"{n} is {list(got)}, expected {list(want)}" for n, want, got in wrong))
    raise WeightsError("\n".join(lines))


def load_tensors(model_dir: str, expected: dict[str, TensorSpec], run: torch.dtype, device,
                 allowed_extra: set[str] = frozenset()) -> dict[str, torch.Tensor]:
    files = open_model_files(model_dir)
    where: dict[str, SafetensorsFile] = {}
    for f in files:
        for name in f.names():
            if name in where:
                raise WeightsError(f"tensor '{name}' is stored twice: {where[name].path} and {f.path}")
            where[name] = f
    check_against(expected, {n: f.shape(n) for n, f in where.items()}, allowed_extra)
    ignored = sorted(n for n in where if n not in expected)
    if ignored:     # allowed and unused (the reference decides by presence: src/graph_builder.cpp:250-253)
        warnings.warn(f"{model_dir}: stored but not used by this configuration: {', '.join(ignored)}",
                      stacklevel=2)
    out: dict[str, torch.Tensor] = {}
    for name, spec in expected.items():
        f = where[name]
        stored = f.stored_dtype(name)
        if spec.integer != (not stored.is_floating_point):
            kind = "an integer table" if spec.integer else "a floating-point tensor"
            raise WeightsError(f"tensor '{name}' is stored as {stored}, expected {kind}")
        target = run_dtype_of(stored, run, spec.integer)
        out[name] = _upload(f.tensor(name), target, torch.device(device))
    return out


def _upload(stored: torch.Tensor, target: torch.dtype, device: torch.device) -> torch.Tensor:
    """The tensor on the device in the dtype it runs in. On the GPU the bytes go up as they are
    stored and the conversion is the library's own kernel (bf16 -> f32 is the 16-bit shift of
    tools/quant_bench/ref_qwen3.py:60; f32 -> bf16 rounds to nearest even)."""
    if device.type != "cuda" or not stored.is_floating_point() or stored.dtype == target:
        return stored.to(device=device, dtype=target).contiguous()
    from ..kernels import ops
    raw = stored.contiguous().to(device)
    out = torch.empty(raw.shape, dtype=target, device=device)
    ops.cast(out, raw)
    return out
