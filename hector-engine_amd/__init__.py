"""Qwen2 dense generation library for one MI355X (package folder ``hector-engine_amd``).

Python entry point:

    import hector_engine_amd as he
    engine = he.Engine("model_dir", dtype="bfloat16", max_tokens=8192)
    results = he.generate(engine, [[5, 17, 3], [9, 2]], max_new_tokens=16,
                          sampling=he.SamplingConfig(temperature=0.8, seed=7))

Heavy modules load on first use, so the configuration, weights and cache
bookkeeping import without a GPU.
"""
from __future__ import annotations

__all__ = ["Engine", "StepEntry", "generate", "GenerationResult", "Session", "SamplingConfig", "Sampler",
           "load_config", "register_architecture", "register_part", "register_init", "register_route",
           "write_random_model", "build_kernels"]

_LAZY = {
    "Engine": ("engine.engine", "Engine"),
    "StepEntry": ("engine.engine", "StepEntry"),
    "generate": ("engine.generate", "generate"),
    "GenerationResult": ("engine.generate", "GenerationResult"),
    "Session": ("engine.session", "Session"),
    "SamplingConfig": ("sampling.sampler", "SamplingConfig"),
    "Sampler": ("sampling.sampler", "Sampler"),
    "load_config": ("registry", "load_config"),
    "register_architecture": ("registry", "register_architecture"),
    "register_part": ("parts.base", "register_part"),
    "register_init": ("weights.random_init", "register_init"),
    "register_route": ("kernels.routes", "register_route"),
    "write_random_model": ("weights.random_init", "write_random_model"),
}


def __getattr__(name: str):
    if name in _LAZY:
        import importlib
        module, attr = _LAZY[name]
        value = getattr(importlib.import_module(f"{__name__}.{module}"), attr)
        globals()[name] = value
        return value
    raise AttributeError(f"module '{__name__}' has no attribute '{name}'")


def build_kernels(force: bool = True) -> str:
    """Compiles the HIP kernel library for gfx950; returns its path."""
    from .kernels.lib import _build_module
    return _build_module().build(force=force)
