"""The one registry from an architecture's name (config.json `architectures[0]`)
to its typed configuration and its model description.

An architecture registers `(config class, spec builder)`; the spec builder
turns the typed configuration into a :class:`ModelSpec` - data only - and the
generic :class:`DecoderModel` assembles the parts from it. The reference keeps
runtime registries of the same spirit for dtypes, ops and kernels
(src/dtype.hpp:73-99, src/optype.hpp:60-83) and names architectures in a table
(src/hnf_loader.hpp:128-138).
"""
from __future__ import annotations

from typing import Callable

from .config.base import ConfigError, ModelConfig, architecture_name, load_config_dict
from .parts.base import BuildEnv, ModelSpec

_architectures: dict[str, tuple[type, Callable[[ModelConfig], ModelSpec]]] = {}


def register_architecture(name: str, config_cls: type, spec_builder: Callable[[ModelConfig], ModelSpec]) -> None:
    _architectures[name] = (config_cls, spec_builder)


def registered_architectures() -> list[str]:
    return sorted(_architectures)


def _lookup(name: str):
    from . import architectures  # noqa: F401  (registers the built-in architecture)
    try:
        return _architectures[name]
    except KeyError:
        raise ConfigError(f"architecture '{name}' is not registered; registered: "
                          f"{registered_architectures()}") from None


def config_from_dict(data: dict) -> ModelConfig:
    config_cls, _ = _lookup(architecture_name(data))
    return config_cls.from_dict(data)


def load_config(model_dir: str) -> ModelConfig:
    return config_from_dict(load_config_dict(model_dir))


def model_spec(config: ModelConfig) -> ModelSpec:
    _, builder = _lookup(config.architecture)
    return builder(config)


def build_model(config: ModelConfig, env: BuildEnv):
    from .engine.model import DecoderModel
    return DecoderModel(model_spec(config), env)
