"""Typed reading of config.json.

A model configuration is a dataclass whose fields are read from the
architecture's own config.json keys by :func:`read_fields`; nothing that the
file gives is repeated in code. The reference keeps a string->variant map with
typed accessors and defaults (src/hnf_loader.hpp:423-499); here each
architecture has a typed dataclass instead and errors name the key.
"""
from __future__ import annotations

import dataclasses
import json
import os
from typing import Any

REQUIRED = object()


class ConfigError(ValueError):
    """A config.json that cannot be used; the message names the key."""


def _coerce(key: str, value: Any, kind: type) -> Any:
    if kind is bool:
        if isinstance(value, bool):
            return value
        if isinstance(value, int) and value in (0, 1):  # int -> bool as the reference coerces
            return bool(value)
    elif kind is int:
        if isinstance(value, bool):
            pass
        elif isinstance(value, int):
            return value
        elif isinstance(value, float) and value == int(value):
            return int(value)
    elif kind is float:
        if isinstance(value, (int, float)) and not isinstance(value, bool):
            return float(value)
    elif kind is str:
        if isinstance(value, str):
            return value
    raise ConfigError(f"config key '{key}': expected {kind.__name__}, got {value!r}")


def read_field(data: dict, key: str, kind: type, default: Any = REQUIRED) -> Any:
    """data[key] as `kind`; a missing or null key gives the default or an error."""
    value = data.get(key)
    if value is None:
        if default is REQUIRED:
            raise ConfigError(f"config key '{key}' is required")
        return default
    return _coerce(key, value, kind)


def read_int_list(data: dict, key: str, default: Any = REQUIRED) -> list[int] | None:
    """An int or a list of ints (eos_token_id is either)."""
    value = data.get(key)
    if value is None:
        if default is REQUIRED:
            raise ConfigError(f"config key '{key}' is required")
        return default
    if isinstance(value, list):
        return [_coerce(key, v, int) for v in value]
    return [_coerce(key, value, int)]


def load_config_dict(model_dir: str) -> dict:
    path = os.path.join(model_dir, "config.json")
    try:
        with open(path) as f:
            data = json.load(f)
    except FileNotFoundError:
        raise ConfigError(f"{path} not found") from None
    except json.JSONDecodeError as exc:
        raise ConfigError(f"{path}: not valid JSON: {exc}") from None
    if not isinstance(data, dict):
        raise ConfigError(f"{path}: top level must be an object")
    return data


def stop_token_ids(model_dir: str | None, config: "ModelConfig") -> list[int]:
    """The token ids that end a sequence when the caller names none: `eos_token_id` of the
    folder's generation_config.json when that file has the key (an instruction-tuned
    checkpoint lists its end-of-turn id there beside the end-of-text id), else `eos_token_id`
    of config.json, else none. The reference takes the id from the model's own files too
    (src/inference_session.cpp:357)."""
    if model_dir is not None:
        path = os.path.join(model_dir, "generation_config.json")
        if os.path.exists(path):
            try:
                with open(path) as f:
                    data = json.load(f)
            except json.JSONDecodeError as exc:
                raise ConfigError(f"{path}: not valid JSON: {exc}") from None
            if not isinstance(data, dict):
                raise ConfigError(f"{path}: top level must be an object")
            ids = read_int_list(data, "eos_token_id", None)
            if ids is not None:
                return ids
    return list(getattr(config, "eos_token_id", None) or [])


def architecture_name(data: dict) -> str:
    """architectures[0], the name the registry is keyed by."""
    archs = data.get("architectures")
    if isinstance(archs, list) and archs and isinstance(archs[0], str):
        return archs[0]
    raise ConfigError("config key 'architectures' must be a non-empty list of names")


@dataclasses.dataclass
class ModelConfig:
    """Base of every architecture's typed configuration."""

    architecture: str

    @classmethod
    def from_dict(cls, data: dict) -> "ModelConfig":
        raise NotImplementedError

    def to_dict(self) -> dict:
        """The config.json this configuration is read back from."""
        raise NotImplementedError

    def save(self, model_dir: str) -> None:
        os.makedirs(model_dir, exist_ok=True)
        with open(os.path.join(model_dir, "config.json"), "w") as f:
            json.dump(self.to_dict(), f, indent=2)
