"""Typed configurations read from config.json."""
from .base import ConfigError, ModelConfig, architecture_name, load_config_dict, read_field, read_int_list
from .qwen2 import Qwen2Config
