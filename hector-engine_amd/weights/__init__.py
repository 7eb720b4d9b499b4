"""Weights: safetensors by tensor name, and the random-weights mode."""
from .loader import check_against, load_tensors, run_dtype_of
from .random_init import random_tensors, register_init, write_random_model
from .safetensors_io import SafetensorsFile, WeightsError, open_model_files, write_safetensors
