"""Parts a layer is put together from, and their registries."""
from . import attention, block, embedding, mlp, norm, rotary  # noqa: F401  (register the built-in parts)
from .base import (Block, BuildEnv, FeedForward, KVNeed, LayerCache, LayerSpec, Mixer, ModelSpec,
                   Norm, Part, PartSpec, PositionEncoding, ResidualStream, ScheduleEntry,
                   StepContext, TensorSpec, build_part, param, register_part, registered)
