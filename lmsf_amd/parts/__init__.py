"""Parts a model is put together from. Importing this package registers the built-in kinds."""
from .base import (Block, CacheBinding, CacheSpec, FeedForward, LayerSpec, Mixer, ModelSpec, Norm, Part,
                   PartSpec, PositionEncoding, Runtime, ScheduleEntry, StateSpec, TensorDecl, build_part,
                   part_class, register_part, unregister_part)
from . import attention, block, embedding, mlp, norm, rotary  # noqa: F401  (registration)
from .linear import FusedLinear, Linear

__all__ = ["Block", "CacheBinding", "CacheSpec", "FeedForward", "LayerSpec", "Mixer", "ModelSpec", "Norm", "Part",
           "PartSpec", "PositionEncoding", "Runtime", "ScheduleEntry", "StateSpec", "TensorDecl", "build_part",
           "part_class", "register_part", "unregister_part", "FusedLinear", "Linear"]
