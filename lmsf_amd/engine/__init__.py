from .batch import GroupView, StepContext, StepEntry
from .core import EngineCore, load_engine_core, resolve_dtype
from .executor import ModelExecutor, StepError

__all__ = ["GroupView", "StepContext", "StepEntry", "EngineCore", "load_engine_core", "resolve_dtype",
           "ModelExecutor", "StepError"]
