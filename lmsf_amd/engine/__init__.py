from .args import EngineArgs
from .batch import GroupView, StepContext, StepEntry
from .core import EngineCore, load_engine_core, resolve_dtype
from .executor import ModelExecutor, StepError
from .llm_engine import LLM, LLMEngine
from .outputs import CompletionOutput, RequestOutput
from .scheduler import ScheduledSequence, Scheduler, SchedulerConfig, StepPlan
from .sequence import RequestMetrics, Sequence, SequenceState

__all__ = ["EngineArgs", "GroupView", "StepContext", "StepEntry", "EngineCore", "load_engine_core", "resolve_dtype",
           "ModelExecutor", "StepError", "LLM", "LLMEngine", "CompletionOutput", "RequestOutput", "ScheduledSequence",
           "Scheduler", "SchedulerConfig", "StepPlan", "RequestMetrics", "Sequence", "SequenceState"]
