"""lmsf_amd: a small, whole LLM inference engine for one MI355X.

    from lmsf_amd import LLM, SamplingParams
    outs = LLM(model="/path/to/model").generate([[1, 2, 3]], SamplingParams(temperature=0.0, max_tokens=16))
"""
__version__ = "0.1.0"

_LAZY = {
    "LLM": "engine", "LLMEngine": "engine", "EngineArgs": "engine", "RequestOutput": "engine",
    "CompletionOutput": "engine", "StepEntry": "engine", "load_engine_core": "engine",
    "SamplingParams": "sampling",
}


def __getattr__(name):
    if name in _LAZY:
        import importlib
        return getattr(importlib.import_module("." + _LAZY[name], __name__), name)
    raise AttributeError("module %r has no attribute %r" % (__name__, name))


__all__ = sorted(_LAZY)
