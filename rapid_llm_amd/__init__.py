"""rapid_llm_amd: a small, whole inference engine for one MI355X GPU.

Importing the package touches neither the GPU nor the compiler; the heavy names are
resolved on first use (the reference does the same, rapid_llm/__init__.py:33-61).
"""

__version__ = "0.1.0"

_LAZY = {
    "LLM": ("rapid_llm_amd.engine.llm", "LLM"),
    "Scheduler": ("rapid_llm_amd.engine.scheduler", "Scheduler"),
    "SamplingParams": ("rapid_llm_amd.sampling.params", "SamplingParams"),
    "PositionLogprobs": ("rapid_llm_amd.sampling.logprobs", "PositionLogprobs"),
    "RequestOutput": ("rapid_llm_amd.engine.outputs", "RequestOutput"),
    "CompletionOutput": ("rapid_llm_amd.engine.outputs", "CompletionOutput"),
    "EngineConfig": ("rapid_llm_amd.config.engine_config", "EngineConfig"),
    "ModelRunner": ("rapid_llm_amd.engine.step", "ModelRunner"),
    "StepEntry": ("rapid_llm_amd.engine.step", "StepEntry"),
    "write_random_model": ("rapid_llm_amd.weights.random_init", "write_random_model"),
}


def __getattr__(name):
    try:
        module, attr = _LAZY[name]
    except KeyError:
        raise AttributeError(f"module 'rapid_llm_amd' has no attribute {name!r}") from None
    import importlib

    return getattr(importlib.import_module(module), attr)


__all__ = sorted(_LAZY) + ["__version__"]
