"""mini-vllm_amd: a small, whole inference engine for one MI355X GPU.

``LLM`` is the Python entry point (``LLM(model=...).generate(prompts, sampling_params)``),
``EngineConfig`` and ``SamplingParams`` carry its options. Everything heavier is imported when
it is first used.
"""
from .config import ConfigError, EngineConfig, SamplingParams

__version__ = "0.1.0"
__all__ = ["ConfigError", "EngineConfig", "SamplingParams", "LLM", "RequestOutput"]


def __getattr__(name):
    if name in ("LLM", "RequestOutput"):
        from .engine import llm as _llm
        return getattr(_llm, name)
    raise AttributeError(f"module {__name__!r} has no attribute {name!r}")
