"""An LLM inference engine for one AMD Instinct MI355X (gfx950): Llama dense decoder.

``LLMEngine`` and ``SamplingParams`` are exported lazily, so that importing a
subpackage (configuration, cache manager, scheduler) does not pull in torch
extensions (the reference exports the same two names the same way,
inference_engine/__init__.py:1-9).
"""

__version__ = "0.1.0"


def __getattr__(name):
    if name == "LLMEngine":
        from .engine.llm_engine import LLMEngine
        return LLMEngine
    if name == "SamplingParams":
        from .sampling.params import SamplingParams
        return SamplingParams
    if name == "EngineConfig":
        from .config.engine_config import EngineConfig
        return EngineConfig
    raise AttributeError(name)
