"""A single-GPU inference engine for Qwen3 dense on AMD MI355X (gfx950).

Public names follow the reference's (ullm/__init__.py:1-17)."""
from .config.engine_config import EngineConfig
from .engine.request import FinishReason
from .sampling.params import SamplingParams

__all__ = ["LLM", "EngineConfig", "SamplingParams", "FinishReason", "GenerateOutput", "RequestOutput"]


def __getattr__(name):
    # the entry point pulls in torch and the kernels; configuration and parameters do not need them
    if name in ("LLM", "GenerateOutput", "RequestOutput"):
        from . import llm
        return getattr(llm, name)
    raise AttributeError(name)
