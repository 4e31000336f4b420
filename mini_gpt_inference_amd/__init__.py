"""An MI355X-native inference engine for the GPT-2-style decoder of mini-gpt-inference."""

from .config.engine_config import EngineConfig, SamplingParams
from .config.model_config import GPTConfig
from .engine.request import Request, RequestOutput

__all__ = ["EngineConfig", "SamplingParams", "GPTConfig", "Request", "RequestOutput", "LLMEngine"]


def __getattr__(name):
    if name == "LLMEngine":   # imported late: it needs torch and the native libraries
        from .engine.llm_engine import LLMEngine
        return LLMEngine
    raise AttributeError(name)
