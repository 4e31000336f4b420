"""An MI355X-native inference engine for the GPT-2-style decoder of mini-gpt-inference."""

from .config.engine_config import EngineConfig, SamplingParams
from .engine.request import Request, RequestOutput

__all__ = ["EngineConfig", "SamplingParams", "GPTConfig", "Request", "RequestOutput", "LLMEngine"]


def __getattr__(name):
    if name == "LLMEngine":   # imported late: it needs torch and the native libraries
        from .engine.llm_engine import LLMEngine
        return LLMEngine
    if name == "GPTConfig":   # the one architecture's configuration class lives in its module under models/
        from .models.gpt2_mini import GPTConfig
        return GPTConfig
    raise AttributeError(name)
