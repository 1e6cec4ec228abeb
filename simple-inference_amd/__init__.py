"""An LLM inference engine for one AMD Instinct MI355X: from a request's tokens to its next token."""

from . import models  # noqa: F401  (registers the architectures)
from .config import EngineConfig, LlamaConfig, preset, register_architecture
from .engine import Engine, Request, RequestState
from .sampling import SamplingParams

__all__ = ["EngineConfig", "LlamaConfig", "preset", "register_architecture", "Engine", "Request",
           "RequestState", "SamplingParams"]
