from .model_config import ConfigError, LlamaConfig, RopeScaling, read_config_json
from .engine_config import EngineConfig, resolve_dtype
from .registry import (
    Architecture, UnknownArchitecture, architecture_of, get_architecture,
    known_architectures, register_architecture, unregister_architecture,
)
from .presets import PRESETS, preset

__all__ = [
    "ConfigError", "LlamaConfig", "RopeScaling", "read_config_json",
    "EngineConfig", "resolve_dtype",
    "Architecture", "UnknownArchitecture", "architecture_of", "get_architecture",
    "known_architectures", "register_architecture", "unregister_architecture",
    "PRESETS", "preset",
]
