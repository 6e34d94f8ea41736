from .engine_config import DTYPES, EngineConfig, dtype_from_name
from .model_config import ConfigError, Qwen25VLConfig, TextConfig, read_config_json
from .registry import known_architectures, register_architecture, resolve_architecture

__all__ = [
    "ConfigError", "Qwen25VLConfig", "TextConfig", "read_config_json", "EngineConfig", "DTYPES",
    "dtype_from_name", "register_architecture", "resolve_architecture", "known_architectures",
]
