from .engine_config import DTYPES, EngineConfig, dtype_from_name
from .model_config import ConfigError, Qwen25VLConfig, TextConfig, read_config_json
from .registry import (Architecture, RawConfig, architecture_entry, architecture_name, config_to_dict,
                       known_architectures, load_config, register_architecture, resolve_architecture)

__all__ = [
    "ConfigError", "Qwen25VLConfig", "TextConfig", "read_config_json", "EngineConfig", "DTYPES",
    "dtype_from_name", "register_architecture", "resolve_architecture", "known_architectures",
    "Architecture", "RawConfig", "architecture_entry", "architecture_name", "config_to_dict", "load_config",
]
