"""A single-GPU inference engine for the Qwen2.5-VL text decoder on MI355X (gfx950).

The public names follow the reference package (reference src/qwen25vl_lite/__init__.py:30-47):
``Qwen25VLConfig``, ``TextConfig``, ``build_model``, ``load_weights``, ``EngineConfig``,
``ModelRunner``, ``LLMEngine``, ``RequestOutput``, ``SamplingParams``; ``LLM`` wraps them.
"""

from .config import (ConfigError, EngineConfig, Qwen25VLConfig, TextConfig, known_architectures,
                     register_architecture, resolve_architecture)
from .models import DecoderModel, ModelSpec, build_model
from .weights import WeightsError, fill_random, load_weights, write_random_model

__version__ = "0.1.0"

__all__ = [
    "ConfigError", "EngineConfig", "Qwen25VLConfig", "TextConfig", "known_architectures", "register_architecture",
    "resolve_architecture", "DecoderModel", "ModelSpec", "build_model", "WeightsError", "fill_random",
    "load_weights", "write_random_model", "ModelRunner", "LLMEngine", "LLM", "RequestOutput", "SamplingParams",
]


def __getattr__(name):
    # The engine pulls in the kernels; keep `import qwen25vl_lite_amd` light for config-only users.
    if name in ("ModelRunner",):
        from .engine.runner import ModelRunner
        return ModelRunner
    if name in ("LLMEngine", "RequestOutput", "EngineStats"):
        from .engine import scheduler
        return getattr(scheduler, name)
    if name == "LLM":
        from .engine.llm import LLM
        return LLM
    if name == "SamplingParams":
        from .sampling.params import SamplingParams
        return SamplingParams
    raise AttributeError(name)
