"""Model specs and the generic decoder.  Importing the package registers the architectures."""

from . import qwen25vl_text  # noqa: F401  (registration)
from .decoder import DecoderModel
from .spec import LayerSpec, ModelSpec, RunEntry

__all__ = ["DecoderModel", "LayerSpec", "ModelSpec", "RunEntry", "build_model"]


def build_model(config, dtype=None, device="cuda:0") -> DecoderModel:
    """The model the configuration's architecture name stands for, without weights
    (reference model.py:232-243)."""
    import torch

    from ..config.registry import resolve_architecture

    spec = resolve_architecture(config.architecture)(config)
    return DecoderModel(spec, dtype or torch.float32, device)
