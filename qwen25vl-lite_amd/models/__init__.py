"""Model specs and the generic decoder.  Importing the package registers the architectures."""

from . import qwen25vl_text  # noqa: F401  (registration)
from .decoder import DecoderModel
from .spec import LayerSpec, ModelSpec, RunEntry

__all__ = ["DecoderModel", "LayerSpec", "ModelSpec", "RunEntry", "build_model"]


def build_model(config, dtype=None, device="cuda:0", *, architecture=None) -> DecoderModel:
    """The model the configuration's architecture name stands for, without weights
    (reference model.py:232-243).  ``config`` is what :func:`~qwen25vl_lite_amd.config.load_config`
    returns (it carries ``architecture``), or any object its architecture's ``build_spec`` takes
    together with the ``architecture`` name."""
    import torch

    from ..config.registry import resolve_architecture

    spec = resolve_architecture(architecture or config.architecture)(config)
    return DecoderModel(spec, dtype or torch.float32, device)
