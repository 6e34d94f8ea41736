"""One registry from an architecture's name to its model.

``config.json`` names the architecture (``architectures[0]``, else ``model_type``).  An
architecture is registered as a function from the parsed configuration to a
:class:`~qwen25vl_lite_amd.models.spec.ModelSpec`: the list of layers, the parts each is
made of, the order in which they run and the checkpoint names of their tensors.  The
reference has no registry (its model class is fixed in code, reference
src/qwen25vl_lite/model.py:76-88); this is where another architecture is added.
"""

from __future__ import annotations

from typing import Callable, Dict, List

__all__ = ["register_architecture", "resolve_architecture", "known_architectures"]

_ARCHITECTURES: Dict[str, Callable] = {}


def register_architecture(name: str, build_spec: Callable, *, replace: bool = False) -> None:
    """Register ``build_spec(config) -> ModelSpec`` under an architecture name."""
    if name in _ARCHITECTURES and not replace:
        raise ValueError(f"architecture {name!r} is already registered")
    _ARCHITECTURES[name] = build_spec


def known_architectures() -> List[str]:
    return sorted(_ARCHITECTURES)


def resolve_architecture(name: str) -> Callable:
    try:
        return _ARCHITECTURES[name]
    except KeyError:
        raise KeyError(
            f"architecture {name!r} is not registered; known: {known_architectures()}") from None
