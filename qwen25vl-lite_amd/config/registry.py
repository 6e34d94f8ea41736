"""One registry from an architecture's name to its model.

``config.json`` names the architecture (``architectures[0]``, else ``model_type``).  An
architecture is registered as two functions: ``read_config(raw)`` turns the parsed
``config.json`` into the architecture's own configuration object (it alone knows its keys), and
``build_spec(config)`` turns that into a :class:`~qwen25vl_lite_amd.models.spec.ModelSpec`: the
list of layers, the parts each is made of, the order in which they run and the checkpoint names
of their tensors.  Everything that starts from a model folder (:func:`load_config`) looks the
name up first and lets the entry read the rest, so nothing outside an architecture's own module
knows its keys.  The reference has no registry (its model class is fixed in code, reference
src/qwen25vl_lite/model.py:76-88); this is where another architecture is added.
"""

from __future__ import annotations

import json
import os
from dataclasses import dataclass
from typing import Any, Callable, Dict, List, Optional

__all__ = ["Architecture", "RawConfig", "register_architecture", "resolve_architecture", "known_architectures",
           "architecture_entry", "architecture_name", "load_config", "config_to_dict"]


class RawConfig:
    """The configuration of an architecture that registers no reader of its own: the keys of
    ``config.json`` as attributes and items, unchanged."""

    def __init__(self, raw: Dict[str, Any]):
        self.raw = dict(raw)

    @property
    def architecture(self) -> str:
        return architecture_name(self.raw)

    def __getattr__(self, key: str):
        try:
            return self.__dict__["raw"][key]
        except KeyError:
            raise AttributeError(f"config.json has no key {key!r}") from None

    def __getitem__(self, key: str):
        return self.raw[key]

    def get(self, key: str, default=None):
        return self.raw.get(key, default)

    def to_dict(self) -> Dict[str, Any]:
        return dict(self.raw)


@dataclass(frozen=True)
class Architecture:
    name: str
    build_spec: Callable[[Any], Any]
    read_config: Callable[[Dict[str, Any]], Any] = RawConfig


_ARCHITECTURES: Dict[str, Architecture] = {}


def register_architecture(name: str, build_spec: Callable, read_config: Optional[Callable] = None, *,
                          replace: bool = False) -> None:
    """Register an architecture: ``build_spec(config) -> ModelSpec`` and, if its configuration
    is more than the raw keys, ``read_config(raw dict) -> config`` (which validates them)."""
    if name in _ARCHITECTURES and not replace:
        raise ValueError(f"architecture {name!r} is already registered")
    _ARCHITECTURES[name] = Architecture(name, build_spec, read_config or RawConfig)


def known_architectures() -> List[str]:
    return sorted(_ARCHITECTURES)


def architecture_entry(name: str) -> Architecture:
    try:
        return _ARCHITECTURES[name]
    except KeyError:
        raise KeyError(
            f"architecture {name!r} is not registered; known: {known_architectures()}") from None


def resolve_architecture(name: str) -> Callable:
    """``build_spec`` of the named architecture."""
    return architecture_entry(name).build_spec


def architecture_name(raw: Dict[str, Any]) -> str:
    """The registry key a ``config.json`` names: ``architectures[0]``, else ``model_type``."""
    archs = raw.get("architectures") or ()
    if archs:
        return str(archs[0])
    if raw.get("model_type"):
        return str(raw["model_type"])
    raise ValueError("config.json names no architecture (neither 'architectures' nor 'model_type')")


def load_config(source) -> Any:
    """The configuration object of a model: ``source`` is a model folder, a path to a
    ``config.json``, or the parsed dictionary.  The architecture named in it reads it."""
    if isinstance(source, dict):
        raw, where = source, None
    else:
        path = source if str(source).endswith(".json") else os.path.join(source, "config.json")
        if not os.path.isfile(path):
            raise FileNotFoundError(
                f"no config.json under {source!r}; point --model at a folder that holds config.json "
                "and model.safetensors")
        with open(path, "r", encoding="utf-8") as fh:
            raw = json.load(fh)
        if not isinstance(raw, dict):
            raise ValueError(f"{path} does not hold a JSON object")
        where = os.path.abspath(os.path.dirname(path))
    config = architecture_entry(architecture_name(raw)).read_config(raw)
    if where is not None:
        try:
            object.__setattr__(config, "name_or_path", where)
        except (AttributeError, TypeError):
            pass
    return config


def config_to_dict(config) -> Dict[str, Any]:
    """What :func:`load_config` reads back as the same configuration."""
    if isinstance(config, dict):
        return dict(config)
    return config.to_dict()
