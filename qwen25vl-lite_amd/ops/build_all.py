"""Compile every kernel library the package can ask for."""

from __future__ import annotations

from typing import List

from .library import build_library

__all__ = ["LIBRARIES", "build_everything"]

# (source stem, -D options)
LIBRARIES = [
    ("elementwise", {}),
    ("attention_generic", {}),
    ("gemm_f32", {}),
    ("sample", {}),
]


def build_everything(force: bool = False, quiet: bool = False) -> List[str]:
    return [build_library(stem, defines, force=force, quiet=quiet) for stem, defines in LIBRARIES]
