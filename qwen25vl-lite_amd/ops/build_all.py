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
    ("gemm_skinny", {}),
    # the matrix-core attention is compiled per head size; these are the sizes the tests and the
    # benchmark use, any other multiple of 16 is compiled at its first use
    ("attention_mfma", {"HD": 128}),
    ("attention_mfma", {"HD": 16}),
    ("attention_mfma", {"HD": 48}),
    ("attention_mfma", {"HD": 80}),
]


def build_everything(force: bool = False, quiet: bool = False) -> List[str]:
    return [build_library(stem, defines, force=force, quiet=quiet) for stem, defines in LIBRARIES]
