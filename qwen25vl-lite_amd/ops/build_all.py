"""Compile every kernel library the package can ask for."""

from __future__ import annotations

import os
from typing import List

from .library import build_library

__all__ = ["LIBRARIES", "build_everything"]

# (source stem, -D options)
LIBRARIES = [
    ("elementwise", {}),
    ("attention_generic", {}),
    ("gemm_f32", {}),
    ("sample", {}),
    ("gemm_resident", {}),
    ("gemm_resident", {"RK": 4}),
    ("gemm_split", {}),
    ("peaks", {}),
    # the matrix-core attention is compiled per head size; these are the sizes the tests and the
    # benchmark use, any other multiple of 16 is compiled at its first use
    ("attention_mfma", {"HD": 128}),
    ("attention_mfma", {"HD": 16}),
    ("attention_mfma", {"HD": 48}),
    ("attention_mfma", {"HD": 80}),
    ("attention_mfma", {"HD": 256}),
    ("attention_mfma", {"HD": 32}),
    ("attention_mfma", {"HD": 64}),
    ("attention_mfma", {"HD": 96}),
    ("attention_mfma", {"HD": 112}),
    # the kind whose waves carry three column tiles (long prompts)
    ("attention_mfma", {"HD": 128, "BLK_CT": 3}),
    ("attention_mfma", {"HD": 48, "BLK_CT": 3}),
]


def build_everything(force: bool = False, quiet: bool = False) -> List[str]:
    built = [build_library(stem, defines, force=force, quiet=quiet) for stem, defines in LIBRARIES]
    # libraries of sources that have changed since are of no use to anyone
    keep = {os.path.basename(p) for p in built}
    for directory in {os.path.dirname(p) for p in built}:
        for name in os.listdir(directory):
            if name.endswith(".so") and name not in keep:
                os.remove(os.path.join(directory, name))
    return built
