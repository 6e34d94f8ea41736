"""Random weights for a configuration and a seed.

The reference package has no such mode (its tests build a library model under a seed and
save it, reference tests/conftest.py:76-86).  Here every tensor is drawn from a generator
seeded by ``(seed, tensor name)``, so a tensor's values do not depend on the order or the
set of tensors drawn.  How a tensor is drawn is its part's word (``ParamSpec.init``): N(0, std)
unless it says otherwise (a norm's weight: 1 + N(0, std)).
"""

from __future__ import annotations

import hashlib
import json
import os
from typing import Dict, Iterator, Optional, Tuple

import torch

from ..config.registry import config_to_dict
from .safetensors_io import write_safetensors

__all__ = ["random_tensors", "write_random_model", "fill_random"]


def _seed_for(seed: int, name: str) -> int:
    digest = hashlib.blake2b(f"{seed}:{name}".encode(), digest_size=8).digest()
    return int.from_bytes(digest, "little") & 0x7FFFFFFFFFFFFFFF


def _draw(name: str, shape, seed: int, std: float, device, dtype: torch.dtype, init: str = "normal") -> torch.Tensor:
    if init in ("zeros", "ones"):
        return torch.full(tuple(shape), float(init == "ones"), dtype=dtype, device=device)
    if init not in ("normal", "around_one"):
        raise ValueError(f"{name}: no rule to draw a tensor with init {init!r}")
    gen = torch.Generator(device=device)
    gen.manual_seed(_seed_for(seed, name))
    t = torch.empty(tuple(shape), dtype=torch.float32, device=device)
    t.normal_(0.0, std, generator=gen)
    if init == "around_one":
        t += 1.0
    return t.to(dtype)


def random_tensors(model, seed: int, std: float = 0.02, *, device="cpu",
                   dtype: Optional[torch.dtype] = None) -> Iterator[Tuple[str, torch.Tensor]]:
    """``(canonical name, tensor)`` for every tensor the model expects (the head too, unless
    the model ties it to the embedding table)."""
    for name, spec in model.expected_tensors().items():
        if name == model.spec.head_name and model.spec.tie_word_embeddings:
            continue
        if spec.role == "int":
            raise ValueError(f"no rule to draw the integer table {name}")
        yield name, _draw(name, spec.shape, seed, std, device, dtype or torch.float32, spec.init)


def write_random_model(config, out_dir: str, seed: int, *, std: float = 0.02,
                       dtype: torch.dtype = torch.bfloat16) -> str:
    """Write a model folder (``config.json``, ``model.safetensors``) with random weights.

    ``config`` is a configuration object of any registered architecture (or the dictionary of
    its ``config.json``).  Tensors are stored in ``dtype`` under the names the architecture's
    spec gives them in a checkpoint (for the Qwen2.5-VL decoder the released checkpoints'
    ``model.language_model.layers...``, ``lm_head.weight``)."""
    from ..config.registry import load_config
    from ..models import build_model

    os.makedirs(out_dir, exist_ok=True)
    if isinstance(config, dict):
        config = load_config(config)
    model = build_model(config, torch.float32, "meta")
    tensors: Dict[str, torch.Tensor] = {}
    for name, t in random_tensors(model, seed, std, dtype=dtype):
        tensors[model.spec.store_name(name)] = t
    with open(os.path.join(out_dir, "config.json"), "w", encoding="utf-8") as fh:
        json.dump(config_to_dict(config), fh, indent=1)
    write_safetensors(os.path.join(out_dir, "model.safetensors"), tensors)
    return out_dir


def fill_random(model, seed: int, std: float = 0.02) -> None:
    """Give a model on the GPU random weights without a file: each tensor is drawn on the
    device (large models need no host copy) and handed to its part."""
    from .loader import kept_dtype

    expected = model.expected_tensors()
    for part, names in model.part_groups():
        tensors = {}
        for local, name in names.items():
            if name == model.spec.head_name and model.spec.tie_word_embeddings:
                continue
            spec = expected[name]
            tensors[local] = _draw(name, spec.shape, seed, std, model.device, kept_dtype(spec.role, model.dtype),
                                   spec.init)
        if tensors:
            model.load_part(part, tensors)
    if model.spec.tie_word_embeddings:
        model.tie_head()
