"""The description of a model as data: its layers, the parts of each, the run list.

An architecture is a function from a parsed configuration to a :class:`ModelSpec`.  The
generic :class:`~qwen25vl_lite_amd.models.decoder.DecoderModel` builds any spec; it never
looks at the architecture's name.
"""

from __future__ import annotations

from dataclasses import dataclass, field
from typing import Callable, List, Optional

from ..parts.base import PartSpec

__all__ = ["LayerSpec", "RunEntry", "ModelSpec"]


@dataclass(frozen=True)
class LayerSpec:
    """One layer: a block part (which names its norms, mixer and feed-forward) and the
    checkpoint prefix of its tensors, e.g. ``layers.3.``."""

    block: PartSpec
    prefix: str


@dataclass(frozen=True)
class RunEntry:
    """One step of the run list: run ``layer``.  ``cache_from`` names an earlier entry of the
    run list whose cache this entry reads instead of writing its own."""

    layer: int
    cache_from: Optional[int] = None


@dataclass
class ModelSpec:
    hidden_size: int
    vocab_size: int
    layers: List[LayerSpec]
    run: List[RunEntry]
    final_norm: PartSpec
    tie_word_embeddings: bool
    position_rows: int = 3
    embed_name: str = "embed_tokens.weight"
    final_norm_prefix: str = "norm."
    head_name: str = "lm_head.weight"
    # checkpoint tensor name -> canonical name, or None for a tensor this model ignores
    map_name: Callable[[str], Optional[str]] = field(default=lambda name: name)
    # canonical name -> the name a written model folder stores the tensor under
    store_name: Callable[[str], str] = field(default=lambda name: name)
    eos_token_id: Optional[int] = None
    # the parts at the two ends; None: a plain token table and a plain linear head of [vocab, hidden].
    # Their tensors go by ``embed_name`` / ``head_name`` with the last component replaced by the part's own names.
    embed: Optional[PartSpec] = None
    head: Optional[PartSpec] = None
