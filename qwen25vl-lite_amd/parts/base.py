"""What a layer is made of: the interfaces of the parts and the data a step hands them.

A part is built from a dictionary of its own sizes and constants and never learns which
model it sits in.  It declares the tensors it needs (by local name and shape), receives
them once, and then transforms activations of a flat batch of tokens.

Kinds of parts and what each must provide:

* ``Norm``: ``forward(stream) -> x``.  Folds the stream's pending addend into the float32
  residual and returns the normalised activations in the run dtype.
* ``Mixer``: ``forward(x, step, slot) -> y`` for ``x`` of ``[N, hidden]``; it may keep keys and
  values in pages (``cache_need()``) and/or a state of fixed size per request
  (``state_need()``), both handed to it through ``slot``.
* ``FeedForward``: ``forward(x, step) -> y``.
  A mixer or feed-forward may add ``y`` into ``step.residual`` (the float32 residual, if the block
  offers it) itself and return None; one that sets ``takes_lazy_norm`` may be handed
  :class:`~qwen25vl_lite_amd.ops.linear.NormedRows` instead of a tensor and passes it to its first
  product, which then computes the norm on the way.
* ``PositionEncoding``: ``rotary_tables(head_dim, device)`` gives the per-frequency inverse
  frequencies and the row of the position tensor each frequency reads.
* ``Block``: ``forward(stream, step, slot)`` arranges two norms, a mixer and a feed-forward.

New kinds are added with :func:`register_part` and named in a model's layer specs.
"""

from __future__ import annotations

from dataclasses import dataclass, field
from typing import Any, Callable, Dict, List, Optional, Sequence, Tuple

import torch

__all__ = [
    "ParamSpec", "PartSpec", "CacheNeed", "StateNeed", "LayerSlot", "GroupStep", "StepContext", "ResidualStream",
    "Part", "Norm", "Mixer", "FeedForward", "PositionEncoding", "Block", "register_part", "build_part",
    "known_parts", "Embedding", "Head",
]


@dataclass(frozen=True)
class ParamSpec:
    """A tensor a part needs.  ``role`` decides how it is kept on the device:
    ``"matrix"`` and ``"table"`` in the run dtype (bfloat16 or float32), ``"vector"`` in
    float32 (norm weights, biases: they enter float32 arithmetic), ``"int"`` as int32.
    ``init`` says how the random-weights mode draws it: ``"normal"`` N(0, std),
    ``"around_one"`` 1 + N(0, std) (a gain), ``"zeros"``, ``"ones"``."""

    shape: Tuple[int, ...]
    role: str = "matrix"
    init: str = "normal"


@dataclass(frozen=True)
class PartSpec:
    """A part named by its registered kind, with its sizes and constants."""

    kind: str
    params: Dict[str, Any] = field(default_factory=dict)


@dataclass(frozen=True)
class CacheNeed:
    """Keys and values a mixer keeps per token.  ``window`` None: all keys stay; a number:
    only the last ``window`` keys are read, older pages may be given back."""

    num_kv_heads: int
    head_dim: int
    window: Optional[int] = None


@dataclass(frozen=True)
class StateNeed:
    """A state of fixed size a mixer keeps per request (zeroed when a request starts)."""

    shape: Tuple[int, ...]
    dtype: torch.dtype = torch.float32


@dataclass
class LayerSlot:
    """What one entry of the run list owns in the cache: its group and cache layer, whether
    it writes keys and values (an entry that reads another's cache does not), and its state."""

    group: Optional[int] = None
    k_cache: Optional[torch.Tensor] = None  # [pages, nkv, page_size, hd]
    v_cache: Optional[torch.Tensor] = None  # [pages, nkv, hd, page_size]
    writes: bool = True
    state: Optional[torch.Tensor] = None    # [max_num_seqs, *StateNeed.shape]
    # a block with several mixers: each one's slot under the mixer's sub-part name (this slot is
    # the first of them)
    by_part: Dict[str, "LayerSlot"] = field(default_factory=dict)


@dataclass
class GroupStep:
    """A cache group's view of a step: where each token's keys and values go, and the pages
    of each request of the batch (row r, entry i = page of tokens i*page_size ...; -1 = none)."""

    slot_mapping: torch.Tensor  # int32 [N]
    block_table: torch.Tensor   # int32 [R, width]
    page_size: int


@dataclass
class StepContext:
    """One step's batch on the device: N tokens of R requests, each request a contiguous run."""

    num_tokens: int
    num_reqs: int
    token_ids: torch.Tensor     # int32 [N]
    positions: torch.Tensor     # int32 [rows, N]
    token_req: torch.Tensor     # int32 [N]   row of the request in this batch
    token_seqpos: torch.Tensor  # int32 [N]   index of the token in its sequence
    cu_q: torch.Tensor          # int32 [R+1] where each request's run starts
    ctx_len: torch.Tensor       # int32 [R]   tokens of the request in the cache after this step
    req_slots: torch.Tensor     # int32 [R]   the request's state slot
    groups: List[GroupStep]
    logit_rows: torch.Tensor    # int32 [M]
    cu_q_host: Sequence[int] = ()
    ctx_len_host: Sequence[int] = ()
    req_slots_host: Sequence[int] = ()
    max_q_len: int = 0
    max_ctx_len: int = 0
    dtype: torch.dtype = torch.float32
    residual: Optional[torch.Tensor] = None   # set by a block while a part may add its result in place
    derived: Dict[Any, Any] = field(default_factory=dict)   # per-step arrays kernels derive once (tile lists)
    # tensors computed from the step's values once per forward pass (rotation tables): a context
    # that is run again with new values (a captured step) starts each pass with this empty
    per_pass: Dict[Any, Any] = field(default_factory=dict)


@dataclass
class ResidualStream:
    """The residual sum in float32 and an addend that has not been folded in yet.  The next
    norm adds ``pending`` to ``h`` in float32 in the same kernel that normalises."""

    h: torch.Tensor                          # float32 [N, hidden]
    pending: Optional[torch.Tensor] = None   # float32 or run dtype [N, hidden]


class Part:
    """Base of all parts.  ``graph_safe`` says that ``forward`` only launches device work whose
    shape depends on the step's shape alone (no host reads of device data, no host loops over
    the step's values: requests, positions, state rows and pages are found through the step's
    device tensors), so a decode step through it may be captured in a HIP graph and replayed
    with other values in the same buffers.  It promises nothing about running a step twice: a
    mixer may advance its per-request state on every pass (the engine puts the state rows back
    after the passes it runs to warm a new graph up)."""

    graph_safe: bool = False
    takes_lazy_norm: bool = False   # forward accepts NormedRows in place of the normalised tensor

    def __init__(self, dtype: torch.dtype, device: torch.device):
        self.dtype = dtype
        self.device = device

    def param_specs(self) -> Dict[str, ParamSpec]:
        return {}

    def load(self, tensors: Dict[str, torch.Tensor]) -> None:
        """Receive the tensors of :meth:`param_specs`, already on the device in their kept dtype."""

    def sub_parts(self) -> Dict[str, "Part"]:
        return {}


class Norm(Part):
    def forward(self, stream: ResidualStream, rows: Optional[torch.Tensor] = None, lazy: bool = False):
        """Fold ``stream.pending`` into ``stream.h`` and return the normalised rows; with ``lazy`` it
        may return :class:`~qwen25vl_lite_amd.ops.linear.NormedRows` instead of computing them."""
        raise NotImplementedError


class Mixer(Part):
    def cache_need(self) -> Optional[CacheNeed]:
        return None

    def state_need(self) -> Optional[StateNeed]:
        return None

    def forward(self, x: torch.Tensor, step: StepContext, slot: LayerSlot) -> torch.Tensor:
        raise NotImplementedError


class FeedForward(Part):
    def forward(self, x: torch.Tensor, step: StepContext) -> torch.Tensor:
        raise NotImplementedError


class PositionEncoding(Part):
    num_rows: int = 1

    def rotary_tables(self, head_dim: int) -> Tuple[torch.Tensor, torch.Tensor]:
        """``(inv_freq float32 [rot/2], freq_row int32 [rot/2])`` on the device."""
        raise NotImplementedError

    def table_key(self, head_dim: int):
        """A hashable value that is equal for encodings with equal tables: layers whose encodings
        agree share what a step derives from the tables.  Default: this instance only."""
        return (id(self), head_dim)


class Block(Part):
    def forward(self, stream: ResidualStream, step: StepContext, slot: LayerSlot) -> ResidualStream:
        raise NotImplementedError


class Embedding(Part):
    """Token ids to the start of the residual sum.  ``table`` is the tensor a tied head shares."""

    table: Optional[torch.Tensor] = None

    def forward(self, token_ids: torch.Tensor, step: StepContext) -> torch.Tensor:
        """int32 ``[N]`` -> float32 ``[N, hidden]``."""
        raise NotImplementedError


class Head(Part):
    """Normalised rows to logits."""

    def forward(self, x, step: StepContext) -> torch.Tensor:
        """``[rows, hidden]`` -> float32 ``[rows, vocab]``."""
        raise NotImplementedError

    def tie(self, embedding: Embedding) -> None:
        """Use the embedding's table instead of a tensor of its own (a model that ties the two)."""
        raise NotImplementedError


_REGISTRY: Dict[str, Dict[str, Callable[..., Part]]] = {
    "norm": {}, "mixer": {}, "ffn": {}, "position": {}, "block": {}, "embedding": {}, "head": {},
}


def register_part(category: str, kind: str, factory: Callable[..., Part], *, replace: bool = False) -> None:
    """Register ``factory(params, dtype, device) -> Part`` under ``category``/``kind``."""
    if category not in _REGISTRY:
        raise KeyError(f"unknown part category {category!r}; known: {sorted(_REGISTRY)}")
    if kind in _REGISTRY[category] and not replace:
        raise ValueError(f"{category} part {kind!r} is already registered")
    _REGISTRY[category][kind] = factory


def known_parts(category: str) -> List[str]:
    return sorted(_REGISTRY[category])


def build_part(category: str, spec: PartSpec, dtype: torch.dtype, device: torch.device) -> Part:
    try:
        factory = _REGISTRY[category][spec.kind]
    except KeyError:
        raise KeyError(f"no {category} part of kind {spec.kind!r}; known: {known_parts(category)}") from None
    return factory(dict(spec.params), dtype, device)
