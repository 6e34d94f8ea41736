"""A decoder built from a :class:`ModelSpec`: embedding, the run list of layers, the final
norm and the output head (reference src/qwen25vl_lite/text.py:209-279, model.py:84-86, 200-202).
"""

from __future__ import annotations

from typing import Dict, List, Optional, Tuple

import torch

from ..cache.manager import CacheGroupSpec
from ..parts.base import (Block, CacheNeed, LayerSlot, Mixer, ParamSpec, Part, PartSpec, ResidualStream, StateNeed,
                          StepContext, build_part)
from .spec import ModelSpec

__all__ = ["DecoderModel"]


def _collect(part: Part, prefix: str, out: Dict[str, Tuple[Part, str, ParamSpec]]) -> None:
    for local, spec in part.param_specs().items():
        out[prefix + local] = (part, local, spec)
    for name, sub in part.sub_parts().items():
        _collect(sub, f"{prefix}{name}.", out)


def _prefix_of(name: str) -> str:
    """``"a.b.weight"`` -> ``"a.b."``: where the tensors of the part behind a named tensor go."""
    return name[:name.rfind(".") + 1]


def _mixers_of(block: Part, prefix: str = "") -> List[Tuple[str, Mixer]]:
    """Every mixer inside a block, however deep, with its dotted sub-part name."""
    found: List[Tuple[str, Mixer]] = []
    for name, sub in block.sub_parts().items():
        if isinstance(sub, Mixer):
            found.append((prefix + name, sub))
        else:
            found.extend(_mixers_of(sub, f"{prefix}{name}."))
    return found


class DecoderModel:
    """Holds the parts and runs a step over them.  Tensors arrive through :meth:`load_part`."""

    def __init__(self, spec: ModelSpec, dtype: torch.dtype, device):
        self.spec = spec
        self.dtype = dtype
        self.device = torch.device(device)
        self.blocks: List[Block] = [build_part("block", ls.block, dtype, self.device) for ls in spec.layers]
        self.final_norm = build_part("norm", spec.final_norm, dtype, self.device)
        sizes = {"vocab_size": spec.vocab_size, "hidden_size": spec.hidden_size}
        self.embedding = build_part("embedding", spec.embed or PartSpec("token_table", sizes), dtype, self.device)
        self.head_part = build_part("head", spec.head or PartSpec("linear", sizes), dtype, self.device)
        self._has_weights = False

        # The run list: which cache layer and state every mixer of every entry owns.  The lists
        # below have one element per (run entry, mixer of its block), in run order ("places");
        # entry_places[i] names the places of entry i by the mixer's sub-part name.  A block with
        # one mixer, the usual case, has one place.
        self.group_needs: List[CacheNeed] = []
        self.group_layers: List[int] = []
        self.entry_places: List[Dict[str, int]] = []
        self.entry_group: List[Optional[int]] = []
        self.entry_cache_layer: List[Optional[int]] = []
        self.entry_writes: List[bool] = []
        self.entry_state: List[Optional[StateNeed]] = []
        for i, entry in enumerate(spec.run):
            if not 0 <= entry.layer < len(self.blocks):
                raise ValueError(f"run entry {i} names layer {entry.layer}, which does not exist")
            mixers = _mixers_of(self.blocks[entry.layer])
            if entry.cache_from is not None:
                src = entry.cache_from
                if not 0 <= src < i:
                    raise ValueError(f"run entry {i} must read the cache of an earlier entry that writes one")
                if not any(m.cache_need() is not None for _, m in mixers):
                    raise ValueError(f"run entry {i} reads a cache but its mixer keeps none")
            places: Dict[str, int] = {}
            for name, mixer in mixers:
                need = mixer.cache_need()
                places[name] = len(self.entry_state)
                self.entry_state.append(mixer.state_need())
                if need is None:
                    self.entry_group.append(None)
                    self.entry_cache_layer.append(None)
                    self.entry_writes.append(False)
                    continue
                if entry.cache_from is not None:
                    src_place = self.entry_places[entry.cache_from].get(name)
                    if src_place is None or self.entry_group[src_place] is None or not self.entry_writes[src_place]:
                        raise ValueError(f"run entry {i} must read the cache of an earlier entry that writes one")
                    if self.group_needs[self.entry_group[src_place]] != need:
                        raise ValueError(
                            f"run entry {i} reads the cache of entry {entry.cache_from}, whose shape or window differs")
                    self.entry_group.append(self.entry_group[src_place])
                    self.entry_cache_layer.append(self.entry_cache_layer[src_place])
                    self.entry_writes.append(False)
                    continue
                if need not in self.group_needs:
                    self.group_needs.append(need)
                    self.group_layers.append(0)
                g = self.group_needs.index(need)
                self.entry_group.append(g)
                self.entry_cache_layer.append(self.group_layers[g])
                self.entry_writes.append(True)
                self.group_layers[g] += 1
            self.entry_places.append(places)

        self.params: Dict[str, Tuple[Optional[Part], str, ParamSpec]] = {}
        _collect(self.embedding, _prefix_of(spec.embed_name), self.params)
        for ls, block in zip(spec.layers, self.blocks):
            _collect(block, ls.prefix, self.params)
        _collect(self.final_norm, spec.final_norm_prefix, self.params)
        _collect(self.head_part, _prefix_of(spec.head_name), self.params)
        for name in (spec.embed_name, spec.head_name):
            if name not in self.params:
                raise ValueError(f"the spec names the tensor {name}, which neither end of the model declares")

    # ------------------------------------------------------------------ structure
    @property
    def graph_safe(self) -> bool:
        """True if every part may run under HIP graph capture."""
        def safe(part) -> bool:
            return part.graph_safe and all(safe(s) for s in part.sub_parts().values())
        return all(safe(b) for b in self.blocks) and safe(self.final_norm) and safe(self.embedding) and safe(self.head_part)

    def cache_groups(self) -> List[CacheGroupSpec]:
        return [CacheGroupSpec(need, n) for need, n in zip(self.group_needs, self.group_layers)]

    def expected_tensors(self) -> Dict[str, ParamSpec]:
        """Canonical tensor name -> what is expected under it."""
        return {name: spec for name, (_, _, spec) in self.params.items()}

    def part_groups(self) -> List[Tuple[Optional[Part], Dict[str, str]]]:
        """Tensors grouped by the part that takes them: ``(part, {local: canonical})``."""
        groups: Dict[int, Tuple[Optional[Part], Dict[str, str]]] = {}
        for name, (part, local, _) in self.params.items():
            key = id(part) if part is not None else hash(name)
            groups.setdefault(key, (part, {}))[1][local] = name
        return list(groups.values())

    def load_part(self, part: Part, tensors: Dict[str, torch.Tensor]) -> None:
        part.load(tensors)
        self._has_weights = True

    def tie_head(self) -> None:
        self.head_part.tie(self.embedding)

    @property
    def embed(self) -> Optional[torch.Tensor]:
        """The token table (what a tied head shares)."""
        return self.embedding.table

    @property
    def head(self) -> Optional[torch.Tensor]:
        """The built-in head's matrix (None for a head of another kind)."""
        return getattr(self.head_part, "weight", None)

    def make_slots(self, storage, state_tensors: List[Optional[torch.Tensor]]) -> List[LayerSlot]:
        """One slot per run entry.  ``state_tensors`` has one element per place (see
        ``entry_state``).  The slot of an entry is its first mixer's; a block with several
        mixers finds each one's under the mixer's sub-part name in ``slot.by_part``."""
        def place_slot(p: int) -> LayerSlot:
            g, layer = self.entry_group[p], self.entry_cache_layer[p]
            return LayerSlot(
                group=g,
                k_cache=storage.k[g][layer] if g is not None else None,
                v_cache=storage.v[g][layer] if g is not None else None,
                writes=self.entry_writes[p],
                state=state_tensors[p],
            )

        slots = []
        for places in self.entry_places:
            by_part = {name: place_slot(p) for name, p in places.items()}
            first = next(iter(by_part.values()), LayerSlot(writes=False))
            first.by_part = by_part
            slots.append(first)
        return slots

    # ------------------------------------------------------------------ the step
    def forward(self, step: StepContext, slots: List[LayerSlot]) -> torch.Tensor:
        """Run the step's tokens through the run list; float32 logits ``[M, vocab]`` at
        ``step.logit_rows``."""
        if not self._has_weights:
            raise RuntimeError("the model has no weights yet")
        stream = ResidualStream(self.embedding.forward(step.token_ids, step))
        for entry, slot in zip(self.spec.run, slots):
            stream = self.blocks[entry.layer].forward(stream, step, slot)
        if step.logit_rows.shape[0] == 0:
            return torch.empty((0, self.spec.vocab_size), dtype=torch.float32, device=self.device)
        x = self.final_norm.forward(stream, rows=step.logit_rows)
        return self.head_part.forward(x, step)
