"""Attention over the paged cache (reference src/qwen25vl_lite/text.py:69-185).

``q = x Wq^T + bq`` and likewise k, v; queries and keys are rotated by the position encoding;
keys (rotated) and values go into the request's pages; every token attends to the keys of its
request up to itself (``scale * q.k``, softmax in float32, GQA: query head h reads key head
``h // (heads / kv_heads)``), within ``window`` keys if the layer has one; then ``Wo``.
"""

from __future__ import annotations

from typing import Dict, Optional

import torch

from ..ops import kernels, skinny
from ..ops.attention import paged_attention
from ..ops.linear import NormedRows, linear, linear_into
from .base import (CacheNeed, LayerSlot, Mixer, ParamSpec, PartSpec, StepContext, build_part, register_part)

# 33 to 48 rows: the projection cut along its inner size (slabs) and the rotation's kernel behind it beat the
# fused kernel on teams of blocks (7B sizes: a step of 33 rows 4.14 ms against 4.24, of 48 rows 4.34 against 4.39,
# of 64 rows 4.68 against 4.67)
SPLIT_ROWS = (33, 48)

__all__ = ["PagedAttention"]


class PagedAttention(Mixer):
    """params: ``hidden_size``, ``num_heads``, ``num_kv_heads``, ``head_dim``, ``qkv_bias``,
    ``window`` (None: all keys), ``scale`` (None: ``head_dim ** -0.5``, reference text.py:78),
    ``position`` (a :class:`PartSpec` of category ``position``), ``kv_shared`` (True: the layer
    has no key/value projections and reads the cache another layer wrote)."""

    graph_safe = True
    takes_lazy_norm = True

    def __init__(self, params, dtype, device):
        super().__init__(dtype, device)
        self.hidden = int(params["hidden_size"])
        self.nq = int(params["num_heads"])
        self.nkv = int(params["num_kv_heads"])
        self.hd = int(params["head_dim"])
        self.qkv_bias = bool(params.get("qkv_bias", False))
        self.window: Optional[int] = params.get("window")
        scale = params.get("scale")
        self.scale = float(scale) if scale is not None else self.hd ** -0.5
        self.kv_shared = bool(params.get("kv_shared", False))
        if self.nq % self.nkv:
            raise ValueError(f"{self.nq} heads are not a multiple of {self.nkv} key/value heads")
        pos: PartSpec = params["position"]
        self.position = build_part("position", pos, dtype, device)
        self.w_in: Optional[torch.Tensor] = None
        self.b_in: Optional[torch.Tensor] = None
        self.w_out: Optional[torch.Tensor] = None

    def cache_need(self) -> CacheNeed:
        return CacheNeed(self.nkv, self.hd, self.window)

    def param_specs(self) -> Dict[str, ParamSpec]:
        specs = {"q_proj.weight": ParamSpec((self.nq * self.hd, self.hidden))}
        if not self.kv_shared:
            specs["k_proj.weight"] = ParamSpec((self.nkv * self.hd, self.hidden))
            specs["v_proj.weight"] = ParamSpec((self.nkv * self.hd, self.hidden))
        if self.qkv_bias:
            specs["q_proj.bias"] = ParamSpec((self.nq * self.hd,), "vector")
            if not self.kv_shared:
                specs["k_proj.bias"] = ParamSpec((self.nkv * self.hd,), "vector")
                specs["v_proj.bias"] = ParamSpec((self.nkv * self.hd,), "vector")
        specs["o_proj.weight"] = ParamSpec((self.hidden, self.nq * self.hd))
        return specs

    def load(self, tensors):
        names = ["q_proj"] if self.kv_shared else ["q_proj", "k_proj", "v_proj"]
        # One product for q, k and v: the three matrices are stacked by rows.
        self.w_in = torch.cat([tensors[f"{n}.weight"] for n in names], dim=0).contiguous()
        self.b_in = torch.cat([tensors[f"{n}.bias"] for n in names]).contiguous() if self.qkv_bias else None
        self.w_out = tensors["o_proj.weight"]

    def named_weights(self) -> Dict[str, torch.Tensor]:
        """Views of the stacked tensors under their checkpoint names."""
        out, row = {}, 0
        for name, heads in (("q_proj", self.nq), ("k_proj", self.nkv), ("v_proj", self.nkv)):
            if self.kv_shared and name != "q_proj":
                continue
            rows = heads * self.hd
            out[f"{name}.weight"] = self.w_in[row:row + rows]
            if self.b_in is not None:
                out[f"{name}.bias"] = self.b_in[row:row + rows]
            row += rows
        out["o_proj.weight"] = self.w_out
        return out

    def forward(self, x: torch.Tensor, step: StepContext, slot: LayerSlot) -> torch.Tensor:
        if slot.group is None or slot.k_cache is None:
            raise RuntimeError("attention needs a cache slot")
        group = step.groups[slot.group]
        write = slot.writes and not self.kv_shared
        if slot.writes == self.kv_shared:
            raise RuntimeError("a layer without key/value projections must read another layer's cache, "
                               "and a layer with them must write its own")
        inv_freq, freq_row = self.position.rotary_tables(self.hd)
        q = self._project_few_rows(x, step, group, slot, write, inv_freq, freq_row)
        if q is None:
            q = self._project(x, step, group, slot, write, inv_freq, freq_row)
        o = paged_attention(q, slot.k_cache, slot.v_cache, group.block_table, step, self.nq, self.window, self.scale)
        return linear_into(step.residual, o, self.w_out)

    def _project(self, x, step, group, slot, write, inv_freq, freq_row) -> torch.Tensor:
        # Projections are written out in float32 (the accumulator, unrounded): bias, rotation and
        # the residual sum then happen in float32 and each stored value is rounded once.
        m, k = x.shape
        if (SPLIT_ROWS[0] <= m <= SPLIT_ROWS[1] and self.dtype == torch.bfloat16 and isinstance(x, torch.Tensor)
                and x.dtype == torch.bfloat16 and self.hd % 4 == 0 and inv_freq.shape[0] % 4 == 0
                and skinny.takes_split(m, k, self.w_in) and x.stride(1) == 1 and x.stride(0) % 8 == 0
                and x.data_ptr() % 16 == 0):
            qkv = skinny.split_product(self.w_in, x)   # slabs of partial sums: the rotation's kernel adds them
        else:
            qkv = linear(x, self.w_in, out_dtype=torch.float32)
        cs = self._rotation_table(step, inv_freq, freq_row, m)
        return kernels.rope_kv_write(
            qkv, self.b_in, step.positions, inv_freq, freq_row,
            group.slot_mapping if write else None, slot.k_cache if write else None, slot.v_cache if write else None,
            self.nq, self.nkv if write else 0, self.hd, group.page_size, out_dtype=self.dtype, cs=cs)

    def _rotation_table(self, step, inv_freq, freq_row, n: int) -> torch.Tensor:
        """Cosines and sines of the step's angles: computed once per pass and position encoding,
        by the first layer that needs them, and read by every head of every layer."""
        key = ("rope_cs", self.position.table_key(self.hd))
        cs = step.per_pass.get(key)
        if cs is None:
            cs = step.per_pass[key] = kernels.rope_table(step.positions, inv_freq, freq_row, n)
        return cs

    def _project_few_rows(self, x, step, group, slot, write, inv_freq, freq_row) -> Optional[torch.Tensor]:
        """A decode step's few bfloat16 rows: projection, bias, rotation and cache write in one
        kernel (the float32 sums never leave it)."""
        lazy = isinstance(x, NormedRows)
        m, k = x.shape
        if not lazy and SPLIT_ROWS[0] <= m <= SPLIT_ROWS[1]:
            return None
        if self.dtype != torch.bfloat16 or not skinny.takes_qkv_rope(
                m, k, self.w_in, self.hd, inv_freq.shape[0], slot.k_cache.dtype if write else None, norm=lazy):
            return None
        if not lazy and (x.dtype != torch.bfloat16 or x.stride(1) != 1 or x.stride(0) % 8 or x.data_ptr() % 16):
            return None
        cs = self._rotation_table(step, inv_freq, freq_row, m)
        src = dict(h=x.h, norm_weight=x.weight, eps=x.eps) if lazy else dict(x=x)
        return skinny.qkv_rope_product(
            self.w_in, cs, bias=self.b_in, slots=group.slot_mapping if write else None,
            k_cache=slot.k_cache if write else None, v_cache=slot.v_cache if write else None,
            num_q_heads=self.nq, num_kv_heads=self.nkv if write else 0, head_dim=self.hd,
            page_size=group.page_size, **src)


register_part("mixer", "paged_attention", PagedAttention)
