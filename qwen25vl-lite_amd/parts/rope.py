"""Rotary position encodings as tables for the rotation kernel.

The kernel rotates the pair ``(f, f + rot/2)`` of every head by the angle
``float32(position[freq_row[f]]) * inv_freq[f]``.  A position encoding is therefore a choice
of ``inv_freq`` and ``freq_row``:

* MRoPE (reference src/qwen25vl_lite/rope.py:26-33, 48-96): ``inv_freq[f] = theta^(-2f/hd)``;
  the three section counts, repeated as a list over both halves of the head, give frequency
  ``f`` the row 0, 1 or 2 (t, h, w) according to the section it falls in.
* Plain 1-D RoPE: every frequency reads row 0; ``rotary_dim`` below the head size leaves the
  remaining channels unrotated.
"""

from __future__ import annotations

from typing import Tuple

import torch

from .base import PositionEncoding, register_part

__all__ = ["MRoPE", "RoPE1D", "inverse_frequencies"]


def inverse_frequencies(rotary_dim: int, theta: float) -> torch.Tensor:
    """``1 / theta^(2f / rotary_dim)`` in float32, as the reference builds it (rope.py:32-33)."""
    idx = torch.arange(0, rotary_dim, 2, dtype=torch.float32)
    return 1.0 / (float(theta) ** (idx / rotary_dim))


class MRoPE(PositionEncoding):
    """params: ``theta``, ``sections`` (three counts adding up to half the head size)."""

    num_rows = 3

    graph_safe = True

    def __init__(self, params, dtype, device):
        super().__init__(dtype, device)
        self.theta = float(params["theta"])
        self.sections = tuple(int(s) for s in params["sections"])
        if len(self.sections) != 3:
            raise ValueError("MRoPE takes three section counts (t, h, w)")
        self._tables = {}

    def table_key(self, head_dim: int):
        return ("mrope", self.theta, self.sections, head_dim)

    def rotary_tables(self, head_dim: int) -> Tuple[torch.Tensor, torch.Tensor]:
        if head_dim not in self._tables:
            half = head_dim // 2
            if sum(self.sections) != half:
                # reference rope.py:89-93
                raise ValueError(f"mrope sections {self.sections} do not cover half the head size {half}")
            rows = []
            for row, count in enumerate(self.sections):
                rows += [row] * count
            self._tables[head_dim] = (
                inverse_frequencies(head_dim, self.theta).to(self.device),
                torch.tensor(rows, dtype=torch.int32, device=self.device),
            )
        return self._tables[head_dim]


class RoPE1D(PositionEncoding):
    """params: ``theta``, optional ``rotary_dim`` (default: the whole head)."""

    num_rows = 1

    graph_safe = True

    def __init__(self, params, dtype, device):
        super().__init__(dtype, device)
        self.theta = float(params["theta"])
        self.rotary_dim = params.get("rotary_dim")
        self._tables = {}

    def table_key(self, head_dim: int):
        return ("rope", self.theta, self.rotary_dim, head_dim)

    def rotary_tables(self, head_dim: int) -> Tuple[torch.Tensor, torch.Tensor]:
        if head_dim not in self._tables:
            rot = int(self.rotary_dim) if self.rotary_dim is not None else head_dim
            if rot % 2 or rot > head_dim:
                raise ValueError(f"rotary_dim {rot} must be even and at most the head size {head_dim}")
            self._tables[head_dim] = (
                inverse_frequencies(rot, self.theta).to(self.device),
                torch.zeros(rot // 2, dtype=torch.int32, device=self.device),
            )
        return self._tables[head_dim]


register_part("position", "mrope", MRoPE)
register_part("position", "rope", RoPE1D)
