"""Dispatch of bfloat16 products with few rows to the hand-written skinny kernel."""

from __future__ import annotations

from typing import Optional

import torch

__all__ = ["try_linear"]


def try_linear(x: torch.Tensor, weight: torch.Tensor, bias: Optional[torch.Tensor],
               out_dtype: Optional[torch.dtype]) -> Optional[torch.Tensor]:
    """The product through the skinny kernel, or None if the shape is not one it takes."""
    return None
