"""Dispatch to the matrix-core attention kernel (bfloat16, head sizes in steps of 16)."""

from __future__ import annotations

from typing import Optional

import torch

__all__ = ["try_attention"]


def try_attention(q, k_cache, v_cache, block_table, step, num_q_heads: int, window: Optional[int],
                  scale: float) -> Optional[torch.Tensor]:
    """The attention through the matrix-core kernel, or None if it does not take this shape."""
    return None
