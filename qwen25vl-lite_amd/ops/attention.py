"""Choice of the attention kernel for a step."""

from __future__ import annotations

from typing import Optional

import torch

from . import kernels

__all__ = ["paged_attention"]


def paged_attention(q: torch.Tensor, k_cache: torch.Tensor, v_cache: torch.Tensor, block_table: torch.Tensor,
                    step, num_q_heads: int, window: Optional[int], scale: float) -> torch.Tensor:
    """Attention of the step's tokens over their requests' pages.

    bfloat16 with a head size in steps of 16 runs on the matrix cores; everything else
    (float32, other head sizes) runs through the float32-arithmetic kernel.
    """
    if q.dtype == torch.bfloat16:
        from . import attention_mfma
        out = attention_mfma.try_attention(q, k_cache, v_cache, block_table, step, num_q_heads, window, scale)
        if out is not None:
            return out
    return kernels.paged_attention_generic(q, k_cache, v_cache, block_table, step.token_req, step.token_seqpos,
                                           num_q_heads, window, scale)
