"""Matrix products of the step: ``x @ weight.T`` for ``weight`` as a Linear stores it.

float32 runs through the hand-written FMA kernel (true 32-bit, fixed summation order).
bfloat16 uses the hand-written skinny kernel for the few rows of a decode step and the
vendor library's matrix product otherwise, which is also what the reference's engine uses
for its projections (reference src/qwen25vl_lite/text.py:61-66, 80-90).
"""

from __future__ import annotations

from typing import Optional

import torch

from . import kernels

__all__ = ["linear"]


def linear(x: torch.Tensor, weight: torch.Tensor, bias: Optional[torch.Tensor] = None,
           out_dtype: Optional[torch.dtype] = None, allow_slabs: bool = False) -> torch.Tensor:
    """``x [M, K] @ weight[N, K].T (+ bias)``.  ``out_dtype`` float32 is allowed for
    bfloat16 operands (the products are accumulated in float32 either way).  With ``allow_slabs``
    the result may come as partial sums ``[S, M, N]`` whose consumer adds them up (the residual
    add + norm kernel does); without it the result is always ``[M, N]``."""
    if not x.is_cuda:
        raise kernels.KernelError("linear has no CPU path: its tensors must be on the GPU")
    if x.dtype == torch.float32:
        return kernels.gemm_f32(x, weight, bias)
    if x.dtype != torch.bfloat16 or weight.dtype != torch.bfloat16:
        raise kernels.KernelError(f"linear: operands {x.dtype}/{weight.dtype} are not built")
    from . import skinny
    out = skinny.try_linear(x, weight, bias, out_dtype, allow_slabs)
    if out is not None:
        return out
    if out_dtype == torch.float32:
        y = torch.mm(x, weight.t(), out_dtype=torch.float32)  # float32 accumulator written out unrounded
    else:
        y = torch.nn.functional.linear(x, weight)
    if bias is not None:
        y = y + bias.to(y.dtype)
    return y
