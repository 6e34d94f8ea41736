"""RMSNorm (reference src/qwen25vl_lite/layers.py:14-31)."""

from __future__ import annotations

from typing import Dict, Optional

import torch

from ..ops import kernels, skinny
from ..ops.linear import NormedRows
from .base import Norm, ParamSpec, ResidualStream, register_part

__all__ = ["RMSNorm"]


class RMSNorm(Norm):
    """``x * rsqrt(mean(x^2) + eps) * weight`` with the statistics in float32 and ``eps``
    inside the root; the weight is used as stored (not ``1 + weight``).

    params: ``size`` (row width), ``eps``.
    """

    graph_safe = True

    def __init__(self, params, dtype, device):
        super().__init__(dtype, device)
        self.size = int(params["size"])
        self.eps = float(params["eps"])
        self.weight: Optional[torch.Tensor] = None

    def param_specs(self) -> Dict[str, ParamSpec]:
        return {"weight": ParamSpec((self.size,), "vector", init="around_one")}

    def load(self, tensors):
        self.weight = tensors["weight"]

    def forward(self, stream: ResidualStream, rows: Optional[torch.Tensor] = None, lazy: bool = False):
        if (lazy and rows is None and stream.pending is None and self.dtype == torch.bfloat16
                and self.size % 8 == 0 and skinny.folds_norm(stream.h.shape[0], self.size, stream.h.device)):
            # a decode step: the product that follows computes the norm on the way
            return NormedRows(stream.h, self.weight, self.eps, self.dtype)
        out = kernels.add_rmsnorm(stream.h, stream.pending, self.weight, self.eps, self.dtype, rows=rows)
        if rows is None:
            stream.pending = None  # folded into h
        return out


register_part("norm", "rms_norm", RMSNorm)
