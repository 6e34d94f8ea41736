"""SwiGLU feed-forward (reference src/qwen25vl_lite/text.py:56-66)."""

from __future__ import annotations

from typing import Dict, Optional

import torch

from ..ops import kernels
from ..ops.linear import linear
from .base import FeedForward, ParamSpec, StepContext, register_part

__all__ = ["SwiGLU"]


class SwiGLU(FeedForward):
    """``down(silu(gate(x)) * up(x))`` without biases.

    params: ``hidden_size``, ``intermediate_size``.
    """

    graph_safe = True

    def __init__(self, params, dtype, device):
        super().__init__(dtype, device)
        self.hidden = int(params["hidden_size"])
        self.inter = int(params["intermediate_size"])
        self.w_gate_up: Optional[torch.Tensor] = None
        self.w_down: Optional[torch.Tensor] = None

    def param_specs(self) -> Dict[str, ParamSpec]:
        return {
            "gate_proj.weight": ParamSpec((self.inter, self.hidden)),
            "up_proj.weight": ParamSpec((self.inter, self.hidden)),
            "down_proj.weight": ParamSpec((self.hidden, self.inter)),
        }

    def load(self, tensors):
        # gate and up share their input: one product of [2 I, H], gate rows first.
        self.w_gate_up = torch.cat([tensors["gate_proj.weight"], tensors["up_proj.weight"]], dim=0).contiguous()
        self.w_down = tensors["down_proj.weight"]

    def named_weights(self) -> Dict[str, torch.Tensor]:
        return {"gate_proj.weight": self.w_gate_up[:self.inter], "up_proj.weight": self.w_gate_up[self.inter:],
                "down_proj.weight": self.w_down}

    def forward(self, x: torch.Tensor, step: StepContext) -> torch.Tensor:
        gate_up = linear(x, self.w_gate_up)
        return linear(kernels.swiglu(gate_up), self.w_down, out_dtype=torch.float32, allow_slabs=True)


register_part("ffn", "swiglu", SwiGLU)
