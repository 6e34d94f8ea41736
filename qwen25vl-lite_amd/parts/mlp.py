"""SwiGLU feed-forward (reference src/qwen25vl_lite/text.py:56-66)."""

from __future__ import annotations

from typing import Dict, Optional

import torch

from ..ops.linear import gate_up_swiglu, linear_into
from .base import FeedForward, ParamSpec, StepContext, register_part

__all__ = ["SwiGLU"]


class SwiGLU(FeedForward):
    """``down(silu(gate(x)) * up(x))`` without biases.

    params: ``hidden_size``, ``intermediate_size``.
    """

    graph_safe = True
    takes_lazy_norm = True

    def __init__(self, params, dtype, device):
        super().__init__(dtype, device)
        self.hidden = int(params["hidden_size"])
        self.inter = int(params["intermediate_size"])
        # gate and up rows alternate in groups of 8 where the size allows: a 16-row tile of the
        # product then holds 8 features' gate and up and can apply the activation itself
        self.grouped = self.inter % 8 == 0
        self.w_gate_up: Optional[torch.Tensor] = None
        self.w_down: Optional[torch.Tensor] = None

    def param_specs(self) -> Dict[str, ParamSpec]:
        return {
            "gate_proj.weight": ParamSpec((self.inter, self.hidden)),
            "up_proj.weight": ParamSpec((self.inter, self.hidden)),
            "down_proj.weight": ParamSpec((self.hidden, self.inter)),
        }

    def load(self, tensors):
        # gate and up share their input: one product of [2 I, H]
        gate, up = tensors["gate_proj.weight"], tensors["up_proj.weight"]
        if self.grouped:
            both = torch.stack([gate.view(-1, 8, self.hidden), up.view(-1, 8, self.hidden)], dim=1)
            self.w_gate_up = both.reshape(2 * self.inter, self.hidden).contiguous()
        else:
            self.w_gate_up = torch.cat([gate, up], dim=0).contiguous()
        self.w_down = tensors["down_proj.weight"]

    def named_weights(self) -> Dict[str, torch.Tensor]:
        if self.grouped:
            both = self.w_gate_up.view(-1, 2, 8, self.hidden)
            gate, up = both[:, 0].reshape(self.inter, self.hidden), both[:, 1].reshape(self.inter, self.hidden)
        else:
            gate, up = self.w_gate_up[:self.inter], self.w_gate_up[self.inter:]
        return {"gate_proj.weight": gate, "up_proj.weight": up, "down_proj.weight": self.w_down}

    def forward(self, x, step: StepContext):
        act = gate_up_swiglu(x, self.w_gate_up, self.grouped)
        return linear_into(step.residual if step is not None else None, act, self.w_down)


register_part("ffn", "swiglu", SwiGLU)
