"""The arrangement of parts in a layer (reference src/qwen25vl_lite/text.py:188-206)."""

from __future__ import annotations

from typing import Dict

from .base import Block, LayerSlot, Part, PartSpec, ResidualStream, StepContext, build_part, register_part

__all__ = ["PreNormBlock"]


class PreNormBlock(Block):
    """``h += mixer(norm1(h)); h += ffn(norm2(h))``.

    params: ``norm1``, ``mixer``, ``norm2``, ``ffn`` (:class:`PartSpec` each) and ``names``,
    the checkpoint sub-name of each of the four.  Each sum into ``h`` happens in float32,
    inside the following norm's kernel or, in a decode step, inside the product that ends the
    mixer or the feed-forward.
    """

    graph_safe = True

    def __init__(self, params, dtype, device):
        super().__init__(dtype, device)
        self.norm1 = build_part("norm", params["norm1"], dtype, device)
        self.mixer = build_part("mixer", params["mixer"], dtype, device)
        self.norm2 = build_part("norm", params["norm2"], dtype, device)
        self.ffn = build_part("ffn", params["ffn"], dtype, device)
        self.names: Dict[str, str] = dict(params["names"])

    def sub_parts(self) -> Dict[str, Part]:
        return {self.names["norm1"]: self.norm1, self.names["mixer"]: self.mixer,
                self.names["norm2"]: self.norm2, self.names["ffn"]: self.ffn}

    def forward(self, stream: ResidualStream, step: StepContext, slot: LayerSlot) -> ResidualStream:
        x = self.norm1.forward(stream, lazy=self.mixer.takes_lazy_norm)
        step.residual = stream.h            # the mixer may add its result in place and return None
        stream.pending = self.mixer.forward(x, step, slot)
        y = self.norm2.forward(stream, lazy=self.ffn.takes_lazy_norm)
        step.residual = stream.h
        stream.pending = self.ffn.forward(y, step)
        step.residual = None
        return stream


register_part("block", "pre_norm", PreNormBlock)
