"""The two ends of the decoder that touch the vocabulary: the token table and the output head
(reference src/qwen25vl_lite/text.py:209-213, 275-279; model.py:84-86 for the tied head)."""

from __future__ import annotations

from typing import Dict, Optional

import torch

from ..ops import kernels
from ..ops.linear import linear
from .base import Embedding, Head, ParamSpec, register_part

__all__ = ["TokenTable", "LinearHead"]


class TokenTable(Embedding):
    """Row ``id`` of a ``[vocab, hidden]`` table, widened to float32.

    params: ``vocab_size``, ``hidden_size``.
    """

    graph_safe = True

    def __init__(self, params, dtype, device):
        super().__init__(dtype, device)
        self.vocab, self.hidden = int(params["vocab_size"]), int(params["hidden_size"])
        self.table: Optional[torch.Tensor] = None

    def param_specs(self) -> Dict[str, ParamSpec]:
        return {"weight": ParamSpec((self.vocab, self.hidden), "table")}

    def load(self, tensors):
        self.table = tensors["weight"]

    def forward(self, token_ids, step):
        return kernels.embed_gather(token_ids, self.table)


class LinearHead(Head):
    """``x @ weight.T`` in float32, ``weight`` being ``[vocab, hidden]`` or the tied token table.

    params: ``vocab_size``, ``hidden_size``.
    """

    graph_safe = True

    def __init__(self, params, dtype, device):
        super().__init__(dtype, device)
        self.vocab, self.hidden = int(params["vocab_size"]), int(params["hidden_size"])
        self.weight: Optional[torch.Tensor] = None

    def param_specs(self) -> Dict[str, ParamSpec]:
        return {"weight": ParamSpec((self.vocab, self.hidden), "matrix")}

    def load(self, tensors):
        self.weight = tensors["weight"]

    def tie(self, embedding):
        if embedding.table is None or tuple(embedding.table.shape) != (self.vocab, self.hidden):
            raise ValueError("a tied head needs the embedding's table of [vocab, hidden]")
        self.weight = embedding.table

    def forward(self, x, step):
        return linear(x, self.weight, out_dtype=torch.float32)


register_part("embedding", "token_table", TokenTable)
register_part("head", "linear", LinearHead)
