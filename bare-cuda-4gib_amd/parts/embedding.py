"""Token embedding and output head."""
from __future__ import annotations

from typing import Dict

import torch

from ..csrc import ops
from ..weights.loader import WeightSpec
from .base import Part, register_part
from .linear import linear


class Embedding(Part):
    """x[t, :] = float(table[ids[t], :]) * scale, nothing added; scale 1 unless a design names one
    (reference: engine/kernels/embedding_lookup.cu:16-31)."""
    category = "embedding"
    graph_safe = True     # launches kernels only: may run inside a captured graph

    def __init__(self, vocab_size: int, hidden_size: int, scale: float = 1.0):
        self.vocab_size, self.hidden_size, self.scale = int(vocab_size), int(hidden_size), float(scale)
        self.table = None

    def weight_specs(self) -> Dict[str, WeightSpec]:
        return {"weight": WeightSpec((self.vocab_size, self.hidden_size), kind="table")}

    def bind(self, tensors, rt) -> None:
        self.table = tensors["weight"]

    def forward(self, ctx) -> torch.Tensor:
        return ops.embed_gather(self.table, ctx.token_ids, factor=self.scale)

    def add_to(self, x: torch.Tensor, ctx) -> torch.Tensor:
        """x += the embedding of the step's tokens, in place on the float32 stream."""
        return ops.embed_add(self.table, ctx.token_ids, x, factor=self.scale)

    def beside(self, x: torch.Tensor, ctx, out_dtype: torch.dtype) -> torch.Tensor:
        """[T, 2 H] in ``out_dtype``: the stream's rows, each followed by the embedding of the row's token."""
        return ops.embed_beside(x, self.table, ctx.token_ids, out_dtype, factor=self.scale)


class LMHead(Part):
    """logits = h W^T in float32 (reference: engine/src/model.cpp:612-615).  If
    ``tied_to`` names the embedding table's tensor and the file has no weight
    of the head's own, the table is used."""
    category = "head"
    graph_safe = True     # launches kernels only: may run inside a captured graph

    def __init__(self, vocab_size: int, hidden_size: int, tied_to=None):
        self.vocab_size, self.hidden_size, self.tied_to = int(vocab_size), int(hidden_size), tied_to
        self.weight = None

    def weight_specs(self) -> Dict[str, WeightSpec]:
        return {"weight": WeightSpec((self.vocab_size, self.hidden_size), optional=self.tied_to is not None)}

    def bind(self, tensors, rt) -> None:
        self.weight = ops.StreamedWeight(tensors["weight"])

    accepts_lazy_norm = True

    def forward(self, h) -> torch.Tensor:
        return linear(h, self.weight, out_dtype=torch.float32)


register_part("embedding", "embedding", Embedding)
register_part("head", "lm_head", LMHead)
