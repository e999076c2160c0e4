"""Token embedding and output head."""
from __future__ import annotations

from typing import Dict

import torch

from ..csrc import ops
from ..weights.loader import WeightSpec
from .base import Part, register_part
from .linear import linear


class Embedding(Part):
    """x[t, :] = float(table[ids[t], :]); no scaling, nothing added
    (reference: engine/kernels/embedding_lookup.cu:16-31)."""
    category = "embedding"
    graph_safe = True     # launches kernels only: may run inside a captured graph

    def __init__(self, vocab_size: int, hidden_size: int):
        self.vocab_size, self.hidden_size = int(vocab_size), int(hidden_size)
        self.table = None

    def weight_specs(self) -> Dict[str, WeightSpec]:
        return {"weight": WeightSpec((self.vocab_size, self.hidden_size), kind="table")}

    def bind(self, tensors, rt) -> None:
        self.table = tensors["weight"]

    def forward(self, ctx) -> torch.Tensor:
        return ops.embed_gather(self.table, ctx.token_ids)


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
