"""Token embedding: one row of the table per token, as 32-bit rows of the residual
stream; an id outside the vocabulary reads row 0 (src/model.c:6148-6162).
"""
from __future__ import annotations

from typing import Dict

from .base import Part, ParamSpec, register_embedding


class TokenEmbedding(Part):
    def __init__(self, vocab_size: int, hidden_size: int, scale: float = 1.0, weight_name: str = "weight"):
        self.vocab_size, self.hidden_size, self.scale = int(vocab_size), int(hidden_size), float(scale)
        self.weight_name = weight_name
        self.weight = None

    def param_specs(self) -> Dict[str, ParamSpec]:
        return {self.weight_name: ParamSpec((self.vocab_size, self.hidden_size), role="matrix")}

    def bind(self, tensors, rt) -> None:
        self.rt = rt
        self.weight = tensors[self.weight_name]

    def share_table(self, table) -> None:
        """Gather from ``table`` from now on: the same values in another layout (a tied output
        head's packed copy), so that the model keeps the table once."""
        if tuple(table.shape) != (self.vocab_size, self.hidden_size):
            raise ValueError(f"a table of {tuple(table.shape)} cannot stand for one of {(self.vocab_size, self.hidden_size)}")
        self.weight = table

    def forward(self, ctx, token_ids):
        return self.rt.ops.embedding(self.weight, token_ids, self.scale)


register_embedding("token_embedding", TokenEmbedding)
