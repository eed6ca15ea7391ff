"""The output head: ``logits = W h`` in 32-bit, with ``W`` its own tensor or the
embedding table when the model ties them (src/model.c:2353-2366, :6481).
"""
from __future__ import annotations

from typing import Dict

import torch

from .base import Part, ParamSpec, register_head


class LinearHead(Part):
    def __init__(self, vocab_size: int, hidden_size: int, tied: bool = False, weight_name: str = "weight"):
        self.vocab_size, self.hidden_size, self.tied = int(vocab_size), int(hidden_size), bool(tied)
        self.weight_name = weight_name
        self.weight = None

    def param_specs(self) -> Dict[str, ParamSpec]:
        if self.tied:
            return {}
        return {self.weight_name: ParamSpec((self.vocab_size, self.hidden_size), role="matrix")}

    def bind(self, tensors, rt, tied_to=None) -> None:
        """``tied_to``: the embedding part whose table a tied head uses."""
        self.rt = rt
        weight = getattr(tied_to, "weight", None) if self.tied else tensors[self.weight_name]
        if weight is None:
            raise ValueError("a tied head needs the embedding table")
        # In the kernels' own order where they have one.  A tied head shares one buffer with the
        # embedding (src/model.c:2354 aliases the pointer): where the table is
        # packed for the head's product, the embedding gathers its rows from the packed table too.
        self.weight = rt.ops.pack_weight(weight)
        if self.tied and self.weight is not weight and hasattr(tied_to, "share_table"):
            tied_to.share_table(self.weight)

    def forward(self, ctx, h):
        return self.rt.ops.linear(h, self.weight, out_dtype=torch.float32)


register_head("linear", LinearHead)
