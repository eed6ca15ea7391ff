"""A model: the parts of a ``ModelSpec``, built, bound to their tensors, and run.

The forward pass is the reference's, step by step
(src/model.c:6148-6483): embedding, the layers in their run order,
then final norm and output head on the rows whose logits are wanted only
(:6478-6481).
"""
from __future__ import annotations

from typing import Dict, List, Optional

import torch

from ..config import ModelSpec
from ..parts.base import Block, ParamSpec, Runtime, make_block, make_part


class Model:
    def __init__(self, spec: ModelSpec):
        spec.validate()
        self.spec = spec
        self.embedding = make_part("embedding", spec.embedding)
        self.blocks: List[Block] = []
        for ls in spec.layers:
            self.blocks.append(make_block(
                ls.block,
                make_part("mixer", ls.mixer) if ls.mixer is not None else None,
                make_part("feed_forward", ls.feed_forward) if ls.feed_forward is not None else None,
                {name: make_part("norm", ps) for name, ps in ls.norms.items()}))
        self.final_norm = make_part("norm", spec.final_norm)
        self.head = make_part("head", spec.head)
        self.rt: Optional[Runtime] = None

    # ------------------------------------------------------------------ tensors
    def _named_parts(self):
        yield self.spec.embedding.prefix, self.embedding
        for ls, blk in zip(self.spec.layers, self.blocks):
            for name, ps in ls.norms.items():
                yield ps.prefix, blk.norms[name]
            if ls.mixer is not None:
                yield ls.mixer.prefix, blk.mixer
            if ls.feed_forward is not None:
                yield ls.feed_forward.prefix, blk.feed_forward
        yield self.spec.final_norm.prefix, self.final_norm
        yield self.spec.head.prefix, self.head

    def capturable(self) -> bool:
        """Whether a step's launches are the same for any data (every part says so)."""
        return all(part.capturable for _, part in self._named_parts())

    def expected(self) -> Dict[str, ParamSpec]:
        out: Dict[str, ParamSpec] = {}
        for prefix, part in self._named_parts():
            for rel, ps in part.param_specs().items():
                name = prefix + rel
                if name in out:
                    raise ValueError(f"two parts claim the tensor {name}")
                out[name] = ps
        return out

    @staticmethod
    def expected_tensors(spec: ModelSpec) -> Dict[str, ParamSpec]:
        return Model(spec).expected()

    def bind(self, tensors: Dict[str, torch.Tensor], rt: Runtime) -> None:
        """Give every part its tensors (``tensors`` is emptied as parts take theirs)."""
        self.rt = rt
        for prefix, part in self._named_parts():
            mine = {rel: tensors.pop(prefix + rel) for rel in part.param_specs() if prefix + rel in tensors}
            if part is self.head:
                part.bind(mine, rt, tied_to=self.embedding)
            else:
                part.bind(mine, rt)

    # ------------------------------------------------------------------ what the cache must hold
    def cache_needs(self):
        """Per entry of the run order: (KVSpec or None, StateSpec or None, cache_of)."""
        kv, st, of = [], [], []
        for step in self.spec.order:
            mixer = self.blocks[step.layer].mixer
            kv.append(mixer.kv_spec() if mixer is not None else None)
            st.append(mixer.state_spec() if mixer is not None and step.cache_of is None else None)
            of.append(step.cache_of)
        return kv, st, of

    # ------------------------------------------------------------------ forward
    def forward(self, ctx, caches) -> torch.Tensor:
        """Run the step's tokens through every layer; returns the residual stream ``[T, E]`` (32-bit)."""
        x = self.embedding.forward(ctx, ctx.token_ids)
        order = self.spec.order
        h = None            # the result of the next block's first norm, if the block before made it
        for i, step in enumerate(order):
            block = self.blocks[step.layer]
            if block.chained:
                after = self.blocks[order[i + 1].layer].entry_norm() if i + 1 < len(order) else None
                h = block.forward(ctx, caches[i], x, h=h, after=after)
            else:
                block.forward(ctx, caches[i], x)
                h = None
        return x

    def logits(self, ctx, x: torch.Tensor, rows: torch.Tensor) -> torch.Tensor:
        """32-bit logits ``[len(rows), V]`` of the rows ``rows`` of ``x``."""
        h = self.final_norm.forward(ctx, x, rows=rows)
        return self.head.forward(ctx, h)
