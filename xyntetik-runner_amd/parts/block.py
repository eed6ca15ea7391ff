"""Arrangements of a layer's parts around the 32-bit residual stream.

"prenorm": ``x += mixer(norm(x)); x += feed_forward(norm(x))`` — norm, projections,
rotation, cache write, attention, output, add, norm, feed-forward, add, every layer
alike (/root/reference/src/model.c:6168-6473).
"""
from __future__ import annotations

from .base import Block, register_block


class PreNormBlock(Block):
    def forward(self, ctx, cache, x) -> None:
        h = self.mixer_norm.forward(ctx, x)
        self.mixer.forward_add(ctx, cache, h, x)
        h = self.feed_forward_norm.forward(ctx, x)
        self.feed_forward.forward_add(ctx, h, x)


register_block("prenorm", PreNormBlock)
