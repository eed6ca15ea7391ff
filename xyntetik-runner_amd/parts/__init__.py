from .base import (Part, Norm, PositionEncoding, QKTransform, Mixer, FeedForward, Block, ParamSpec, KVSpec, StateSpec,
                   RotaryParams, Runtime, make_part, make_block, unregister, register_norm, register_position,
                   register_qk_transform, register_mixer, register_feed_forward, register_block, register_embedding, register_head)
from . import norm, rotary, embedding, head, mlp, attention, block    # noqa: F401  (registers the built-in parts)
from .norm import RMSNorm
from .rotary import Rotary, NoPosition, rotary_inv_freq
from .embedding import TokenEmbedding
from .head import LinearHead
from .mlp import GatedMLP
from .attention import PagedAttention
from .block import PreNormBlock

__all__ = [
    "Part", "Norm", "PositionEncoding", "QKTransform", "Mixer", "FeedForward", "Block", "ParamSpec", "KVSpec", "StateSpec",
    "RotaryParams", "Runtime", "make_part", "make_block", "unregister", "register_norm", "register_position",
    "register_qk_transform", "register_mixer", "register_feed_forward", "register_block", "register_embedding", "register_head",
    "RMSNorm", "Rotary", "NoPosition", "rotary_inv_freq", "TokenEmbedding", "LinearHead", "GatedMLP",
    "PagedAttention", "PreNormBlock",
]
