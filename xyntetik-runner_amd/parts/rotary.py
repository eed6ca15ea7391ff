"""Rotary position encoding: the frequency table and its scaling rules.

``inv_freq[j] = theta^(-2j / rotary_dim)`` (src/model.c:285-289).
The reference then divides by per-dimension factors that the model file brings for
"llama 3.x long-context models" (:291-297) and does not compute them itself; the
"llama3" rule below computes the same divisors from ``rope_scaling``:

    wavelen = 2*pi / inv_freq
    wavelen < orig / high_freq_factor  : unchanged
    wavelen > orig / low_freq_factor   : inv_freq / factor
    otherwise, with s = (orig / wavelen - low) / (high - low):
                                         (1 - s) * inv_freq / factor + s * inv_freq

"linear" divides every frequency by ``factor`` (src/model.c:317-321).
The rotation itself (pairing, angle = position * inv_freq in 32-bit) is applied by
the kernel that writes keys to the cache (src/model.c:3514-3532).
"""
from __future__ import annotations

import math
from typing import Any, Mapping, Optional

import torch

from .base import PositionEncoding, RotaryParams, register_position


def rotary_inv_freq(rotary_dim: int, theta: float, scaling: Optional[Mapping[str, Any]] = None) -> torch.Tensor:
    """The table as float64 on the CPU."""
    if rotary_dim <= 0 or rotary_dim % 2:
        raise ValueError(f"rotary width {rotary_dim} must be positive and even")
    j = torch.arange(rotary_dim // 2, dtype=torch.float64)
    inv = torch.pow(torch.tensor(float(theta), dtype=torch.float64), -2.0 * j / rotary_dim)
    if not scaling:
        return inv
    kind = scaling.get("rope_type", scaling.get("type", "default"))
    if kind in (None, "default"):
        return inv
    factor = float(scaling["factor"])
    if kind == "linear":
        return inv / factor
    if kind == "llama3":
        low = float(scaling.get("low_freq_factor", 1.0))
        high = float(scaling.get("high_freq_factor", 4.0))
        orig = float(scaling["original_max_position_embeddings"])
        wavelen = 2.0 * math.pi / inv
        smooth = (orig / wavelen - low) / (high - low)
        mid = (1.0 - smooth) * inv / factor + smooth * inv
        out = torch.where(wavelen > orig / low, inv / factor, inv)
        between = (wavelen <= orig / low) & (wavelen >= orig / high)
        return torch.where(between, mid, out)
    raise ValueError(f"rope scaling {kind!r} is not supported")


class Rotary(PositionEncoding):
    def __init__(self, head_dim: int, theta: float, rotary_dim: Optional[int] = None,
                 scaling: Optional[Mapping[str, Any]] = None, interleaved: bool = False, mscale: float = 1.0):
        self.head_dim = int(head_dim)
        self.rotary_dim = int(rotary_dim) if rotary_dim is not None else self.head_dim
        if self.rotary_dim > self.head_dim:
            raise ValueError(f"rotary width {self.rotary_dim} exceeds head size {self.head_dim}")
        self.theta, self.scaling = float(theta), dict(scaling) if scaling else None
        self.interleaved, self.mscale = bool(interleaved), float(mscale)
        self._params: Optional[RotaryParams] = None

    def bind(self, tensors, rt) -> None:
        self.rt = rt
        table = rotary_inv_freq(self.rotary_dim, self.theta, self.scaling).to(torch.float32).to(rt.device)
        # the class is part of the key: a subclass that computes another table must not share this one's
        key = (type(self).__qualname__, self.rotary_dim, self.theta,
               repr(sorted(self.scaling.items())) if self.scaling else None)
        self._params = RotaryParams(table, self.rotary_dim, self.interleaved, self.mscale, table_key=key)

    def rotary(self) -> Optional[RotaryParams]:
        return self._params


class NoPosition(PositionEncoding):
    """Queries and keys go to attention as they are."""

    def __init__(self, **_):
        pass

    def bind(self, tensors, rt) -> None:
        self.rt = rt


register_position("rotary", Rotary)
register_position("none", NoPosition)
