"""Per-request sampling options and the sampler's state.

The options are the reference's five knobs with its defaults for an unknown model
family: temperature, top-k, top-p, min-p and a repeat penalty over the last 256
tokens (src/sample.h:9-20).  ``temperature <= 0`` asks for the argmax
and applies no penalty (src/sample.c:141-172).  The random numbers come
from xorshift64, one draw for each sampled token; state 0 is a fixed point, so seed 0 is
refused, and an absent seed is taken from the clock
(src/sample.c:13-20, src/main.c:833-845).
"""
from __future__ import annotations

import time
from dataclasses import dataclass, field
from typing import List, Optional

RECENT_WINDOW = 256
_MASK = 0xFFFFFFFFFFFFFFFF


@dataclass(frozen=True)
class SamplingParams:
    temperature: float = 0.0
    top_k: int = 0                 # 0 = off
    top_p: float = 1.0
    min_p: float = 0.0             # 0 = off
    repeat_penalty: float = 1.0    # 1 = off
    seed: Optional[int] = None
    max_new_tokens: int = 256      # -1 = until a stop token or the context is full
    ignore_eos: bool = False

    def __post_init__(self):
        if self.seed is not None and (self.seed & _MASK) == 0:
            raise ValueError("seed 0 is not usable: state 0 is a fixed point of the sampler's generator")
        if self.top_k < 0:
            raise ValueError(f"top_k {self.top_k} is negative")
        if not (0.0 <= self.top_p <= 1.0):
            raise ValueError(f"top_p {self.top_p} is outside [0, 1]")
        if not (0.0 <= self.min_p <= 1.0):
            raise ValueError(f"min_p {self.min_p} is outside [0, 1]")
        if self.repeat_penalty <= 0.0:
            raise ValueError(f"repeat_penalty {self.repeat_penalty} must be positive")

    @property
    def greedy(self) -> bool:
        return not (self.temperature > 0.0)


def xorshift64(state: int) -> int:
    x = state & _MASK
    x ^= (x << 13) & _MASK
    x ^= x >> 7
    x ^= (x << 17) & _MASK
    return x


class SamplerState:
    """What a request's sampler remembers between tokens: generator state and recent window."""

    def __init__(self, params: SamplingParams):
        self.params = params
        if params.seed is not None:
            self.rng = params.seed & _MASK
        else:
            self.rng = (int(time.time()) ^ 0x9E3779B97F4A7C15) & _MASK or 1
        self.recent: List[int] = [0] * RECENT_WINDOW
        self.n_recent = 0
        self.head = 0

    def draw(self) -> float:
        """The next uniform number in [0, 1): the top 24 bits of the next state."""
        self.rng = xorshift64(self.rng)
        return (self.rng >> 40) / 16777216.0

    def accept(self, token: int) -> None:
        """Record a token (prompt or generated) in the ring of the last 256
        (src/sample.c:27-31)."""
        self.recent[self.head] = int(token)
        self.head = (self.head + 1) % RECENT_WINDOW
        if self.n_recent < RECENT_WINDOW:
            self.n_recent += 1
