"""A generation request as the scheduler sees it."""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Hashable, List, Optional

from ..sampling.params import SamplerState, SamplingParams

WAITING, RUNNING, FINISHED = "waiting", "running", "finished"


class Request:
    def __init__(self, req_id: Hashable, prompt: List[int], params: SamplingParams):
        if not prompt:
            raise ValueError("a request needs at least one prompt token")
        self.id = req_id
        self.prompt = [int(t) for t in prompt]
        self._n_prompt = len(self.prompt)      # (the prompt never changes)
        self.params = params
        self.output: List[int] = []
        self.n_computed = 0          # tokens of prompt + output whose keys and values are cached
        self.status = WAITING
        self.finish_reason: Optional[str] = None
        self.sampler = SamplerState(params)
        self.n_accepted = 0          # tokens already recorded in the sampler's recent window
        self.n_preempted = 0

    @property
    def tokens(self) -> List[int]:
        return self.prompt + self.output

    def token_slice(self, a: int, b: int) -> List[int]:
        """``tokens[a:b]`` without putting prompt and output together first."""
        n = self._n_prompt
        if a >= n:
            return self.output[a - n:b - n]
        if b <= n:
            return self.prompt[a:b]
        return self.prompt[a:] + self.output[:b - n]

    @property
    def n_tokens(self) -> int:
        return self._n_prompt + len(self.output)

    @property
    def remaining(self) -> int:
        """Tokens that still have to run before the next one can be sampled."""
        return self._n_prompt + len(self.output) - self.n_computed

    @property
    def finished(self) -> bool:
        return self.status == FINISHED
