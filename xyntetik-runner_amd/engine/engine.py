"""The generation engine: requests in, tokens out.

``Engine.step`` is one turn of the loop: the scheduler plans, the step function runs
the plan as one batch, the sampler picks a token for every request whose last token
has run, and finished requests give back what they hold.  The first generated token
is sampled from the logits of the prompt's last position, as in the reference
(/root/reference/src/engine.c:1939-1956); unlike it, no step is run for a token after
which nothing will be sampled.
"""
from __future__ import annotations

import itertools
import time
from dataclasses import dataclass
from typing import Dict, Hashable, Iterable, List, Optional, Sequence, Union

import torch

from ..sampling import Sampler, SamplingParams
from .batch import StepEntry
from .request import Request
from .runner import ModelRunner
from .scheduler import Scheduler, StepPlan


@dataclass
class StepOutput:
    req_id: Hashable
    token: Optional[int]          # None: the request ended without a new token (stop token, failure)
    finished: bool
    finish_reason: Optional[str] = None


@dataclass
class EngineStats:
    steps: int = 0
    prompt_tokens: int = 0
    generated_tokens: int = 0
    preemptions: int = 0
    prefill_seconds: float = 0.0
    decode_seconds: float = 0.0


class Engine:
    def __init__(self, runner: ModelRunner, max_batched_tokens: int = 2048, max_running: int = 64,
                 max_model_len: Optional[int] = None, stop_ids: Optional[Sequence[int]] = None):
        self.runner = runner
        spec = runner.spec
        stops = list(spec.eos_token_ids) if stop_ids is None else list(stop_ids)
        self.scheduler = Scheduler(
            runner.manager, max_batched_tokens=max_batched_tokens,
            max_running=min(max_running, runner.manager.slots.size),
            max_model_len=max_model_len or spec.max_position, stop_ids=stops)
        self.sampler = Sampler(runner.ops, runner.device, exempt_ids=stops)
        self.requests: Dict[Hashable, Request] = {}
        self.stats = EngineStats()
        self._ids = itertools.count()

    # ------------------------------------------------------------------ requests
    def add_request(self, prompt: Sequence[int], params: Optional[SamplingParams] = None,
                    req_id: Optional[Hashable] = None) -> Hashable:
        rid = next(self._ids) if req_id is None else req_id
        if rid in self.requests:
            raise ValueError(f"request id {rid!r} is in use")
        req = Request(rid, list(prompt), params or SamplingParams())
        self.scheduler.add(req)
        self.requests[rid] = req
        return rid

    def has_work(self) -> bool:
        return self.scheduler.has_work()

    # ------------------------------------------------------------------ one step
    def step(self) -> List[StepOutput]:
        plan = self.scheduler.schedule()
        outs: List[StepOutput] = []
        self.stats.preemptions += len(plan.preempted)
        for req in plan.failed:
            outs.append(StepOutput(req.id, None, True, req.finish_reason))
        if not plan.entries:
            if not plan.failed and self.scheduler.has_work():
                raise RuntimeError("the scheduler has work but could plan nothing")
            return outs
        entries = []
        for req, n in plan.entries:
            toks = req.token_slice(req.n_computed, req.n_computed + n)
            last = req.n_computed + n == req.n_tokens
            entries.append(StepEntry(req.id, toks, [n - 1] if last else []))
            # the sampler's window sees every token of the request once, prompt included
            # (/root/reference/src/engine.c:881)
            upto = req.n_computed + n
            for t in req.token_slice(req.n_accepted, upto):
                req.sampler.accept(t)
            req.n_accepted = max(req.n_accepted, upto)
        t0 = time.perf_counter()
        logits = self.runner.step(entries)
        ready = self.scheduler.ran(plan)
        if ready:
            tokens = self.sampler.sample(logits, [r.sampler for r in ready])
            for req, tok in zip(ready, tokens):
                before = len(req.output)
                done = self.scheduler.accept(req, tok)
                new = req.output[-1] if len(req.output) > before else None
                if new is not None:
                    self.stats.generated_tokens += 1
                outs.append(StepOutput(req.id, new, done, req.finish_reason))
        dt = time.perf_counter() - t0
        if any(n > 1 for _, n in plan.entries):
            self.stats.prefill_seconds += dt
        else:
            self.stats.decode_seconds += dt
        self.stats.steps += 1
        return outs

    # ------------------------------------------------------------------ whole generations
    def generate(self, prompts: Sequence[Sequence[int]],
                 params: Union[SamplingParams, Sequence[SamplingParams], None] = None) -> List[List[int]]:
        """Generate for every prompt (lists of token ids); returns the new tokens of each."""
        if params is None or isinstance(params, SamplingParams):
            params = [params or SamplingParams()] * len(prompts)
        ids = [self.add_request(p, sp) for p, sp in zip(prompts, params)]
        self.stats.prompt_tokens += sum(len(p) for p in prompts)
        while self.has_work():
            self.step()
        out = []
        for rid in ids:
            req = self.requests.pop(rid)
            if req.finish_reason == "cache_full":
                raise RuntimeError(f"request {rid!r} does not fit the cache even alone "
                                   f"({self.scheduler.capacity_tokens()} positions)")
            out.append(list(req.output))
        return out
