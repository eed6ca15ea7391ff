"""The scheduler: which requests run which tokens in the next step.

Continuous batching with prompts cut into portions under a token budget:

* every step has at most ``max_batched_tokens`` tokens;
* running requests come first, in the order they were admitted: one token for each
  request that is decoding, then further portions of prompts that are under way;
* then waiting requests are admitted first-come first-served while fewer than
  ``max_running`` run, a state slot is free, budget is left and the first portion's
  pages are free; a portion may be any size down to what is left of the budget;
* when a running request cannot get the pages for its next tokens, the request
  admitted last is preempted: its pages and slot go back, it returns to the *front*
  of the waiting queue and is later recomputed from its prompt plus what it has
  generated (a request's cache rows depend on its own tokens only, so the recomputed
  rows equal the lost ones); the request that needs the pages is never preempted for
  itself while another runs, and a request that does not fit when it runs alone
  finishes with reason "cache_full";
* a request ends on a stop token (unless told to ignore it), after ``max_new_tokens``,
  or when it has ``max_model_len`` tokens.

The reference serves prompt chunks and decode steps by turns through a FIFO ticket
lock and gathers waiting sequences into decode microbatches
(src/scheduler.c:101-125, :153-220), with a fixed cache per slot so
that running out cannot happen; its finishing rules are kept
(src/engine.c:1834-1854).  This file is host logic only.
"""
from __future__ import annotations

from collections import deque
from dataclasses import dataclass, field
from typing import Deque, Dict, Hashable, List, Optional, Sequence, Tuple

from ..cache import CacheManager, OutOfPages
from .request import FINISHED, RUNNING, WAITING, Request


@dataclass
class StepPlan:
    entries: List[Tuple[Request, int]] = field(default_factory=list)    # (request, tokens to run)
    preempted: List[Request] = field(default_factory=list)
    failed: List[Request] = field(default_factory=list)

    @property
    def n_tokens(self) -> int:
        return sum(n for _, n in self.entries)


class Scheduler:
    def __init__(self, manager: CacheManager, max_batched_tokens: int = 2048, max_running: int = 64,
                 max_model_len: int = 4096, stop_ids: Sequence[int] = ()):
        if max_batched_tokens < 1 or max_running < 1:
            raise ValueError("the token budget and the number of running requests must be at least 1")
        self.manager = manager
        self.max_batched_tokens = max_batched_tokens
        self.max_running = max_running
        self.max_model_len = max_model_len
        self.stop_ids = set(int(s) for s in stop_ids)
        self.waiting: Deque[Request] = deque()
        self.running: List[Request] = []

    # ------------------------------------------------------------------ intake
    def capacity_tokens(self) -> int:
        """The most tokens a request can hold (layers that keep a window of keys set no limit)."""
        return self.manager.capacity_tokens()

    def add(self, req: Request) -> None:
        if req.n_tokens >= self.max_model_len:
            raise ValueError(f"request {req.id!r}: prompt of {req.n_tokens} tokens does not fit a context of "
                             f"{self.max_model_len} (a context of at least {req.n_tokens + 1} would)")
        if req.n_tokens + 1 > self.capacity_tokens():
            raise ValueError(f"request {req.id!r}: prompt of {req.n_tokens} tokens does not fit the cache "
                             f"({self.capacity_tokens()} positions)")
        req.status = WAITING
        self.waiting.append(req)

    def has_work(self) -> bool:
        return bool(self.waiting or self.running)

    # ------------------------------------------------------------------ one step's plan
    def _preempt(self, req: Request, plan: StepPlan) -> None:
        self.manager.release(req.id)
        self.running.remove(req)
        plan.entries = [(r, n) for r, n in plan.entries if r is not req]
        req.n_computed = 0
        req.status = WAITING
        req.n_preempted += 1
        self.waiting.appendleft(req)
        plan.preempted.append(req)

    def schedule(self) -> StepPlan:
        plan = StepPlan()
        budget = self.max_batched_tokens
        mgr = self.manager
        portion = mgr.max_portion()         # what the pools of windowed layers let one request run in a step
        # running requests: decoding ones first, then prompts under way
        order, prompts = [], []
        for r in self.running:
            (order if r.remaining == 1 else prompts).append(r)
        order += prompts
        for req in order:
            if budget <= 0 or (plan.preempted and req not in self.running):      # nothing left / preempted meanwhile
                continue
            n = min(req.remaining, budget, portion)
            while True:
                try:
                    mgr.reserve(req.id, req.n_computed + n)
                    break
                except OutOfPages:
                    victim = self.running[-1]
                    if victim is req:
                        others = [r for r in self.running if r is not req]
                        if not others:
                            victim = None
                        else:
                            victim = others[-1]
                    if victim is None:
                        # alone and still too big for the cache
                        if n > 1:
                            n = max(1, n // 2)      # a smaller portion may still fit
                            continue
                        self.manager.release(req.id)
                        self.running.remove(req)
                        req.status, req.finish_reason = FINISHED, "cache_full"
                        plan.failed.append(req)
                        n = 0
                        break
                    budget += sum(m for r, m in plan.entries if r is victim)
                    self._preempt(victim, plan)
            if n > 0:
                plan.entries.append((req, n))
                budget -= n
        # admission, first come first served
        while self.waiting and budget > 0 and len(self.running) < self.max_running and mgr.can_admit():
            req = self.waiting[0]
            if req in plan.preempted:
                break                  # preempted in this very step: it waits for the next one
            n = min(req.remaining, budget, portion)
            mgr.admit(req.id)
            try:
                mgr.reserve(req.id, n)
            except OutOfPages:
                mgr.release(req.id)
                if not self.running:
                    # nothing else holds pages, so it will never fit
                    self.waiting.popleft()
                    req.status, req.finish_reason = FINISHED, "cache_full"
                    plan.failed.append(req)
                    continue
                break
            self.waiting.popleft()
            req.status = RUNNING
            self.running.append(req)
            plan.entries.append((req, n))
            budget -= n
        return plan

    # ------------------------------------------------------------------ after the step
    def ran(self, plan: StepPlan) -> List[Request]:
        """Record that the plan's tokens are cached; returns the requests whose next token can be sampled."""
        ready = []
        for req, n in plan.entries:
            req.n_computed += n
            if req.remaining == 0:
                ready.append(req)
        return ready

    def accept(self, req: Request, token: int) -> bool:
        """Take a sampled token; returns True if the request is finished
        (src/engine.c:1834-1854, :1878)."""
        p = req.params
        if token in self.stop_ids and not p.ignore_eos:
            return self._finish(req, "stop")          # the stop token is neither kept nor run
        req.output.append(int(token))
        if p.max_new_tokens >= 0 and len(req.output) >= p.max_new_tokens:
            return self._finish(req, "length")
        if req.n_tokens >= self.max_model_len:
            return self._finish(req, "context")
        return False

    def _finish(self, req: Request, reason: str) -> bool:
        req.status, req.finish_reason = FINISHED, reason
        if req in self.running:
            self.running.remove(req)
            self.manager.release(req.id)
        return True

    def abort(self, req: Request, reason: str = "aborted") -> None:
        if req in self.waiting:
            self.waiting.remove(req)
            req.status, req.finish_reason = FINISHED, reason
        elif req in self.running:
            self._finish(req, reason)
