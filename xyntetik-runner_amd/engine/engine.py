"""The generation engine: requests in, tokens out.

``Engine.step`` is one turn of the loop: the scheduler plans, the step function runs
the plan as one batch, the sampler picks a token for every request whose last token
has run, and finished requests give back what they hold.  In steady decoding the next
step's kernels are queued before the host reads this step's tokens (``_launch_ahead``), so
the GPU does not wait for the host's turn.  The first generated token
is sampled from the logits of the prompt's last position, as in the reference
(src/engine.c:1939-1956); unlike it, no step is run for a token after
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
from ..cache import OutOfPages
from .request import RUNNING, Request
from .runner import ModelRunner
from .scheduler import Scheduler, StepPlan


@dataclass
class StepOutput:
    req_id: Hashable
    token: Optional[int]          # None: the request ended without a new token (stop token, failure)
    finished: bool
    finish_reason: Optional[str] = None
    request: Optional[Request] = None      # with ``finished``: the request as it ended (the engine keeps it no longer)


@dataclass
class EngineStats:
    steps: int = 0
    prompt_tokens: int = 0
    generated_tokens: int = 0
    preemptions: int = 0
    steps_ahead: int = 0          # decode steps queued before the host had read the tokens before them
    prefill_seconds: float = 0.0
    decode_seconds: float = 0.0


@dataclass
class _Launched:
    """A step whose kernels are queued."""
    plan: StepPlan
    ready: List[Request]                 # the requests a token is picked for, row by row
    tokens: Optional[torch.Tensor]       # their picks, on the device (None: nothing is picked)
    t0: float
    pure_decode: bool                    # one token of every request, through a recorded graph
    ahead: bool = False
    host_tokens: Optional[torch.Tensor] = None      # the picks' copy in pinned memory, queued right behind them
    copied: Optional[torch.cuda.Event] = None
    rows: Optional[List[int]] = None                # the rows of host_tokens that `ready` still names

    def start_copy(self) -> None:
        """Queue the copy of the picks to the host now: asked for later, it would wait behind
        whatever was queued meanwhile (the step after this one)."""
        if self.tokens is not None:
            self.host_tokens = torch.empty(self.tokens.shape, dtype=self.tokens.dtype, pin_memory=True)
            self.host_tokens.copy_(self.tokens, non_blocking=True)
            self.copied = torch.cuda.Event()
            self.copied.record()

    def read_tokens(self) -> List[int]:
        self.copied.synchronize()
        return self.host_tokens.tolist()

    @property
    def decode(self) -> bool:
        return all(n == 1 for _, n in self.plan.entries)


class Engine:
    def __init__(self, runner: ModelRunner, max_batched_tokens: int = 2048, max_running: int = 64,
                 max_model_len: Optional[int] = None, stop_ids: Optional[Sequence[int]] = None,
                 run_ahead: bool = True):
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
        self.run_ahead = run_ahead
        self._ahead: Optional[_Launched] = None

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

    def abort(self, req_id: Hashable, reason: str = "aborted") -> Request:
        """Take a request out between two steps; what it holds goes back, and it is returned as it ended."""
        req = self.requests.pop(req_id)
        self.scheduler.abort(req, reason)
        return req

    # ------------------------------------------------------------------ one step
    def step(self) -> List[StepOutput]:
        outs: List[StepOutput] = []
        cur = self._take_step_ahead()
        if cur is None:
            plan = self.scheduler.schedule()
            self.stats.preemptions += len(plan.preempted)
            for req in plan.failed:
                outs.append(self._ended(StepOutput(req.id, None, True, req.finish_reason), req))
            if not plan.entries:
                if not plan.failed and self.scheduler.has_work():
                    raise RuntimeError("the scheduler has work but could plan nothing")
                return outs
            cur = self._launch(plan)
        # While the GPU works on this step: queue the one after it, if nothing the host will
        # learn from this step's tokens can change its plan except that a request may end.
        if self.run_ahead and cur.tokens is not None:
            self._ahead = self._launch_ahead(cur)
        if cur.tokens is not None:
            tokens = cur.read_tokens()                   # waits for the step
            if cur.rows is not None:
                tokens = [tokens[i] for i in cur.rows]
            for req, tok in zip(cur.ready, tokens):
                before = len(req.output)
                done = self.scheduler.accept(req, int(tok))
                new = req.output[-1] if len(req.output) > before else None
                if new is not None:
                    self.stats.generated_tokens += 1
                out = StepOutput(req.id, new, done, req.finish_reason)
                outs.append(self._ended(out, req) if done else out)
        dt = time.perf_counter() - cur.t0
        if cur.decode:
            self.stats.decode_seconds += dt
        else:
            self.stats.prefill_seconds += dt
        self.stats.steps += 1
        return outs

    def _ended(self, out: StepOutput, req: Request) -> StepOutput:
        """A request that is over leaves the engine's table with the output that reports its end."""
        self.requests.pop(req.id, None)
        out.request = req
        return out

    def _record(self, plan: StepPlan) -> List[Request]:
        """The plan's tokens are cached: every request's sampler window sees its tokens once, prompt
        included (src/engine.c:881); returns the requests whose next token is sampled."""
        ready = self.scheduler.ran(plan)
        for req, _ in plan.entries:
            for t in req.token_slice(req.n_accepted, req.n_computed):
                req.sampler.accept(t)
            req.n_accepted = max(req.n_accepted, req.n_computed)
        return ready

    def _launch(self, plan: StepPlan) -> "_Launched":
        entries = []
        for req, n in plan.entries:
            toks = req.token_slice(req.n_computed, req.n_computed + n)
            last = req.n_computed + n == req.n_tokens
            entries.append(StepEntry(req.id, toks, [n - 1] if last else []))
        t0 = time.perf_counter()
        logits = self.runner.step(entries)
        ready = self._record(plan)
        tokens = self.sampler.launch(logits, [r.sampler for r in ready]) if ready else None
        decode = all(n == 1 for _, n in plan.entries)
        cur = _Launched(plan, ready, tokens, t0, decode and len(ready) == len(plan.entries)
                        and self.runner.takes_token_source(entries))
        cur.start_copy()
        return cur

    def _launch_ahead(self, cur: "_Launched") -> Optional["_Launched"]:
        """Queue the decode step after ``cur`` before ``cur``'s tokens are known to the host: its
        tokens go from the sampler's result to the step's input on the device.  Only when the next
        plan is certain but for requests ending: every running request is decoding in ``cur``,
        nobody waits, nobody reaches a length limit with this token, and no pick depends on
        earlier tokens.  A request that ends with ``cur``'s token has run one token too far,
        which nobody sees: its row is dropped and its pages are given back with the rest."""
        sch = self.scheduler
        reqs = cur.ready
        if not cur.pure_decode or sch.waiting or len(reqs) != len(sch.running):
            return None
        if self.sampler.uses_history([r.sampler for r in reqs]):
            return None
        for r in reqs:
            p = r.params
            if (p.max_new_tokens >= 0 and len(r.output) + 1 >= p.max_new_tokens) or r.n_tokens + 1 >= sch.max_model_len:
                return None
        entries = [StepEntry(r.id, [0], [0]) for r in reqs]
        if not self.runner.takes_token_source(entries):
            return None
        t0 = time.perf_counter()
        try:
            logits = self.runner.step(entries, token_source=cur.tokens)
        except OutOfPages:
            return None                  # the scheduler decides who makes room, in its own turn
        tokens = self.sampler.launch(logits, [r.sampler for r in reqs])
        nxt = _Launched(StepPlan(entries=[(r, 1) for r in reqs]), list(reqs), tokens, t0, True, ahead=True)
        nxt.start_copy()
        self.stats.steps_ahead += 1
        return nxt

    def _take_step_ahead(self) -> Optional["_Launched"]:
        """The step that was queued ahead, now that the tokens before it are accepted: the
        requests that went on, in the rows they were given (None if there is no such step)."""
        cur, self._ahead = self._ahead, None
        if cur is None:
            return None
        rows = [i for i, r in enumerate(cur.ready) if r.status == RUNNING]
        if not rows:
            return None
        if len(rows) < len(cur.ready):
            cur.rows = rows                      # of the picks as they were copied to the host
            cur.tokens = cur.tokens[torch.tensor(rows, dtype=torch.long, device=cur.tokens.device)]
            cur.ready = [cur.ready[i] for i in rows]
            cur.plan = StepPlan(entries=[(r, 1) for r in cur.ready])
        self._record(cur.plan)
        return cur

    # ------------------------------------------------------------------ whole generations
    def generate(self, prompts: Sequence[Sequence[int]],
                 params: Union[SamplingParams, Sequence[SamplingParams], None] = None) -> List[List[int]]:
        """Generate for every prompt (lists of token ids); returns the new tokens of each."""
        if params is None or isinstance(params, SamplingParams):
            params = [params or SamplingParams()] * len(prompts)
        ids = [self.add_request(p, sp) for p, sp in zip(prompts, params)]
        self.stats.prompt_tokens += sum(len(p) for p in prompts)
        ended: Dict[Hashable, Request] = {}
        while self.has_work():
            for o in self.step():
                if o.finished:
                    ended[o.req_id] = o.request
        out = []
        for rid in ids:
            req = ended[rid]
            if req.finish_reason == "cache_full":
                raise RuntimeError(f"request {rid!r} does not fit the cache even alone "
                                   f"({self.scheduler.capacity_tokens()} positions)")
            out.append(list(req.output))
        return out
