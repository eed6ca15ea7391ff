"""The step function: run a batch of (request, its next tokens) from the cache.

``ModelRunner.step`` takes entries cut anywhere: portions of prompts beside single
decoded tokens.  It reserves pages, runs only the tokens it is given as one batch,
records that the requests have grown, and returns 32-bit logits at the wanted
places, in the order of the entries and of each entry's ``want``.
"""
from __future__ import annotations

import os
from typing import Dict, Hashable, List, Optional, Sequence

import torch

from ..cache import CacheManager, CacheStorage, OutOfPages, cache_groups, memory_budget, size_pools
from ..config import ModelSpec, load_config
from ..csrc.ops import load_ops
from ..parts.base import Runtime
from ..weights import SafetensorsStore, load_state, load_tensors
from .batch import StepContext, StepEntry
from .model import Model

_DTYPES = {"float32": torch.float32, "fp32": torch.float32, "bfloat16": torch.bfloat16, "bf16": torch.bfloat16}


def parse_dtype(name) -> torch.dtype:
    if isinstance(name, torch.dtype):
        if name not in (torch.float32, torch.bfloat16):
            raise ValueError(f"the engine runs in float32 or bfloat16, not {name}")
        return name
    try:
        return _DTYPES[str(name)]
    except KeyError:
        raise ValueError(f"dtype {name!r}: expected bfloat16 or float32") from None


class ModelRunner:
    def __init__(self, spec: ModelSpec, tensors_or_store, dtype, max_tokens: Optional[int] = None, page_size: int = 64,
                 max_requests: int = 64, device: str = "cuda:0", use_graphs: bool = True, consume_state: bool = False,
                 max_step_tokens: Optional[int] = None, gpu_memory_fraction: float = 0.9,
                 max_model_len: Optional[int] = None):
        """``max_tokens``: cache positions over all live requests.  None sizes the cache from the
        card instead: ``gpu_memory_fraction`` of its memory, less what is in use once the weights
        are bound and what a step's activations take, but no more than ``max_requests`` requests of
        ``max_model_len`` tokens (default: the model's context) can fill; ``CacheTooSmall`` if not even
        one such request fits.  ``max_step_tokens``: the most tokens a step will bring (None: any
        number); layers that keep a window of keys get pools for that instead of for ``max_tokens``."""
        if not torch.cuda.is_available():
            raise RuntimeError("no GPU: this engine runs on an MI355X only and has no CPU path")
        self.device = torch.device(device)
        torch.cuda.set_device(self.device)
        self.dtype = parse_dtype(dtype)
        self.spec = spec
        self.ops = load_ops()
        self.rt = Runtime(self.device, self.dtype, self.ops)
        self.model = Model(spec)
        expected = self.model.expected()
        if isinstance(tensors_or_store, SafetensorsStore):
            tensors = load_tensors(tensors_or_store, expected, self.dtype, self.device)
        else:
            tensors = load_state(tensors_or_store, expected, self.dtype, self.device, consume=consume_state)
        self.model.bind(tensors, self.rt)
        del tensors
        kv, st, of = self.model.cache_needs()
        self.page_size = page_size
        specs, owners = cache_groups(kv, of)
        elt = torch.empty((), dtype=self.dtype).element_size()
        if max_tokens is not None:
            sizes = size_pools(specs, owners, page_size, elt, max_requests, max_step_tokens, max_tokens=max_tokens)
        else:
            torch.cuda.synchronize(self.device)
            free, total = torch.cuda.mem_get_info(self.device)
            # what torch holds without having handed it out is as good as free
            free += torch.cuda.memory_reserved(self.device) - torch.cuda.memory_allocated(self.device)
            working = max(1 << 30, (max_step_tokens or 2048) << 20)     # a step's activations, generously
            sizes = size_pools(specs, owners, page_size, elt, max_requests, max_step_tokens,
                               budget_bytes=memory_budget(total, free, gpu_memory_fraction, working),
                               max_model_len=max_model_len or spec.max_position)
        self.storage = CacheStorage(kv, st, of, page_size, lambda s: sizes[specs.index(s)], max_requests,
                                    self.dtype, self.device)
        assert self.storage.group_specs == specs
        self.manager = CacheManager(specs, page_size, self.storage.group_pages, max_requests)
        self.vocab_size = spec.vocab_size
        from .graphs import DecodeGraphs
        self.graphs = DecodeGraphs(self) if use_graphs else None

    @classmethod
    def from_folder(cls, model_dir: str, dtype="bfloat16", **kw) -> "ModelRunner":
        arch, cfg = load_config(model_dir)
        spec = arch.build_spec(cfg)
        store = SafetensorsStore.open_folder(model_dir)
        try:
            return cls(spec, store, dtype, **kw)
        finally:
            store.close()

    # ------------------------------------------------------------------ requests
    def has(self, req_id: Hashable) -> bool:
        return req_id in self.manager.requests

    def start(self, req_id: Hashable) -> None:
        self.manager.admit(req_id)

    def finish(self, req_id: Hashable) -> None:
        self.manager.release(req_id)

    def length(self, req_id: Hashable) -> int:
        return self.manager.get(req_id).n_tokens

    # ------------------------------------------------------------------ the step
    def step(self, entries: Sequence[StepEntry], token_source: Optional[torch.Tensor] = None) -> Optional[torch.Tensor]:
        """Run ``entries`` as one batch; logits ``[wanted, V]`` float32 on the device (None if nothing is wanted).

        ``token_source`` (int32 on the device, one per entry): the entries' single tokens are
        taken from there instead (theirs are placeholders), so that a decode step can be queued
        before the host has seen the tokens the step before it picked.  Only for steps that a
        recorded graph runs (``takes_token_source``)."""
        entries = [e for e in entries if len(e.tokens) > 0]
        if not entries:
            return None
        if token_source is not None and not self.takes_token_source(entries):
            raise ValueError("tokens on the device are taken only by a recorded decode step")
        mgr = self.manager
        seen = set()
        for e in entries:
            if e.req_id in seen:
                raise ValueError(f"request {e.req_id!r} appears twice in one step")
            seen.add(e.req_id)
            for w in e.want:
                if not (0 <= w < len(e.tokens)):
                    raise ValueError(f"request {e.req_id!r}: wanted place {w} is outside its {len(e.tokens)} tokens")
        # Everything the step needs is counted before anything is taken: a state slot for every
        # request that is new, pages for all entries.  If it does not fit the step raises and
        # nothing has changed: no request admitted, no slot or page held.
        new = [e for e in entries if not self.has(e.req_id)]
        if len(new) > mgr.slots.n_free:
            raise OutOfPages(f"this step starts {len(new)} requests, {mgr.slots.n_free} of {mgr.slots.size} state slots are free")
        need = [0] * len(mgr.groups)
        for e in entries:
            if self.has(e.req_id):
                per = mgr.pages_needed(e.req_id, mgr.get(e.req_id).n_tokens + len(e.tokens))
            else:
                per = mgr.pages_needed_new(len(e.tokens))
            need = [a + b for a, b in zip(need, per)]
        for gi, g in enumerate(mgr.groups):
            if need[gi] > g.pool.n_free:
                raise OutOfPages(f"this step needs {need[gi]} new pages in group {gi}, {g.pool.n_free} of {g.pool.size} are free")
        for e in new:
            self.start(e.req_id)
        rcs = [mgr.get(e.req_id) for e in entries]
        try:
            for e, rc in zip(entries, rcs):
                mgr.reserve(e.req_id, rc.n_tokens + len(e.tokens))
            out = self._run(entries, rcs, token_source)
        except BaseException:
            # a step that failed leaves no request behind that it started and no page it reserved
            started = {e.req_id for e in new}
            for e in entries:
                if e.req_id in started:
                    mgr.release(e.req_id)
                else:
                    mgr.trim(e.req_id)
            raise
        for e, rc in zip(entries, rcs):
            mgr.advance(e.req_id, rc.n_tokens + len(e.tokens))
        return out

    def _run(self, entries, rcs, token_source) -> Optional[torch.Tensor]:
        mgr = self.manager
        if self.graphs is not None and self.graphs.applies(entries):
            out = self._step_graph(entries, rcs, token_source)
        else:
            ctx = StepContext(self.ops, self.device, entries, rcs, len(mgr.groups))
            self._zero_fresh_state(ctx)
            x = self.model.forward(ctx, self.storage.layers)
            out = self.model.logits(ctx, x, ctx.want_rows) if ctx.n_want else None
        return out

    def takes_token_source(self, entries: Sequence[StepEntry]) -> bool:
        return self.graphs is not None and self.graphs.applies(list(entries))

    def _step_graph(self, entries, rcs, token_source=None) -> Optional[torch.Tensor]:
        """A step of single tokens through a captured graph; the result is valid until the next step."""
        for e in entries:
            if any(w != 0 for w in e.want):
                raise ValueError(f"request {e.req_id!r}: wanted place outside its one token")
        self._zero_state_rows([rc.slot for rc in rcs if rc.fresh])
        logits = self.graphs.run(entries, rcs, token_source)
        rows = [i for i, e in enumerate(entries) for _ in e.want]
        if not rows:
            return None
        if rows == list(range(len(entries))):
            return logits
        return logits[torch.tensor(rows, dtype=torch.long, device=self.device)]

    def _zero_fresh_state(self, ctx: StepContext) -> None:
        self._zero_state_rows(ctx.fresh_slots_host)

    def _zero_state_rows(self, slots: List[int]) -> None:
        """The state rows of requests that use their slot for the first time begin at zero."""
        if not slots:
            return
        rows = None
        for lc in self.storage.layers:
            if lc.state is None:
                continue
            if rows is None:
                rows = torch.tensor(slots, dtype=torch.int32, device=self.device)
            self.ops.fill_rows_(lc.state, rows, len(slots), 0)
