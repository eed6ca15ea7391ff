"""HIP graphs for decode steps.

A step in which every request brings one token launches a few hundred short kernels;
launching them one by one from Python costs more than running them.  Such a step is
therefore captured once per *bucket* (batch size rounded up to a power of two, and the
number of key ranges each request's attention is split into) and replayed afterwards.
Everything a step's kernels read that changes from step to step -- token ids, positions,
block tables, the attention work list -- lives in one device buffer at fixed addresses
that is refilled with a single copy before each replay, the way the reference keeps the
position and the cache pointers of its captured decode step in device memory
(src/cuda.c:4388-4411, :4242-4264).  Rows that pad a batch up to its
bucket read and write the null page and their logits are dropped.

No memset is recorded: the step's kernels write every byte they later read.
"""
from __future__ import annotations

import gc
from typing import Dict, List, Optional, Tuple

import numpy as np
import torch

from ..cache import NULL_PAGE
from .batch import ATTN_MIN_RANGE, ATTN_STREAM_SLOTS, ATTN_TILE, AttentionPlan, StepEntry

BUCKETS = (1, 2, 4, 8, 16, 32, 64, 128, 256, 512)
SPLITS = (1, 2, 4, 8, 16, 32)


def bucket_for(n: int) -> Optional[int]:
    for b in BUCKETS:
        if n <= b:
            return b
    return None


def splits_for(batch_cap: int, max_tiles: int, n_kv_heads: int) -> int:
    """Key ranges per request: one round of workgroups, and no range shorter than it pays."""
    want = max(1, min(ATTN_STREAM_SLOTS // (batch_cap * n_kv_heads), max_tiles // ATTN_MIN_RANGE))
    best = 1
    for s in SPLITS:
        if s <= want:
            best = s
    return best


class StaticDecodeContext:
    """A ``StepContext`` for one token per request whose device arrays never move."""

    def __init__(self, ops, device, batch_cap: int, n_splits: int, table_widths: List[int],
                 windowed: Optional[List[bool]] = None, max_tiles: Optional[int] = None, *, null_slot: int):
        """``n_splits``: the most key ranges a request is cut into; ``max_tiles``: the longest request's
        tiles when the context is made.  Every attention plan (group size, window, key/value heads)
        gets a number of key ranges of its own from these: a windowed layer, or one with more
        key/value heads, needs fewer ranges to fill the chip than the bucket's longest request
        with the fewest heads."""
        self.ops, self.device = ops, device
        self.max_tiles = max_tiles
        self.null_slot = null_slot          # the state row of the rows that pad the batch
        # groups whose requests give pages back while they live (their table rows are rewritten every step)
        self.windowed = list(windowed) if windowed is not None else [True] * len(table_widths)
        self.B = self.T = batch_cap
        self.S = n_splits
        self.table_width = list(table_widths)
        self.q_lens = [1] * batch_cap
        self.max_q_len = 1
        self.n_want = batch_cap
        B = batch_cap
        # [token_ids B][positions B][req_of_token B][cu_q B+1][seq_lens B][slots B][fresh B][starts B][want B]
        # [tables ...][plans ...]
        self._sizes = [B, B, B, B + 1, B, B, B, B, B] + [B * w for w in self.table_width]
        self._plan_keys: List[Tuple[int, Optional[int], int]] = []
        self._plans: Dict[Tuple[int, Optional[int], int], AttentionPlan] = {}
        self._plan_off: Dict[Tuple[int, Optional[int], int], int] = {}
        self._plan_splits: Dict[Tuple[int, Optional[int], int], int] = {}
        self._alloc()
        self.fresh_slots_host: List[int] = []
        self._copied = None
        self.shared = {}        # what parts make once a pass over the layers and share (a rotation's table)

    def _alloc(self) -> None:
        B = self.B
        n_plan = sum(B * self._plan_splits[k] * 8 + B * 7 for k in self._plan_keys)
        offs = np.concatenate([[0], np.cumsum(self._sizes)]).astype(np.int64)
        total = int(offs[-1]) + n_plan
        self._offs = offs
        self._host = torch.zeros((total,), dtype=torch.int32).pin_memory()
        # what each row of each block table in the pinned buffer holds: (the request's cache record, pages)
        self._rows = [[None] * B for _ in self.table_width]
        for g, w in enumerate(self.table_width):
            tab = self._host.numpy()[offs[9 + g]:offs[10 + g]].reshape(B, w)
            tab[:] = -1
            tab[:, 0] = NULL_PAGE
        self._dev = torch.zeros((total,), dtype=torch.int32, device=self.device)
        d, o = self._dev, offs
        self.token_ids, self.positions, self.req_of_token = d[o[0]:o[1]], d[o[1]:o[2]], d[o[2]:o[3]]
        self.cu_q, self.seq_lens_dev, self.slots = d[o[3]:o[4]], d[o[4]:o[5]], d[o[5]:o[6]]
        self.fresh, self.starts_dev, self.want_rows = d[o[6]:o[7]], d[o[7]:o[8]], d[o[8]:o[9]]
        self._tables = [d[o[9 + g]:o[10 + g]].view(B, w) for g, w in enumerate(self.table_width)]
        base = int(offs[-1])
        for k in self._plan_keys:
            S = self._plan_splits[k]
            self._plan_off[k] = base
            items = d[base:base + B * S * 8]
            jobs = d[base + B * S * 8:base + B * S * 8 + B * 7]
            self._plans[k] = AttentionPlan(items, B * S, jobs if S > 1 else None, B if S > 1 else 0,
                                           B * S if S > 1 else 0)
            base += B * S * 8 + B * 7

    def block_table(self, group: int) -> torch.Tensor:
        return self._tables[group]

    @property
    def slots_host(self):
        raise RuntimeError("this step is recorded as a graph: a part with state reads its rows' slots from "
                           "ctx.slots (on the device), or sets capturable = False to be run eagerly")

    def attention_plan(self, group: int, group_size: int, window: Optional[int], n_kv_heads: int,
                       page_size: int = 64) -> AttentionPlan:
        key = (group_size, window, n_kv_heads)
        if key not in self._plans:
            if torch.cuda.is_current_stream_capturing():
                raise RuntimeError("an attention plan was first asked for during graph capture")
            tiles = self.max_tiles
            if tiles is not None and window:
                tiles = min(tiles, -(-window // ATTN_TILE) + 1)
            self._plan_splits[key] = self.S if tiles is None else min(self.S, splits_for(self.B, tiles, n_kv_heads))
            self._plan_keys.append(key)
            self._alloc()
            self.fill(*self._last)
        return self._plans[key]

    # ------------------------------------------------------------------ per step
    def fill(self, entries: List[StepEntry], rcs, token_source: Optional[torch.Tensor] = None) -> None:
        """Write this step's data into the pinned buffer and copy it to the device; the tokens
        come from ``token_source`` (on the device) if there is one."""
        if self._copied is not None:
            self._copied.synchronize()          # the last copy has read the pinned buffer
        self._last = (entries, rcs, token_source)
        self.shared.clear()
        B, S, o = self.B, self.S, self._offs
        n = len(entries)
        h = self._host.numpy()
        starts = np.zeros(B, dtype=np.int32)
        starts[:n] = [rc.n_tokens for rc in rcs]
        tok = np.zeros(B, dtype=np.int32)
        tok[:n] = [e.tokens[0] for e in entries]
        h[o[0]:o[1]] = tok
        h[o[1]:o[2]] = starts
        h[o[2]:o[3]] = np.arange(B, dtype=np.int32)
        h[o[3]:o[4]] = np.arange(B + 1, dtype=np.int32)
        h[o[4]:o[5]] = starts + 1
        slots = np.full(B, self.null_slot, dtype=np.int32)
        slots[:n] = [rc.slot for rc in rcs]
        h[o[5]:o[6]] = slots
        h[o[6]:o[7]] = 0
        h[o[7]:o[8]] = starts
        h[o[8]:o[9]] = np.arange(B, dtype=np.int32)
        for g, w in enumerate(self.table_width):
            tab = h[o[9 + g]:o[10 + g]].reshape(B, w)
            held = self._rows[g]
            for b in range(B):
                rc = rcs[b] if b < n else None
                if rc is None:
                    if held[b] is not None:
                        tab[b, :] = -1
                        tab[b, 0] = NULL_PAGE
                        held[b] = None
                    continue
                t = rc.tables[g]
                # a table only grows at its end while its request lives, unless a window gives pages
                # back or a step that failed gave back what it had reserved (which `version` counts)
                if (not self.windowed[g] and held[b] is not None and held[b][0] is rc
                        and held[b][1] == len(t) and held[b][2] == rc.version):
                    continue
                if len(t) > w:
                    raise ValueError("a request outgrew the block table of its graph bucket")
                tab[b, :] = -1
                tab[b, 0] = NULL_PAGE
                tab[b, :len(t)] = t
                held[b] = (rc, len(t), rc.version)
        self.starts = [int(s) for s in starts]
        self.seq_lens = [s + 1 for s in self.starts]
        self.max_seq_len = max(self.seq_lens)
        for key in self._plan_keys:
            self._fill_plan(h, self._plan_off[key], key, starts)
        self._dev.copy_(self._host, non_blocking=True)
        ev = torch.cuda.Event()
        ev.record()
        self._copied = ev
        if token_source is not None:
            self.token_ids[:n].copy_(token_source)

    def _fill_plan(self, h, base: int, key, starts) -> None:
        group_size, window, _ = key
        B, S = self.B, self._plan_splits[key]
        items = h[base:base + B * S * 8].reshape(B, S, 8)
        jobs = h[base + B * S * 8:base + B * S * 8 + B * 7].reshape(B, 7)
        hi = starts.astype(np.int64) + 1                          # keys [lo, hi)
        lo = np.zeros(B, dtype=np.int64)
        if window:
            lo = np.maximum(0, starts.astype(np.int64) - window + 1)
        lo = (lo // ATTN_TILE) * ATTN_TILE
        tiles = -(-(hi - lo) // ATTN_TILE)
        per = np.maximum(1, -(-tiles // S)) * ATTN_TILE           # keys per range
        s_idx = np.arange(S, dtype=np.int64)[None, :]
        kb = lo[:, None] + s_idx * per[:, None]
        ke = np.minimum(hi[:, None], kb + per[:, None])
        empty = kb >= ke
        kb = np.where(empty, 0, kb)
        ke = np.where(empty, 0, ke)
        items[:, :, 0] = np.arange(B)[:, None]
        items[:, :, 1] = 0
        items[:, :, 2] = kb
        items[:, :, 3] = ke
        items[:, :, 4] = (np.arange(B)[:, None] * S + s_idx) if S > 1 else -1
        items[:, :, 5] = np.arange(B)[:, None]
        items[:, :, 6] = 1
        items[:, :, 7] = starts[:, None]
        jobs[:, 0] = np.arange(B)
        jobs[:, 1] = 0
        jobs[:, 2] = np.arange(B) * S
        jobs[:, 3] = S
        jobs[:, 4] = 1
        jobs[:, 5] = np.arange(B)
        jobs[:, 6] = 1


class DecodeGraphs:
    """Captured decode steps of one ``ModelRunner``, by bucket."""

    def __init__(self, runner):
        self.runner = runner
        self.graphs: Dict[Tuple[int, int, int], Tuple[StaticDecodeContext, torch.cuda.CUDAGraph, torch.Tensor]] = {}
        self.pool = None
        kv, st, _ = runner.model.cache_needs()
        # parts that look at their data on the host are served eagerly (`capturable` False)
        self.usable = runner.model.capturable()
        # the bucket's number of key ranges is that of the group with the fewest key/value heads
        # (the one that needs most ranges to fill the chip); every plan then takes what it needs
        self.kv_heads = min((k.num_kv_heads for k in kv if k is not None), default=1)
        self.replays = 0
        self.captures = 0

    def applies(self, entries: List[StepEntry]) -> bool:
        return self.usable and all(len(e.tokens) == 1 for e in entries) and bucket_for(len(entries)) is not None

    def run(self, entries: List[StepEntry], rcs, token_source: Optional[torch.Tensor] = None) -> torch.Tensor:
        """Logits ``[len(entries), V]`` of a step of single tokens (pages are reserved already).
        ``token_source``: the tokens, on the device (the entries' own are placeholders)."""
        r = self.runner
        n = len(entries)
        cap = bucket_for(n)
        max_len = max(rc.n_tokens for rc in rcs) + 1
        # block tables as wide as the longest request needs, in steps of 32 pages
        pages = max(max(len(t) for t in rc.tables) for rc in rcs) if r.manager.groups else 1
        w = -(-max(1, pages) // 32) * 32
        width = [w] * len(r.manager.groups)
        S = splits_for(cap, -(-max_len // ATTN_TILE), self.kv_heads)
        key = (cap, S, w)
        hit = self.graphs.get(key)
        if hit is not None:
            ctx, graph, logits = hit
            ctx.fill(entries, rcs, token_source)
            graph.replay()
            self.replays += 1
            return logits[:n]
        # first time: run the step eagerly on the static context, then record it for later
        ctx = StaticDecodeContext(r.ops, r.device, cap, S, width,
                                  windowed=[g.spec.window is not None for g in r.manager.groups],
                                  max_tiles=-(-max_len // ATTN_TILE), null_slot=r.storage.null_slot)
        ctx.fill(entries, rcs, token_source)
        x = r.model.forward(ctx, r.storage.layers)
        out = r.model.logits(ctx, x, ctx.want_rows)
        torch.cuda.synchronize()
        graph = torch.cuda.CUDAGraph()
        # No garbage collection while the stream records: an earlier step's context that a
        # collection frees gives back pinned memory, which is no operation a recording allows
        # (the process aborts).  Cycles are collected before, and again afterwards as usual.
        gc.collect()
        gc_was_on = gc.isenabled()
        gc.disable()
        ctx.shared.clear()          # what the eager pass left is not part of the recording
        try:
            with torch.cuda.graph(graph, pool=self.pool):
                gx = r.model.forward(ctx, r.storage.layers)
                glogits = r.model.logits(ctx, gx, ctx.want_rows)
        finally:
            if gc_was_on:
                gc.enable()
        if self.pool is None:
            self.pool = graph.pool()
        ctx.shared.clear()          # a table made while recording belongs to the graph's memory
        self.graphs[key] = (ctx, graph, glogits)
        self.captures += 1
        return out[:n]
