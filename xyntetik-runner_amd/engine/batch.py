"""One step's batch as the kernels see it.

A step is a list of entries (request, its next tokens, the places whose logits are
wanted).  All tokens of all entries are laid out one after another ("rows"); per
row the device gets its token id, its position in its request and the index of its
request in this batch; per request and cache group the block table.  One pinned
host buffer carries all of it to the device in a single copy.

The reference has two narrower primitives, n consecutive tokens of one sequence
(src/model.h:667-670) and one token each of up to 8 sequences with
per-column position and cache pointers (src/model.h:796-807,
src/cuda.c:4213-4236); an entry list covers both and their mixtures.
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Hashable, List, Optional, Sequence

import numpy as np
import torch


@dataclass
class AttentionPlan:
    """The work list of the MFMA attention kernel for one step, cache group, group size and window.

    ``items [c + n, 8]`` int32 on the device: request, first row of a row block, first key,
    end key, partial slot (-1: the item covers all keys of its block and writes the output),
    the request's first row in the step, its number of tokens, its first position.  The first
    ``n_cta_items`` are blocks of 128 rows that a workgroup takes together (its wave w the rows
    from ``row0 + 32 w``, with partial slot ``slot + w``), the other ``n_items`` blocks of 32
    rows, one wave each.
    ``jobs [m, 7]``: request, first row of 32, first slot, number of slots to merge, the
    distance between them, the request's first row in the step and its number of tokens.
    """
    items: torch.Tensor
    n_items: int
    jobs: Optional[torch.Tensor]
    n_jobs: int
    n_slots: int
    n_cta_items: int = 0


# The first four are the attention kernels' shapes.  The last three are tuning, not limits: they
# say how much work gives every one of an MI355X's 256 compute units a workgroup, measured on the
# 8B shape's attention; on another chip or shape they cost speed, never correctness.
ATTN_ROWS = 32          # query rows (token x head-in-group) per work item
ATTN_TILE = 32          # keys per tile; items begin and end on tile edges
ATTN_CTA_ROWS = 128     # rows of an item that a whole workgroup takes
ATTN_CTA_MIN_ROWS = 64  # a request brings at least this many rows to be served by workgroups
ATTN_STREAM_SLOTS = 256 # workgroups of the streaming kernel that run at a time (one a compute unit)
ATTN_MIN_RANGE = 4      # tiles: the shortest key range worth a workgroup
ATTN_CTA_FILL = 256     # 128-row items (times key/value heads) that give every compute unit one workgroup


def key_ranges(tiles: int, share: float) -> int:
    """Into how many key ranges a 32-row block of ``tiles`` tiles is cut, given its share of
    the workgroups that run at a time.

    Measured on MI355X (batch 1-64, 2k and 8k context): the streaming kernel is fastest with
    one round of workgroups and ranges as long as that allows; a range under 4 tiles costs more
    to start and to merge than to run.
    """
    return max(1, min(int(share), tiles // ATTN_MIN_RANGE))


def plan_attention(starts, q_lens, group_size: int, window: Optional[int], n_kv_heads: int,
                   page_size: int = 64, cta_tiles: Optional[int] = None):
    """Host side of ``AttentionPlan``: ``(cta_items, items, jobs, n_slots)`` as plain Python ints.

    ``cta_tiles`` fixes the most tiles a 128-row item may cover (for measurements); by
    default it follows from how many such items the step has.
    """
    blocks, cta_blocks = [], []
    total_tiles = 0
    q0s, acc = [], 0
    for n in q_lens:
        q0s.append(acc)
        acc += n

    def key_range(s, n, row0, rows):
        tok_lo = row0 // group_size
        tok_hi = min(n - 1, (row0 + rows - 1) // group_size)
        lo = 0 if not window else max(0, s + tok_lo - window + 1)
        lo = (lo // ATTN_TILE) * ATTN_TILE
        hi = s + tok_hi + 1
        return lo, hi, -(-(hi - lo) // ATTN_TILE)

    for b, (s, n) in enumerate(zip(starts, q_lens)):
        rows = n * group_size
        if rows >= ATTN_CTA_MIN_ROWS and page_size >= ATTN_TILE:
            for row0 in range(0, rows, ATTN_CTA_ROWS):
                cta_blocks.append((b, row0) + key_range(s, n, row0, ATTN_CTA_ROWS))
            continue
        for row0 in range(0, rows, ATTN_ROWS):
            blk = (b, row0) + key_range(s, n, row0, ATTN_ROWS)
            blocks.append(blk)
            total_tiles += blk[4]
    items, cta_items, jobs, slot = [], [], [], 0
    # longest first: workgroups are started in list order, and a long item started last
    # would run on alone at the end
    cta_blocks.sort(key=lambda blk: -blk[4])
    blocks.sort(key=lambda blk: -blk[4])

    if cta_blocks:
        chunk = cta_tiles
        if chunk is None:
            # A workgroup (two sets of four waves) fills a compute unit.  Whole blocks when they give
            # at least half the units one each: the merge of split blocks costs more than the units
            # left idle (512 tokens after 4,096, 8 key/value heads: 86 us whole, 86 us in ranges of
            # 32 tiles, 101 us in ranges of 16; 512 tokens from 0: 17 us whole, 26 us split).
            # Fewer blocks are cut into about as many ranges as there are units (128 tokens after
            # 8,000: 145 us whole, 44 us in ranges of 32 tiles, 58 us in ranges of 16).
            if len(cta_blocks) * n_kv_heads >= ATTN_CTA_FILL // 2:
                chunk = 1 << 30
            else:
                work = sum(blk[4] for blk in cta_blocks)
                chunk = max(8, -(-work * n_kv_heads // ATTN_CTA_FILL))
        for b, row0, lo, hi, tiles in cta_blocks:
            parts = -(-tiles // chunk)
            if parts <= 1:
                cta_items.append((b, row0, lo, hi, -1, q0s[b], q_lens[b], starts[b]))
                continue
            per = -(-tiles // parts)
            first = slot
            k = lo
            while k < hi:
                e = min(hi, k + per * ATTN_TILE)
                cta_items.append((b, row0, k, e, slot, q0s[b], q_lens[b], starts[b]))
                slot += ATTN_CTA_ROWS // ATTN_ROWS
                k = e
            n_parts = (slot - first) // (ATTN_CTA_ROWS // ATTN_ROWS)
            rows = q_lens[b] * group_size
            for w in range(ATTN_CTA_ROWS // ATTN_ROWS):
                if row0 + w * ATTN_ROWS < rows:
                    jobs.append((b, row0 + w * ATTN_ROWS, first + w, n_parts, ATTN_CTA_ROWS // ATTN_ROWS, q0s[b], q_lens[b]))

    budget = max(1, ATTN_STREAM_SLOTS // n_kv_heads)       # items that run at a time
    for b, row0, lo, hi, tiles in blocks:
        parts = 1 if len(blocks) >= budget else key_ranges(tiles, budget * tiles / total_tiles)
        if parts <= 1:
            items.append((b, row0, lo, hi, -1, q0s[b], q_lens[b], starts[b]))
            continue
        per = -(-tiles // parts)
        first = slot
        k = lo
        while k < hi:
            e = min(hi, k + per * ATTN_TILE)
            items.append((b, row0, k, e, slot, q0s[b], q_lens[b], starts[b]))
            slot += 1
            k = e
        jobs.append((b, row0, first, slot - first, 1, q0s[b], q_lens[b]))
    return cta_items, items, jobs, slot


@dataclass
class StepEntry:
    req_id: Hashable
    tokens: Sequence[int]
    want: Sequence[int] = ()        # indices into ``tokens`` whose logits are wanted


class StepContext:
    """Device views of one step's metadata, handed to every part."""

    def __init__(self, ops, device, entries: List[StepEntry], request_caches, n_groups: int, pad_to: int = 0):
        self.ops = ops
        self.device = device
        self.entries = entries
        B = len(entries)
        q_lens = [len(e.tokens) for e in entries]
        T = sum(q_lens)
        self.B, self.T = B, T
        self.q_lens = q_lens
        self.starts = [rc.n_tokens for rc in request_caches]            # position of each entry's first token
        self.seq_lens = [s + n for s, n in zip(self.starts, q_lens)]    # length after this step
        self.max_q_len = max(q_lens) if q_lens else 0
        self.max_seq_len = max(self.seq_lens) if B else 0
        nb = [max((len(rc.tables[g]) for rc in request_caches), default=0) for g in range(n_groups)]
        self.table_width = [max(1, w) for w in nb]
        want_rows: List[int] = []
        row0 = 0
        for e, n in zip(entries, q_lens):
            for w in e.want:
                if not (0 <= w < n):
                    raise ValueError(f"request {e.req_id!r}: wanted place {w} is outside its {n} tokens")
                want_rows.append(row0 + w)
            row0 += n
        self.n_want = len(want_rows)

        # ---- pack: [token_ids T][positions T][req_of_token T][cu_q B+1][seq_lens B][slots B][fresh B]
        #            [want W][table g: B * width_g]...
        sizes = [T, T, T, B + 1, B, B, B + B, self.n_want] + [B * w for w in self.table_width]
        offs = np.concatenate([[0], np.cumsum(sizes)]).astype(np.int64)
        total = int(offs[-1])
        host = torch.empty((max(total, 1),), dtype=torch.int32, pin_memory=True)
        h = host.numpy()
        tok, pos, rot = h[offs[0]:offs[1]], h[offs[1]:offs[2]], h[offs[2]:offs[3]]
        cu = h[offs[3]:offs[4]]
        cu[0] = 0
        r = 0
        for b, (e, n) in enumerate(zip(entries, q_lens)):
            tok[r:r + n] = np.asarray(e.tokens, dtype=np.int64).astype(np.int32)
            pos[r:r + n] = np.arange(self.starts[b], self.starts[b] + n, dtype=np.int32)
            rot[r:r + n] = b
            r += n
            cu[b + 1] = r
        h[offs[4]:offs[5]] = self.seq_lens
        h[offs[5]:offs[6]] = [rc.slot for rc in request_caches]
        h[offs[6]:offs[6] + B] = [1 if rc.fresh else 0 for rc in request_caches]
        h[offs[6] + B:offs[7]] = self.starts
        h[offs[7]:offs[8]] = want_rows
        for g in range(n_groups):
            w = self.table_width[g]
            tab = h[offs[8 + g]:offs[9 + g]].reshape(B, w)
            tab[:] = -1
            for b, rc in enumerate(request_caches):
                t = rc.tables[g]
                tab[b, :len(t)] = t
        dev = host.to(device, non_blocking=True)
        self._host = host      # keep the pinned buffer alive until the copy has run
        self.token_ids = dev[offs[0]:offs[1]]
        self.positions = dev[offs[1]:offs[2]]
        self.req_of_token = dev[offs[2]:offs[3]]
        self.cu_q = dev[offs[3]:offs[4]]
        self.seq_lens_dev = dev[offs[4]:offs[5]]
        self.slots = dev[offs[5]:offs[6]]
        self.fresh = dev[offs[6]:offs[6] + B]
        self.starts_dev = dev[offs[6] + B:offs[7]]
        self.want_rows = dev[offs[7]:offs[8]]
        self._tables = [dev[offs[8 + g]:offs[9 + g]].view(B, self.table_width[g]) for g in range(n_groups)]
        self.fresh_slots_host = [rc.slot for rc in request_caches if rc.fresh]
        self.slots_host = [rc.slot for rc in request_caches]
        self._plans = {}
        self.shared = {}        # what parts make once a step and share between layers (a rotation's table)

    def attention_plan(self, group: int, group_size: int, window: Optional[int], n_kv_heads: int,
                       page_size: int = 64) -> AttentionPlan:
        """The MFMA attention work list, made once per step and shared by all layers that can."""
        key = (group_size, window, n_kv_heads, page_size)
        plan = self._plans.get(key)
        if plan is None:
            cta_items, items, jobs, n_slots = plan_attention(self.starts, self.q_lens, group_size, window,
                                                             n_kv_heads, page_size)
            flat = [v for it in cta_items + items for v in it] + [v for j in jobs for v in j]
            host = torch.tensor(flat, dtype=torch.int32).pin_memory()
            dev = host.to(self.device, non_blocking=True)
            nc, ni, nj = len(cta_items), len(items), len(jobs)
            nw = (nc + ni) * 8
            plan = AttentionPlan(dev[:nw], ni, dev[nw:] if nj else None, nj, n_slots, nc)
            plan._host = host
            self._plans[key] = plan
        return plan

    def block_table(self, group: int) -> torch.Tensor:
        """``[B, width]`` int32: page of each block of each request of this step, -1 where none."""
        return self._tables[group]
