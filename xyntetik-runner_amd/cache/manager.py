"""The cache manager: which pages and which state slot each live request holds.

Keys and values live in pages of ``page_size`` positions.  Layers whose needs are
equal (``KVSpec``: heads, head size, all keys or a window of them) form a *group*;
a group has a pool of pages of its own and every request has one block table per
group: entry ``i`` is the page that holds positions ``[i*page_size, (i+1)*page_size)``,
or -1 once a window has passed it.  Beside the pages every request holds one *slot*
for state of fixed size (zeroed by the step function before its first use), whether
or not any layer has such state.

The reference keeps one contiguous cache per sequence and never gives rows back
while the process lives (src/model.c:3089-3101, :3351-3354); what it
does promise is kept here per request: row i of a request is a function of its
tokens [0, i] only (src/engine.c:218-221) and the tokens recorded for
a request are exactly those whose rows are cached (src/engine.c:852-861).

Page 0 of every group is never handed out: padded rows of a batch write there.
This file is pure host logic; ``storage.py`` owns the device tensors.
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Dict, Hashable, List, Optional, Sequence, Union

from ..parts.base import KVSpec
from .pages import OutOfPages, Pool

NULL_PAGE = 0


@dataclass
class GroupInfo:
    spec: KVSpec
    page_size: int
    pool: Pool


@dataclass
class RequestCache:
    req_id: Hashable
    slot: int
    n_tokens: int = 0                      # positions [0, n_tokens) are cached
    tables: List[List[int]] = field(default_factory=list)   # one block table per group
    fresh: bool = True                     # the slot has not been used by this request yet
    version: int = 0                       # counts the times a table lost pages at its end (`trim`)


def first_needed_position(n_tokens: int, window: Optional[int]) -> int:
    """The lowest position a query at position ``n_tokens`` (the next one) can still read."""
    if window is None:
        return 0
    return max(0, n_tokens - window + 1)


def pages_for_spec(spec: KVSpec, page_size: int, max_tokens: int, max_requests: int,
                   max_step_tokens: Optional[int] = None) -> int:
    """How many pages a group needs so that ``max_requests`` requests holding ``max_tokens`` tokens
    together can run steps of up to ``max_step_tokens`` tokens (None: of any size).

    A group that keeps every key needs the tokens' pages.  A group that keeps a window needs, for
    every request, the pages its window touches plus the one being filled and the one not yet
    given back, and, over all requests of a step, the pages of the step's tokens: a portion's pages
    are all held until the portion is cached.
    """
    full = max(1, -(-int(max_tokens) // page_size))
    if spec.window is None or max_step_tokens is None:
        return full
    per_request = -(-spec.window // page_size) + 2
    return min(full, max_requests * per_request + -(-int(max_step_tokens) // page_size))


class CacheManager:
    def __init__(self, group_specs: Sequence[KVSpec], page_size: int, pages_per_group: Union[int, Sequence[int]],
                 n_slots: int):
        """``pages_per_group``: one number for all groups or one per group (see ``pages_for_spec``)."""
        if page_size < 1 or page_size & (page_size - 1):
            raise ValueError(f"page size {page_size} must be a power of two")
        sizes = [pages_per_group] * len(group_specs) if isinstance(pages_per_group, int) else list(pages_per_group)
        if len(sizes) != len(group_specs):
            raise ValueError(f"{len(sizes)} pool sizes for {len(group_specs)} groups")
        if any(n < 1 for n in sizes) or (isinstance(pages_per_group, int) and pages_per_group < 1):
            raise ValueError("a group needs at least one page")
        self.page_size = page_size
        self.groups = [GroupInfo(s, page_size, Pool(n, first=1, what="page")) for s, n in zip(group_specs, sizes)]
        self.slots = Pool(n_slots, what="state slot")
        self.requests: Dict[Hashable, RequestCache] = {}
        self._no_pages = [0] * len(self.groups)
        self._windowed = [gi for gi, g in enumerate(self.groups) if g.spec.window is not None]

    # ------------------------------------------------------------------ sizes
    @property
    def pages_per_group(self) -> int:
        """The pool size of the first group (of every group, when they were given one number)."""
        return self.groups[0].pool.size if self.groups else 0

    def all_free(self) -> bool:
        """No page of any group and no state slot is out."""
        return all(g.pool.n_out == 0 for g in self.groups) and self.slots.n_out == 0

    def capacity_tokens(self) -> int:
        """The most tokens one request can hold: what the smallest pool of a group that keeps every
        key holds.  A group that keeps a window gives pages back as a request grows and sets no limit."""
        full = [g.pool.size * self.page_size for g in self.groups if g.spec.window is None]
        return min(full) if full else 1 << 62

    def max_portion(self) -> int:
        """The most tokens of one request that a step can run, whatever its length: the pages of a
        windowed group must hold the window behind the portion's first token and the portion
        (groups that keep every key limit a request's length, not its portions)."""
        best = 1 << 62
        for g in self.groups:
            if g.spec.window is not None:
                behind = -(-g.spec.window // self.page_size) + 1
                best = min(best, max(1, (g.pool.size - behind) * self.page_size))
        return best

    def pages_for(self, n_tokens: int) -> int:
        return -(-n_tokens // self.page_size)

    def free_pages(self, group: int = 0) -> int:
        return self.groups[group].pool.n_free

    # ------------------------------------------------------------------ life of a request
    def admit(self, req_id: Hashable) -> RequestCache:
        if req_id in self.requests:
            raise ValueError(f"request {req_id!r} is already live")
        slot = self.slots.take()            # OutOfPages if every slot is taken
        rc = RequestCache(req_id, slot, 0, [[] for _ in self.groups])
        self.requests[req_id] = rc
        return rc

    def can_admit(self) -> bool:
        return self.slots.n_free > 0

    def _new_pages_needed(self, rc: RequestCache, new_len: int) -> List[int]:
        want = self.pages_for(new_len)
        for t in rc.tables:
            if len(t) < want:
                break
        else:
            return self._no_pages           # the usual case of a decoded token (callers only read it)
        need = []
        for gi, g in enumerate(self.groups):
            have = len(rc.tables[gi])
            # pages wholly below the window of the first new query are never read or written
            lo_page = first_needed_position(rc.n_tokens, g.spec.window) // self.page_size
            need.append(sum(1 for i in range(have, want) if i >= lo_page))
        return need

    def can_reserve(self, req_id: Hashable, new_len: int, spare: Optional[List[int]] = None) -> bool:
        """Whether ``reserve`` would succeed; ``spare`` pages per group are treated as already spoken for."""
        rc = self.requests[req_id]
        need = self._new_pages_needed(rc, new_len)
        for gi, g in enumerate(self.groups):
            if need[gi] > g.pool.n_free - (spare[gi] if spare else 0):
                return False
        return True

    def pages_needed(self, req_id: Hashable, new_len: int) -> List[int]:
        return self._new_pages_needed(self.requests[req_id], new_len)

    def pages_needed_new(self, new_len: int) -> List[int]:
        """Pages per group that a request not yet admitted needs for its first ``new_len`` tokens
        (all of them: a window gives pages back only once the tokens are cached)."""
        return [self.pages_for(new_len)] * len(self.groups)

    def trim(self, req_id: Hashable) -> None:
        """Give back the pages reserved beyond the tokens the request holds (for a step that
        reserved and then did not run)."""
        rc = self.requests[req_id]
        keep = self.pages_for(rc.n_tokens)
        for gi, g in enumerate(self.groups):
            table = rc.tables[gi]
            while len(table) > keep:
                page = table.pop()
                rc.version += 1             # who copied the table must not take its length for its contents
                if page >= 0:
                    g.pool.give(page)

    def reserve(self, req_id: Hashable, new_len: int) -> None:
        """Make positions ``[n_tokens, new_len)`` writable in every group, or raise and change nothing."""
        rc = self.requests[req_id]
        if new_len < rc.n_tokens:
            raise ValueError(f"request {req_id!r} holds {rc.n_tokens} tokens, cannot shrink to {new_len}")
        need = self._new_pages_needed(rc, new_len)
        if need is self._no_pages:
            return
        for gi, g in enumerate(self.groups):
            if need[gi] > g.pool.n_free:
                raise OutOfPages(f"request {req_id!r} needs {need[gi]} more pages in group {gi}, "
                                 f"{g.pool.n_free} of {g.pool.size} free")
        for gi, g in enumerate(self.groups):
            table = rc.tables[gi]
            lo_page = first_needed_position(rc.n_tokens, g.spec.window) // self.page_size
            for i in range(len(table), self.pages_for(new_len)):
                table.append(g.pool.take() if i >= lo_page else -1)

    def advance(self, req_id: Hashable, new_len: int) -> None:
        """Positions below ``new_len`` are now cached; give back pages a window has passed."""
        rc = self.requests[req_id]
        if self.pages_for(new_len) > min((len(t) for t in rc.tables), default=self.pages_for(new_len)):
            raise ValueError(f"request {req_id!r}: {new_len} tokens were not reserved")
        rc.n_tokens = new_len
        rc.fresh = False
        for gi in self._windowed:
            g = self.groups[gi]
            lo_page = first_needed_position(new_len, g.spec.window) // self.page_size
            table = rc.tables[gi]
            for i in range(min(lo_page, len(table))):
                if table[i] >= 0:
                    g.pool.give(table[i])
                    table[i] = -1

    def release(self, req_id: Hashable) -> None:
        """The request is over (finished or preempted): everything it holds goes back."""
        rc = self.requests.pop(req_id)
        for gi, g in enumerate(self.groups):
            for p in rc.tables[gi]:
                if p >= 0:
                    g.pool.give(p)
        self.slots.give(rc.slot)

    # ------------------------------------------------------------------ views
    def get(self, req_id: Hashable) -> RequestCache:
        return self.requests[req_id]

    def tokens_held(self) -> int:
        return sum(rc.n_tokens for rc in self.requests.values())

    def check(self) -> None:
        """No page lost, held twice or freed twice; tables cover exactly what each request holds."""
        for gi, g in enumerate(self.groups):
            g.pool.check()
            held = [p for rc in self.requests.values() for p in rc.tables[gi] if p >= 0]
            if len(held) != len(set(held)):
                raise AssertionError(f"group {gi}: a page is in two block tables")
            if set(held) != g.pool._out:
                raise AssertionError(f"group {gi}: pages out {sorted(g.pool._out)} differ from pages in tables {sorted(held)}")
            if NULL_PAGE in held:
                raise AssertionError("the null page is in a block table")
        self.slots.check()
        slots = [rc.slot for rc in self.requests.values()]
        if len(slots) != len(set(slots)) or set(slots) != self.slots._out:
            raise AssertionError("state slots out differ from state slots held")
        for rc in self.requests.values():
            for gi, g in enumerate(self.groups):
                lo = first_needed_position(rc.n_tokens, g.spec.window)
                for pos in range(lo, rc.n_tokens):
                    if rc.tables[gi][pos // self.page_size] < 0:
                        raise AssertionError(f"request {rc.req_id!r}: position {pos} of group {gi} has no page")
