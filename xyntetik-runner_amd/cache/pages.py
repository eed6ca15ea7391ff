"""Pools of numbered resources: cache pages and state slots.

A pool hands out ids from a free list and takes them back; the id most recently
given back is handed out next, so a page is used again soon after it is freed.
An id is never out twice, and giving back an id that is not out is an error.
"""
from __future__ import annotations

from typing import List


class OutOfPages(RuntimeError):
    """The pool cannot cover what was asked; nothing was taken."""


class Pool:
    def __init__(self, size: int, first: int = 0, what: str = "page"):
        if size < 0:
            raise ValueError(f"a pool of {size} {what}s")
        self.size, self.first, self.what = size, first, what
        # ids first .. first+size-1; the lowest id is handed out first
        self._free: List[int] = list(range(first + size - 1, first - 1, -1))
        self._out = set()

    @property
    def n_free(self) -> int:
        return len(self._free)

    @property
    def n_out(self) -> int:
        return len(self._out)

    def take(self) -> int:
        if not self._free:
            raise OutOfPages(f"no free {self.what} (all {self.size} are in use)")
        i = self._free.pop()
        self._out.add(i)
        return i

    def take_many(self, n: int) -> List[int]:
        if n > len(self._free):
            raise OutOfPages(f"{n} {self.what}s wanted, {len(self._free)} of {self.size} free")
        return [self.take() for _ in range(n)]

    def give(self, i: int) -> None:
        if i not in self._out:
            raise ValueError(f"{self.what} {i} is given back but is not out")
        self._out.remove(i)
        self._free.append(i)

    def check(self) -> None:
        """No id lost, none held twice."""
        free = set(self._free)
        if len(free) != len(self._free):
            raise AssertionError(f"a {self.what} is on the free list twice")
        if free & self._out:
            raise AssertionError(f"{self.what}s {sorted(free & self._out)} are both free and out")
        everything = set(range(self.first, self.first + self.size))
        if free | self._out != everything:
            raise AssertionError(f"{self.what}s {sorted(everything - free - self._out)} are lost")
