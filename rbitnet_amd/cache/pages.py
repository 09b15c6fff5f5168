"""Bookkeeping of the cache on the host: which slots and pages are free, which
sequence holds which pages.  Pure Python, no GPU: the whole of it is testable
without one.

A *slot* belongs to one sequence from `alloc` to `free`: it carries the sequence's
length and indexes its fixed-size state.  A *page* holds the keys and values of
PAGE_SIZE consecutive positions; a sequence of length n holds ceil(n / PAGE_SIZE)
pages per storage group (fewer behind a window).  Both are handed out lowest id
first and reused after they are given back.  Holding something twice, giving it
back twice and asking for more than there is are errors, never silent.
"""
from __future__ import annotations

import heapq
from typing import Dict, List, Optional

from ..errors import CacheError

PAGE_SIZE = 64


def pages_for(n_tokens: int) -> int:
    return (n_tokens + PAGE_SIZE - 1) // PAGE_SIZE


class FreeList:
    """Ids 0..n-1, lowest free id first."""

    def __init__(self, n: int, what: str):
        self.n = int(n)
        self.what = what
        self._free = list(range(self.n))
        heapq.heapify(self._free)
        self._held = set()

    @property
    def n_free(self) -> int:
        return len(self._free)

    @property
    def n_held(self) -> int:
        return len(self._held)

    def held(self) -> List[int]:
        return sorted(self._held)

    def take(self) -> int:
        if not self._free:
            raise CacheError(f"no free {self.what} left (all {self.n} are in use)")
        i = heapq.heappop(self._free)
        self._held.add(i)
        return i

    def give_back(self, i: int) -> None:
        if not 0 <= i < self.n:
            raise CacheError(f"{self.what} {i} does not exist (there are {self.n})")
        if i not in self._held:
            raise CacheError(f"{self.what} {i} is not in use (freed twice?)")
        self._held.remove(i)
        heapq.heappush(self._free, i)

    def check(self) -> None:
        """No id lost, none both free and held, none twice."""
        free = sorted(self._free)
        if len(set(free)) != len(free):
            raise CacheError(f"a {self.what} is in the free list twice")
        if set(free) & self._held:
            raise CacheError(f"a {self.what} is both free and in use")
        if len(free) + len(self._held) != self.n:
            raise CacheError(f"a {self.what} was lost: {len(free)} free + {len(self._held)} held != {self.n}")


class PageTable:
    """The pages of each slot for one storage group.  Logical page i of a slot covers
    positions [i * PAGE_SIZE, (i + 1) * PAGE_SIZE).  With a window, pages that lie wholly
    behind every future query's reach are given back early; their entries stay in the
    table as -1 and are never read."""

    def __init__(self, n_pages: int, window: Optional[int] = None):
        self.pool = FreeList(n_pages, "cache page")
        self.window = window
        self.tables: Dict[int, List[int]] = {}

    def open(self, slot: int) -> None:
        if slot in self.tables:
            raise CacheError(f"slot {slot} already has a page table")
        self.tables[slot] = []

    def ensure(self, slot: int, n_tokens: int) -> bool:
        """Make the slot's pages cover positions < n_tokens.  True if pages were added.
        All or nothing: when the pool runs out, the pages taken so far go back."""
        table = self.tables[slot]
        need = pages_for(n_tokens) - len(table)
        if need <= 0:
            return False
        if need > self.pool.n_free:
            raise CacheError(
                f"cache full: slot {slot} needs {need} more pages of {PAGE_SIZE} tokens, "
                f"{self.pool.n_free} of {self.pool.n} are free")
        for _ in range(need):
            table.append(self.pool.take())
        return True

    def release_behind(self, slot: int, length: int) -> int:
        """With a window w, a query at position p >= length reads keys > p - w, so keys
        below length - w + 1 are dead.  Returns how many pages were given back."""
        if self.window is None:
            return 0
        dead_pages = max(0, length - self.window + 1) // PAGE_SIZE
        table = self.tables[slot]
        n = 0
        for i in range(min(dead_pages, len(table))):
            if table[i] >= 0:
                self.pool.give_back(table[i])
                table[i] = -1
                n += 1
        return n

    def close(self, slot: int) -> None:
        if slot not in self.tables:
            raise CacheError(f"slot {slot} has no page table (freed twice?)")
        for p in self.tables.pop(slot):
            if p >= 0:
                self.pool.give_back(p)

    def pages(self, slot: int) -> List[int]:
        return self.tables[slot]

    def check(self) -> None:
        self.pool.check()
        seen = set()
        for slot, table in self.tables.items():
            for p in table:
                if p < 0:
                    continue
                if p in seen:
                    raise CacheError(f"page {p} is held twice")
                seen.add(p)
        if seen != set(self.pool.held()):
            raise CacheError("pages in the tables and pages marked held differ")
