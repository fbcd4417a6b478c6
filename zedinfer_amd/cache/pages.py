"""Fixed pools of pages and of state slots, with O(1) take and give back.

The reference's pool scans for a free block (reference:
src/backend/kvcache/block_pool.cpp:78-103) and keeps reference counts for its
prefix cache; here there is no sharing, so a pool is a stack of free ids.  The
stack is last-in first-out: a page given back is the next one handed out.
"""
from __future__ import annotations

from typing import List


class OutOfPages(RuntimeError):
    """The pool cannot give (or promise) the pages asked for."""


class OutOfSlots(RuntimeError):
    """Every per-request state slot is taken."""


class IdPool:
    """``total`` ids, each either free or held.  Taking from an empty pool, giving back an id
    that is not held, or an id out of range, raises."""

    def __init__(self, total: int, what: str = "page"):
        if total < 0:
            raise ValueError(f"{what} pool size must be non-negative")
        self.total = int(total)
        self.what = what
        self._free: List[int] = list(range(self.total - 1, -1, -1))  # id 0 is handed out first
        self._held = bytearray(self.total)
        self.takes = 0      # ids handed out so far; more than `total` means ids were used again

    @property
    def num_free(self) -> int:
        return len(self._free)

    @property
    def num_held(self) -> int:
        return self.total - len(self._free)

    def take(self) -> int:
        if not self._free:
            raise (OutOfPages if self.what == "page" else OutOfSlots)(f"no free {self.what} (pool of {self.total})")
        i = self._free.pop()
        self._held[i] = 1
        self.takes += 1
        return i

    def give_back(self, i: int) -> None:
        if not (0 <= i < self.total):
            raise ValueError(f"{self.what} {i} is outside the pool of {self.total}")
        if not self._held[i]:
            raise ValueError(f"{self.what} {i} is given back but not held")
        self._held[i] = 0
        self._free.append(i)

    def is_held(self, i: int) -> bool:
        return bool(self._held[i])

    def check(self) -> None:
        """free + held == total, no id twice in the free list, no held id in it."""
        if len(set(self._free)) != len(self._free):
            raise AssertionError(f"{self.what} pool: an id is twice in the free list")
        if any(self._held[i] for i in self._free):
            raise AssertionError(f"{self.what} pool: a held id is in the free list")
        if sum(self._held) + len(self._free) != self.total:
            raise AssertionError(f"{self.what} pool: free + held != total")


class PagePool(IdPool):
    """A page pool that also keeps promises: ``committed`` pages are promised to admitted
    sequences, whether or not they hold them yet.  A sequence never holds more than it was
    promised, so a promise can always be kept."""

    def __init__(self, total: int):
        super().__init__(total, "page")
        self.committed = 0

    @property
    def uncommitted(self) -> int:
        return self.total - self.committed

    def commit(self, n: int) -> None:
        if n < 0 or self.committed + n > self.total:
            raise OutOfPages(f"cannot promise {n} more pages: {self.committed} of {self.total} are promised")
        self.committed += n

    def uncommit(self, n: int) -> None:
        if n < 0 or n > self.committed:
            raise ValueError(f"cannot take back {n} promised pages of {self.committed}")
        self.committed -= n

    def check(self) -> None:
        super().check()
        if not (0 <= self.committed <= self.total):
            raise AssertionError("page pool: promised pages out of range")
