"""Free lists: pages of one pool, and slots for per-request state.

The reference keeps a Python list of free page ids, pops from its end to allocate
and extends it on free, so that pages just given back are used again first
(rollout/cache.py:25, 153, 98). Running out raises KVCapacityError, a MemoryError
(rollout/engine.py:9-10, rollout/cache.py:139-140).
"""
from __future__ import annotations

from typing import Iterable, List


class KVCapacityError(MemoryError):
    """The cache cannot hold what was asked for (pages or request slots)."""


class FreeList:
    """Ids 0..count-1; last freed, first reused. Refuses to free an id twice or one it never gave."""

    def __init__(self, count: int, what: str = "page"):
        self.count = int(count)
        self.what = what
        self._free: List[int] = list(range(self.count - 1, -1, -1))
        self._is_free = [True] * self.count

    def available(self) -> int:
        return len(self._free)

    def in_use(self) -> int:
        return self.count - len(self._free)

    def take(self) -> int:
        if not self._free:
            raise KVCapacityError(f"no free {self.what} left (all {self.count} in use)")
        i = self._free.pop()
        self._is_free[i] = False
        return i

    def take_many(self, n: int) -> List[int]:
        if n > len(self._free):
            raise KVCapacityError(
                f"{n} {self.what}s wanted, {len(self._free)} of {self.count} free")
        return [self.take() for _ in range(n)]

    def give_back(self, ids: Iterable[int]) -> None:
        for i in ids:
            if not 0 <= i < self.count:
                raise ValueError(f"{self.what} {i} does not exist (0..{self.count - 1})")
            if self._is_free[i]:
                raise ValueError(f"{self.what} {i} freed twice")
            self._is_free[i] = True
            self._free.append(i)

    def free_ids(self) -> List[int]:
        return list(self._free)
