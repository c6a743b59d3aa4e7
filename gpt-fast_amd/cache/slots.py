"""Bookkeeping of numbered resources (sequence slots, cache pages) on the host.

Pure Python, no device: a free list with checks that no number is handed out twice,
given back twice, or lost.
"""
from typing import List


class CacheFull(RuntimeError):
    """No free slot or page is left."""


class FreeList:
    """Numbers 0..n-1; ``take`` hands out the lowest free one, ``give`` returns one."""

    def __init__(self, n: int, what: str = "item"):
        if n < 0:
            raise ValueError(f"cannot manage {n} {what}s")
        self.n = n
        self.what = what
        self._free: List[int] = list(range(n - 1, -1, -1))    # pop() yields the lowest
        self._held = [False] * n

    @property
    def free(self) -> int:
        return len(self._free)

    @property
    def held(self) -> int:
        return self.n - len(self._free)

    def is_held(self, i: int) -> bool:
        return 0 <= i < self.n and self._held[i]

    def take(self) -> int:
        if not self._free:
            raise CacheFull(f"all {self.n} {self.what}s are in use")
        i = self._free.pop()
        assert not self._held[i], f"{self.what} {i} was on the free list while held"
        self._held[i] = True
        return i

    def give(self, i: int) -> None:
        if not 0 <= i < self.n:
            raise ValueError(f"{self.what} {i} does not exist (there are {self.n})")
        if not self._held[i]:
            raise ValueError(f"{self.what} {i} is given back but is not held")
        self._held[i] = False
        # keep the list sorted descending so that take() stays "lowest first"
        free = self._free
        lo, hi = 0, len(free)
        while lo < hi:
            mid = (lo + hi) // 2
            if free[mid] > i:
                lo = mid + 1
            else:
                hi = mid
        free.insert(lo, i)

    def check(self) -> None:
        """Every number is either free or held, exactly once."""
        seen = set(self._free)
        if len(seen) != len(self._free):
            raise AssertionError(f"a {self.what} is on the free list twice")
        for i in range(self.n):
            if self._held[i] == (i in seen):
                raise AssertionError(f"{self.what} {i} is lost or both free and held")
