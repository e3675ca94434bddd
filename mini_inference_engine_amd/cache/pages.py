"""Free lists of page ids and of state slots.

Page 0 (and slot 0) is scratch: never handed out; padded rows of a captured
decode step write there (inference_engine/block_manager.py:14-19).  Ids are
taken from the left and given back on the right, so a freed page is reused
after the ones freed before it (inference_engine/block_manager.py:39,43).
"""
from __future__ import annotations

from collections import deque


class CacheAccountingError(RuntimeError):
    """A page or slot was given back twice, was never taken, or is scratch."""


class IdPool:
    def __init__(self, count: int, reserved: int = 1, what: str = "page"):
        if count <= reserved:
            raise ValueError(f"need more than {reserved} {what}s, got {count}")
        self.count = count
        self.reserved = reserved
        self.what = what
        self.free = deque(range(reserved, count))
        self._held = [False] * count
        self.low_water = len(self.free)

    @property
    def num_free(self) -> int:
        return len(self.free)

    @property
    def num_usable(self) -> int:
        return self.count - self.reserved

    def take(self, n: int) -> list[int] | None:
        if n > len(self.free):
            return None
        ids = [self.free.popleft() for _ in range(n)]
        for i in ids:
            self._held[i] = True
        self.low_water = min(self.low_water, len(self.free))
        return ids

    def give_back(self, ids) -> None:
        for i in ids:
            if not self.reserved <= i < self.count:
                raise CacheAccountingError(f"{self.what} {i} is scratch or out of range")
            if not self._held[i]:
                raise CacheAccountingError(f"{self.what} {i} given back but not held")
            self._held[i] = False
            self.free.append(i)

    def held(self) -> set[int]:
        return {i for i, h in enumerate(self._held) if h}
