"""Host-side bookkeeping of the cache: slots (one per live sequence) and pages.

Both allocators keep a free list and a set of what is held, so that nothing can
be lost, held twice or given back twice without an error.  The reference has one
sequence and a single write cursor per layer (src/core/kvstorage.h:17-46); the
cursor's role is played here by a length per slot.
"""
from __future__ import annotations

import random
from typing import List


class CacheError(RuntimeError):
    """Wrong use of the cache: a slot freed twice, a position that does not follow, ..."""


class CacheFull(CacheError):
    """No slot or no page left for the request."""


class FreeList:
    """Integers 0..n-1, handed out last-freed first and taken back exactly once.

    At the start they come in rising order, or with `scatter` in a fixed shuffled order.  Pages
    are scattered: sequences that start together get equally many pages one after the other, and
    when that number is a power of two their keys lie at power-of-two distances in memory, which
    the memory channels serve unevenly (measured on MI355X, decode attention of 8 sequences over
    pages in rising order against shuffled ones: 19.5 against 16.9 us at 512 keys, 107 against
    91 us at 4096)."""

    def __init__(self, n: int, what: str, scatter: bool = False):
        if n < 0:
            raise CacheError(f"negative number of {what}s")
        self.n = n
        self.what = what
        self._free: List[int] = list(range(n - 1, -1, -1))  # pop() gives 0 first
        if scatter:
            random.Random(n).shuffle(self._free)
        self._held = set()

    def alloc(self) -> int:
        if not self._free:
            raise CacheFull(f"no free {self.what}: all {self.n} are in use")
        i = self._free.pop()
        self._held.add(i)
        return i

    def free(self, i: int) -> None:
        if i not in self._held:
            raise CacheError(f"{self.what} {i} is not held (freed twice, or never given out)")
        self._held.remove(i)
        self._free.append(i)

    def n_free(self) -> int:
        return len(self._free)

    def holds(self, i: int) -> bool:
        return i in self._held

    def n_held(self) -> int:
        return len(self._held)

    def held(self):
        return sorted(self._held)

    def check(self) -> None:
        """Every index is either free or held, exactly once."""
        if len(self._free) != len(set(self._free)):
            raise CacheError(f"a {self.what} is on the free list twice")
        if self._held & set(self._free):
            raise CacheError(f"a {self.what} is both free and held")
        if len(self._free) + len(self._held) != self.n:
            raise CacheError(f"{self.what}s lost: {len(self._free)} free + {len(self._held)} held != {self.n}")
