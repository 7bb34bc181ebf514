"""Host-side bookkeeping of the cache: which slots and which blocks are in use.

A slot stands for one live sequence. A block holds the keys and values of
BLOCK_TOKENS consecutive tokens of one sequence. Both come from fixed pools
and go back to them when the sequence ends; asking for more than there is, or
giving something back twice, is an error and never silent.
"""
from __future__ import annotations

import heapq
from typing import List

BLOCK_TOKENS = 64   # tokens per block: the unit in which live requests hold cache (the kernel library is asked for its own
                    # number when it is loaded, and refused if that differs)


class CacheFull(RuntimeError):
    """No free slot or block is left."""


class CacheError(RuntimeError):
    """A slot or block was used in a way its state does not allow."""


class Pool:
    """`size` numbered items; the lowest free one is handed out, released ones are used again."""

    def __init__(self, size: int, what: str):
        if size < 0:
            raise ValueError(f"pool of {what}s needs a non-negative size")
        self.size = size
        self.what = what
        self._free: List[int] = list(range(size))               # a heap: the lowest number on top
        self._held = [False] * size

    @property
    def n_free(self) -> int:
        return len(self._free)

    @property
    def n_held(self) -> int:
        return self.size - len(self._free)

    def is_held(self, item: int) -> bool:
        return 0 <= item < self.size and self._held[item]

    def acquire(self) -> int:
        if not self._free:
            raise CacheFull(f"no free {self.what} (all {self.size} are in use)")
        item = heapq.heappop(self._free)
        if self._held[item]:
            raise CacheError(f"{self.what} {item} was on the free list while held")
        self._held[item] = True
        return item

    def release(self, item: int) -> None:
        if not 0 <= item < self.size:
            raise CacheError(f"{self.what} {item} does not exist (pool of {self.size})")
        if not self._held[item]:
            raise CacheError(f"{self.what} {item} is released twice or was never acquired")
        self._held[item] = False
        heapq.heappush(self._free, item)

    def check(self) -> None:
        """Every item is either free once or held; raises CacheError otherwise."""
        free = set(self._free)
        if len(free) != len(self._free):
            raise CacheError(f"a {self.what} is on the free list twice")
        for item in range(self.size):
            if self._held[item] == (item in free):
                raise CacheError(f"{self.what} {item} is " + ("both held and free" if self._held[item] else "lost"))


def blocks_for(tokens: int) -> int:
    return (tokens + BLOCK_TOKENS - 1) // BLOCK_TOKENS
