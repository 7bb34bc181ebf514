"""Host-side bookkeeping of the cache: which slots and which blocks are in use.

A slot stands for one live sequence. A block holds the keys and values of
BLOCK_TOKENS consecutive tokens of one sequence. Both come from fixed pools
and go back to them when the sequence ends; asking for more than there is, or
giving something back twice, is an error and never silent.
"""
from __future__ import annotations

import ctypes

from ..host import ERROR, FULL, OK, last_error, load_host

BLOCK_TOKENS = 64   # tokens per block: the unit in which live requests hold cache (the kernel library is asked for its own
                    # number when it is loaded, and refused if that differs)


class CacheFull(RuntimeError):
    """No free slot or block is left."""


class CacheError(RuntimeError):
    """A slot or block was used in a way its state does not allow."""


def raise_for(status: int) -> None:
    """The host library's verdict as an exception, with its message."""
    if status == FULL:
        raise CacheFull(last_error())
    if status != OK:
        raise CacheError(last_error())


class Pool:
    """`size` numbered items; the lowest free one is handed out, released ones are used again.
    The bookkeeping is the host library's (csrc/host/xrt_host.cpp); `handle` may name a pool that
    someone else owns (the blocks of a group's tables)."""

    def __init__(self, size: int, what: str, handle=None):
        if size < 0:
            raise ValueError(f"pool of {what}s needs a non-negative size")
        self._lib = load_host()
        self.size = size
        self.what = what
        self._owned = handle is None
        self._handle = self._lib.xrt_pool_new(size, what.encode()) if handle is None else handle
        if not self._handle:
            raise CacheError(last_error())

    def __del__(self):
        if getattr(self, "_owned", False) and getattr(self, "_handle", None):
            self._lib.xrt_pool_delete(self._handle)
            self._handle = None

    @property
    def n_free(self) -> int:
        return int(self._lib.xrt_pool_n_free(self._handle))

    @property
    def n_held(self) -> int:
        return self.size - self.n_free

    def is_held(self, item: int) -> bool:
        return bool(self._lib.xrt_pool_is_held(self._handle, int(item)))

    def acquire(self) -> int:
        item = ctypes.c_int(-1)
        raise_for(self._lib.xrt_pool_acquire(self._handle, ctypes.byref(item)))
        return item.value

    def release(self, item: int) -> None:
        raise_for(self._lib.xrt_pool_release(self._handle, int(item)))

    def check(self) -> None:
        """Every item is either free once or held; raises CacheError otherwise."""
        raise_for(self._lib.xrt_pool_check(self._handle))


def blocks_for(tokens: int) -> int:
    return (tokens + BLOCK_TOKENS - 1) // BLOCK_TOKENS
