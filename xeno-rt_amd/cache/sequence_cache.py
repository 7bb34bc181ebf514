"""The cache of all live sequences: keys and values per layer call, in blocks, and
per-sequence state of fixed size.

A slot stands for one sequence and has its own length. Layer calls whose key/
value rows have the same shape and window form a group; a group has storage of
its own (one pool of blocks, one block table) and its own rule for which blocks
a sequence of a given length holds: all of them, or those a window still sees.
Storage of one call: keys [blocks, kv_heads, BLOCK_TOKENS, head_dim], values
[blocks, kv_heads, value_dim, BLOCK_TOKENS]. The order of the BLOCK_TOKENS * head_dim
elements behind the last two dimensions belongs to the kernels that write and read
them (csrc/cache_layout.h: for head sizes that are multiples of 32, the order in
which the decode attention's wavefronts load them; rows otherwise); nothing in
the package looks inside a block.

The reference keeps one paged cache per sequence with rows of all KV heads,
float32 (crates/xrt-runtime/src/kv_cache.rs:4-45); `truncate` follows its
rollback (kv_cache.rs:159-168).
"""
from __future__ import annotations

import ctypes
from dataclasses import dataclass
from typing import Dict, List, Optional

import numpy as np
import torch

from ..staging import staging_for

from ..parts.base import CacheNeeds, KVSpec
from ..host import last_error, load_host
from .allocator import BLOCK_TOKENS, CacheError, CacheFull, Pool, blocks_for, raise_for


@dataclass
class KVView:
    """What an attention kernel needs of one layer call's keys and values."""
    spec: KVSpec
    k: torch.Tensor             # [blocks, kv_heads, BLOCK_TOKENS, head_dim]: per (block, head) the kernels' own order
    v: torch.Tensor             # [blocks, kv_heads, value_dim, BLOCK_TOKENS]: likewise
    block_table: torch.Tensor   # int32 [slots, max_blocks]: logical block -> physical block, -1 = none


@dataclass
class LayerCache:
    kv: Optional[KVView]
    state: Optional[torch.Tensor]   # [slots, *shape]
    writable: bool


class KVGroup:
    """Storage and block accounting of the layer calls that share one KVSpec. Which blocks a sequence holds is kept
    by the host library (csrc/host/xrt_host.cpp), which writes the table that lies here; the device's copy of
    the table is refreshed from it before a step."""

    def __init__(self, spec: KVSpec, calls: List[int], n_blocks: int, max_slots: int,
                 max_blocks_per_sequence: int, dtype: torch.dtype, device):
        self.spec = spec
        self.calls = calls
        self.max_blocks_per_sequence = max_blocks_per_sequence
        self.max_slots = max_slots
        # host table: the truth (the torch view shares the array's memory); device table: what kernels read
        self._table = np.full((max_slots, max_blocks_per_sequence), -1, dtype=np.int32)
        self.table = torch.from_numpy(self._table)
        self.device_table = self.table.to(device)
        self._lib = load_host()
        self._handle = self._lib.xrt_tables_new(n_blocks, max_slots, max_blocks_per_sequence, int(spec.window or 0),
                                                BLOCK_TOKENS, self._table.ctypes.data)
        if not self._handle:
            raise CacheError(last_error())
        self.pool = Pool(n_blocks, "block", handle=self._lib.xrt_tables_pool(self._handle))
        self._added = (ctypes.c_int * max(1, max_blocks_per_sequence))()
        shape_k = (len(calls), n_blocks, spec.n_kv_heads, BLOCK_TOKENS, spec.head_dim)
        shape_v = (len(calls), n_blocks, spec.n_kv_heads, spec.value_width, BLOCK_TOKENS)
        self.k = torch.zeros(shape_k, dtype=dtype, device=device)
        self.v = torch.zeros(shape_v, dtype=dtype, device=device)

    def __del__(self):
        if getattr(self, "_handle", None):
            self._lib.xrt_tables_delete(self._handle)
            self._handle = None

    def first_needed_block(self, length: int) -> int:
        """Lowest logical block that a query at position >= length can still see."""
        return int(self._lib.xrt_tables_first_needed_block(self._handle, int(length)))

    def floor(self, slot: int) -> int:
        """Lowest logical block that the sequence may still hold (a window lets go of those below)."""
        return int(self._lib.xrt_tables_floor(self._handle, int(slot)))

    def held(self, slot: int) -> List[int]:
        row = self._table[slot]
        return [int(b) for b in row[row >= 0]]

    def grow(self, slot: int, new_length: int) -> List[int]:
        """Acquire the blocks that tokens up to new_length need; returns the logical indices added."""
        count = ctypes.c_int(0)
        raise_for(self._lib.xrt_tables_grow(self._handle, int(slot), int(new_length), self._added, ctypes.byref(count)))
        return list(self._added[:count.value])

    def drop(self, slot: int, logicals: List[int]) -> None:
        if logicals:
            array = (ctypes.c_int * len(logicals))(*logicals)
            raise_for(self._lib.xrt_tables_drop(self._handle, int(slot), array, len(logicals)))

    def shrink_to(self, slot: int, length: int) -> None:
        """Release what a sequence of `length` tokens no longer needs: blocks past its end,
        and blocks that have slid out of the window."""
        raise_for(self._lib.xrt_tables_shrink_to(self._handle, int(slot), int(length)))

    def release_all(self, slot: int) -> None:
        raise_for(self._lib.xrt_tables_release_all(self._handle, int(slot)))

    def check(self, slot_held) -> None:
        """No block held by two sequences or by none; free slots hold nothing."""
        flags = (ctypes.c_ubyte * self.max_slots)(*[1 if held else 0 for held in slot_held])
        raise_for(self._lib.xrt_tables_check(self._handle, flags))

    def sync(self) -> None:
        """The rows that changed go to the device through pinned memory, in the order of the stream and
        without waiting for it: a host that prepares the next step while this one runs is not held up."""
        low, high = ctypes.c_int(0), ctypes.c_int(0)
        self._lib.xrt_tables_take_changed(self._handle, ctypes.byref(low), ctypes.byref(high))
        if high.value > low.value:
            staging_for(self.device_table.device).upload(self.table[low.value:high.value], out=self.device_table[low.value:high.value])


class SequenceCache:
    """Slots, their lengths, and the storage of every layer call.

    needs:       for each schedule entry its CacheNeeds, or None if it reads another entry's
    reads_from:  for each schedule entry the entry whose cache it reads (itself if it owns one)
    max_tokens:  tokens that live sequences may hold together, each rounded up to BLOCK_TOKENS
    max_slots:   sequences that may be live together
    max_context: longest sequence
    """

    def __init__(self, needs: List[Optional[CacheNeeds]], reads_from: List[int], max_tokens: int,
                 max_slots: int, max_context: int, dtype: torch.dtype, device):
        if max_tokens <= 0 or max_slots <= 0 or max_context <= 0:
            raise ValueError("max_tokens, max_slots and max_context must be positive")
        self.n_blocks = blocks_for(max_tokens)
        self.max_slots = max_slots
        self.max_context = min(max_context, self.n_blocks * BLOCK_TOKENS)
        self.dtype = dtype
        self.device = torch.device(device)
        self.slots = Pool(max_slots, "slot")
        self.lengths = [0] * max_slots
        self.reads_from = list(reads_from)
        self.needs = list(needs)

        max_blocks = blocks_for(self.max_context)
        self.groups: List[KVGroup] = []
        self._group_of: Dict[int, KVGroup] = {}
        by_spec: Dict[KVSpec, List[int]] = {}
        for call, need in enumerate(needs):
            if need is not None and need.kv is not None:
                by_spec.setdefault(need.kv, []).append(call)
        for spec, calls in by_spec.items():
            group = KVGroup(spec, calls, self.n_blocks, max_slots, max_blocks, dtype, device)
            self.groups.append(group)
            for call in calls:
                self._group_of[call] = group

        self.states: Dict[int, torch.Tensor] = {}
        for call, need in enumerate(needs):
            if need is not None and need.state is not None:
                self.states[call] = torch.zeros((max_slots, *need.state.shape),
                                                dtype=need.state.dtype, device=device)

    # -- slots ---------------------------------------------------------------
    def alloc_slot(self) -> int:
        slot = self.slots.acquire()
        self.lengths[slot] = 0
        for state in self.states.values():
            state[slot].zero_()
        return slot

    def free_slot(self, slot: int) -> None:
        if not self.slots.is_held(slot):
            raise CacheError(f"slot {slot} is freed twice or was never allocated")
        for group in self.groups:
            group.release_all(slot)
        self.lengths[slot] = 0
        self.slots.release(slot)

    def length(self, slot: int) -> int:
        self._require(slot)
        return self.lengths[slot]

    def _require(self, slot: int) -> None:
        if not self.slots.is_held(slot):
            raise CacheError(f"slot {slot} is not allocated")

    # -- growth by a step ----------------------------------------------------
    def reserve(self, slot: int, new_length: int) -> None:
        """Make room for the sequence to grow to new_length; its length is unchanged."""
        self._require(slot)
        if new_length > self.max_context:
            raise CacheError(f"slot {slot}: {new_length} tokens exceed the context limit {self.max_context}")
        grown = []
        try:
            for group in self.groups:
                grown.append((group, group.grow(slot, new_length)))
        except CacheFull:
            for group, added in grown:
                group.drop(slot, added)
            raise

    def commit(self, slot: int, new_length: int) -> None:
        """The step has run: the sequence now has new_length tokens."""
        self._require(slot)
        self.lengths[slot] = new_length
        for group in self.groups:
            if group.spec.window is not None:
                group.shrink_to(slot, new_length)

    def cancel(self, slot: int) -> None:
        """Give back what `reserve` took beyond the sequence's current length."""
        self._require(slot)
        for group in self.groups:
            group.shrink_to(slot, self.lengths[slot])

    def truncate(self, slot: int, length: int) -> None:
        """Forget the tokens from position `length` on (reference: kv_cache.rs:159-168).

        Only for layer calls that keep rows per token; state of fixed size cannot be rolled back."""
        self._require(slot)
        if length > self.lengths[slot]:
            raise CacheError(f"slot {slot}: cannot truncate {self.lengths[slot]} tokens to {length}")
        if self.states and length != self.lengths[slot]:
            raise CacheError("a cache with per-sequence state cannot be truncated")
        for group in self.groups:
            # a window has let go of the blocks below its floor: a shorter sequence that would look there again cannot be had
            if group.spec.window is not None and group.first_needed_block(length) < group.floor(slot):
                raise CacheError(f"slot {slot}: cannot truncate to {length} tokens: a window of {group.spec.window} has "
                                 f"released the keys before {group.floor(slot) * BLOCK_TOKENS}, which a query there would see")
        self.lengths[slot] = length
        for group in self.groups:
            group.shrink_to(slot, length)

    def sync(self) -> None:
        """Bring the device's block tables up to date; call before kernels read them."""
        for group in self.groups:
            group.sync()

    # -- views ---------------------------------------------------------------
    def layer_cache(self, call: int) -> LayerCache:
        source = self.reads_from[call]
        group = self._group_of.get(source)
        kv = None
        if group is not None:
            index = group.calls.index(source)
            kv = KVView(group.spec, group.k[index], group.v[index], group.device_table)
        return LayerCache(kv=kv, state=self.states.get(source), writable=(source == call))

    # -- accounting ----------------------------------------------------------
    def held_blocks(self) -> int:
        return max((group.pool.n_held for group in self.groups), default=0)

    def check(self) -> None:
        """Invariants: no slot or block lost or held twice; free slots hold nothing."""
        self.slots.check()
        held = [self.slots.is_held(slot) for slot in range(self.max_slots)]
        for group in self.groups:
            group.check(held)
