"""The cache's bookkeeping: no slot or block lost, held twice or freed twice."""
import random

import pytest
import torch

from xeno_rt_amd.cache import BLOCK_TOKENS, CacheError, CacheFull, Pool, SequenceCache, blocks_for
from xeno_rt_amd.parts import CacheNeeds, KVSpec, StateSpec


def make_cache(max_tokens=640, max_slots=4, max_context=512, window=None, state=False, calls=3):
    needs = [CacheNeeds(kv=KVSpec(2, 16, window), state=StateSpec((5,)) if state else None) for _ in range(calls)]
    return SequenceCache(needs, list(range(calls)), max_tokens, max_slots, max_context, torch.float32, "cpu")


def test_pool_hands_out_lowest_first_and_reuses():
    pool = Pool(3, "slot")
    assert [pool.acquire() for _ in range(3)] == [0, 1, 2]
    with pytest.raises(CacheFull):
        pool.acquire()
    pool.release(1)
    assert pool.acquire() == 1
    pool.release(0)
    with pytest.raises(CacheError, match="twice"):
        pool.release(0)
    with pytest.raises(CacheError, match="does not exist"):
        pool.release(7)
    pool.check()
    assert pool.n_free == 1 and pool.n_held == 2


def test_blocks_follow_lengths_and_come_back():
    cache = make_cache()
    assert cache.n_blocks == 10 and BLOCK_TOKENS == 64 and blocks_for(65) == 2
    a, b = cache.alloc_slot(), cache.alloc_slot()
    cache.reserve(a, 70); cache.commit(a, 70)
    cache.reserve(b, 64); cache.commit(b, 64)
    assert cache.held_blocks() == 3 and cache.length(a) == 70 and cache.length(b) == 64
    cache.reserve(b, 65); cache.commit(b, 65)            # crossing a block boundary takes one more
    assert cache.held_blocks() == 4
    group = cache.groups[0]
    assert len(set(group.held(a)) | set(group.held(b))) == 4
    cache.check()
    cache.free_slot(a)
    assert cache.held_blocks() == 2
    with pytest.raises(CacheError, match="freed twice"):
        cache.free_slot(a)
    with pytest.raises(CacheError, match="not allocated"):
        cache.reserve(a, 5)
    c = cache.alloc_slot()
    assert c == a and cache.length(c) == 0                # the slot is used again, empty
    assert (group.table[c] < 0).all()
    cache.free_slot(b); cache.free_slot(c)
    assert cache.held_blocks() == 0
    cache.check()


def test_full_cache_refuses_and_rolls_back():
    cache = make_cache(max_tokens=256, max_context=256)
    a, b = cache.alloc_slot(), cache.alloc_slot()
    cache.reserve(a, 129); cache.commit(a, 129)           # 3 of 4 blocks
    with pytest.raises(CacheFull):
        cache.reserve(b, 100)                             # needs 2
    assert cache.held_blocks() == 3                       # nothing kept from the failed attempt
    cache.check()
    with pytest.raises(CacheError, match="context limit"):
        cache.reserve(a, 257)
    cache.reserve(b, 64); cache.commit(b, 64)
    assert cache.held_blocks() == 4
    cache.reserve(a, 150)                                 # still inside a's third block
    cache.cancel(a)
    assert cache.length(a) == 129 and cache.held_blocks() == 4


def test_truncate_gives_back_whole_blocks():
    cache = make_cache()
    a = cache.alloc_slot()
    cache.reserve(a, 200); cache.commit(a, 200)
    assert cache.held_blocks() == 4
    cache.truncate(a, 64)
    assert cache.held_blocks() == 1 and cache.length(a) == 64
    with pytest.raises(CacheError):
        cache.truncate(a, 65)
    cache.check()


def test_groups_with_a_window_keep_only_what_is_still_seen():
    needs = [CacheNeeds(kv=KVSpec(2, 16)), CacheNeeds(kv=KVSpec(2, 16, window=100)), CacheNeeds(kv=KVSpec(2, 16))]
    cache = SequenceCache(needs, [0, 1, 2], 1024, 2, 1024, torch.float32, "cpu")
    assert len(cache.groups) == 2                          # layers of equal needs share storage
    full = next(g for g in cache.groups if g.spec.window is None)
    ring = next(g for g in cache.groups if g.spec.window == 100)
    assert full.calls == [0, 2] and ring.calls == [1] and full.k.shape[0] == 2 and ring.k.shape[0] == 1
    a = cache.alloc_slot()
    cache.reserve(a, 300)
    assert full.pool.n_held == 5 and ring.pool.n_held == 5      # the prompt's own queries see all of it
    cache.commit(a, 300)
    assert full.pool.n_held == 5 and ring.pool.n_held == 2      # keys 201.. stay: blocks 3 and 4
    assert [int(x) >= 0 for x in ring.table[a][:5]] == [False, False, False, True, True]
    for length in range(301, 400):
        cache.reserve(a, length); cache.commit(a, length)
    assert ring.pool.n_held == 3 and full.pool.n_held == 7      # keys 300..399 lie in blocks 4, 5, 6
    cache.check()
    cache.free_slot(a)
    assert ring.pool.n_held == 0 and full.pool.n_held == 0


def test_truncation_below_what_a_window_has_released_is_refused():
    needs = [CacheNeeds(kv=KVSpec(2, 16, window=100))]
    cache = SequenceCache(needs, [0], 1024, 2, 1024, torch.float32, "cpu")
    ring = cache.groups[0]
    a = cache.alloc_slot()
    cache.reserve(a, 600); cache.commit(a, 600)           # a query at 600 sees keys 501..: blocks 0..6 are gone
    held = ring.pool.n_held
    with pytest.raises(CacheError, match="released"):
        cache.truncate(a, 300)                            # a query at 300 would see keys 201..299: released long ago
    assert cache.length(a) == 600 and ring.pool.n_held == held
    cache.truncate(a, 590)                                # a query at 590 sees keys 491..: block 7 is still held
    assert cache.length(a) == 590
    cache.reserve(a, 591); cache.commit(a, 591)
    cache.check()
    cache.free_slot(a)
    assert ring.pool.n_held == 0


def test_values_may_be_wider_or_narrower_than_keys():
    needs = [CacheNeeds(kv=KVSpec(2, 16, value_dim=40)), CacheNeeds(kv=KVSpec(2, 16))]
    cache = SequenceCache(needs, [0, 1], 256, 2, 256, torch.float32, "cpu")
    assert len(cache.groups) == 2                           # another value width is another kind of storage
    wide = cache.layer_cache(0).kv
    assert tuple(wide.k.shape[1:]) == (2, 64, 16) and tuple(wide.v.shape[1:]) == (2, 40, 64)
    assert tuple(cache.layer_cache(1).kv.v.shape[1:]) == (2, 16, 64)
    assert KVSpec(2, 16).value_width == 16 and KVSpec(2, 16, value_dim=40).value_width == 40


def test_state_is_zero_for_every_new_sequence():
    cache = make_cache(state=True)
    a = cache.alloc_slot()
    view = cache.layer_cache(1)
    assert view.state.shape == (4, 5) and view.writable and view.kv.k.shape == (10, 2, 64, 16)
    view.state[a] += 3.0
    cache.free_slot(a)
    assert cache.alloc_slot() == a
    assert float(cache.layer_cache(1).state[a].abs().sum()) == 0.0
    with pytest.raises(CacheError, match="cannot be truncated"):
        cache.reserve(a, 10); cache.commit(a, 10); cache.truncate(a, 5)


def test_a_call_may_read_another_calls_cache():
    needs = [CacheNeeds(kv=KVSpec(1, 16)), None]
    cache = SequenceCache(needs, [0, 0], 128, 1, 128, torch.float32, "cpu")
    own, shared = cache.layer_cache(0), cache.layer_cache(1)
    assert own.writable and not shared.writable
    assert shared.kv.k.data_ptr() == own.kv.k.data_ptr()
    assert cache.groups[0].k.shape[0] == 1


def test_random_traffic_keeps_the_books(seed=0):
    rng = random.Random(seed)
    cache = make_cache(max_tokens=64 * 12, max_slots=5, max_context=300, window=None)
    live = {}
    for _ in range(2000):
        action = rng.random()
        if action < 0.25 and len(live) < 5:
            live[cache.alloc_slot()] = 0
        elif action < 0.4 and live:
            slot = rng.choice(list(live))
            cache.free_slot(slot); del live[slot]
        elif live:
            slot = rng.choice(list(live))
            grow = rng.choice([1, 1, 1, 17, 64, 90])
            try:
                cache.reserve(slot, live[slot] + grow)
            except (CacheFull, CacheError):
                cache.cancel(slot)
            else:
                if rng.random() < 0.9:
                    live[slot] += grow; cache.commit(slot, live[slot])
                else:
                    cache.cancel(slot)
        cache.check()
        assert cache.held_blocks() == sum(blocks_for(n) for n in live.values())
        assert cache.slots.n_held == len(live)
    for slot in list(live):
        cache.free_slot(slot)
    cache.check()
    assert cache.held_blocks() == 0 and cache.slots.n_free == 5
