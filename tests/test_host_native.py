"""The host library (csrc/host/xrt_host.cpp) through its Python face: pools, block tables, the packing of a step
and the loop's decisions, each against a few lines of plain Python that say the same thing; and its own
self-test under the host sanitizers."""
import ctypes
import random
import subprocess

import numpy as np
import pytest
import torch

from xeno_rt_amd.cache.allocator import BLOCK_TOKENS, CacheError, CacheFull, Pool
from xeno_rt_amd.engine.batch import build_batch
from xeno_rt_amd.engine.generate import decide, goes_on_whatever_it_draws, plan_batches


def test_selftest_runs_clean_under_the_sanitizers():
    from xeno_rt_amd.ops import build
    program = build.build_host_selftest(sanitize=True)
    done = subprocess.run([program], capture_output=True, text=True, timeout=120)
    assert done.returncode == 0, done.stdout + done.stderr
    assert "host selftest ok" in done.stdout


def test_a_pool_against_a_set_of_free_numbers():
    generator = random.Random(5)
    pool, free = Pool(37, "thing"), set(range(37))
    for _ in range(3000):
        if generator.random() < 0.55:
            if free:
                item = pool.acquire()
                assert item == min(free)                      # the lowest free one
                free.remove(item)
            else:
                with pytest.raises(CacheFull, match="no free thing"):
                    pool.acquire()
        else:
            item = generator.randrange(37)
            if item in free:
                with pytest.raises(CacheError, match="released twice or was never acquired"):
                    pool.release(item)
            else:
                pool.release(item)
                free.add(item)
        assert pool.n_free == len(free) and pool.n_held == 37 - len(free)
        probe = generator.randrange(-2, 40)
        assert pool.is_held(probe) == (0 <= probe < 37 and probe not in free)
    pool.check()
    with pytest.raises(CacheError, match="does not exist"):
        pool.release(37)


@pytest.mark.parametrize("pad_to", [0, 16])
def test_a_packed_step_against_lists_put_together_by_hand(pad_to):
    generator = random.Random(pad_to)
    for _ in range(50):
        n = generator.randrange(1, 6)
        slots = generator.sample(range(20), n)
        tokens = [[generator.randrange(1000) for _ in range(generator.randrange(1, 9))] for _ in range(n)]
        starts = [generator.randrange(500) for _ in range(n)]
        wants = [sorted(generator.sample(range(len(ids)), generator.randrange(0, len(ids) + 1))) for ids in tokens]
        batch = build_batch(slots, tokens, starts, wants, "cpu", pad_tokens_to=pad_to)
        ids, positions, token_slots, offsets, rows = [], [], [], [0], []
        for slot, new, start, want in zip(slots, tokens, starts, wants):
            rows += [len(ids) + w for w in want]
            ids += new
            positions += range(start, start + len(new))
            token_slots += [slot] * len(new)
            offsets.append(len(ids))
        while len(ids) < pad_to:
            ids.append(0); positions.append(0); token_slots.append(-1)
        assert batch.token_ids.tolist() == ids and batch.positions.tolist() == positions and batch.slots.tolist() == token_slots
        assert batch.sequence_slots.tolist() == slots and batch.sequence_offsets.tolist() == offsets
        assert batch.sequence_starts.tolist() == starts and batch.logit_rows.tolist() == rows
        assert (batch.n_tokens, batch.n_sequences, batch.n_logit_rows) == (len(ids), n, len(rows))
        assert batch.host_counts == [len(new) for new in tokens] and batch.host_slots == slots and batch.host_starts == starts
        assert batch.is_decode == all(len(new) == 1 for new in tokens)
        assert batch.max_count == max(len(new) for new in tokens)
        assert batch.max_context == max(s + len(new) for s, new in zip(starts, tokens))


def test_the_loops_decisions_against_the_reference_s_order():
    """session.rs:115-124: a stop token ends the request and is not kept; else a full context ends it; else the token
    is kept, and ends it if it is the last one allowed."""
    generator = random.Random(9)
    for _ in range(2000):
        stops = frozenset(generator.sample(range(12), generator.randrange(0, 4)))
        token, context = generator.randrange(12), generator.randrange(1, 30)
        history, produced, limit = generator.randrange(0, context + 1), generator.randrange(0, 10), generator.randrange(1, 11)
        if token in stops:
            want = (False, "stop")
        elif history >= context:
            want = (False, "context")
        elif produced + 1 >= limit:
            want = (True, "length")
        else:
            want = (True, None)
        assert decide(token, stops, history, context, produced, limit) == want
        assert goes_on_whatever_it_draws(history, context, produced, limit) == (history + 1 < context and produced + 1 < limit)


def test_batches_against_a_loop_that_fills_them_one_request_at_a_time():
    generator = random.Random(3)
    for _ in range(300):
        n = generator.randrange(0, 12)
        prompts = [generator.randrange(1, 300) for _ in range(n)]
        limits = [generator.randrange(0, 200) for _ in range(n)]
        batch_size, context = generator.randrange(1, 5), generator.randrange(64, 400)
        cache_tokens = BLOCK_TOKENS * generator.randrange(1, 12)
        needs = [-(-min(context, p + l) // BLOCK_TOKENS) * BLOCK_TOKENS for p, l in zip(prompts, limits)]
        if any(need > cache_tokens for need in needs):
            with pytest.raises(ValueError, match="the cache holds"):
                plan_batches(prompts, limits, batch_size, BLOCK_TOKENS, cache_tokens, context)
            continue
        want, current, used = [], [], 0
        for index, need in enumerate(needs):
            if current and (len(current) >= batch_size or used + need > cache_tokens):
                want.append(current)
                current, used = [], 0
            current.append(index)
            used += need
        if current:
            want.append(current)
        assert plan_batches(prompts, limits, batch_size, BLOCK_TOKENS, cache_tokens, context) == want
