"""The matrix-core attention kernels at long contexts, against plain attention in 64-bit:
decode over 32768 keys beside short sequences (the keys are cut into many parts of many blocks),
a prompt of 8192 tokens (64 tiles of queries), a portion of 2048 tokens that continues a cache
of 6144. Random inputs give near-uniform attention, under which one block read wrongly moves the
result by less than any tolerance; so every shape also runs with queries built to pick out one
key each (at a block's first and last place, around the block where the paired tiles of the
prefill kernel change from the early to the late tile, in the last block), and then the result
must be that key's value.

Formulas: crates/xrt-models/src/llama.rs:504-574 (decode), :727-770 (prefill) of the reference.
"""
import math
from types import SimpleNamespace

import pytest
import torch

import cache_order

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
BLOCK = 64


@pytest.fixture(scope="module")
def ops():
    from xeno_rt_amd.ops import load_ops
    return load_ops()


def i32(values):
    return torch.tensor(values, dtype=torch.int32, device=DEV)


def rand(*shape, seed=0, scale=1.0):
    g = torch.Generator().manual_seed(seed)
    return (torch.randn(*shape, generator=g) * scale).to(torch.bfloat16).to(DEV)


def rel(got, want):
    return float((got.double() - want.double()).abs().max()) / max(1e-30, float(want.double().abs().max()))


def long_cache(nkv, hd, lengths, seed):
    """A bfloat16 cache that holds lengths[s] random tokens for slot s; physical blocks in a shuffled order, what lies
    beyond a sequence's end poisoned. Returns (cache, keys, values) with keys[s], values[s] [length, nkv, hd]."""
    per = [(n + BLOCK - 1) // BLOCK for n in lengths]
    n_blocks = sum(per) + 2
    order = torch.randperm(n_blocks, generator=torch.Generator().manual_seed(seed)).tolist()
    k_rows = torch.zeros(n_blocks, nkv, BLOCK, hd, dtype=torch.bfloat16, device=DEV)
    v_rows = torch.zeros(n_blocks, nkv, hd, BLOCK, dtype=torch.bfloat16, device=DEV)
    table = torch.full((len(lengths), max(per) + 1), -1, dtype=torch.int32, device=DEV)
    keys, values = [], []
    for s, n in enumerate(lengths):
        k, v = rand(n, nkv, hd, seed=seed + 10 * s + 1), rand(n, nkv, hd, seed=seed + 10 * s + 2)
        keys.append(k); values.append(v)
        blocks = [order.pop() for _ in range(per[s])]
        table[s, :per[s]] = i32(blocks)
        padded = per[s] * BLOCK
        pad = lambda t: torch.cat([t, torch.full((padded - n, nkv, hd), float("nan"), dtype=t.dtype, device=DEV)])
        index = torch.tensor(blocks, device=DEV)
        k_rows[index] = pad(k).reshape(per[s], BLOCK, nkv, hd).permute(0, 2, 1, 3)
        v_rows[index] = pad(v).reshape(per[s], BLOCK, nkv, hd).permute(0, 2, 3, 1)
    kv = SimpleNamespace(k=cache_order.store_keys(k_rows), v=cache_order.store_values(v_rows), block_table=table)
    return kv, keys, values


def described(slots, counts, starts):
    token_slots, positions, offsets = [], [], [0]
    for slot, count, start in zip(slots, counts, starts):
        token_slots += [slot] * count
        positions += list(range(start, start + count))
        offsets.append(offsets[-1] + count)
    return SimpleNamespace(slots=i32(token_slots), positions=i32(positions), sequence_offsets=i32(offsets),
                           sequence_slots=i32(slots), sequence_starts=i32(starts), n_sequences=len(slots),
                           max_count=max(counts), max_context=max(s + c for s, c in zip(starts, counts)))


def plain_attention(q, positions, keys, values, nh, nkv, hd):
    """q [rows, nh * hd] at absolute positions `positions` of one sequence over its keys and values [n, nkv, hd]:
    softmax(q.k / sqrt(hd)) over the keys 0..position of every row, in 64-bit (llama.rs:727-770)."""
    rows = q.shape[0]
    q = q.double().reshape(rows, nh, hd)
    k, v = keys.double(), values.double()
    hidden = torch.arange(k.shape[0], device=q.device)[None, :] > torch.as_tensor(positions, device=q.device)[:, None]
    out = torch.empty(rows, nh, hd, dtype=torch.float64, device=q.device)
    for head in range(nh):
        kvh = head // (nh // nkv)
        scores = (q[:, head] @ k[:, kvh].t()) / math.sqrt(hd)
        out[:, head] = torch.softmax(scores.masked_fill(hidden, -math.inf), dim=-1) @ v[:, kvh]
    return out.reshape(rows, nh * hd)


def picking_queries(keys, far, nh, nkv, hd):
    """Rows of q/k/v whose query heads are 40 times the key at far[row] (of the head's key/value head): among
    thousands of random keys that key's score stands out by hundreds, and the output is its value."""
    rows = len(far)
    qkv = torch.zeros(rows, (nh + 2 * nkv) * hd, dtype=torch.bfloat16, device=DEV)
    picked = keys[torch.tensor(far, device=DEV)]                          # [rows, nkv, hd]
    qkv[:, :nh * hd] = (picked * 40.0).repeat_interleave(nh // nkv, dim=1).reshape(rows, nh * hd)
    return qkv


def assert_picked(out, values, far, nh, nkv, hd, what):
    want = values[torch.tensor(far, device=DEV)].repeat_interleave(nh // nkv, dim=1).reshape(len(far), nh * hd).float()
    scale = float(want.abs().max())
    worst = ((out.float() - want).abs().amax(dim=1) / scale).cpu()
    bad = torch.nonzero(worst > 2e-2).flatten().tolist()
    assert not bad, f"{what}: rows {bad[:8]} (of {len(bad)}) did not find their keys {[far[r] for r in bad[:8]]}"


# ---- decode ---------------------------------------------------------------------------------

@pytest.mark.parametrize("nh,nkv,hd", [(32, 8, 128), (64, 8, 128), (8, 2, 64)])
def test_decode_over_32768_keys_beside_short_sequences(ops, nh, nkv, hd):
    lengths = [32768, 100, 4097, 1, 20000, 64]
    kv, keys, values = long_cache(nkv, hd, lengths, seed=nh)
    slots = list(range(len(lengths)))
    positions = [n - 1 for n in lengths]
    batch = described(slots, [1] * len(lengths), positions)
    qkv = rand(len(lengths), (nh + 2 * nkv) * hd, seed=3)
    out = torch.full((len(lengths), nh * hd), 7.0, dtype=torch.bfloat16, device=DEV)
    ops.attention(qkv, nh, nkv, hd, kv, batch, out, scale=1.0 / math.sqrt(hd))
    assert torch.isfinite(out).all()
    for s, n in enumerate(lengths):
        want = plain_attention(qkv[s:s + 1, :nh * hd], [n - 1], keys[s], values[s], nh, nkv, hd)
        assert rel(out[s:s + 1], want) < 1e-2, (s, n)
    # one key that must win, wherever it lies among the 32768 (and the 20000 of the other long sequence)
    for far in (0, 63, 64, 1023, 1024, 8191, 16383, 16384, 19999 - 64, 19999):
        picks = [far, 50, 4096, 0, far, 63]
        qkv = torch.cat([picking_queries(keys[s], [f], nh, nkv, hd) for s, f in enumerate(picks)])
        ops.attention(qkv, nh, nkv, hd, kv, batch, out, scale=1.0 / math.sqrt(hd))
        for s, f in enumerate(picks):
            assert_picked(out[s:s + 1], values[s], [f], nh, nkv, hd, f"decode, sequence of {lengths[s]}, key {f}")
    for far in (32767 - 64, 32704, 32767, 20000, 24575, 24576):
        qkv = torch.cat([picking_queries(keys[s], [far if s == 0 else 0], nh, nkv, hd) for s in slots])
        ops.attention(qkv, nh, nkv, hd, kv, batch, out, scale=1.0 / math.sqrt(hd))
        assert_picked(out[:1], values[0], [far], nh, nkv, hd, f"decode over 32768 keys, key {far}")


@pytest.mark.parametrize("batch_size", [1, 8, 64])
def test_decode_finds_keys_at_4096_whatever_the_batch(ops, batch_size):
    """A batch's size decides into how many parts the decode kernel cuts the keys (none at 64 sequences)."""
    nh, nkv, hd = 32, 8, 128
    lengths = [4096] + [4096 - 17 * i for i in range(1, batch_size)]
    kv, keys, values = long_cache(nkv, hd, lengths, seed=batch_size)
    slots = list(range(batch_size))
    batch = described(slots, [1] * batch_size, [n - 1 for n in lengths])
    out = torch.empty(batch_size, nh * hd, dtype=torch.bfloat16, device=DEV)
    for round_, far in enumerate((0, 63, 64, 2047, 2048, 2049, 3000, 4031)):
        picks = [min(n - 1, (far + 64 * s) % n if round_ % 2 else far) for s, n in enumerate(lengths)]
        qkv = torch.cat([picking_queries(keys[s], [f], nh, nkv, hd) for s, f in enumerate(picks)])
        ops.attention(qkv, nh, nkv, hd, kv, batch, out, scale=1.0 / math.sqrt(hd))
        for s, f in enumerate(picks):
            assert_picked(out[s:s + 1], values[s], [f], nh, nkv, hd, f"decode, batch {batch_size}, sequence {s}, key {f}")
    qkv = torch.cat([picking_queries(keys[s], [n - 1], nh, nkv, hd) for s, n in enumerate(lengths)])     # every sequence's last key
    ops.attention(qkv, nh, nkv, hd, kv, batch, out, scale=1.0 / math.sqrt(hd))
    for s, n in enumerate(lengths):
        assert_picked(out[s:s + 1], values[s], [n - 1], nh, nkv, hd, f"decode, batch {batch_size}, sequence {s}, its last key")


# ---- prefill ---------------------------------------------------------------------------------

def keys_to_pick(start, count):
    """For every query row of a step that brings `count` tokens from position `start` on, a key it can see:
    rows take turns over places that a wrong block or a wrong mask would miss."""
    far = []
    for t in range(count):
        pos = start + t
        early_end = (start + 127) // BLOCK * BLOCK           # about where the first tile of 128 queries stops seeing keys
        places = [0, 63, 64, pos, pos - 1, pos - 63, pos - 64, pos // BLOCK * BLOCK, pos // BLOCK * BLOCK - 1,
                  early_end - 1, early_end, early_end + 63, early_end + 64, early_end + 127, early_end + 128,
                  start, start - 1, start // 2, pos // 2, (pos * 7 + 13) % (pos + 1)]
        far.append(min(pos, max(0, places[(t + t // 32) % len(places)])))
    return far


@pytest.mark.parametrize("nh,nkv,hd", [(8, 2, 128), (4, 4, 64)])
@pytest.mark.parametrize("start,count", [(0, 129), (0, 300), (0, 1000), (37, 300), (64, 300), (3096, 1000),
                                         (3967, 129), (1001, 300), (200, 1), (0, 257), (3072, 1024), (91, 385)])
def test_prefill_finds_far_keys_in_every_tile(ops, nh, nkv, hd, start, count):
    """Steps of one, two, three and eight tiles of 128 queries, from position 0 and from positions on and off a
    block's edge (the early tile of a pair then ends after an even or an odd number of blocks), over a cache of up to
    4096 keys. Every query row is checked, each against a key of its own."""
    kv, keys, values = long_cache(nkv, hd, [start + count, 77], seed=start + count)
    far = keys_to_pick(start, count)
    qkv = picking_queries(keys[0], far, nh, nkv, hd)
    # a second, short sequence in the same step, before the long one: the long one's rows then start off a tile's edge
    other = picking_queries(keys[1], list(range(77)), nh, nkv, hd)
    batch = described([1, 0], [77, count], [0, start])
    out = torch.full((77 + count, nh * hd), 7.0, dtype=torch.bfloat16, device=DEV)
    ops.attention(torch.cat([other, qkv]), nh, nkv, hd, kv, batch, out, scale=1.0 / math.sqrt(hd))
    assert_picked(out[:77], values[1], list(range(77)), nh, nkv, hd, "the short sequence beside it")
    assert_picked(out[77:], values[0], far, nh, nkv, hd, f"prefill of {count} tokens from {start}")
    # the last 40 tokens alone (one tile, part of it beyond the step's end), and the last one alone (the decode kernel)
    for tail in (40, 1):
        if count > tail:
            batch = described([0], [tail], [start + count - tail])
            out = torch.full((tail, nh * hd), 7.0, dtype=torch.bfloat16, device=DEV)
            ops.attention(qkv[-tail:].contiguous(), nh, nkv, hd, kv, batch, out, scale=1.0 / math.sqrt(hd))
            assert_picked(out, values[0], far[-tail:], nh, nkv, hd, f"the last {tail} of {start + count} tokens")


@pytest.mark.parametrize("nh,nkv,hd", [(8, 2, 128), (4, 1, 64)])
@pytest.mark.parametrize("start,count", [(0, 8192), (6144, 2048)])
def test_prefill_of_thousands_of_tokens(ops, nh, nkv, hd, start, count):
    """A prompt of 8192 tokens in one step, and 2048 tokens that continue a cache of 6144: random queries against plain
    attention in 64-bit, then queries that each pick out one key."""
    kv, keys, values = long_cache(nkv, hd, [start + count], seed=count + nh)
    batch = described([0], [count], [start])
    qkv = rand(count, (nh + 2 * nkv) * hd, seed=5)
    out = torch.full((count, nh * hd), 7.0, dtype=torch.bfloat16, device=DEV)
    ops.attention(qkv, nh, nkv, hd, kv, batch, out, scale=1.0 / math.sqrt(hd))
    assert torch.isfinite(out).all()
    positions = list(range(start, start + count))
    for first in range(0, count, 2048):                     # the plain scores of 2048 rows at a time
        rows = slice(first, first + 2048)
        want = plain_attention(qkv[rows, :nh * hd], positions[rows], keys[0], values[0], nh, nkv, hd)
        assert rel(out[rows], want) < 1e-2, first
    far = keys_to_pick(start, count)
    ops.attention(picking_queries(keys[0], far, nh, nkv, hd), nh, nkv, hd, kv, batch, out, scale=1.0 / math.sqrt(hd))
    assert_picked(out, values[0], far, nh, nkv, hd, f"prefill of {count} tokens from {start}")
