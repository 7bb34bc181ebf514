"""The order of a cache block, three wordings of it held against each other: the kernel library's (csrc/cache_layout.h,
through its host functions), the C++ reference's (a walk through the block in the decode kernel's order) and the
tests' own (cache_order.py, index arithmetic on tensors), and against offsets worked out by hand from the description."""
import pytest
import torch

import cache_order


def test_places_are_a_permutation_and_keep_pieces_whole():
    for hd in (16, 32, 48, 64, 96, 128, 256):
        keys, values = cache_order.key_places(hd), cache_order.value_places(hd)
        assert sorted(keys.reshape(-1).tolist()) == list(range(64 * hd))
        assert sorted(values.reshape(-1).tolist()) == list(range(64 * hd))
        # 8 dims of a key from a multiple of 8, and 8 tokens of a value dim, are 8 neighbours in the block
        assert torch.equal(keys.view(64, hd // 8, 8), keys.view(64, hd // 8, 8)[:, :, :1] + torch.arange(8))
        assert torch.equal(values.view(hd, 8, 8), values.view(hd, 8, 8)[:, :, :1] + torch.arange(8))
    # a tile of 1 KB of bfloat16 is what one load instruction of the decode kernel takes: for head size 128, the first
    # tile of the keys holds dims 0..31 of keys 0..3, 8..11, 16..19, 24..27 (score tile 0 of the first half)
    keys = cache_order.key_places(128)
    first_tile = {(t, d) for t in range(64) for d in range(128) if int(keys[t, d]) < 512}
    assert first_tile == {(8 * a + b, d) for a in range(4) for b in range(4) for d in range(32)}
    values = cache_order.value_places(128)
    first_tile = {(d, t) for d in range(128) for t in range(64) if int(values[d, t]) < 512}
    assert first_tile == {(d, t) for d in range(16) for t in range(32)}


def test_offsets_worked_out_by_hand():
    # key 13 = 8 * 1 + 4 * 1 + 1: row 4 * 1 + 1 = 5 of score tile 1 of the first half; dim 21: lane group 2 of dims 0..31, element 5.
    # head size 64 has two tiles of 32 dims per score tile: tile (0 * 2 + 1) * 2 + 0 = 2, place 5 + 16 * 2 = 37
    assert int(cache_order.key_places(64)[13, 21]) == (2 * 64 + 37) * 8 + 5
    # value dim 21 = 16 + 5: row 5 of dims 16..31; token 45 = 32 + 8 + 5: second half, lane group 1, element 5; tile 1 * 4 + 1
    assert int(cache_order.value_places(64)[21, 45]) == (5 * 64 + 5 + 16) * 8 + 5
    assert int(cache_order.key_places(48)[13, 21]) == 13 * 48 + 21 and int(cache_order.value_places(48)[21, 45]) == 21 * 64 + 45


def test_the_cpp_reference_keeps_the_same_order():
    from reference_cpp import CppReference
    lib = CppReference().lib
    for hd in (16, 32, 80, 128):
        keys, values = cache_order.key_places(hd), cache_order.value_places(hd)
        for token in (0, 5, 13, 31, 32, 47, 63):
            for dim in range(hd):
                assert lib.xrt_ref_cache_key_offset(token, dim, hd) == int(keys[token, dim])
                assert lib.xrt_ref_cache_value_offset(dim, token, hd) == int(values[dim, token])


@pytest.mark.gpu
def test_the_kernel_library_keeps_the_same_order():
    from xeno_rt_amd.ops import load_ops
    lib = load_ops().lib
    for hd in (16, 32, 48, 64, 128, 256):
        keys, values = cache_order.key_places(hd), cache_order.value_places(hd)
        for token in range(64):
            for dim in range(hd):
                assert lib.xrt_cache_key_offset(token, dim, hd) == int(keys[token, dim])
                assert lib.xrt_cache_value_offset(dim, token, hd) == int(values[dim, token])


def test_store_and_read_back():
    g = torch.Generator().manual_seed(3)
    for hd in (48, 64):
        k, v = torch.randn(3, 2, 64, hd, generator=g), torch.randn(3, 2, hd, 64, generator=g)
        stored_k, stored_v = cache_order.store_keys(k), cache_order.store_values(v)
        assert torch.equal(cache_order.plain_keys(stored_k), k) and torch.equal(cache_order.plain_values(stored_v), v)
        blocks, places = torch.tensor([2, 0, 2]), torch.tensor([5, 63, 40])
        assert torch.equal(cache_order.read_keys(stored_k, blocks, places), k[blocks, :, places, :])
        assert torch.equal(cache_order.read_values(stored_v, blocks, places), v[blocks, :, :, places])
        fresh_k, fresh_v = torch.zeros_like(k), torch.zeros_like(v)
        for block in range(3):
            for place in range(64):
                cache_order.write_key(fresh_k, block, place, k[block, :, place, :])
                cache_order.write_value(fresh_v, block, place, v[block, :, :, place])
        assert torch.equal(fresh_k, stored_k) and torch.equal(fresh_v, stored_v)
