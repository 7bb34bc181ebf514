"""The order of the elements inside a cache block, as the tests know it: written from the description of the
layout (a block of a head whose size is a multiple of 32 lies in tiles of 64 pieces of 8 elements, in the order
in which a wavefront of the decode kernel feeds them to the matrix cores; other head sizes lie in rows), with
index arithmetic on whole tensors. The kernel library and the C++ reference each have their own wording of it;
tests/test_cache_order.py holds the three against each other and against offsets worked out by hand.

A cache tensor keeps the shapes keys [blocks, kv_heads, 64, head_dim], values [blocks, kv_heads, head_dim, 64];
only the order of the 64 * head_dim elements behind the last two dimensions is the library's own."""
import torch

BLOCK = 64


def key_places(head_dim: int) -> torch.Tensor:
    """[64, head_dim]: element offset of (token, dim) of a key within its block."""
    token = torch.arange(BLOCK)[:, None].expand(BLOCK, head_dim)
    dim = torch.arange(head_dim)[None, :].expand(BLOCK, head_dim)
    if head_dim % 32 != 0:
        return token * head_dim + dim
    half, within = token // 32, token % 32               # the block's halves of 32 keys
    score_tile, row = within % 8 // 4, within // 8 * 4 + within % 4      # key 8 a + 4 t + b is row 4 a + b of score tile t
    tile = (half * 2 + score_tile) * (head_dim // 32) + dim // 32
    lane = row + 16 * (dim % 32 // 8)
    return (tile * 64 + lane) * 8 + dim % 8


def value_places(head_dim: int) -> torch.Tensor:
    """[head_dim, 64]: element offset of (dim, token) of a value within its block."""
    dim = torch.arange(head_dim)[:, None].expand(head_dim, BLOCK)
    token = torch.arange(BLOCK)[None, :].expand(head_dim, BLOCK)
    if head_dim % 32 != 0:
        return dim * BLOCK + token
    tile = token // 32 * (head_dim // 16) + dim // 16
    lane = dim % 16 + 16 * (token % 32 // 8)
    return (tile * 64 + lane) * 8 + token % 8


def _flat(cache):
    return cache.view(*cache.shape[:-2], cache.shape[-2] * cache.shape[-1])


def key_index(cache_k, token_in_block):
    """Offsets, on the cache's device, of all dims of the keys at the given places (an int or a tensor of them) of a block."""
    return key_places(cache_k.shape[-1]).to(cache_k.device)[token_in_block]


def value_index(cache_v, token_in_block):
    return value_places(cache_v.shape[-2]).to(cache_v.device)[:, token_in_block]


def write_key(cache_k, block, token_in_block, keys):
    """keys [kv_heads, head_dim] of one token into block `block`."""
    _flat(cache_k)[block][:, key_index(cache_k, token_in_block)] = keys.to(cache_k.dtype)


def write_value(cache_v, block, token_in_block, values):
    _flat(cache_v)[block][:, value_index(cache_v, token_in_block)] = values.to(cache_v.dtype)


def read_keys(cache_k, blocks, token_in_block):
    """Keys [n, kv_heads, head_dim] of n (block, place) pairs."""
    index = key_index(cache_k, token_in_block)                           # [n, head_dim]
    heads = torch.arange(cache_k.shape[1], device=cache_k.device)
    return _flat(cache_k)[blocks[:, None, None], heads[None, :, None], index[:, None, :]]


def read_values(cache_v, blocks, token_in_block):
    index = value_index(cache_v, token_in_block).t()                     # [n, head_dim]
    heads = torch.arange(cache_v.shape[1], device=cache_v.device)
    return _flat(cache_v)[blocks[:, None, None], heads[None, :, None], index[:, None, :]]


def store_keys(plain):
    """A tensor [..., 64, head_dim] of keys in rows, in the cache's order (same shape)."""
    out = torch.empty_like(plain)
    _flat(out)[..., key_places(plain.shape[-1]).reshape(-1).to(plain.device)] = _flat(plain)
    return out


def store_values(plain):
    """A tensor [..., head_dim, 64] of transposed values, in the cache's order (same shape)."""
    out = torch.empty_like(plain)
    _flat(out)[..., value_places(plain.shape[-2]).reshape(-1).to(plain.device)] = _flat(plain)
    return out


def plain_keys(stored):
    return _flat(stored)[..., key_places(stored.shape[-1]).reshape(-1).to(stored.device)].view(stored.shape)


def plain_values(stored):
    return _flat(stored)[..., value_places(stored.shape[-2]).reshape(-1).to(stored.device)].view(stored.shape)
