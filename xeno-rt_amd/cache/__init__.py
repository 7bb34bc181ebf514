"""The cache: slots, blocks, keys and values per layer call, per-sequence state."""
from .allocator import BLOCK_TOKENS, CacheError, CacheFull, Pool, blocks_for
from .sequence_cache import KVGroup, KVView, LayerCache, SequenceCache

__all__ = ["BLOCK_TOKENS", "CacheError", "CacheFull", "Pool", "blocks_for",
           "KVGroup", "KVView", "LayerCache", "SequenceCache"]
