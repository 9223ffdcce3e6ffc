"""Block-granular prefix cache over the paged KV pool.

Mirrors the reference's PrefixCache (src/inference/prefix_cache.py:58-265): full blocks of a
prompt are keyed by a chained 64-bit hash, hash(block_i) = H(hash(block_{i-1}) || token ids of
block i), so a lookup matches exactly the blocks of the longest cached prefix; entries carry
the token ids to rule out collisions, and eviction is least-recently-used among unreferenced
entries first.  Same method names, arguments and return values.

What the reference leaves open is who keeps a cached block alive: its cache stores block ids
only, and the engine allocates fresh blocks for a hit (src/inference/engine.py:587-595,
1108-1113).  Here the cache can be given the BlockPool: an entry then owns one reference of its
block (BlockPool.share), so the block outlives the sequence that filled it and a hit can be
handed to KVCacheManager.allocate_for_sequence(shared_block_ids=...) as real aliases.
"""
import time
from typing import Dict, List, Optional, Tuple

try:
    import xxhash
    _XXHASH_AVAILABLE = True
except ImportError:  # pragma: no cover - xxhash ships with this image
    import hashlib
    _XXHASH_AVAILABLE = False


class CachedBlock:
    __slots__ = ["hash_value", "block_id", "ref_count", "last_access_time", "token_ids"]

    def __init__(self, hash_value: int, block_id: int, token_ids: Tuple[int, ...]):
        self.hash_value = hash_value
        self.block_id = block_id
        self.ref_count = 0            # sequences currently using this entry
        self.last_access_time = time.time()
        self.token_ids = token_ids


class PrefixCache:
    def __init__(self, block_size: int = 16, max_cached_blocks: int = 1024, block_pool=None):
        self._cache: Dict[int, CachedBlock] = {}
        self.block_size = block_size
        self.max_cached_blocks = max_cached_blocks
        self._pool = block_pool
        self.hits = 0
        self.misses = 0
        self._evictions = 0

    def compute_block_hash(self, token_ids: List[int], prev_hash: int = 0) -> int:
        """64-bit hash of one block chained to its predecessor's (0 for the first block)."""
        if _XXHASH_AVAILABLE:
            h = xxhash.xxh64()
            h.update(prev_hash.to_bytes(8, byteorder="little", signed=False))
            for tid in token_ids:
                h.update(int(tid).to_bytes(4, byteorder="little", signed=False))
            return h.intdigest()
        data = prev_hash.to_bytes(8, byteorder="little", signed=False)  # pragma: no cover
        for tid in token_ids:  # pragma: no cover
            data += int(tid).to_bytes(4, byteorder="little", signed=False)
        return int(hashlib.sha256(data).hexdigest()[:16], 16)  # pragma: no cover

    def match_prefix(self, token_ids: List[int]) -> Tuple[int, List[int]]:
        """(tokens matched from the start, physical ids of the matched full blocks).  Each
        matched entry's ref_count goes up by one; release_block undoes it."""
        matched_tokens = 0
        matched_block_ids: List[int] = []
        prev_hash = 0
        for block_idx in range(len(token_ids) // self.block_size):
            block_tokens = token_ids[block_idx * self.block_size:(block_idx + 1) * self.block_size]
            block_hash = self.compute_block_hash(block_tokens, prev_hash)
            cached = self._cache.get(block_hash)
            if cached is not None and tuple(block_tokens) == cached.token_ids:
                cached.last_access_time = time.time()
                cached.ref_count += 1
                matched_tokens += self.block_size
                matched_block_ids.append(cached.block_id)
                prev_hash = block_hash
                self.hits += 1
            else:
                self.misses += 1
                break
        return matched_tokens, matched_block_ids

    def block_hashes(self, token_ids: List[int], num_blocks: Optional[int] = None) -> List[int]:
        """Chained hashes of the first num_blocks full blocks (all of them by default)."""
        n = len(token_ids) // self.block_size
        if num_blocks is not None:
            n = min(n, num_blocks)
        out, prev = [], 0
        for i in range(n):
            prev = self.compute_block_hash(token_ids[i * self.block_size:(i + 1) * self.block_size], prev)
            out.append(prev)
        return out

    def insert(self, token_ids: List[int], block_ids: List[int]):
        """Register the full blocks of a computed prompt.  With a pool attached every new entry
        takes a reference of its block."""
        prev_hash = 0
        num_blocks = min(len(token_ids) // self.block_size, len(block_ids))
        for block_idx in range(num_blocks):
            block_tokens = token_ids[block_idx * self.block_size:(block_idx + 1) * self.block_size]
            block_hash = self.compute_block_hash(block_tokens, prev_hash)
            if len(self._cache) >= self.max_cached_blocks and block_hash not in self._cache:
                self.evict_lru(num_blocks=1)
            entry = self._cache.get(block_hash)
            if entry is None:
                if self._pool is not None:
                    self._pool.share(self._pool.get_block(block_ids[block_idx]))
                self._cache[block_hash] = CachedBlock(block_hash, block_ids[block_idx], tuple(block_tokens))
            else:
                entry.last_access_time = time.time()
            prev_hash = block_hash

    def _drop(self, block_hash: int):
        entry = self._cache.pop(block_hash)
        if self._pool is not None:
            self._pool.free(self._pool.get_block(entry.block_id))

    def evict_lru(self, num_blocks: int = 1):
        """Remove the least recently used entries, unreferenced ones first."""
        evicted = 0
        while evicted < num_blocks and self._cache:
            idle = [(cb.last_access_time, h) for h, cb in self._cache.items() if cb.ref_count <= 0]
            pick = min(idle) if idle else min((cb.last_access_time, h) for h, cb in self._cache.items())
            self._drop(pick[1])
            evicted += 1
            self._evictions += 1

    def release_block(self, block_hash: int):
        cached = self._cache.get(block_hash)
        if cached is not None:
            cached.ref_count = max(0, cached.ref_count - 1)

    def invalidate_all(self):
        """Forget everything (after a weight update the cached K/V are stale)."""
        for block_hash in list(self._cache):
            self._drop(block_hash)

    @property
    def hit_rate(self) -> float:
        total = self.hits + self.misses
        return self.hits / total if total else 0.0

    @property
    def size(self) -> int:
        return len(self._cache)

    def get_stats(self) -> dict:
        return {
            "cached_blocks": len(self._cache),
            "max_cached_blocks": self.max_cached_blocks,
            "utilization": ("%.1f%%" % (100.0 * len(self._cache) / self.max_cached_blocks))
            if self.max_cached_blocks > 0 else "N/A",
            "hits": self.hits,
            "misses": self.misses,
            "hit_rate": "%.1f%%" % (100.0 * self.hit_rate),
            "evictions": self._evictions,
            "block_size": self.block_size,
        }
