"""Block-granular prefix cache over the paged KV pool.

Contract (the public surface of the reference's PrefixCache, src/inference/prefix_cache.py:58-265):
full blocks of a prompt are keyed by a chained 64-bit hash - hash(block i) = xxh64 over the 8
little-endian bytes of hash(block i-1) followed by the block's token ids as 4-byte little-endian
words, 0 standing in before the first block - so `match_prefix` finds exactly the blocks of the
longest cached prefix and returns (matched tokens, their physical block ids); entries remember
their token ids so that a hash collision cannot pass as a hit; eviction removes the least
recently used entry, entries no sequence is using before any other.  Method names, arguments,
return values and the keys of `get_stats` are the reference's.

How it is kept here: token ids are packed once per call into an array('I') and every block is
hashed from a slice of that buffer in a single update; entries live in two recency-ordered
dictionaries - those in use by a sequence and those idle - so a hit, a release and an eviction are
all constant-time moves, where a scan for the oldest time stamp would grow with the cache.

What the reference leaves open is who keeps a cached block alive: its cache stores block ids
only, and the engine allocates fresh blocks for a hit (src/inference/engine.py:587-595,
1108-1113).  Here the cache can be given the BlockPool: an entry then owns one reference of its
block (BlockPool.share), so the block outlives the sequence that filled it and a hit can be
handed to KVCacheManager.allocate_for_sequence(shared_block_ids=...) as real aliases.
"""
import struct
import time
from array import array
from collections import OrderedDict
from typing import Iterator, List, Optional, Sequence, Tuple

try:
    import xxhash

    def _digest64(data: bytes) -> int:
        return xxhash.xxh64_intdigest(data)

    _XXHASH_AVAILABLE = True
except ImportError:  # pragma: no cover - xxhash ships with this image
    import hashlib

    def _digest64(data: bytes) -> int:
        return int.from_bytes(hashlib.sha256(data).digest()[:8], "big")

    _XXHASH_AVAILABLE = False

_PREV = struct.Struct("<Q")


class CachedBlock:
    """One cached full block: its chained hash, the physical block that holds its K/V, how many
    running sequences matched it and have not released it yet, when it was last touched, and
    the token ids it stands for."""
    __slots__ = ("hash_value", "block_id", "ref_count", "last_access_time", "token_ids")

    def __init__(self, hash_value: int, block_id: int, token_ids: Tuple[int, ...]):
        self.hash_value = hash_value
        self.block_id = block_id
        self.ref_count = 0
        self.last_access_time = time.time()
        self.token_ids = token_ids


class PrefixCache:
    def __init__(self, block_size: int = 16, max_cached_blocks: int = 1024, block_pool=None):
        self.block_size = block_size
        self.max_cached_blocks = max_cached_blocks
        self._pool = block_pool
        # hash -> entry, oldest first; an entry is in exactly one of the two
        self._idle: "OrderedDict[int, CachedBlock]" = OrderedDict()
        self._in_use: "OrderedDict[int, CachedBlock]" = OrderedDict()
        self.hits = 0
        self.misses = 0
        self._evictions = 0

    # ------------------------------------------------------------------ hashing

    def compute_block_hash(self, token_ids: Sequence[int], prev_hash: int = 0) -> int:
        """64-bit hash of one block chained to its predecessor's (0 for the first block)."""
        return _digest64(_PREV.pack(prev_hash) + array("I", token_ids).tobytes())

    def _chain(self, token_ids: Sequence[int], limit: Optional[int] = None) -> Iterator[Tuple[int, int, bytes]]:
        """(block index, chained hash, packed token bytes) of the full blocks, hashed lazily: a
        lookup that misses at block 3 never hashes block 4."""
        count = len(token_ids) // self.block_size
        if limit is not None:
            count = min(count, limit)
        if count <= 0:
            return
        packed = array("I", token_ids[:count * self.block_size]).tobytes()
        step = 4 * self.block_size
        link = 0
        for index in range(count):
            piece = packed[index * step:(index + 1) * step]
            link = _digest64(_PREV.pack(link) + piece)
            yield index, link, piece

    def block_hashes(self, token_ids: Sequence[int], num_blocks: Optional[int] = None) -> List[int]:
        """Chained hashes of the first num_blocks full blocks (all of them by default)."""
        return [link for _, link, _ in self._chain(token_ids, num_blocks)]

    # ------------------------------------------------------------------ bookkeeping

    def _find(self, key: int) -> Optional[CachedBlock]:
        entry = self._idle.get(key)
        return entry if entry is not None else self._in_use.get(key)

    def _touch(self, key: int, entry: CachedBlock):
        """Mark as most recently used, in whichever of the two orders the entry belongs to."""
        entry.last_access_time = time.time()
        home, other = (self._in_use, self._idle) if entry.ref_count > 0 else (self._idle, self._in_use)
        other.pop(key, None)
        home[key] = entry
        home.move_to_end(key)

    def _drop(self, key: int):
        entry = self._idle.pop(key, None)
        if entry is None:
            entry = self._in_use.pop(key)
        if self._pool is not None:
            self._pool.free(self._pool.get_block(entry.block_id))

    # ------------------------------------------------------------------ the reference's calls

    def match_prefix(self, token_ids: Sequence[int]) -> Tuple[int, List[int]]:
        """(tokens matched from the start, physical ids of the matched full blocks).  Each
        matched entry's ref_count goes up by one; release_block undoes it."""
        found: List[int] = []
        for _, key, piece in self._chain(token_ids):
            entry = self._find(key)
            if entry is None or array("I", entry.token_ids).tobytes() != piece:
                self.misses += 1          # first block that is not cached (or a colliding hash)
                break
            entry.ref_count += 1
            self._touch(key, entry)
            self.hits += 1
            found.append(entry.block_id)
        return len(found) * self.block_size, found

    def insert(self, token_ids: Sequence[int], block_ids: Sequence[int]):
        """Register the full blocks of a computed prompt.  With a pool attached every new entry
        takes a reference of its block."""
        for index, key, _ in self._chain(token_ids, len(block_ids)):
            entry = self._find(key)
            if entry is not None:
                self._touch(key, entry)
                continue
            if self.size >= self.max_cached_blocks:
                self.evict_lru(num_blocks=1)
            if self._pool is not None:
                self._pool.share(self._pool.get_block(block_ids[index]))
            lo = index * self.block_size
            self._idle[key] = CachedBlock(key, block_ids[index], tuple(token_ids[lo:lo + self.block_size]))

    def evict_lru(self, num_blocks: int = 1):
        """Remove the least recently used entries, unreferenced ones first."""
        for _ in range(num_blocks):
            victims = self._idle or self._in_use
            if not victims:
                return
            self._drop(next(iter(victims)))
            self._evictions += 1

    def release_block(self, block_hash: int):
        """A sequence that matched this entry is done with it."""
        entry = self._in_use.get(block_hash)
        if entry is None:
            return
        entry.ref_count -= 1
        if entry.ref_count > 0:
            return
        entry.ref_count = 0
        # A release is not a use: the entry joins the idle ones at the place its last access
        # gives it, i.e. in front of the idle entries touched since then.
        del self._in_use[block_hash]
        later = []
        for key in reversed(self._idle):
            if self._idle[key].last_access_time <= entry.last_access_time:
                break
            later.append(key)
        self._idle[block_hash] = entry
        for key in reversed(later):
            self._idle.move_to_end(key)

    def invalidate_all(self):
        """Forget everything (after a weight update the cached K/V are stale)."""
        for key in list(self._idle) + list(self._in_use):
            self._drop(key)

    # ------------------------------------------------------------------ figures

    @property
    def hit_rate(self) -> float:
        seen = self.hits + self.misses
        return self.hits / seen if seen else 0.0

    @property
    def size(self) -> int:
        return len(self._idle) + len(self._in_use)

    def get_stats(self) -> dict:
        held, cap = self.size, self.max_cached_blocks
        return {
            "cached_blocks": held,
            "max_cached_blocks": cap,
            "utilization": "%.1f%%" % (100.0 * held / cap) if cap > 0 else "N/A",
            "hits": self.hits,
            "misses": self.misses,
            "hit_rate": "%.1f%%" % (100.0 * self.hit_rate),
            "evictions": self._evictions,
            "block_size": self.block_size,
        }
