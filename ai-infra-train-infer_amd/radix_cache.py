"""Block-granular radix tree over prompt token ids, for prefix reuse in the paged KV pool.

Mirrors the reference's RadixAttentionCache / RadixNode (src/inference/radix_cache.py:35-320):
one tree node per full block of `block_size` tokens, children indexed by the block's first token,
`match_prefix(token_ids) -> (matched_tokens, block_ids)` walks the tree block by block and stops at
the first block that is absent or differs, `insert(token_ids, block_ids)` adds the missing nodes
of a computed prompt.  Because a parent has one child per first token, a block that starts like a
cached sibling but differs later replaces that sibling when nothing has matched it
(ref_count == 0) and is skipped, with the rest of the prompt, when something has
(radix_cache.py:163-212).  Same constructor arguments, methods, counters and stats keys, so the
engine's `use_radix_cache` switch (src/inference/engine.py:366-371) works unchanged.

What is added, as for PrefixCache: given the BlockPool, every node owns one reference of its
block (BlockPool.share), released when the node is evicted, replaced or invalidated, so that a
match can be passed to KVCacheManager.allocate_for_sequence(shared_block_ids=...) as real
aliases.  `release_prefix` undoes the ref_count that `match_prefix` took (the reference never
lowers it: its release_block is a stub, radix_cache.py:237-243, kept here as one).

Where the bookkeeping differs from the reference, on purpose: `node_count` is the number of nodes
in the tree also after a replacement (the reference leaves the count as it was although the
replaced node's subtree goes with it, radix_cache.py:190-192), and eviction never removes a node
of the path being inserted (the reference can detach the node it is about to extend when every
other leaf is referenced, radix_cache.py:215-227).
"""
import time
from dataclasses import dataclass, field
from typing import Dict, List, Optional, Tuple


@dataclass(eq=False)
class RadixNode:
    token_chunk: List[int] = field(default_factory=list)        # the block's tokens (empty: root)
    children: Dict[int, "RadixNode"] = field(default_factory=dict)   # first token -> child
    kv_block_ids: List[int] = field(default_factory=list)       # physical block of this node
    token_count: int = 0
    last_access: float = field(default_factory=time.time)
    ref_count: int = 0                                          # matches not yet released
    parent: Optional["RadixNode"] = field(default=None, repr=False)
    access_seq: int = 0                                         # orders equal time stamps


class RadixAttentionCache:
    def __init__(self, block_size: int = 16, max_nodes: int = 10000, block_pool=None):
        self.root = RadixNode()
        self.block_size = block_size
        self.max_nodes = max_nodes
        self.node_count = 0
        self._pool = block_pool
        self._seq = 0
        self.hits = 0
        self.misses = 0
        self._evictions = 0

    # ---- helpers ----------------------------------------------------------------------------------
    def _touch(self, node: RadixNode):
        self._seq += 1
        node.last_access = time.time()
        node.access_seq = self._seq

    def _blocks(self, token_ids: List[int], limit: Optional[int] = None):
        n = len(token_ids) // self.block_size
        if limit is not None:
            n = min(n, limit)
        for i in range(n):
            yield i, list(token_ids[i * self.block_size:(i + 1) * self.block_size])

    def _new_node(self, parent: RadixNode, tokens: List[int], block_id: int) -> RadixNode:
        if self._pool is not None:
            self._pool.share(self._pool.get_block(block_id))
        node = RadixNode(token_chunk=tokens, kv_block_ids=[block_id], token_count=self.block_size,
                         parent=parent)
        self._touch(node)
        parent.children[tokens[0]] = node
        self.node_count += 1
        return node

    def _drop_subtree(self, node: RadixNode):
        """Detach `node` from its parent and give back the blocks of every node below it."""
        parent = node.parent
        if parent is not None and parent.children.get(node.token_chunk[0]) is node:
            del parent.children[node.token_chunk[0]]
        stack = [node]
        while stack:
            cur = stack.pop()
            stack.extend(cur.children.values())
            self.node_count -= 1
            if self._pool is not None:
                for block_id in cur.kv_block_ids:
                    self._pool.free(self._pool.get_block(block_id))
            cur.children = {}
            cur.parent = None

    # ---- the reference's interface ----------------------------------------------------------------
    def match_prefix(self, token_ids: List[int]) -> Tuple[int, List[int]]:
        """(tokens matched from the start, physical ids of the matched full blocks).  Every
        matched node's ref_count goes up by one; one hit per matched block, one miss for the
        block that ends the walk (radix_cache.py:90-139)."""
        matched_tokens = 0
        matched_block_ids: List[int] = []
        node = self.root
        for _, tokens in self._blocks(token_ids):
            child = node.children.get(tokens[0])
            if child is None or child.token_chunk != tokens:
                self.misses += 1
                break
            self._touch(child)
            child.ref_count += 1
            matched_tokens += self.block_size
            matched_block_ids.extend(child.kv_block_ids)
            self.hits += 1
            node = child
        return matched_tokens, matched_block_ids

    def insert(self, token_ids: List[int], block_ids: List[int]):
        """Add the full blocks of a computed prompt (radix_cache.py:141-227)."""
        node = self.root
        path = set()
        for i, tokens in self._blocks(token_ids, len(block_ids)):
            child = node.children.get(tokens[0])
            if child is not None and child.token_chunk == tokens:
                self._touch(child)                    # already cached: the stored block id stays
            elif child is not None:
                if child.ref_count > 0:
                    break                             # the sibling is in use: give up on the rest
                self._drop_subtree(child)
                child = self._new_node(node, tokens, block_ids[i])
            else:
                if self.node_count >= self.max_nodes:
                    self._evict_lru(protect=path)
                    if self.node_count >= self.max_nodes:
                        break                         # nothing but this prompt's own path is left
                child = self._new_node(node, tokens, block_ids[i])
            path.add(id(child))
            node = child

    def release_prefix(self, token_ids: List[int], num_blocks: Optional[int] = None):
        """Undo one match_prefix of this prompt: lower the ref_count of the nodes it matched
        (all cached full blocks of the prompt, or the first num_blocks of them)."""
        node = self.root
        for _, tokens in self._blocks(token_ids, num_blocks):
            child = node.children.get(tokens[0])
            if child is None or child.token_chunk != tokens:
                break
            child.ref_count = max(0, child.ref_count - 1)
            node = child

    def release_block(self, block_hash: int):
        """Present for callers written against PrefixCache; nodes are not addressed by hash."""

    def invalidate_all(self):
        """Forget everything (after a weight update the cached K/V are stale)."""
        for child in list(self.root.children.values()):
            self._drop_subtree(child)
        self.root = RadixNode()
        self.node_count = 0

    def evict_lru(self, num_blocks: int = 1):
        for _ in range(num_blocks):
            self._evict_lru()

    def _evict_lru(self, protect=()):
        """Remove one leaf: the least recently used unreferenced one, else the least recently
        used of all (radix_cache.py:250-275)."""
        best = None
        stack = [self.root]
        while stack:
            cur = stack.pop()
            for child in cur.children.values():
                if child.children:
                    stack.append(child)
                elif id(child) not in protect:
                    key = (child.ref_count > 0, child.last_access, child.access_seq)
                    if best is None or key < best[0]:
                        best = (key, child)
        if best is not None:
            self._drop_subtree(best[1])
            self._evictions += 1

    @property
    def hit_rate(self) -> float:
        total = self.hits + self.misses
        return self.hits / total if total else 0.0

    @property
    def size(self) -> int:
        return self.node_count

    def get_stats(self) -> dict:
        return {
            "type": "RadixAttentionCache",
            "cached_nodes": self.node_count,
            "max_nodes": self.max_nodes,
            "utilization": ("%.1f%%" % (100.0 * self.node_count / self.max_nodes))
            if self.max_nodes > 0 else "N/A",
            "hits": self.hits,
            "misses": self.misses,
            "hit_rate": "%.1f%%" % (100.0 * self.hit_rate),
            "evictions": self._evictions,
            "block_size": self.block_size,
        }
