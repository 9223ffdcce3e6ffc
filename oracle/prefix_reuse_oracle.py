"""CPU restatement of the reference's prefix-reuse lookups (the checker for PrefixCache and
RadixAttentionCache).

TEST INFRASTRUCTURE ONLY.  Nothing under the product package imports this module; only tests/
do, as the checker.

  longest_cached_prefix   what both caches must return while nothing has been evicted or
                          replaced: the longest run of full blocks, from the start of the query,
                          that some inserted prompt has at the same position with the same
                          predecessors (src/inference/prefix_cache.py:110-150 and
                          src/inference/radix_cache.py:90-139 both stop at the first full block
                          that is not cached); the block ids are those of the prompt that cached
                          each block first (neither cache overwrites an existing entry,
                          prefix_cache.py:178-187, radix_cache.py:163-166).  Brute force over
                          the inserted prompts: no tree, no hash.
  FirstTokenTrie          the radix tree's replacement rule in its smallest form
                          (radix_cache.py:116-137, 155-227): nested dicts, one child per first
                          token of a block; a differing block with the same first token replaces
                          the child (and what hangs below it) when the child was never matched,
                          and stops the insert when it was.

Pinning (tests/test_radix_cache_host.py): FirstTokenTrie equals longest_cached_prefix on streams
whose blocks never share a first token with a differing sibling (random tokens from a large
vocabulary, prompts that branch only at random positions), and the replacement rule is checked on
hand-worked cases: A then B (same first token) -> A and its descendants are gone; A matched once,
then B -> B and its tail are not cached and A still is.
"""
from typing import Dict, List, Sequence, Tuple


def _full_blocks(tokens: Sequence[int], bs: int) -> List[Tuple[int, ...]]:
    return [tuple(tokens[i * bs:(i + 1) * bs]) for i in range(len(tokens) // bs)]


def longest_cached_prefix(inserted: Sequence[Tuple[Sequence[int], Sequence[int]]],
                          query: Sequence[int], bs: int) -> Tuple[int, List[int]]:
    """`inserted` = [(token_ids, block_ids), ...] in insertion order."""
    ids: List[int] = []
    q = _full_blocks(query, bs)
    for depth in range(len(q)):
        owner = None
        for tokens, block_ids in inserted:
            blocks = _full_blocks(tokens, bs)[:len(block_ids)]
            if len(blocks) > depth and blocks[:depth + 1] == q[:depth + 1]:
                owner = block_ids[depth]
                break                                   # first come, first cached
        if owner is None:
            break
        ids.append(owner)
    return len(ids) * bs, ids


class FirstTokenTrie:
    """node = {"tokens": tuple, "block": id, "matched": count, "kids": {first_token: node}}"""

    def __init__(self, bs: int):
        self.bs = bs
        self.kids: Dict[int, dict] = {}

    def match(self, query: Sequence[int]) -> Tuple[int, List[int]]:
        ids, kids = [], self.kids
        for blk in _full_blocks(query, self.bs):
            node = kids.get(blk[0])
            if node is None or node["tokens"] != blk:
                break
            node["matched"] += 1
            ids.append(node["block"])
            kids = node["kids"]
        return len(ids) * self.bs, ids

    def insert(self, tokens: Sequence[int], block_ids: Sequence[int]):
        kids = self.kids
        for blk, bid in zip(_full_blocks(tokens, self.bs), block_ids):
            node = kids.get(blk[0])
            if node is None or node["tokens"] != blk:
                if node is not None and node["matched"] > 0:
                    return
                node = {"tokens": blk, "block": bid, "matched": 0, "kids": {}}
                kids[blk[0]] = node
            kids = node["kids"]

    def count(self) -> int:
        n, stack = 0, [self.kids]
        while stack:
            for node in stack.pop().values():
                n += 1
                stack.append(node["kids"])
        return n
