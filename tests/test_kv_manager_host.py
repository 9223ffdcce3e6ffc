"""Host bookkeeping of the paged pool: allocation, sharing, copy-on-write decisions, prefix cache.

Runs on the CPU: the pool's tensors are tiny CPU tensors here and no kernel is called (the
device copy is covered by tests/test_gpu_block_sharing.py).  The calls the reference has
(src/inference/kv_cache.py:176-212, 318-486; src/inference/prefix_cache.py:58-265) are checked
for the reference's behaviour, the sharing extensions for their invariants.
"""
import warnings

import pytest
import torch

import ai_infra_train_infer_amd as pa

BS = 4


def pool(n=8, cache_dtype="fp16"):
    return pa.BlockPool(n, BS, num_layers=1, num_kv_heads=1, head_dim=8, device="cpu", cache_dtype=cache_dtype)


def refsum(p):
    return sum(b.ref_count for b in p._blocks)


def test_pool_allocate_free_fifo_and_double_free_warns():
    p = pool(3)
    a, b, c = p.allocate(), p.allocate(), p.allocate()
    assert [a.block_id, b.block_id, c.block_id] == [0, 1, 2] and p.allocate() is None
    assert p.num_free_blocks == 0 and p.num_used_blocks == 3 and p.utilization == 1.0
    p.free(b)
    assert p.num_free_blocks == 1 and b.ref_count == 0
    with warnings.catch_warnings(record=True) as w:
        warnings.simplefilter("always")
        p.free(b)
    assert any("Double-free" in str(x.message) for x in w) and p.num_free_blocks == 1
    assert p.allocate().block_id == 1      # freed blocks go to the back of the queue: only one is free


def test_manager_reference_calls():
    p = pool(8)
    m = pa.KVCacheManager(p, BS)
    assert m.can_allocate(4 * BS) and not m.can_allocate(8 * BS)     # keeps one spare block
    t = m.allocate_for_sequence("a", 2 * BS + 1)
    assert t.num_blocks == 3 and t.num_tokens == 2 * BS + 1
    assert [b.is_full for b in t.blocks] == [True, True, False] and t.last_block.token_count == 1
    for _ in range(BS - 1):
        assert m.append_token("a")
    assert t.num_blocks == 3 and t.last_block.is_full
    assert m.append_token("a") and t.num_blocks == 4 and m.get_seq_token_count("a") == 3 * BS + 1
    assert m.get_block_table("a") == [0, 1, 2, 3] and m.get_block_table("nobody") == []
    assert not m.append_token("nobody")
    with pytest.raises(RuntimeError, match="OOM"):
        m.allocate_for_sequence("b", 5 * BS)
    assert p.num_free_blocks == 4                                   # the failed request was rolled back
    e = m.allocate_for_sequence("empty", 0)
    assert e.num_blocks == 0 and m.append_token("empty") and e.num_tokens == 1
    m.free_sequence("a"); m.free_sequence("empty"); m.free_sequence("a")
    assert p.num_free_blocks == 8 and refsum(p) == 0
    assert m.get_stats()["active_sequences"] == 0


def test_fork_shares_everything_and_first_writer_copies():
    p = pool(8)
    m = pa.KVCacheManager(p, BS)
    m.allocate_for_sequence("p", BS + 2)            # blocks 0 (full), 1 (2 of 4 tokens)
    kids = ["k0", "k1", "k2"]
    for k in kids:
        m.fork_sequence("p", k)
    assert all(m.get_block_table(k) == [0, 1] for k in kids) and p.num_used_blocks == 2
    assert p.get_block(0).ref_count == 4 and p.get_block(1).ref_count == 4
    # every sample appends one token: the first three writers move to copies, the last owner stays
    slots = {}
    for s in ["p"] + kids:
        assert m.append_token(s)
        slots[s] = m.next_slot(s)
    tables = {s: m.get_block_table(s) for s in ["p"] + kids}
    assert all(t[0] == 0 for t in tables.values())                       # the full block stays shared
    lasts = [t[1] for t in tables.values()]
    assert len(set(lasts)) == 4 and lasts.count(1) == 1                   # private last blocks, one is the original
    assert sorted(m.pending_copies) == sorted((1, b) for b in lasts if b != 1)
    assert all(slot == tables[s][1] * BS + 2 for s, slot in slots.items())   # token index 2 of the last block
    assert all(p.get_block(b).ref_count == 1 for b in lasts) and p.get_block(0).ref_count == 4
    # no writer ever targets a block with another owner
    for s, slot in slots.items():
        assert p.get_block(slot // BS).ref_count == 1
    for s in ["p"] + kids:
        m.free_sequence(s)
    assert p.num_free_blocks == 8 and refsum(p) == 0


def test_fork_at_block_boundary_needs_no_copy():
    p = pool(6)
    m = pa.KVCacheManager(p, BS)
    m.allocate_for_sequence("p", 2 * BS)
    m.fork_sequence("p", "k")
    assert m.append_token("p") and m.append_token("k")
    assert m.pending_copies == [] and m.get_block_table("p")[:2] == m.get_block_table("k")[:2]
    assert m.get_block_table("p")[2] != m.get_block_table("k")[2]


def test_append_fails_cleanly_when_the_copy_cannot_be_allocated():
    p = pool(2)
    m = pa.KVCacheManager(p, BS)
    m.allocate_for_sequence("p", BS + 1)
    m.fork_sequence("p", "k")
    before = (m.get_block_table("k"), p.get_block(1).ref_count, m.get_seq_token_count("k"))
    assert not m.append_token("k")
    assert (m.get_block_table("k"), p.get_block(1).ref_count, m.get_seq_token_count("k")) == before
    assert m.pending_copies == []


def test_shared_prefix_allocation_and_validation():
    p = pool(8)
    m = pa.KVCacheManager(p, BS)
    m.allocate_for_sequence("a", 3 * BS)
    t = m.allocate_for_sequence("b", 2 * BS + 3, shared_block_ids=[0, 1])
    assert t.get_physical_block_ids()[:2] == [0, 1] and t.num_blocks == 3 and t.num_tokens == 2 * BS + 3
    assert p.get_block(0).ref_count == 2 and p.get_block(2).ref_count == 1
    assert m.can_allocate(4 * BS, num_shared_blocks=2)
    with pytest.raises(RuntimeError, match="shared blocks hold more"):
        m.allocate_for_sequence("c", BS, shared_block_ids=[0, 1])
    with pytest.raises(RuntimeError, match="not a full, live block"):
        m.allocate_for_sequence("c", 3 * BS, shared_block_ids=[0, 7])
    assert p.get_block(0).ref_count == 2                               # rolled back
    m.free_sequence("a")
    assert p.get_block(0).ref_count == 1 and p.num_used_blocks == 3    # b keeps the prefix alive
    m.free_sequence("b")
    assert p.num_free_blocks == 8


def test_prefix_cache_reference_behaviour():
    c = pa.PrefixCache(block_size=BS, max_cached_blocks=3)
    prompt = list(range(100, 100 + 3 * BS + 2))
    assert c.match_prefix(prompt) == (0, []) and c.misses == 1
    c.insert(prompt, [5, 6, 7, 8])
    assert c.size == 3                                                  # only full blocks
    assert c.match_prefix(prompt) == (3 * BS, [5, 6, 7])
    other = prompt[:BS] + [1] * (2 * BS)
    assert c.match_prefix(other) == (BS, [5])                           # chain breaks at block 1
    shifted = [9] + prompt
    assert c.match_prefix(shifted)[0] == 0
    # chained hash: same tokens, different predecessor -> different key
    assert c.compute_block_hash(prompt[BS:2 * BS], 0) != c.block_hashes(prompt)[1]
    assert c.block_hashes(prompt, 2) == c.block_hashes(prompt)[:2]
    # LRU: entries in use survive while an idle one exists
    for h in c.block_hashes(prompt)[1:]:
        c.release_block(h); c.release_block(h)
    c.insert([7] * BS, [9])
    assert c.size == 3 and c.match_prefix(prompt)[0] == BS             # an idle entry of the old prompt went
    assert c.get_stats()["evictions"] == 1 and 0.0 < c.hit_rate < 1.0
    c.invalidate_all()
    assert c.size == 0


def test_prefix_cache_keeps_blocks_alive_and_feeds_shared_allocation():
    p = pool(8)
    m = pa.KVCacheManager(p, BS)
    c = pa.PrefixCache(block_size=BS, max_cached_blocks=16, block_pool=p)
    prompt = list(range(2 * BS + 1))
    m.allocate_for_sequence("first", len(prompt))
    c.insert(prompt, m.get_block_table("first"))
    m.free_sequence("first")
    assert p.num_used_blocks == 2 and p.get_block(0).ref_count == 1    # the cache owns the two full blocks
    n, ids = c.match_prefix(prompt)
    assert (n, ids) == (2 * BS, [0, 1])
    t = m.allocate_for_sequence("second", len(prompt), shared_block_ids=ids)
    assert t.get_physical_block_ids()[:2] == [0, 1] and p.get_block(0).ref_count == 2
    c.invalidate_all()
    assert p.get_block(0).ref_count == 1                               # the sequence still holds them
    m.free_sequence("second")
    assert p.num_free_blocks == 8 and refsum(p) == 0


def test_copy_blocks_on_cpu_pool_fails_loudly():
    p = pool(4)
    with pytest.raises(RuntimeError, match="no CPU path"):
        p.copy_blocks([(0, 1)])
    p.copy_blocks([])            # nothing to do is fine anywhere


def test_duplicate_sequence_ids_are_refused():
    p = pool(8)
    m = pa.KVCacheManager(p, BS)
    m.allocate_for_sequence("a", BS + 1)
    with pytest.raises(RuntimeError, match="already has a block table"):
        m.allocate_for_sequence("a", 1)
    with pytest.raises(RuntimeError, match="already has a block table"):
        m.fork_sequence("a", "a")
    assert p.num_used_blocks == 2                   # nothing leaked, nothing replaced
    m.free_sequence("a")
    m.allocate_for_sequence("a", 1)
    assert p.num_used_blocks == 1


def test_chained_copies_are_cut_into_ordered_launches():
    cut = pa.KVCacheManager._ordered_batches
    assert cut([]) == []
    assert cut([(1, 2), (3, 4), (1, 5)]) == [[(1, 2), (3, 4), (1, 5)]]          # shared sources are fine
    assert cut([(1, 2), (2, 3)]) == [[(1, 2)], [(2, 3)]]                          # reads what the first writes
    assert cut([(1, 2), (7, 1)]) == [[(1, 2)], [(7, 1)]]                          # overwrites what the first reads
    assert cut([(1, 2), (3, 2), (4, 5)]) == [[(1, 2)], [(3, 2), (4, 5)]]          # same destination twice


def test_a_freed_source_reused_as_destination_is_copied_in_order():
    """Nearly full pool: block 0 is queued as a copy's source, its last owner leaves, and a later
    copy-on-write is handed block 0 as its destination.  The launches keep the queue's order."""
    p = pool(4)
    m = pa.KVCacheManager(p, BS)
    m.allocate_for_sequence("a", 2)                 # block 0, half full
    m.fork_sequence("a", "b")
    assert m.append_token("b")                      # b moves to a copy: (0 -> 1)
    m.free_sequence("a")                            # block 0 loses its last owner: free again
    m.allocate_for_sequence("c", 2)                 # block 2
    m.fork_sequence("c", "d")
    assert m.append_token("d")                      # (2 -> 3)
    m.fork_sequence("c", "g")
    assert m.append_token("g")                      # the only free block is 0: (2 -> 0)
    assert m.pending_copies == [(0, 1), (2, 3), (2, 0)]
    launched = []
    p.copy_blocks = lambda pairs: launched.append(list(pairs))
    m.apply_copies()
    assert launched == [[(0, 1), (2, 3)], [(2, 0)]] and m.pending_copies == []


def test_prefix_hash_is_the_documented_xxh64_chain():
    """compute_block_hash == xxh64 over (previous hash as 8 LE bytes) + (token ids as 4-byte LE
    words), fed here one word at a time through the streaming interface."""
    import xxhash
    c = pa.PrefixCache(block_size=BS)
    toks, prev = [7, 0, 2 ** 31 + 5, 151935], 0x0123456789ABCDEF
    h = xxhash.xxh64()
    h.update(prev.to_bytes(8, "little"))
    for t in toks:
        h.update(t.to_bytes(4, "little"))
    assert c.compute_block_hash(toks, prev) == h.intdigest()
    first = xxhash.xxh64(b"\0" * 8 + b"".join(t.to_bytes(4, "little") for t in toks)).intdigest()
    assert c.block_hashes(toks + toks) == [first, c.compute_block_hash(toks, first)]


def test_prefix_cache_eviction_order():
    c = pa.PrefixCache(block_size=1, max_cached_blocks=3)
    c.insert([10], [0]); c.insert([20], [1]); c.insert([30], [2])
    assert c.match_prefix([10]) == (1, [0])         # 10 is in use and now the most recently touched
    c.insert([40], [3])                             # evicts the oldest idle entry: 20
    assert c.match_prefix([20])[0] == 0 and c.size == 3
    c.release_block(c.compute_block_hash([10]))     # 10 idle again, but still younger than 30
    c.insert([50], [4])                             # so 30 goes
    assert c.match_prefix([30])[0] == 0
    assert c.match_prefix([10]) == (1, [0]) and c.match_prefix([40]) == (1, [3])
    # everything in use: the least recently used of them is evicted all the same
    assert c.match_prefix([50]) == (1, [4])
    c.insert([60], [5])
    assert c.size == 3 and c.match_prefix([10])[0] == 0 and c.get_stats()["evictions"] == 3


def test_manager_records_who_shares_a_prefix():
    """The first-block index follows allocation with shared blocks, forks, the private copy of a shared
    first block and frees; shared_prefix_groups answers from it without walking unrelated tables."""
    p = pool(64)
    m = pa.KVCacheManager(p, BS)
    a = m.allocate_for_sequence("a", 4 * BS + 1).get_physical_block_ids()          # 4 full blocks + 1 token
    assert m.sharing_candidates() == []
    m.allocate_for_sequence("b", 4 * BS + 2, shared_block_ids=a[:4])                 # a prefix-cache hit on a's 4 full blocks
    m.allocate_for_sequence("c", 3 * BS)                                            # shares nothing
    m.fork_sequence("a", "a2")
    assert m.sharing_candidates() == [["a", "a2", "b"]]
    # the batch's rows in any order; heads 2 / 1: up to 8 rows per group; partitions of two blocks
    groups = m.shared_prefix_groups(["c", "b", "a", "a2"], 2, 1, 2 * BS)
    assert groups == [([1, 2, 3], 4 * BS)]
    assert m.shared_prefix_groups(["c", "a"], 2, 1, 2 * BS) == []                   # a's sharers are not in this batch
    assert m.shared_prefix_groups(["c", "b", "a"], 32, 1, 2 * BS) == []             # no room for a second row per group
    # a sequence whose only block is shared gets a private first block when it appends: it leaves its set
    m.allocate_for_sequence("s", 2)
    m.fork_sequence("s", "s2")
    assert sorted(map(tuple, m.sharing_candidates())) == [("a", "a2", "b"), ("s", "s2")]
    assert m.append_token("s2")
    assert m.sharing_candidates() == [["a", "a2", "b"]]
    m.free_sequence("b")
    m.free_sequence("a")
    assert m.sharing_candidates() == [] and m.shared_prefix_groups(["a2", "c"], 2, 1, 2 * BS) == []
    for s in ("a2", "c", "s", "s2"):
        m.free_sequence(s)
    assert m._by_first_block == {} and m._first_block_of == {} and p.num_free_blocks == 64
