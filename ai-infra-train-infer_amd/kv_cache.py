"""Device tensors of the paged KV cache.

Mirrors the tensor half of the reference's BlockPool (src/inference/kv_cache.py:31-39,
131-174, 233-258): one tensor [2, num_layers, num_blocks, block_size, num_kv_heads, head_dim]
(index 0 = K, 1 = V) in the model dtype or float8_e4m3fn, plus, for fp8, two fp32 scale
tensors [num_layers, num_blocks, block_size] initialised to one.

The host-side bookkeeping follows the reference too (Block :42-62, BlockPool.allocate / free
:176-212, BlockTable :261-315, KVCacheManager :318-486, same names and return conventions) and
adds what the reference's ref_count was declared for but never did: a physical block can
belong to several sequences (a cached prefix, the prompt of K samples), and a sequence that
appends to a block it shares first gets a private copy of it (copy-on-write, one
`pa_copy_blocks` launch for all layers).  The reference's K-sample path notes that its prefix
match cannot skip any prefill until this exists (src/inference/engine.py:1108-1113).

Sizing note for MI355X: one GPU holds 288 GB, so the pool is a single allocation; at the
Qwen3-0.6B shape (8 KV heads x 128) a token costs 4 KiB per layer in fp16 and 2 KiB + 8 B
in fp8.
"""
import warnings
from collections import deque
from dataclasses import dataclass
from typing import Dict, Iterable, List, Optional, Set, Tuple

import torch

# fp8 probe, as the reference does at src/inference/kv_cache.py:32-39
try:
    _FP8_DTYPE = torch.float8_e4m3fn
    torch.tensor([1.0], dtype=_FP8_DTYPE)
    HAS_FP8 = True
except (AttributeError, RuntimeError):  # pragma: no cover - torch too old
    HAS_FP8 = False
    _FP8_DTYPE = None


@dataclass
class Block:
    """One physical block: room for block_size tokens of K and V in every layer."""
    block_id: int
    ref_count: int = 0       # owners: sequences' tables and prefix-cache entries
    token_count: int = 0     # tokens written so far (<= block_size)
    is_full: bool = False
    hash_value: Optional[int] = None

    def reset(self):
        self.ref_count = 0
        self.token_count = 0
        self.is_full = False
        self.hash_value = None


class BlockPool:
    """Owns the KV tensors of all layers and the free list of their blocks."""

    def __init__(self, num_blocks: int, block_size: int, num_layers: int, num_kv_heads: int,
                 head_dim: int, dtype: torch.dtype = torch.float16, device: str = "cuda",
                 cache_dtype: str = "fp16"):
        self.num_blocks = num_blocks
        self.block_size = block_size
        self.num_layers = num_layers
        self.num_kv_heads = num_kv_heads
        self.head_dim = head_dim
        self.dtype = dtype
        self.device = device
        if cache_dtype == "fp8":
            if HAS_FP8:
                self.cache_dtype = "fp8"
            else:  # pragma: no cover
                self.cache_dtype = "fp16"
                warnings.warn("FP8 KV cache requested but torch.float8_e4m3fn is unavailable; "
                              "falling back to FP16.", RuntimeWarning)
        else:
            self.cache_dtype = "fp16"
        self._blocks: List[Block] = [Block(block_id=i) for i in range(num_blocks)]
        self._free_queue: deque = deque(range(num_blocks))
        self._used_set: Set[int] = set()
        self._kv_cache: Optional[torch.Tensor] = None
        self.k_scale: Optional[torch.Tensor] = None
        self.v_scale: Optional[torch.Tensor] = None
        self._allocate_gpu_memory()

    # ---------------------------------------------------------------- block bookkeeping (host)

    def allocate(self) -> Optional[Block]:
        """A free block with ref_count 1, or None when the pool is exhausted."""
        if not self._free_queue:
            return None
        block = self._blocks[self._free_queue.popleft()]
        block.reset()
        block.ref_count = 1
        self._used_set.add(block.block_id)
        return block

    def share(self, block: Block) -> Block:
        """One more owner for a block that is in use."""
        if block.ref_count <= 0:
            raise RuntimeError("BlockPool.share: block %d is not allocated" % block.block_id)
        block.ref_count += 1
        return block

    def free(self, block: Block):
        """Drop one owner; the block returns to the free list with the last one."""
        if block.ref_count <= 0:
            warnings.warn("Double-free detected for block %d (ref_count=%d). Ignoring."
                          % (block.block_id, block.ref_count))
            return
        block.ref_count -= 1
        if block.ref_count <= 0:
            block.reset()
            self._used_set.discard(block.block_id)
            self._free_queue.append(block.block_id)

    def get_block(self, block_id: int) -> Block:
        return self._blocks[block_id]

    @property
    def num_free_blocks(self) -> int:
        return len(self._free_queue)

    @property
    def num_used_blocks(self) -> int:
        return len(self._used_set)

    @property
    def utilization(self) -> float:
        return self.num_used_blocks / self.num_blocks if self.num_blocks else 0.0

    def copy_blocks(self, pairs: Iterable[Tuple[int, int]]):
        """block dst := block src for every (src, dst), in all layers, K, V and fp8 scales.
        One launch per tensor on the current stream."""
        pairs = [(int(a), int(b)) for a, b in pairs]
        if not pairs:
            return
        from . import _native
        kv = self._kv_cache
        if not kv.is_cuda:
            raise RuntimeError("BlockPool.copy_blocks: the pool is on %s; this package has no CPU path"
                               % kv.device)
        lib = _native.load()
        dev_pairs = torch.tensor(pairs, dtype=torch.int32).pin_memory().to(kv.device, non_blocking=True)
        stream = torch.cuda.current_stream(kv.device).cuda_stream
        block_bytes = self.block_size * self.num_kv_heads * self.head_dim * kv.element_size()
        todo = [(kv, 2 * self.num_layers, block_bytes)]
        if self.k_scale is not None:
            todo += [(self.k_scale, self.num_layers, self.block_size * 4),
                     (self.v_scale, self.num_layers, self.block_size * 4)]
        for t, planes, bb in todo:
            rc = lib.pa_copy_blocks(t.data_ptr(), planes, self.num_blocks * bb, bb, self.num_blocks,
                                    dev_pairs.data_ptr(), len(pairs), stream)
            if rc != 0:
                raise RuntimeError("pa_copy_blocks failed (%d): %s"
                                   % (rc, lib.pa_last_error().decode("utf-8", "replace")))

    # ---------------------------------------------------------------- device tensors

    def _allocate_gpu_memory(self):
        alloc_dtype = _FP8_DTYPE if self.cache_dtype == "fp8" else self.dtype
        shape = (2, self.num_layers, self.num_blocks, self.block_size, self.num_kv_heads,
                 self.head_dim)
        try:
            self._kv_cache = torch.zeros(shape, dtype=alloc_dtype, device=self.device)
        except RuntimeError as e:
            # the reference drops to a CPU tensor here; a CPU pool cannot be served by the
            # HIP kernels, so the failure is reported instead
            raise RuntimeError("KV cache allocation of %d blocks failed on %s: %s"
                               % (self.num_blocks, self.device, e)) from e
        if self.cache_dtype == "fp8":
            sshape = (self.num_layers, self.num_blocks, self.block_size)
            self.k_scale = torch.ones(sshape, dtype=torch.float32, device=self.device)
            self.v_scale = torch.ones(sshape, dtype=torch.float32, device=self.device)

    @property
    def kv_cache_tensor(self) -> Optional[torch.Tensor]:
        """[2, num_layers, num_blocks, block_size, num_kv_heads, head_dim]"""
        return self._kv_cache

    def get_flattened_kv_cache(self) -> Optional[torch.Tensor]:
        """View [2, num_layers, num_blocks*block_size, num_kv_heads, head_dim] (slot-indexed)."""
        if self._kv_cache is None:
            return None
        s = self._kv_cache.shape
        return self._kv_cache.view(s[0], s[1], s[2] * s[3], s[4], s[5])

    def layer_views(self, layer: int):
        """(k_cache, v_cache, k_scale, v_scale) of one layer, as ModelRunner binds them
        (src/inference/model_runner.py:102-116)."""
        ks = self.k_scale[layer] if self.k_scale is not None else None
        vs = self.v_scale[layer] if self.v_scale is not None else None
        return self._kv_cache[0, layer], self._kv_cache[1, layer], ks, vs

    def bind_to_model(self, model: torch.nn.Module):
        """Bind layer views to every PagedAttention module in module order."""
        from .attention import PagedAttention
        layer = 0
        for module in model.modules():
            if isinstance(module, PagedAttention):
                k, v, ks, vs = self.layer_views(layer)
                module.k_cache, module.v_cache = k, v
                module.cache_dtype = self.cache_dtype
                if ks is not None:
                    module.k_scale, module.v_scale = ks, vs
                layer += 1
        return layer


class BlockTable:
    """Logical -> physical block map of one sequence (src/inference/kv_cache.py:261-315)."""

    def __init__(self, block_size: int):
        self._blocks: List[Block] = []
        self._block_size = block_size
        # tokens of THIS sequence in its last block; a shared block's own token_count may run
        # ahead of a sequence that has not yet written its copy
        self._last_tokens = 0

    def append_block(self, block: Block):
        self._blocks.append(block)
        self._last_tokens = block.token_count

    def get_physical_block_ids(self) -> List[int]:
        return [b.block_id for b in self._blocks]

    @property
    def last_block(self) -> Optional[Block]:
        return self._blocks[-1] if self._blocks else None

    @property
    def num_blocks(self) -> int:
        return len(self._blocks)

    @property
    def num_tokens(self) -> int:
        if not self._blocks:
            return 0
        return (len(self._blocks) - 1) * self._block_size + self._last_tokens

    @property
    def blocks(self) -> List[Block]:
        return self._blocks


class KVCacheManager:
    """Allocates, shares and frees the blocks of sequences (src/inference/kv_cache.py:318-486).

    On top of the reference's calls: `allocate_for_sequence(..., shared_block_ids=[...])` makes the
    first logical blocks aliases of blocks that already hold the prefix (a prefix-cache hit),
    `fork_sequence` starts a sample that shares everything its parent has, and `append_token`
    copies a shared last block before the sequence writes into it.  Copies are queued; the
    caller runs `apply_copies()` before the step's KV store.
    """

    def __init__(self, block_pool: BlockPool, block_size: int = 16):
        self._pool = block_pool
        self._block_size = block_size
        self._seq_tables: Dict[object, BlockTable] = {}
        self._pending_copies: List[Tuple[int, int]] = []
        # Which sequences may share a prefix, recorded where sharing is made (a prefix-cache hit, a fork)
        # and dropped where it ends (free, a private copy of the first block): sequences that share
        # anything share their first physical block, so the index is first block id -> sequences.
        self._by_first_block: Dict[int, Set[object]] = {}
        self._first_block_of: Dict[object, int] = {}

    # -- who shares with whom -----------------------------------------------------------------

    def _index_first_block(self, seq_id):
        """Keep the first-block index in step with the sequence's table."""
        table = self._seq_tables.get(seq_id)
        new = table.blocks[0].block_id if table is not None and table.blocks else None
        old = self._first_block_of.get(seq_id)
        if new == old:
            return
        if old is not None:
            members = self._by_first_block.get(old)
            if members is not None:
                members.discard(seq_id)
                if not members:
                    del self._by_first_block[old]
            del self._first_block_of[seq_id]
        if new is not None:
            self._by_first_block.setdefault(new, set()).add(seq_id)
            self._first_block_of[seq_id] = new

    def sharing_candidates(self) -> List[List[object]]:
        """Sets of live sequences that start with the same physical block, i.e. that share a prefix
        (only sets of two or more)."""
        return [sorted(m, key=repr) for m in self._by_first_block.values() if len(m) > 1]

    def shared_prefix_groups(self, seq_ids, num_q_heads: int, num_kv_heads: int, partition_size: int):
        """Groups of the given sequences that share a prefix of whole partitions, as
        [([index into seq_ids, ...], shared_tokens)] - what attention.shared_prefix_descriptors takes for a
        batch whose rows are seq_ids.  Only sequences the index names as sharers are looked at: a batch
        without sharing costs one dictionary lookup per row."""
        from .attention import find_prefix_groups_anywhere
        rows = [i for i, s in enumerate(seq_ids)
                if len(self._by_first_block.get(self._first_block_of.get(s, -1), ())) > 1]
        if len(rows) < 2:
            return []
        tables = [self._seq_tables[seq_ids[i]].get_physical_block_ids() for i in rows]
        lens = [self._seq_tables[seq_ids[i]].num_tokens for i in rows]
        return find_prefix_groups_anywhere(tables, lens, self._block_size, num_q_heads, num_kv_heads, partition_size,
                                           rows=rows)

    # -- allocation ---------------------------------------------------------------------------

    def allocate_for_sequence(self, seq_id, num_initial_tokens: int = 0,
                              shared_block_ids: Optional[List[int]] = None) -> BlockTable:
        """Block table for a new sequence of num_initial_tokens tokens.  shared_block_ids are full
        blocks that already hold the first len(shared) * block_size tokens; they gain an owner
        instead of being allocated.  Raises RuntimeError (after rolling back) when out of blocks."""
        if seq_id in self._seq_tables:
            # replacing the table would leak every block the sequence already owns
            raise RuntimeError("allocate_for_sequence: seq %s already has a block table "
                               "(free_sequence it first)" % (seq_id,))
        table = BlockTable(self._block_size)
        shared = list(shared_block_ids or [])
        needed = (num_initial_tokens + self._block_size - 1) // self._block_size
        if len(shared) * self._block_size > num_initial_tokens:
            raise RuntimeError("allocate_for_sequence: %d shared blocks hold more than the %d tokens "
                               "of seq %s" % (len(shared), num_initial_tokens, seq_id))
        for bid in shared:
            block = self._pool.get_block(bid)
            if block.ref_count <= 0 or not block.is_full:
                for b in table.blocks:
                    self._pool.free(b)
                raise RuntimeError("allocate_for_sequence: shared block %d is not a full, live block" % bid)
            table.append_block(self._pool.share(block))
        for i in range(len(shared), needed):
            block = self._pool.allocate()
            if block is None:
                for b in table.blocks:
                    self._pool.free(b)
                raise RuntimeError("OOM: Cannot allocate %d blocks for seq %s. Free: %d"
                                   % (needed - len(shared), seq_id, self._pool.num_free_blocks))
            block.token_count = min(self._block_size, num_initial_tokens - i * self._block_size)
            block.is_full = block.token_count == self._block_size
            table.append_block(block)
        self._seq_tables[seq_id] = table
        self._index_first_block(seq_id)
        return table

    def fork_sequence(self, parent_id, child_id) -> BlockTable:
        """A new sequence that shares every block of its parent, the partly filled last one
        included; whichever of them appends to that block first gets a private copy."""
        parent = self._seq_tables.get(parent_id)
        if parent is None:
            raise RuntimeError("fork_sequence: unknown parent %s" % (parent_id,))
        if child_id in self._seq_tables:
            raise RuntimeError("fork_sequence: seq %s already has a block table" % (child_id,))
        table = BlockTable(self._block_size)
        for block in parent.blocks:
            table.append_block(self._pool.share(block))
        table._last_tokens = parent._last_tokens
        self._seq_tables[child_id] = table
        self._index_first_block(child_id)
        return table

    def append_token(self, seq_id) -> bool:
        """Room for one more token of the sequence; False when the pool is exhausted (nothing
        changes then).  Writing into a block with other owners first moves the sequence to a copy."""
        table = self._seq_tables.get(seq_id)
        if table is None:
            return False
        last = table.last_block
        if last is None or table._last_tokens == self._block_size:
            block = self._pool.allocate()
            if block is None:
                return False
            block.token_count = 1
            block.is_full = self._block_size == 1
            table.append_block(block)
            if table.num_blocks == 1:
                self._index_first_block(seq_id)
            return True
        if last.ref_count > 1:
            block = self._pool.allocate()
            if block is None:
                return False
            self._pending_copies.append((last.block_id, block.block_id))
            self._pool.free(last)
            block.token_count = table._last_tokens + 1
            block.is_full = block.token_count == self._block_size
            table._blocks[-1] = block
            table._last_tokens = block.token_count
            if table.num_blocks == 1:
                self._index_first_block(seq_id)           # the private copy is the sequence's first block now
            return True
        last.token_count = table._last_tokens + 1
        last.is_full = last.token_count == self._block_size
        table._last_tokens = last.token_count
        return True

    def next_slot(self, seq_id) -> int:
        """Slot of the sequence's newest token (call after append_token), as slot_mapping wants it."""
        table = self._seq_tables[seq_id]
        return table.last_block.block_id * self._block_size + table._last_tokens - 1

    @property
    def pending_copies(self) -> List[Tuple[int, int]]:
        return list(self._pending_copies)

    @staticmethod
    def _ordered_batches(pairs: List[Tuple[int, int]]) -> List[List[Tuple[int, int]]]:
        """Cut the queue, in order, into batches in which no block is written by one pair and read
        or written by another: the pairs of one launch run concurrently, launches run in order.
        A queue can chain when the pool is nearly full: block X is queued as the source of (X, Y),
        its last owner frees it, and the next copy-on-write is handed X as its destination."""
        batches, current, reads, writes = [], [], set(), set()
        for src, dst in pairs:
            if src in writes or dst in writes or dst in reads:
                batches.append(current)
                current, reads, writes = [], set(), set()
            current.append((src, dst))
            reads.add(src)
            writes.add(dst)
        if current:
            batches.append(current)
        return batches

    def apply_copies(self):
        """Run the queued copy-on-write copies on the current stream, in queue order."""
        pending, self._pending_copies = self._pending_copies, []
        for batch in self._ordered_batches(pending):
            self._pool.copy_blocks(batch)

    def free_sequence(self, seq_id):
        table = self._seq_tables.pop(seq_id, None)
        if table is None:
            return
        self._index_first_block(seq_id)
        for block in table.blocks:
            self._pool.free(block)

    # -- queries --------------------------------------------------------------------------------

    def can_allocate(self, num_tokens: int, num_shared_blocks: int = 0) -> bool:
        """Room for a new sequence of num_tokens tokens plus one spare block for decode growth."""
        needed = (num_tokens + self._block_size - 1) // self._block_size - num_shared_blocks
        return self._pool.num_free_blocks >= needed + 1

    def get_block_table(self, seq_id) -> List[int]:
        table = self._seq_tables.get(seq_id)
        return table.get_physical_block_ids() if table is not None else []

    def get_seq_token_count(self, seq_id) -> int:
        table = self._seq_tables.get(seq_id)
        return table.num_tokens if table is not None else 0

    def get_stats(self) -> dict:
        pool = self._pool
        shared = sum(1 for bid in pool._used_set if pool.get_block(bid).ref_count > 1)
        return {
            "total_blocks": pool.num_blocks,
            "used_blocks": pool.num_used_blocks,
            "free_blocks": pool.num_free_blocks,
            "shared_blocks": shared,
            "utilization": "%.1f%%" % (100.0 * pool.utilization),
            "active_sequences": len(self._seq_tables),
            "block_size": self._block_size,
            "memory_bytes": (pool.num_blocks * self._block_size * 2 * pool.num_layers * pool.num_kv_heads
                             * pool.head_dim * pool.kv_cache_tensor.element_size()),
        }
