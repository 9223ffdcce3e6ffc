"""The caller side of the paged-attention path: per-step metadata, cache binding, graph replay.

Mirrors the part of the reference's ModelRunner that feeds the attention layers
(src/inference/model_runner.py): `bind_kv_cache` / `_bind_kv_cache_to_model` (:78-116),
`prepare_prefill` (:464-540), `prepare_decode` (:542-588), `_prepare_block_tables` (:814-828),
`run` (:128-165), `run_batch_decode` (:639-708), `sample` (:590-634) and the decode graph capture /
replay (:710-810).  Same sequence dictionaries in,
same context out (int32 `slot_mapping`, `context_lens`, `cu_seqlens_*`, `block_tables` padded with
-1).  What differs is how the metadata reaches the GPU:

  * the reference builds the block table with one Python assignment per entry
    (`tables[i, j] = block_id`, 16 384 device writes at batch 64 / ctx 4096) and a fresh
    torch.tensor(...) per field; here the fields of a step are built with numpy row copies side by
    side in one pinned staging buffer and shipped with one asynchronous copy;
  * graph replay copies into static device buffers and pads with slot -1 / context 0, exactly as
    the reference does, but capture needs no host synchronisation inside the model;
  * `run_batch_decode` gets its slot mapping from a kernel instead of two `.item()` reads per
    sequence, so a decode step driven by device-resident tables never waits for the GPU;
  * `DecodeState` keeps block tables, context lengths, positions, slots and input ids of the
    running batch on the GPU between steps: a step uploads at most one block id per sequence
    (the block its new token opens) and advances everything else with one small kernel, and the
    graphs recorded over it (`capture_decode_state_graphs`) replay without a single input copy.

The reference's shipped mode around a HuggingFace model (`bind_hf_model`, `_hf_prefill_forward`,
`_hf_decode_forward`, `_store_hf_*`, `_load_kv_from_paged_cache`, :118-462) is here too, with its
per-entry slot loops and index gathers replaced by one gather kernel per layer, and so is its mock
mode (a runner without a model returns random logits).
"""
from dataclasses import dataclass
from typing import Dict, List, Optional, Tuple

import numpy as np
import torch

from .attention import PagedAttention
from .context import get_context, reset_context, set_context


@dataclass
class ModelRunnerConfig:
    num_layers: int = 32
    num_heads: int = 32
    num_kv_heads: int = 8
    head_dim: int = 128
    hidden_size: int = 4096
    vocab_size: int = 151936
    block_size: int = 16
    max_num_blocks: int = 1024          # widest block table a sequence may have
    dtype: torch.dtype = torch.float16
    device: str = "cuda"
    enable_cuda_graph: bool = True
    max_cuda_graph_batch_size: int = 64
    # decode steps read a prefix that several rows share as the same blocks (n samples of a prompt,
    # forks of a cached prefix) once per group of rows instead of once per row.  The groups are kept
    # where the rows are: DecodeState updates them when a row is admitted or retired, prepare_decode
    # keeps the last step's groups for as long as the batch's first blocks stay what they were.
    share_prefix_decode: bool = True
    prefix_partition_sizes: Tuple[int, ...] = (1024, 512)     # tokens; coarsest first
    # Recorded decode launches cannot be resized, and one sized for the width of the block tables
    # (max_num_blocks) is a poor fit for a batch of rows a fraction of that long.  Graphs over a
    # DecodeState are therefore recorded per context bucket - launches sized for rows of up to that many
    # tokens - and a step replays the smallest bucket that holds its longest row (the host knows the
    # lengths).  None: the table's width and every half of the one before down to 2048 tokens.
    decode_context_buckets: Optional[Tuple[int, ...]] = None
    # also record, where the launch policy would shape it differently, a graph for ragged batches (rows
    # 0.45 of the bucket long on average), replayed when the mean length is below 0.7 of the bucket
    ragged_decode_graphs: bool = True


# mean row length, as a share of the context bucket, that the graphs for ragged batches are recorded for
# (rows between a quarter of the bucket and the whole of it: batches with longer rows take the next bucket)
_RAGGED_GRAPH_MEAN = 0.45


def slots_for_range(block_table, start, end, block_size):
    """Physical slots of token positions [start, end) of one sequence (numpy int32)."""
    pos = np.arange(start, end, dtype=np.int64)
    bt = np.asarray(block_table, dtype=np.int64)
    return (bt[pos // block_size] * block_size + pos % block_size).astype(np.int32)


class DecodeState:
    """Decode metadata of up to `max_batch` sequences, resident on the GPU between steps.

    What prepare_decode rebuilds and uploads every step (src/inference/model_runner.py:542-588,
    814-828) lives here in fixed tensors: `block_tables` [max_batch, max_blocks] int32 (-1 =
    unused), `context_lens` [max_batch] int32 (0 = free row), `positions` int64, `slot_mapping`
    int32, `input_ids` int64.  A sequence occupies one row from `admit` (after its prefill) to
    `retire`; `step` makes every active row one token longer.  Free rows are inert in the
    kernels (slot -1, context 0), so any prefix [0, n) with n >= `rows_in_use` is a valid batch,
    which is what graph replay needs.  The host keeps only counters (lengths, tables) to know
    when a sequence needs its next block; it never reads the device tensors back.
    """

    def __init__(self, max_batch: int, max_blocks_per_seq: int, block_size: int, num_blocks: int,
                 device: str = "cuda", num_q_heads: Optional[int] = None, num_kv_heads: Optional[int] = None,
                 prefix_partition_sizes: Tuple[int, ...] = (1024, 512)):
        """num_q_heads / num_kv_heads: give them and the state also keeps the groups of rows that share
        a prefix as the same physical blocks (rebuilt when a row is admitted or retired, never per
        step), as device descriptors for pa_decode_shared_prefix; prefix_partition_sizes are the
        partition sizes such a launch may use, coarsest first."""
        dev = torch.device(device)
        self.max_batch, self.max_blocks = int(max_batch), int(max_blocks_per_seq)
        self.block_size, self.num_blocks = int(block_size), int(num_blocks)
        self.block_tables = torch.full((max_batch, max_blocks_per_seq), -1, dtype=torch.int32, device=dev)
        self.context_lens = torch.zeros(max_batch, dtype=torch.int32, device=dev)
        self.positions = torch.zeros(max_batch, dtype=torch.long, device=dev)
        self.slot_mapping = torch.full((max_batch,), -1, dtype=torch.int32, device=dev)
        self.input_ids = torch.zeros(max_batch, dtype=torch.long, device=dev)
        self._new_blocks = torch.full((max_batch,), -1, dtype=torch.int32, device=dev)
        self._fresh = torch.zeros(max_batch, dtype=torch.int32, device=dev)   # 1: admitted since the last step
        # two pinned staging buffers used in turn; an event marks when the copy out of one is done
        self._stage = [[torch.full((max_batch,), -1, dtype=torch.int32).pin_memory(), None] for _ in range(2)]
        self._turn = 0
        self._fresh_rows = set()                        # host copy of the same
        self._lens = np.zeros(max_batch, dtype=np.int64)    # tokens in the cache, per row (0 = free)
        self._ntab = np.zeros(max_batch, dtype=np.int64)    # block ids held, per row
        self._tables = [[] for _ in range(max_batch)]       # the block ids themselves
        # ---- rows that share prefixes ---------------------------------------------------------------
        self._heads = (int(num_q_heads), int(num_kv_heads)) if num_q_heads and num_kv_heads else None
        self.max_group_rows = 16 // max(1, self._heads[0] // self._heads[1]) if self._heads else 0
        self.prefix_partition_sizes = tuple(sorted(
            (int(x) for x in prefix_partition_sizes if int(x) > 0 and int(x) % self.block_size == 0 and int(x) % 16 == 0
             and int(x) <= self.max_blocks * self.block_size), reverse=True))
        self.tracks_prefixes = self.max_group_rows >= 2 and bool(self.prefix_partition_sizes) and max_batch >= 2
        self.max_groups = max_batch // 2
        self.prefix_partition_size: Optional[int] = None    # of the groups now on the device; None: no groups
        self.prefix_groups_host: List[Tuple[List[int], int]] = []
        self._groups_dirty = False
        if self.tracks_prefixes:
            # one buffer, so that an update is one copy: group_desc [G, 4] | group_rows [B] | row_skip [B]
            self._groups_dev = torch.zeros(4 * self.max_groups + 2 * max_batch, dtype=torch.int32, device=dev)
            self._group_desc = self._groups_dev[:4 * self.max_groups].view(-1, 4)
            self._group_rows = self._groups_dev[4 * self.max_groups:4 * self.max_groups + max_batch]
            self._row_skip = self._groups_dev[4 * self.max_groups + max_batch:]

    @property
    def rows_in_use(self) -> int:
        """One past the highest active row."""
        used = np.flatnonzero(self._lens)
        return int(used[-1]) + 1 if used.size else 0

    def active_rows(self) -> List[int]:
        return np.flatnonzero(self._lens).tolist()

    def known_lengths(self, batch: Optional[int] = None) -> Tuple[int, float]:
        """(longest, mean) context length over the first `batch` rows (default: the rows in use), free
        rows counted as 0: what the host knows without asking the device."""
        n = self.rows_in_use if batch is None else int(batch)
        if n <= 0:
            return 0, 0.0
        lens = self._lens[:n]
        return int(lens.max()), float(lens.sum()) / n

    def num_tokens(self, row: int) -> int:
        return int(self._lens[row])

    def admit(self, block_table: List[int], num_cached_tokens: int, next_token: int) -> int:
        """Give a prefilled sequence (its `num_cached_tokens` tokens are in the cache, `next_token`
        is the one sampled from the prefill) the lowest free row; returns the row."""
        if num_cached_tokens <= 0:
            raise RuntimeError("DecodeState.admit: a sequence enters decode with at least one cached token")
        if len(block_table) > self.max_blocks or len(block_table) * self.block_size < num_cached_tokens:
            raise RuntimeError("DecodeState.admit: block table does not fit the state or the tokens")
        free = np.flatnonzero((self._lens == 0) & (self._ntab == 0))
        if not free.size:
            raise RuntimeError("DecodeState.admit: all %d rows are in use" % self.max_batch)
        row = int(free[0])
        host_row = torch.full((self.max_blocks,), -1, dtype=torch.int32)
        host_row[:len(block_table)] = torch.tensor(block_table, dtype=torch.int32)
        self.block_tables[row].copy_(host_row.pin_memory(), non_blocking=True)
        self.context_lens[row].fill_(int(num_cached_tokens))
        self.input_ids[row].fill_(int(next_token))
        self._fresh[row].fill_(1)
        self._fresh_rows.add(row)
        self._lens[row] = int(num_cached_tokens)
        self._tables[row] = list(block_table)
        self._ntab[row] = len(block_table)
        self._groups_dirty = self.tracks_prefixes
        return row

    def reserve(self, block_table: List[int]) -> int:
        """Give a sequence that has not finished its prefill the lowest free row: its block table goes to
        the device now (prefill chunks can take it from there: ModelRunner.prepare_prefill(state=...)), the
        row stays out of the decode steps until activate().  Returns the row."""
        if not block_table or len(block_table) > self.max_blocks:
            raise RuntimeError("DecodeState.reserve: block table empty or wider than the state")
        free = np.flatnonzero((self._lens == 0) & (self._ntab == 0))
        if not free.size:
            raise RuntimeError("DecodeState.reserve: all %d rows are in use" % self.max_batch)
        row = int(free[0])
        host_row = torch.full((self.max_blocks,), -1, dtype=torch.int32)
        host_row[:len(block_table)] = torch.tensor(block_table, dtype=torch.int32)
        self.block_tables[row].copy_(host_row.pin_memory(), non_blocking=True)
        self._tables[row] = list(block_table)
        self._ntab[row] = len(block_table)
        return row

    def activate(self, row: int, num_cached_tokens: int, next_token: int):
        """A reserved row joins the decode steps: its `num_cached_tokens` tokens are in the cache and
        `next_token` is the one its last prefill chunk produced."""
        if self._lens[row] != 0 or self._ntab[row] == 0:
            raise RuntimeError("DecodeState.activate: row %d is not a reserved row" % row)
        if num_cached_tokens <= 0 or self._ntab[row] * self.block_size < num_cached_tokens:
            raise RuntimeError("DecodeState.activate: the row's block table does not hold %d tokens" % num_cached_tokens)
        self.context_lens[row].fill_(int(num_cached_tokens))
        self.input_ids[row].fill_(int(next_token))
        self._fresh[row].fill_(1)
        self._fresh_rows.add(row)
        self._lens[row] = int(num_cached_tokens)
        self._groups_dirty = self.tracks_prefixes

    def retire(self, row: int) -> List[int]:
        """Free a row; returns the block ids the sequence held."""
        self.context_lens[row].fill_(0)
        self._fresh_rows.discard(row)
        blocks, self._tables[row], self._lens[row], self._ntab[row] = self._tables[row], [], 0, 0
        self._groups_dirty = self.tracks_prefixes
        return blocks

    # ---- rows that share prefixes ---------------------------------------------------------------------
    # Full blocks never change while one of their owners lives, so what a set of rows shares is fixed
    # from the moment the last of them is admitted until the first of them retires: the groups are
    # rebuilt on those two events only, on the host, from the block-id lists the state already keeps
    # (rows that share anything share their first block: one dictionary pass finds the candidates),
    # and shipped to the device in one small copy.  A step costs nothing.

    def sync_prefix_groups(self):
        """Bring the device descriptors up to date with the rows admitted and retired since the last
        call.  Called by step() and set_context(); a launch over descriptors that still name a retired
        row would skip that row's group."""
        if not self._groups_dirty:
            return
        from .attention import choose_prefix_partition, find_prefix_groups_anywhere
        self._groups_dirty = False
        active = self.active_rows()
        tables = [self._tables[r] for r in active]
        lens = [int(self._lens[r]) for r in active]
        hq, hkv = self._heads

        def find(size):
            return find_prefix_groups_anywhere(tables, lens, self.block_size, hq, hkv, size, rows=active)

        size, groups = choose_prefix_partition(find, self.prefix_partition_sizes)
        groups = groups[:self.max_groups]
        had = self.prefix_partition_size is not None
        self.prefix_partition_size, self.prefix_groups_host = (size, groups) if groups else (None, [])
        if not groups and not had:
            return                                     # nothing on the device names a row
        host = torch.zeros(self._groups_dev.numel(), dtype=torch.int32)
        desc = host[:4 * self.max_groups].view(-1, 4)
        rows_flat = host[4 * self.max_groups:4 * self.max_groups + self.max_batch]
        skip = host[4 * self.max_groups + self.max_batch:]
        cursor = 0
        for i, (members, tokens) in enumerate(groups):
            parts = tokens // size
            desc[i, 0], desc[i, 1], desc[i, 2] = cursor, len(members), parts
            for r in members:
                rows_flat[cursor] = r
                skip[r] = parts
                cursor += 1
        self._groups_dev.copy_(host.pin_memory(), non_blocking=True)

    def prefix_groups(self, batch: int, partition_size: Optional[int] = None, for_graph: bool = False,
                      longest_context: Optional[int] = None):
        """PrefixGroups over the state's device descriptors for the first `batch` rows, or None when
        no rows share a prefix.  for_graph: the descriptors at their full capacity whatever they hold
        now (empty groups cost a workgroup that returns at once), for partition_size - what a
        recorded launch must be sized with; longest_context: the rows the launch will serve hold at
        most that many tokens (a prefix cannot be longer than the rows that share it)."""
        from .attention import PrefixGroups
        if not self.tracks_prefixes:
            return None
        if for_graph:
            size = int(partition_size)
            tokens = self.max_blocks * self.block_size
            if longest_context:
                tokens = min(tokens, int(longest_context))
            parts = -(-tokens // size)
            return PrefixGroups(size, self._group_desc, self._group_rows, self._row_skip[:batch], self.max_groups,
                                self.max_group_rows, parts, 0)
        self.sync_prefix_groups()
        if self.prefix_partition_size is None:
            return None
        size = self.prefix_partition_size
        groups = self.prefix_groups_host
        return PrefixGroups(size, self._group_desc, self._group_rows, self._row_skip[:batch], len(groups),
                            max(len(m) for m, _ in groups), max(t for _, t in groups) // size, 0, groups=groups)

    def rows_needing_block(self) -> List[int]:
        """Active rows whose next token opens a block they do not have yet."""
        bs = self.block_size
        lens = self._lens
        return np.flatnonzero((lens > 0) & (lens % bs == 0) & (lens // bs >= self._ntab)).tolist()

    def step(self, new_blocks: Optional[Dict[int, int]] = None, next_tokens: Optional[torch.Tensor] = None):
        """Advance every active row by one token.  new_blocks: {row: block id} for the rows of
        rows_needing_block(), and for rows whose last block has just been replaced by a private
        copy (copy-on-write): the id lands in the table column the new token falls into; next_tokens: device int64 [>= rows_in_use], row r's entry being the
        token the previous step produced for row r (the sampler's output as it is); rows admitted
        since that step keep the token they were admitted with."""
        from . import _native
        lib = _native.load()
        self.sync_prefix_groups()
        if next_tokens is not None:
            next_tokens = next_tokens.reshape(-1)
            if not next_tokens.is_cuda or next_tokens.dtype != torch.long or not next_tokens.is_contiguous():
                raise RuntimeError("DecodeState.step: next_tokens must be a contiguous int64 GPU tensor")
            # the highest row that takes its input from next_tokens (active, not admitted since the last step)
            last_fed = next((r for r in np.flatnonzero(self._lens)[::-1].tolist() if r not in self._fresh_rows), -1)
            if last_fed >= next_tokens.numel():
                raise RuntimeError("DecodeState.step: next_tokens has no entry for row %d" % last_fed)
            if next_tokens.numel() < self.max_batch:      # the kernel indexes it by row
                padded = torch.zeros(self.max_batch, dtype=torch.long, device=next_tokens.device)
                padded[:next_tokens.numel()] = next_tokens
                next_tokens = padded
        need = self.rows_needing_block()
        if need:
            missing = [r for r in need if not new_blocks or r not in new_blocks]
            if missing:
                raise RuntimeError("DecodeState.step: rows %s need a new block" % missing)
        new_ptr = None
        if new_blocks:
            host, event = self._stage[self._turn]
            if event is not None:
                event.synchronize()                       # the copy that last read this buffer
            host.fill_(-1)
            for row, block in new_blocks.items():
                if self._lens[row] <= 0 or self._lens[row] // self.block_size >= self.max_blocks:
                    raise RuntimeError("DecodeState.step: row %d cannot take a block" % row)
                host[row] = int(block)
                col = self._lens[row] // self.block_size          # the block the new token falls into
                if col < len(self._tables[row]):
                    self._tables[row][col] = int(block)          # copy-on-write: a private copy replaces it
                else:
                    self._tables[row].append(int(block))
                    self._ntab[row] += 1
            self._new_blocks.copy_(host, non_blocking=True)
            done = torch.cuda.Event()
            done.record()
            self._stage[self._turn][1] = done
            self._turn ^= 1
            new_ptr = self._new_blocks.data_ptr()
        stream = torch.cuda.current_stream(self.block_tables.device).cuda_stream
        rc = lib.pa_decode_advance(self.block_tables.data_ptr(), self.block_tables.stride(0),
                                   self.context_lens.data_ptr(), self.positions.data_ptr(),
                                   self.slot_mapping.data_ptr(), new_ptr, self.input_ids.data_ptr(),
                                   next_tokens.data_ptr() if next_tokens is not None else None,
                                   self._fresh.data_ptr(), self.max_batch, self.max_blocks,
                                   self.block_size, self.num_blocks, stream)
        _native.check(rc, "pa_decode_advance")
        self._lens[self._lens > 0] += 1
        self._fresh_rows.clear()

    def set_context(self, batch: Optional[int] = None, share_prefixes: bool = True,
                    graph_partition_size: Optional[int] = None, lengths="host"):
        """Point the attention layers at the first `batch` rows (default: the rows in use).
        share_prefixes: hand them the groups of rows that share a prefix, when there are any;
        graph_partition_size: the descriptors at full capacity for that partition size instead (what
        a graph is recorded over).  lengths: what the launches may assume about the rows - "host": the
        lengths the host has counted (an eager step), (longest, mean): these (a recorded launch serves
        every batch that fits them; mean 0 = rows as long as the longest), None: nothing beyond the
        width of the tables."""
        n = self.rows_in_use if batch is None else batch
        if isinstance(lengths, str):
            longest, mean = self.known_lengths(n)
        elif lengths is None:
            longest, mean = 0, 0.0
        else:
            longest, mean = int(lengths[0]), float(lengths[1])
        groups = None
        if graph_partition_size is not None:
            groups = self.prefix_groups(n, graph_partition_size, for_graph=True, longest_context=longest or None)
        elif share_prefixes:
            groups = self.prefix_groups(n)
        set_context(False, slot_mapping=self.slot_mapping[:n], context_lens=self.context_lens[:n],
                    block_tables=self.block_tables[:n], prefix_groups=groups,
                    longest_context_len=longest, mean_context_len=mean)
        return n


class ModelRunner:
    """prepare_prefill / prepare_decode -> run -> logits, around a model that owns
    PagedAttention layers."""

    def __init__(self, model: Optional[torch.nn.Module], config: ModelRunnerConfig):
        self.model = model
        self.config = config
        self.block_size = config.block_size
        self._kv_cache: Optional[torch.Tensor] = None
        self._k_scale = self._v_scale = None
        self._cache_dtype = "fp16"
        self._graphs: Dict[tuple, torch.cuda.CUDAGraph] = {}      # (batch size, context bucket, for ragged batches)
        self._graph_outputs: Dict[tuple, torch.Tensor] = {}
        self._graph_buckets: List[int] = []
        self._graph_pool = None
        self._graph_vars: Optional[Dict[str, torch.Tensor]] = None
        self._graph_batch_sizes: List[int] = []
        # (id of the DecodeState, batch size, shared-prefix partition size or None, context bucket, for ragged batches)
        self._state_graphs: Dict[tuple, Tuple[torch.cuda.CUDAGraph, torch.Tensor]] = {}
        self._state_buckets: Dict[int, List[int]] = {}      # id of the DecodeState -> context buckets recorded, ascending
        self._hf_model: Optional[torch.nn.Module] = None
        self._state_graph_lookup: Dict[tuple, object] = {}
        self._prefix_groups_kept = None          # (signature of the batch, PrefixGroups or None) of the last decode step
        # pinned staging buffers for the uploads of prepare_decode and prepare_prefill, used in turn; an event marks when the copy
        # out of one is done.  (A fresh pinned tensor per step comes out of torch's caching host
        # allocator, which hands a block out again only after its copy has run: a host that prepares
        # steps faster than the GPU takes them makes it allocate a new block every step.)
        self._decode_stage = [[None, None] for _ in range(4)]
        self._table_rows = {}          # prepare_decode: (length, first id, last id) -> (copy of the block-id list, int32 row)
        self._decode_stage_turn = 0
        # how run_decode_state ran its steps: replays of a graph recorded over the shared-prefix launch,
        # replays of a plain graph, eager forwards
        self.decode_state_stats = {"shared_prefix_graph": 0, "plain_graph": 0, "ragged_graph": 0, "eager": 0}

    # ---------------------------------------------------------------- cache binding

    def bind_kv_cache(self, kv_cache_tensor, k_scale=None, v_scale=None, cache_dtype="fp16"):
        """kv_cache_tensor [2, layers, blocks, block_size, kv_heads, head_dim]; scales
        [layers, blocks, block_size] for fp8."""
        self._kv_cache = kv_cache_tensor
        self._k_scale, self._v_scale = k_scale, v_scale
        self._cache_dtype = cache_dtype
        if self.model is not None:
            self._bind_kv_cache_to_model()

    def _bind_kv_cache_to_model(self):
        layer = 0
        for module in self.model.modules():
            if isinstance(module, PagedAttention):
                module.k_cache = self._kv_cache[0, layer]
                module.v_cache = self._kv_cache[1, layer]
                module.cache_dtype = self._cache_dtype
                if self._k_scale is not None:
                    module.k_scale = self._k_scale[layer]
                if self._v_scale is not None:
                    module.v_scale = self._v_scale[layer]
                layer += 1

    # ---------------------------------------------------------------- metadata

    def _device(self):
        return self.config.device if torch.cuda.is_available() else "cpu"

    def _to_device(self, arr, dtype):
        t = torch.from_numpy(np.ascontiguousarray(arr)).to(dtype)
        dev = self._device()
        if dev == "cpu":
            return t
        return t.pin_memory().to(dev, non_blocking=True)

    def _staging(self, nbytes):
        """The next pinned staging buffer of the ring, at least nbytes long (uint8), and its ring slot;
        _upload(slot, nbytes) ships its first nbytes.  Waits for the copy that last left the buffer
        (as many steps ago as the ring has buffers)."""
        slot = self._decode_stage[self._decode_stage_turn]
        self._decode_stage_turn = (self._decode_stage_turn + 1) % len(self._decode_stage)
        if slot[1] is not None:
            slot[1].synchronize()
        if slot[0] is None or slot[0].numel() < nbytes:
            slot[0] = torch.empty(max(2 * nbytes, 1 << 16), dtype=torch.uint8).pin_memory()
        return slot[0][:nbytes], slot

    def _upload(self, slot, nbytes):
        """One asynchronous copy of the staging buffer's first nbytes to a fresh device tensor."""
        dev = torch.empty(nbytes, dtype=torch.uint8, device=self._device())
        dev.copy_(slot[0][:nbytes], non_blocking=True)
        if slot[1] is None:
            slot[1] = torch.cuda.Event()
        slot[1].record()
        return dev

    def _prepare_block_tables(self, sequences, device=None):
        """[num_seqs, max_blocks] int32, padded with -1; None when no sequence has a table."""
        lists = [seq.get("block_table", []) for seq in sequences]
        if not lists or all(len(bt) == 0 for bt in lists):
            return None
        width = max(len(bt) for bt in lists)
        tables = np.full((len(lists), width), -1, dtype=np.int32)
        for i, bt in enumerate(lists):
            if len(bt):
                tables[i, :len(bt)] = bt
        return self._to_device(tables, torch.int32)

    def prepare_prefill(self, sequences: List[dict], state: Optional["DecodeState"] = None
                        ) -> Tuple[torch.Tensor, torch.Tensor]:
        """sequences: dicts with 'token_ids', 'block_table', 'num_cached_tokens',
        'num_scheduled_tokens'.  Sets the global context; returns (input_ids, positions).

        On the GPU the step's metadata goes up in ONE copy - the chunk's token ids, the two cumulative
        length arrays and (when a sequence has a cached prefix or a cache to write) the block tables,
        side by side in one pinned buffer - and positions and slots are computed there by
        pa_prefill_metadata; the reference builds them in Python loops and ships every field on its own
        (src/inference/model_runner.py:464-540).  With `state` and a 'state_row' in every dict (a row
        the sequence holds in the DecodeState: DecodeState.reserve) the tables are not sent at all:
        they are the state's own rows, which stay on the device from the first chunk to the last
        decode step."""
        if self._device() == "cpu":
            return self._prepare_prefill_host(sequences)
        from .attention import prefill_metadata
        dev = torch.device(self._device())
        S = len(sequences)
        starts = [seq["num_cached_tokens"] for seq in sequences]
        counts = [seq["num_scheduled_tokens"] for seq in sequences]
        total = sum(counts)
        from_state = state is not None and S > 0 and all("state_row" in seq for seq in sequences)
        lists = [seq.get("block_table", []) for seq in sequences]
        any_table = any(len(bt) for bt in lists)
        has_prefix = any(st > 0 for st in starts)
        width = 0 if from_state or not any_table else max(len(bt) for bt in lists)
        # one pinned staging buffer: ids int64 [total] | cu_q int32 [S+1] | cu_k int32 [S+1] | rows int32 [S] | tables int32 [S, width]
        n32 = 2 * (S + 1) + S + S * width
        stage, slot = self._staging(8 * total + 4 * n32)
        ids = stage[:8 * total].view(torch.long)
        meta = stage[8 * total:].view(torch.int32)
        ids_np, meta_np = ids.numpy(), meta.numpy()
        cu_q, cu_k = meta_np[:S + 1], meta_np[S + 1:2 * (S + 1)]
        rows_np = meta_np[2 * (S + 1):2 * (S + 1) + S]
        tables_np = meta_np[2 * (S + 1) + S:].reshape(S, width) if width else None
        cu_q[0] = cu_k[0] = 0
        cursor = max_q = max_k = 0
        if tables_np is not None:
            tables_np.fill(-1)
        for i, seq in enumerate(sequences):
            start, n = starts[i], counts[i]
            ids_np[cursor:cursor + n] = seq["token_ids"][start:start + n]
            cursor += n
            cu_q[i + 1] = cu_q[i] + n
            cu_k[i + 1] = cu_k[i] + start + n
            max_q, max_k = max(max_q, n), max(max_k, start + n)
            rows_np[i] = seq["state_row"] if from_state else i
            if tables_np is not None and len(lists[i]):
                tables_np[i, :len(lists[i])] = lists[i]
        on_dev = self._upload(slot, 8 * total + 4 * n32)
        input_ids = on_dev[:8 * total].view(torch.long)
        meta_dev = on_dev[8 * total:].view(torch.int32)
        cu_q_dev, cu_k_dev = meta_dev[:S + 1], meta_dev[S + 1:2 * (S + 1)]
        rows_dev = meta_dev[2 * (S + 1):2 * (S + 1) + S]
        num_blocks = self._kv_cache.shape[2] if self._kv_cache is not None else 2 ** 31 // self.block_size - 1
        if from_state:
            positions, slot_mapping = prefill_metadata(cu_q_dev, cu_k_dev, total, state.block_tables, self.block_size,
                                                       num_blocks, row_index=rows_dev)
            block_tables = state.block_tables.index_select(0, rows_dev.long()) if has_prefix else None
        elif width:
            tables_dev = meta_dev[2 * (S + 1) + S:].view(S, width)
            positions, slot_mapping = prefill_metadata(cu_q_dev, cu_k_dev, total, tables_dev, self.block_size, num_blocks)
            block_tables = tables_dev if has_prefix else None
        else:
            positions, slot_mapping = prefill_metadata(cu_q_dev, cu_k_dev, total)
            block_tables = None
        set_context(is_prefill=True, cu_seqlens_q=cu_q_dev, cu_seqlens_k=cu_k_dev, max_seqlen_q=max_q, max_seqlen_k=max_k,
                    slot_mapping=slot_mapping, block_tables=block_tables)
        return input_ids, positions

    def _prepare_prefill_host(self, sequences: List[dict]) -> Tuple[torch.Tensor, torch.Tensor]:
        """prepare_prefill with every field built on the host (numpy row copies): what a machine without
        a GPU runs, and what the device path is checked against."""
        ids, pos, slots = [], [], []
        cu_q, cu_k = [0], [0]
        max_q = max_k = 0
        has_prefix = False
        for seq in sequences:
            start = seq["num_cached_tokens"]
            n = seq["num_scheduled_tokens"]
            end = start + n
            ids.append(np.asarray(seq["token_ids"][start:end], dtype=np.int64))
            pos.append(np.arange(start, end, dtype=np.int64))
            bt = seq.get("block_table", [])
            if bt:
                slots.append(slots_for_range(bt, start, end, self.block_size))
            cu_q.append(cu_q[-1] + n)
            cu_k.append(cu_k[-1] + end)
            max_q, max_k = max(max_q, n), max(max_k, end)
            has_prefix = has_prefix or start > 0
        input_ids = self._to_device(np.concatenate(ids) if ids else np.zeros(0, np.int64), torch.long)
        positions = self._to_device(np.concatenate(pos) if pos else np.zeros(0, np.int64), torch.long)
        slot_mapping = self._to_device(np.concatenate(slots), torch.int32) if slots else None
        block_tables = self._prepare_block_tables(sequences) if has_prefix else None
        set_context(
            is_prefill=True,
            cu_seqlens_q=self._to_device(np.asarray(cu_q), torch.int32),
            cu_seqlens_k=self._to_device(np.asarray(cu_k), torch.int32),
            max_seqlen_q=max_q, max_seqlen_k=max_k,
            slot_mapping=slot_mapping, block_tables=block_tables,
        )
        return input_ids, positions

    def prepare_decode(self, sequences: List[dict]) -> Tuple[torch.Tensor, torch.Tensor]:
        """sequences: dicts with 'token_ids', 'block_table', optional 'last_block_num_tokens'.
        One token per sequence; context_lens counts the token being written."""
        n = len(sequences)
        bs = self.block_size
        ids_l, lens_l, slots_l = [], [], []
        for seq in sequences:
            toks = seq["token_ids"]
            length = len(toks)
            last = seq.get("last_block_num_tokens", None)
            if last is None:
                last = ((length - 1) % bs) + 1
            ids_l.append(toks[-1])
            lens_l.append(length)
            slots_l.append(seq["block_table"][-1] * bs + last - 1)
        ids = np.array(ids_l, np.int64)
        lens = np.array(lens_l, np.int32)
        pos = lens.astype(np.int64) - 1
        slots = np.array(slots_l, np.int32)
        groups = None
        if getattr(self.config, "share_prefix_decode", False) and self._device() != "cpu":
            groups = self._decode_prefix_groups([seq["block_table"] for seq in sequences], lens.tolist())
        hints = dict(
            prefix_groups=groups,
            # the host has the lengths: the attention launch is sized for these rows, not for full tables
            longest_context_len=int(lens.max()) if n else 0,
            mean_context_len=float(lens.mean()) if n else 0.0,
        )
        lists = [seq.get("block_table", []) for seq in sequences]
        width = max((len(bt) for bt in lists), default=0)
        if self._device() == "cpu" or n == 0 or width == 0:
            set_context(
                is_prefill=False,
                slot_mapping=self._to_device(slots, torch.int32),
                context_lens=self._to_device(lens, torch.int32),
                block_tables=self._prepare_block_tables(sequences),
                **hints,
            )
            return self._to_device(ids, torch.long), self._to_device(pos, torch.long)
        # On the GPU the five fields go up side by side in one pinned buffer, as ONE copy (each field
        # on its own, as the reference ships them (src/inference/model_runner.py:542-588), costs a
        # pinned staging block and a copy apiece: 0.2 ms of host time per step); every field starts on
        # a 16-byte boundary:  ids int64 [n] | positions int64 [n] | slots int32 [n] | lens int32 [n] | tables int32 [n, width]
        pad = lambda nbytes: -(-nbytes // 16) * 16
        o_pos = pad(8 * n)
        o_slots = o_pos + pad(8 * n)
        o_lens = o_slots + pad(4 * n)
        o_tables = o_lens + pad(4 * n)
        nbytes = o_tables + 4 * n * width
        pinned, slot = self._staging(nbytes)
        stage = pinned.numpy()
        stage[0:8 * n].view(np.int64)[:] = ids
        stage[o_pos:o_pos + 8 * n].view(np.int64)[:] = pos
        stage[o_slots:o_slots + 4 * n].view(np.int32)[:] = slots
        stage[o_lens:o_lens + 4 * n].view(np.int32)[:] = lens
        tables = stage[o_tables:].view(np.int32).reshape(n, width)
        tables.fill(-1)
        # Turning a sequence's Python list of block ids into int32 costs more than everything else in
        # this function (8192 integers at batch 64 x ctx 2048), and the lists change once in block_size
        # steps.  The rows of the last step are kept, found again by (length, first id, last id) and
        # reused only when the kept copy of the list still equals the caller's list (a comparison at
        # C speed); whatever else changed - an appended block, a copied-on-write block, a new
        # sequence in the slot - is converted afresh.
        kept, fresh = self._table_rows, {}
        for i, bt in enumerate(lists):
            length = len(bt)
            if length:
                if type(bt) is list:
                    key = (length, bt[0], bt[-1])
                    hit = kept.get(key)
                    if hit is None or hit[0] != bt:
                        hit = (list(bt), np.asarray(bt, dtype=np.int32))
                    fresh[key] = hit
                    tables[i, :length] = hit[1]
                else:
                    tables[i, :length] = bt
        self._table_rows = fresh
        dev = self._upload(slot, nbytes)
        set_context(
            is_prefill=False,
            slot_mapping=dev[o_slots:o_slots + 4 * n].view(torch.int32),
            context_lens=dev[o_lens:o_lens + 4 * n].view(torch.int32),
            block_tables=dev[o_tables:].view(torch.int32).view(n, width),
            **hints,
        )
        return dev[0:8 * n].view(torch.long), dev[o_pos:o_pos + 8 * n].view(torch.long)

    def _decode_prefix_groups(self, tables, lens):
        """Groups of rows that share a prefix, for prepare_decode.  Finding them walks block-id lists,
        so the last result is kept and reused while it provably still holds: same batch size, same
        first block in every row (rows that share anything share their first block, so new sharing
        cannot appear without one of these changing), and every member of every group still has its
        group's last shared block where it was and a context that covers the shared tokens (shared
        blocks are full blocks, which never change while an owner lives).  A step with an unchanged
        batch costs one pass over the rows."""
        cfg = self.config
        if 16 // max(1, cfg.num_heads // cfg.num_kv_heads) < 2:
            return None
        key = (len(tables),) + tuple(t[0] if len(t) else -1 for t in tables)
        kept = self._prefix_groups_kept
        if kept is not None and kept[0] == key:
            pg = kept[1]
            if pg is None:
                return None
            bs = self.block_size
            for members, tokens in pg.groups:
                last = tokens // bs - 1
                lead = tables[members[0]]
                if any(len(tables[r]) <= last or tables[r][last] != lead[last] or lens[r] < tokens for r in members):
                    break
            else:
                return pg
        sizes = [x for x in cfg.prefix_partition_sizes if x % self.block_size == 0 and x % 16 == 0]
        pg = None
        if sizes:
            from .attention import choose_prefix_partition, find_prefix_groups_anywhere, shared_prefix_descriptors
            size, groups = choose_prefix_partition(
                lambda x: find_prefix_groups_anywhere(tables, lens, self.block_size, cfg.num_heads, cfg.num_kv_heads, x),
                sizes)
            if groups:
                pg = shared_prefix_descriptors(groups, len(tables), self._device(), size)
        self._prefix_groups_kept = (key, pg)
        return pg

    # ---------------------------------------------------------------- forward

    @torch.inference_mode()
    def run(self, input_ids, positions, is_prefill=True):
        if self._hf_model is not None:
            return self._run_hf_model(input_ids, positions, is_prefill)
        if self.model is None:
            # the reference's mock mode (src/inference/model_runner.py:152-158): a runner without a
            # model answers with random logits, so that a scheduler can be exercised on its own
            logits = torch.randn(input_ids.shape[0], self.config.vocab_size, device=input_ids.device,
                                 dtype=torch.float32)
            reset_context()
            return logits
        use_graph = (not is_prefill and self.config.enable_cuda_graph and self._graph_vars is not None
                     and any(b >= input_ids.size(0) for b in self._graph_batch_sizes))
        if use_graph:
            logits = self._run_with_cuda_graph(input_ids, positions)
        else:
            logits = self.model(input_ids, positions=positions)
        reset_context()
        return logits

    @torch.inference_mode()
    def run_batch_decode(self, input_ids, positions, block_tables, context_lens):
        """One decode step for a batch whose metadata is already on the GPU: input_ids [batch] or
        [batch, 1], positions [batch] (of the token being written), block_tables [batch, max_blocks]
        int32, context_lens [batch] int32 (counting that token) -> logits [batch, vocab]
        (src/inference/model_runner.py:639-708)."""
        from .attention import slot_mapping
        if input_ids.dim() == 2:
            input_ids = input_ids.squeeze(1)
        num_blocks = self._kv_cache.shape[2] if self._kv_cache is not None else 2 ** 31 // self.block_size - 1
        slots = slot_mapping(positions, block_tables, self.block_size, num_blocks)
        set_context(is_prefill=False, slot_mapping=slots, context_lens=context_lens, block_tables=block_tables)
        return self.run(input_ids, positions, is_prefill=False)

    # ---------------------------------------------------------------- HuggingFace-style models
    # The reference's shipped kv_cache mode (src/inference/model_runner.py:118-462): the model is
    # a HuggingFace causal LM that knows nothing of paging; its K/V are written into the paged pool
    # after the forward and rebuilt from the pool as past_key_values before every decode step.
    # Same methods and call order; the pool traffic goes through pa_kv_store and pa_gather_kv.

    def bind_hf_model(self, model: torch.nn.Module):
        self._hf_model = model

    def _run_hf_model(self, input_ids, positions, is_prefill):
        ctx = get_context()
        if is_prefill:
            logits = self._hf_prefill_forward(input_ids, positions, ctx)
        else:
            logits = self._hf_decode_forward(input_ids, positions, ctx)
        reset_context()
        return logits

    def _hf_prefill_forward(self, input_ids, positions, ctx):
        """One sequence [num_tokens]: full forward, K/V of every layer into the pool, logits
        [num_tokens, vocab] (model_runner.py:192-230)."""
        ids2 = input_ids.unsqueeze(0) if input_ids.dim() == 1 else input_ids
        pos2 = positions.unsqueeze(0) if positions.dim() == 1 else positions
        mask = torch.ones(1, ids2.shape[1], dtype=torch.long, device=input_ids.device)
        outputs = self._hf_model(input_ids=ids2, position_ids=pos2, attention_mask=mask, use_cache=True)
        if ctx.slot_mapping is not None and self._kv_cache is not None:
            self._store_hf_kv_to_paged_cache(outputs.past_key_values, ctx.slot_mapping)
        return outputs.logits.squeeze(0)

    def _hf_decode_forward(self, input_ids, positions, ctx):
        """One token per sequence: past_key_values gathered from the pool, single-token forward,
        the new token's K/V into the pool, logits [batch, vocab] (model_runner.py:232-285)."""
        ids2 = input_ids.unsqueeze(1) if input_ids.dim() == 1 else input_ids
        pos2 = positions.unsqueeze(1) if positions.dim() == 1 else positions
        past, mask = None, None
        if ctx.context_lens is not None:
            max_past_len = int(ctx.context_lens.max().item()) - 1       # the reference's one host read
            past = self._load_kv_from_paged_cache(ctx.block_tables, ctx.context_lens, max_past_len)
            mask = torch.ones(ids2.shape[0], max_past_len + 1, dtype=torch.long, device=input_ids.device)
        outputs = self._hf_model(input_ids=ids2, position_ids=pos2, attention_mask=mask,
                                 past_key_values=past, use_cache=True)
        if ctx.slot_mapping is not None and self._kv_cache is not None:
            self._store_hf_decode_kv_to_cache(outputs.past_key_values, ctx)
        return outputs.logits.squeeze(1)

    def _pool_layer(self, layer_idx):
        if self._k_scale is not None or self._kv_cache.element_size() == 1:
            raise RuntimeError("the HuggingFace path stores K/V unscaled: bind an fp16 or bf16 pool")
        return self._kv_cache[0, layer_idx], self._kv_cache[1, layer_idx]

    def _store_hf_kv_to_paged_cache(self, past_key_values, slot_mapping):
        """Prefill: [1, kv_heads, seq, dim] per layer -> the slots of the sequence
        (model_runner.py:287-312)."""
        from .attention import store_kv_cache
        for layer_idx in range(self.config.num_layers):
            k, v = self._extract_layer_kv(past_key_values, layer_idx)
            k_cache, v_cache = self._pool_layer(layer_idx)
            k = k.squeeze(0).transpose(0, 1).contiguous().to(k_cache.dtype)
            v = v.squeeze(0).transpose(0, 1).contiguous().to(v_cache.dtype)
            store_kv_cache(k, v, k_cache, v_cache, slot_mapping)

    def _store_hf_decode_kv_to_cache(self, past_key_values, ctx):
        """Decode: the last position of [batch, kv_heads, past + 1, dim] per layer -> each
        sequence's new slot (model_runner.py:314-338)."""
        from .attention import store_kv_cache
        for layer_idx in range(self.config.num_layers):
            k, v = self._extract_layer_kv(past_key_values, layer_idx)
            k_cache, v_cache = self._pool_layer(layer_idx)
            k_new = k[:, :, -1, :].contiguous().to(k_cache.dtype)        # [batch, kv_heads, dim]
            v_new = v[:, :, -1, :].contiguous().to(v_cache.dtype)
            store_kv_cache(k_new, v_new, k_cache, v_cache, ctx.slot_mapping)

    def _load_kv_from_paged_cache(self, block_tables, context_lens, max_past_len: Optional[int] = None):
        """past_key_values for a decode step: per layer K, V [batch, kv_heads, max_past_len, dim]
        with each sequence's first context_len - 1 positions from the pool and zeros after
        (model_runner.py:340-420).  None when there is no cache or nothing cached yet.  Returned
        as a transformers DynamicCache when that class is importable, else as a tuple of (K, V)."""
        from .attention import gather_kv_cache
        if self._kv_cache is None or block_tables is None or context_lens is None:
            return None
        if max_past_len is None:
            max_past_len = int(context_lens.max().item()) - 1
        if max_past_len <= 0:
            return None
        layers = []
        for layer_idx in range(self.config.num_layers):
            k_cache, v_cache = self._pool_layer(layer_idx)
            layers.append(gather_kv_cache(k_cache, v_cache, block_tables, context_lens, max_past_len, len_offset=1))
        try:
            from transformers import DynamicCache
            cache = DynamicCache()
            for layer_idx, (k, v) in enumerate(layers):
                cache.update(k, v, layer_idx)
            return cache
        except ImportError:
            return tuple(layers)

    @staticmethod
    def _extract_layer_kv(past_key_values, layer_idx: int):
        """(K, V) of one layer, each [batch, kv_heads, seq, dim], from the cache classes of
        transformers 5.x (.layers) and 4.x (.key_cache) or a legacy tuple (model_runner.py:435-462)."""
        if hasattr(past_key_values, "layers"):
            layer = past_key_values.layers[layer_idx]
            return layer.keys, layer.values
        if hasattr(past_key_values, "key_cache"):
            return past_key_values.key_cache[layer_idx], past_key_values.value_cache[layer_idx]
        layer_kv = past_key_values[layer_idx]
        if isinstance(layer_kv, (tuple, list)):
            return layer_kv[0], layer_kv[1]
        raise ValueError("Unsupported past_key_values format: %s" % type(past_key_values))

    # ---------------------------------------------------------------- sampling

    def sample(self, logits: torch.Tensor, temperature: float = 0.7, top_p: float = 0.9,
               uniforms: Optional[torch.Tensor] = None) -> List[int]:
        """Token ids for logits [batch, vocab], as a list like the reference's sample()
        (src/inference/model_runner.py:590-634); `sample_tokens` is the same without the copy to
        the host."""
        from .attention import sample_tokens
        return sample_tokens(logits, temperature, top_p, uniforms).tolist()

    # ---------------------------------------------------------------- decode graphs

    @torch.inference_mode()
    def capture_cuda_graphs(self, batch_sizes: Optional[List[int]] = None,
                            context_buckets: Optional[List[int]] = None):
        """Record HIP graphs of the decode forward over shared static inputs: one per batch size
        (src/inference/model_runner.py:710-760) and, because the static block tables are max_num_blocks
        wide whatever the batch holds, per context bucket (launches sized for rows of up to that many
        tokens; default config.decode_context_buckets) and, where the launch policy cuts a ragged batch
        differently, once more for ragged batches.  A step replays the graph that fits the lengths
        prepare_decode has passed on (InferenceContext.longest_context_len / mean_context_len); a context
        without them takes the graph sized for the tables' width."""
        if not torch.cuda.is_available() or self.model is None:
            return
        if batch_sizes is None:
            max_bs = min(self.config.max_cuda_graph_batch_size, 64)
            batch_sizes = [1, 2, 4, 8] + list(range(16, max_bs + 1, 16))
        from .attention import sizing_graph_workspace
        self._graph_batch_sizes = sorted(batch_sizes)
        max_bs = max(batch_sizes)
        dev = self.config.device
        self._reserve_decode_workspace(max_bs)
        width = self.config.max_num_blocks * self.block_size
        self._graph_buckets = self._buckets_for_width(width, context_buckets)
        gv = {
            "input_ids": torch.zeros(max_bs, dtype=torch.long, device=dev),
            "positions": torch.zeros(max_bs, dtype=torch.long, device=dev),
            "slot_mapping": torch.full((max_bs,), -1, dtype=torch.int32, device=dev),
            "context_lens": torch.zeros(max_bs, dtype=torch.int32, device=dev),
            "block_tables": torch.zeros(max_bs, self.config.max_num_blocks, dtype=torch.int32, device=dev),
        }
        for bs in reversed(self._graph_batch_sizes):
            for bucket in self._graph_buckets:
                flavours = [False]
                if getattr(self.config, "ragged_decode_graphs", True) and self._ragged_launch_differs(bs, bucket):
                    flavours.append(True)
                for ragged in flavours:
                    graph = torch.cuda.CUDAGraph()
                    hints = dict(longest_context_len=bucket if bucket < width else 0,
                                 mean_context_len=_RAGGED_GRAPH_MEAN * bucket if ragged else 0.0)
                    set_context(False, slot_mapping=gv["slot_mapping"][:bs], context_lens=gv["context_lens"][:bs],
                                block_tables=gv["block_tables"][:bs], **hints)
                    # warm-up outside the capture: library handles, allocator warm-up
                    with sizing_graph_workspace():
                        self.model(gv["input_ids"][:bs], positions=gv["positions"][:bs])
                    torch.cuda.synchronize()
                    set_context(False, slot_mapping=gv["slot_mapping"][:bs], context_lens=gv["context_lens"][:bs],
                                block_tables=gv["block_tables"][:bs], **hints)
                    with torch.cuda.graph(graph, pool=self._graph_pool):
                        out = self.model(gv["input_ids"][:bs], positions=gv["positions"][:bs])
                    if self._graph_pool is None:
                        self._graph_pool = graph.pool()
                    self._graphs[(bs, bucket, ragged)] = graph
                    self._graph_outputs[(bs, bucket, ragged)] = out
                    torch.cuda.synchronize()
                    reset_context()
        self._graph_vars = gv

    def _reserve_decode_workspace(self, max_batch):
        """Size the device's partition workspace for the finest split any decode launch of up to
        max_batch rows can choose, before anything is recorded: a workspace never grows inside a
        capture, and one that a graph has recorded is never freed."""
        from .attention import decode_workspace_bytes, reserve_decode_workspace
        cfg = self.config
        reserve_decode_workspace(torch.device(cfg.device),
                                 decode_workspace_bytes(max_batch, cfg.num_heads, cfg.head_dim), for_graphs=True)

    def _run_with_cuda_graph(self, input_ids, positions):
        bs = input_ids.size(0)
        ctx = get_context()
        graph_bs = next((x for x in self._graph_batch_sizes if x >= bs), None)
        # the smallest context bucket that holds the longest row the host knows of (none known: the widest)
        longest = getattr(ctx, "longest_context_len", 0) or self._graph_buckets[-1]
        bucket = next((b for b in self._graph_buckets if b >= longest), None)
        mean = getattr(ctx, "mean_context_len", 0.0)
        ragged = bucket is not None and 0 < mean < 0.7 * bucket and (graph_bs, bucket, True) in self._graphs
        key = (graph_bs, bucket, ragged)
        if graph_bs is None or key not in self._graphs:
            return self.model(input_ids, positions=positions)
        gv = self._graph_vars
        gv["input_ids"][:bs] = input_ids
        gv["positions"][:bs] = positions
        gv["slot_mapping"].fill_(-1)                 # padded rows write nothing
        if ctx.slot_mapping is not None:
            gv["slot_mapping"][:bs] = ctx.slot_mapping
        gv["context_lens"].zero_()                   # padded rows read nothing
        if ctx.context_lens is not None:
            gv["context_lens"][:bs] = ctx.context_lens
        if ctx.block_tables is not None:
            bt = ctx.block_tables
            gv["block_tables"][:bs, :bt.size(1)] = bt    # the tail stays stale, as in the reference
        self._graphs[key].replay()
        return self._graph_outputs[key][:bs]

    # ---------------------------------------------------------------- decode over a DecodeState

    @torch.inference_mode()
    def _buckets_for_width(self, width: int, given=None) -> List[int]:
        """Context buckets (tokens, ascending) for block tables `width` tokens wide; the last one is the
        width.  given None: config.decode_context_buckets, and without those the width and every half
        of the one before down to 2048 tokens."""
        if given is None:
            given = getattr(self.config, "decode_context_buckets", None)
        if given is None:
            buckets, b = [], width
            while b >= 2048:
                buckets.append(b)
                b //= 2
        else:
            buckets = [int(b) for b in given if 0 < int(b) < width]
        return sorted(set(buckets) | {width})

    def _context_buckets(self, state: DecodeState) -> List[int]:
        """Context buckets that graphs over `state` are recorded for."""
        return self._buckets_for_width(state.max_blocks * state.block_size)

    def _ragged_launch_differs(self, bs: int, bucket: int) -> bool:
        """Whether the launch policy shapes a ragged batch of `bs` rows of up to `bucket` tokens
        differently from a full one (only then is a second graph worth recording)."""
        from .attention import choose_partition
        cfg = self.config
        elem = 1 if self._cache_dtype == "fp8" else 2
        full = choose_partition(bs, cfg.num_heads, cfg.num_kv_heads, bucket, cfg.head_dim, elem)
        ragged = choose_partition(bs, cfg.num_heads, cfg.num_kv_heads, bucket, cfg.head_dim, elem,
                                  mean_context=_RAGGED_GRAPH_MEAN * bucket)
        return full != ragged

    def capture_decode_state_graphs(self, state: DecodeState, batch_sizes: Optional[List[int]] = None,
                                    context_buckets: Optional[List[int]] = None):
        """Record the decode forward over the first n rows of `state` for each n: the graph's
        inputs are the state's own tensors, so a replay needs no copies at all.

        A recorded launch cannot be resized, so each n is recorded per context bucket (launches sized for
        rows of up to that many tokens; default: config.decode_context_buckets) and, where the launch
        policy would split a ragged batch differently from a full one, once more for ragged batches;
        run_decode_state replays the graph that fits the lengths the host has counted.  When the state
        keeps groups of rows that share a prefix (and config.share_prefix_decode), one more graph per n,
        bucket and partition size is recorded over its group descriptors - at their full capacity, empty
        groups included - and replayed whenever the state holds a group."""
        from .attention import sizing_graph_workspace
        if not torch.cuda.is_available() or self.model is None:
            return
        if batch_sizes is None:
            batch_sizes = sorted({b for b in (1, 2, 4, 8, 16, 32, 64, 128, 256) if b < state.max_batch}
                                 | {state.max_batch})
        self._reserve_decode_workspace(max(batch_sizes))
        width = state.max_blocks * state.block_size
        buckets = self._buckets_for_width(width, context_buckets)
        self._state_buckets[id(state)] = sorted(set(self._state_buckets.get(id(state), [])) | set(buckets))
        prefix_sizes = []
        if state.tracks_prefixes and getattr(self.config, "share_prefix_decode", False):
            prefix_sizes = list(state.prefix_partition_sizes)
        for bs in sorted(batch_sizes, reverse=True):
            for bucket in buckets:
                variants = [(None, False)]
                if getattr(self.config, "ragged_decode_graphs", True) and self._ragged_launch_differs(bs, bucket):
                    variants.append((None, True))
                if bs >= 2:
                    variants += [(psize, False) for psize in prefix_sizes if psize <= bucket]
                for psize, ragged in variants:
                    lengths = (bucket, _RAGGED_GRAPH_MEAN * bucket if ragged else 0.0)
                    state.set_context(bs, share_prefixes=False, graph_partition_size=psize, lengths=lengths)
                    with sizing_graph_workspace():
                        self.model(state.input_ids[:bs], positions=state.positions[:bs])     # library handles, allocator warm-up
                    torch.cuda.synchronize()
                    graph = torch.cuda.CUDAGraph()
                    with torch.cuda.graph(graph, pool=self._graph_pool):
                        out = self.model(state.input_ids[:bs], positions=state.positions[:bs])
                    if self._graph_pool is None:
                        self._graph_pool = graph.pool()
                    self._state_graphs[(id(state), bs, psize, bucket, ragged)] = (graph, out)
                    self._state_graph_lookup.clear()
                    torch.cuda.synchronize()
                    reset_context()

    def _state_graph_for(self, state, rows, partition_size, longest=0, mean=0.0):
        """The graph recorded over `state` for the smallest batch size >= rows and the smallest context
        bucket >= longest (for the given shared-prefix partition size, None = the plain launch; the one
        for ragged batches when there is one and `mean` is below 0.7 of the bucket), or None."""
        bucket = next((b for b in self._state_buckets.get(id(state), ()) if b >= longest), None)
        if bucket is None:
            return None
        ragged = partition_size is None and 0 < mean < 0.7 * bucket
        key = (id(state), rows, partition_size, bucket, ragged)
        hit = self._state_graph_lookup.get(key, False)
        if hit is False:
            hit = None
            for flavour in ((True, False) if ragged else (False,)):
                sizes = sorted(bs for (sid, bs, ps, bk, rg) in self._state_graphs
                               if sid == id(state) and ps == partition_size and bk == bucket and rg == flavour and bs >= rows)
                if sizes:
                    hit = self._state_graphs[(id(state), sizes[0], partition_size, bucket, flavour)] + (flavour,)
                    break
            self._state_graph_lookup[key] = hit
        return hit

    @torch.inference_mode()
    def run_decode_state(self, state: DecodeState) -> torch.Tensor:
        """Logits [rows_in_use, vocab] of the step `state.step()` has just prepared."""
        if self.model is None:
            raise RuntimeError("ModelRunner.run_decode_state: no model bound")
        n = state.rows_in_use
        share = getattr(self.config, "share_prefix_decode", False)
        state.sync_prefix_groups()
        if self.config.enable_cuda_graph and id(state) in self._state_buckets:
            psize = state.prefix_partition_size if share else None
            longest, mean = state.known_lengths(n)
            for want in ((psize, None) if psize is not None else (None,)):
                hit = self._state_graph_for(state, n, want, longest, mean)
                if hit is not None:
                    graph, out, ragged = hit
                    graph.replay()
                    self.decode_state_stats["shared_prefix_graph" if want is not None else
                                            "ragged_graph" if ragged else "plain_graph"] += 1
                    return out[:n]
        self.decode_state_stats["eager"] += 1
        state.set_context(n, share_prefixes=share)
        logits = self.model(state.input_ids[:n], positions=state.positions[:n])
        reset_context()
        return logits

    def invalidate_cuda_graphs(self):
        """Drop every recorded graph (after a weight update)."""
        self._state_graphs.clear()
        self._state_graph_lookup.clear()
        self._state_buckets.clear()
        self._prefix_groups_kept = None
        self._graphs.clear()
        self._graph_outputs.clear()
        self._graph_pool = None
        self._graph_vars = None
        self._graph_batch_sizes = []
