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
    torch.tensor(...) per field; here every field is filled in one pinned host staging buffer
    with numpy row copies and shipped with a single asynchronous copy per step;
  * graph replay copies into static device buffers and pads with slot -1 / context 0, exactly as
    the reference does, but capture needs no host synchronisation inside the model;
  * `run_batch_decode` gets its slot mapping from a kernel instead of two `.item()` reads per
    sequence, so a decode step driven by device-resident tables never waits for the GPU.

HF-model KV gathering and mock logits are outside this path and are not rebuilt.
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


def slots_for_range(block_table, start, end, block_size):
    """Physical slots of token positions [start, end) of one sequence (numpy int32)."""
    pos = np.arange(start, end, dtype=np.int64)
    bt = np.asarray(block_table, dtype=np.int64)
    return (bt[pos // block_size] * block_size + pos % block_size).astype(np.int32)


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
        self._graphs: Dict[int, torch.cuda.CUDAGraph] = {}
        self._graph_outputs: Dict[int, torch.Tensor] = {}
        self._graph_pool = None
        self._graph_vars: Optional[Dict[str, torch.Tensor]] = None
        self._graph_batch_sizes: List[int] = []

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

    def prepare_prefill(self, sequences: List[dict]) -> Tuple[torch.Tensor, torch.Tensor]:
        """sequences: dicts with 'token_ids', 'block_table', 'num_cached_tokens',
        'num_scheduled_tokens'.  Sets the global context; returns (input_ids, positions)."""
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
        ids = np.empty(n, np.int64)
        pos = np.empty(n, np.int64)
        slots = np.empty(n, np.int32)
        lens = np.empty(n, np.int32)
        for i, seq in enumerate(sequences):
            toks = seq["token_ids"]
            position = len(toks) - 1
            last = seq.get("last_block_num_tokens", None)
            if last is None:
                last = (position % self.block_size) + 1
            ids[i] = toks[-1]
            pos[i] = position
            slots[i] = seq["block_table"][-1] * self.block_size + last - 1
            lens[i] = len(toks)
        set_context(
            is_prefill=False,
            slot_mapping=self._to_device(slots, torch.int32),
            context_lens=self._to_device(lens, torch.int32),
            block_tables=self._prepare_block_tables(sequences),
        )
        return self._to_device(ids, torch.long), self._to_device(pos, torch.long)

    # ---------------------------------------------------------------- forward

    @torch.inference_mode()
    def run(self, input_ids, positions, is_prefill=True):
        if self.model is None:
            raise RuntimeError("ModelRunner.run: no model bound")
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
        if self.model is None:
            raise RuntimeError("ModelRunner.run_batch_decode: no model bound")
        from .attention import slot_mapping
        if input_ids.dim() == 2:
            input_ids = input_ids.squeeze(1)
        num_blocks = self._kv_cache.shape[2] if self._kv_cache is not None else 2 ** 31 // self.block_size - 1
        slots = slot_mapping(positions, block_tables, self.block_size, num_blocks)
        set_context(is_prefill=False, slot_mapping=slots, context_lens=context_lens, block_tables=block_tables)
        return self.run(input_ids, positions, is_prefill=False)

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
    def capture_cuda_graphs(self, batch_sizes: Optional[List[int]] = None):
        """Record one HIP graph of the decode forward per batch size over shared static inputs."""
        if not torch.cuda.is_available() or self.model is None:
            return
        if batch_sizes is None:
            max_bs = min(self.config.max_cuda_graph_batch_size, 64)
            batch_sizes = [1, 2, 4, 8] + list(range(16, max_bs + 1, 16))
        self._graph_batch_sizes = sorted(batch_sizes)
        max_bs = max(batch_sizes)
        dev = self.config.device
        gv = {
            "input_ids": torch.zeros(max_bs, dtype=torch.long, device=dev),
            "positions": torch.zeros(max_bs, dtype=torch.long, device=dev),
            "slot_mapping": torch.full((max_bs,), -1, dtype=torch.int32, device=dev),
            "context_lens": torch.zeros(max_bs, dtype=torch.int32, device=dev),
            "block_tables": torch.zeros(max_bs, self.config.max_num_blocks, dtype=torch.int32, device=dev),
        }
        for bs in reversed(self._graph_batch_sizes):
            graph = torch.cuda.CUDAGraph()
            set_context(False, slot_mapping=gv["slot_mapping"][:bs], context_lens=gv["context_lens"][:bs],
                        block_tables=gv["block_tables"][:bs])
            # warm-up outside the capture: allocates the partition workspace and library handles
            self.model(gv["input_ids"][:bs], positions=gv["positions"][:bs])
            torch.cuda.synchronize()
            with torch.cuda.graph(graph, pool=self._graph_pool):
                out = self.model(gv["input_ids"][:bs], positions=gv["positions"][:bs])
            if self._graph_pool is None:
                self._graph_pool = graph.pool()
            self._graphs[bs] = graph
            self._graph_outputs[bs] = out
            torch.cuda.synchronize()
            reset_context()
        self._graph_vars = gv

    def _run_with_cuda_graph(self, input_ids, positions):
        bs = input_ids.size(0)
        graph_bs = next((x for x in self._graph_batch_sizes if x >= bs), None)
        if graph_bs is None or graph_bs not in self._graphs:
            return self.model(input_ids, positions=positions)
        ctx = get_context()
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
        self._graphs[graph_bs].replay()
        return self._graph_outputs[graph_bs][:bs]

    def invalidate_cuda_graphs(self):
        """Drop every recorded graph (after a weight update)."""
        self._graphs.clear()
        self._graph_outputs.clear()
        self._graph_pool = None
        self._graph_vars = None
        self._graph_batch_sizes = []
