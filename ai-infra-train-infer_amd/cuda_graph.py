"""Decode steps recorded as HIP graphs, one per padded batch size.

Mirrors the reference's CUDAGraphRunner (src/inference/cuda_graph.py:30-233): `capture` records
`model_forward_fn(input_ids, positions, **extra_buffers)` over static input buffers for one batch
size, `replay` copies the live inputs into the buffers of the smallest recorded size that fits,
launches the graph and returns the first `batch_size` rows of its output; `is_captured`,
`invalidate`, `get_stats` and the default size ladder are the reference's.  On ROCm
torch.cuda.CUDAGraph is a hipGraph, so one replay is one launch for the whole step.

What a paged decode step needs on top, and the reference leaves to chance: the rows between the
live batch and the padded size must be inert.  The reference zero-fills every extra buffer
(cuda_graph.py:108-110) and never resets the padding on replay, so a padded row writes its K/V to
slot 0 (block 0, a live block) and attends over whatever the previous, larger batch left in its
row.  Here a buffer is created with, and before every replay reset to, its padding value:
`slot_mapping` -1 (the writers skip it), everything else 0 (`context_lens` 0: the row reads
nothing and its output is zero).  Other names take a value through `buffer_fill={name: value}`.

The recorded region must not allocate: the partitioned decode launches take their partials from
the device's workspace for graphs, which the warm-up runs (outside the recording) have sized.
"""
from typing import Callable, Dict, List, Optional, Tuple

import torch

_PADDING = {"slot_mapping": -1}


class CUDAGraphRunner:
    def __init__(self, max_batch_size: int = 32, supported_batch_sizes: Optional[List[int]] = None):
        if supported_batch_sizes is None:
            supported_batch_sizes = [b for b in (1, 2, 4, 8, 16, 32, 64, 128) if b <= max_batch_size] or [1]
        self.max_batch_size = max_batch_size
        self.supported_batch_sizes = sorted(supported_batch_sizes)
        self._graphs: Dict[int, "torch.cuda.CUDAGraph"] = {}
        self._input_buffers: Dict[int, Dict[str, torch.Tensor]] = {}
        self._output_buffers: Dict[int, torch.Tensor] = {}
        self._fill: Dict[int, Dict[str, int]] = {}
        self._graph_pool = None
        self._replay_count = 0
        self._capture_count = 0

    def capture(self, model_forward_fn: Callable, batch_size: int, input_ids_shape: Tuple[int, ...] = None,
                hidden_size: int = 4096, device: str = "cuda", dtype: torch.dtype = torch.float16,
                num_warmup: int = 3, buffer_fill: Optional[Dict[str, int]] = None, **extra_buffer_shapes):
        """Record model_forward_fn for `batch_size`.  extra_buffer_shapes: name -> shape of an int32
        input buffer (block_tables, slot_mapping, context_lens ...) passed to the function by
        keyword.  The output buffer is whatever the function returns (its first dimension must be
        the batch); `input_ids_shape`, `hidden_size` and `dtype` are accepted for the reference's
        signature only.  Does nothing without a GPU, like the reference."""
        if not torch.cuda.is_available():
            return
        fill = dict(_PADDING)
        fill.update(buffer_fill or {})
        buffers = {
            "input_ids": torch.zeros(batch_size, dtype=torch.long, device=device),
            "positions": torch.zeros(batch_size, dtype=torch.long, device=device),
        }
        for name, shape in extra_buffer_shapes.items():
            buffers[name] = torch.full(tuple(shape), fill.get(name, 0), dtype=torch.int32, device=device)
        extra = {name: buffers[name] for name in extra_buffer_shapes}
        from .attention import sizing_graph_workspace
        with torch.inference_mode():
            with sizing_graph_workspace():
                for _ in range(max(1, num_warmup)):     # sizes the graphs' workspace and library handles
                    model_forward_fn(buffers["input_ids"], buffers["positions"], **extra)
            torch.cuda.synchronize()
            graph = torch.cuda.CUDAGraph()
            with torch.cuda.graph(graph, pool=self._graph_pool):
                out = model_forward_fn(buffers["input_ids"], buffers["positions"], **extra)
        if not isinstance(out, torch.Tensor) or out.dim() == 0 or out.size(0) != batch_size:
            raise RuntimeError("CUDAGraphRunner.capture: the forward must return a tensor with %d rows" % batch_size)
        if self._graph_pool is None:
            self._graph_pool = graph.pool()
        self._graphs[batch_size] = graph
        self._input_buffers[batch_size] = buffers
        self._output_buffers[batch_size] = out
        self._fill[batch_size] = {name: fill.get(name, 0) for name in extra_buffer_shapes}
        self._capture_count += 1
        torch.cuda.synchronize()

    def replay(self, batch_size: int, input_ids: torch.Tensor, positions: Optional[torch.Tensor] = None,
               **kwargs) -> Optional[torch.Tensor]:
        """Output rows [:batch_size] (a copy), or None when no recorded size fits: the caller then
        runs the step eagerly."""
        padded = self._get_padded_batch_size(batch_size)
        if padded is None or padded not in self._graphs:
            return None
        buffers = self._input_buffers[padded]
        buffers["input_ids"][:batch_size].copy_(input_ids.reshape(-1)[:batch_size])
        if positions is not None:
            buffers["positions"][:batch_size].copy_(positions.reshape(-1)[:batch_size])
        for name, pad in self._fill[padded].items():
            buf = buffers[name]
            if buf.dim() > 0 and buf.shape[0] == padded:
                buf[batch_size:].fill_(pad)                     # padding rows stay inert
            value = kwargs.get(name)
            if isinstance(value, torch.Tensor):
                window = tuple(slice(0, min(a, b)) for a, b in zip(value.shape, buf.shape))
                buf[window].copy_(value[window])
        self._graphs[padded].replay()
        self._replay_count += 1
        return self._output_buffers[padded][:batch_size].clone()

    def _get_padded_batch_size(self, actual_batch_size: int) -> Optional[int]:
        for b in self.supported_batch_sizes:
            if b >= actual_batch_size:
                return b
        return None

    def is_captured(self, batch_size: int) -> bool:
        padded = self._get_padded_batch_size(batch_size)
        return padded is not None and padded in self._graphs

    def invalidate(self):
        """Drop every graph: after a weight update the recorded launches point at stale state."""
        self._graphs.clear()
        self._input_buffers.clear()
        self._output_buffers.clear()
        self._fill.clear()
        self._graph_pool = None

    def get_stats(self) -> dict:
        return {
            "captured_sizes": list(self._graphs.keys()),
            "total_captures": self._capture_count,
            "total_replays": self._replay_count,
            "graph_pool_active": self._graph_pool is not None,
            "supported_batch_sizes": self.supported_batch_sizes,
        }
