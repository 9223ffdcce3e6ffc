"""Device tensors of the paged KV cache.

Mirrors the tensor half of the reference's BlockPool (src/inference/kv_cache.py:31-39,
131-174, 233-258): one tensor [2, num_layers, num_blocks, block_size, num_kv_heads, head_dim]
(index 0 = K, 1 = V) in the model dtype or float8_e4m3fn, plus, for fp8, two fp32 scale
tensors [num_layers, num_blocks, block_size] initialised to one.  The host-side block
bookkeeping (free list, per-sequence tables) is not part of this package.

Sizing note for MI355X: one GPU holds 288 GB, so the pool is a single allocation; at the
Qwen3-0.6B shape (8 KV heads x 128) a token costs 4 KiB per layer in fp16 and 2 KiB + 8 B
in fp8.
"""
import warnings
from typing import Optional

import torch

# fp8 probe, as the reference does at src/inference/kv_cache.py:32-39
try:
    _FP8_DTYPE = torch.float8_e4m3fn
    torch.tensor([1.0], dtype=_FP8_DTYPE)
    HAS_FP8 = True
except (AttributeError, RuntimeError):  # pragma: no cover - torch too old
    HAS_FP8 = False
    _FP8_DTYPE = None


class BlockPool:
    """Owns the KV tensors of all layers; hands out per-layer views."""

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
        self._kv_cache: Optional[torch.Tensor] = None
        self.k_scale: Optional[torch.Tensor] = None
        self.v_scale: Optional[torch.Tensor] = None
        self._allocate_gpu_memory()

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
