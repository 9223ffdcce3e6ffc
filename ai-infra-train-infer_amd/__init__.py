"""MI355X (gfx950) paged-attention hot path for the ai-infra-train-infer inference engine.

Exports the names a caller would import from the reference's src/inference package for
this path (src/inference/__init__.py:18-68): the context functions, the KV tensors of the
block pool, store_kv_cache and the two attention modules.  Compute is done by hand-written
HIP kernels behind a C ABI (include/paged_attn.h, libpaged_attn.so next to this file).

The directory name contains a hyphen, so import it through the `ai_infra_train_infer_amd`
loader module at the repository root.
"""
from .context import InferenceContext, set_context, get_context, reset_context
from .kv_cache import Block, BlockPool, BlockTable, KVCacheManager, HAS_FP8, _FP8_DTYPE
from .prefix_cache import PrefixCache, CachedBlock
from .radix_cache import RadixAttentionCache, RadixNode
from .cuda_graph import CUDAGraphRunner
from .attention import (
    PagedAttention,
    PartitionedPagedAttention,
    store_kv_cache,
    qk_norm_rope_store,
    sample_tokens,
    slot_mapping,
    prefill_metadata,
    gather_kv_cache,
    add_rms_norm,
    silu_mul,
    paged_decode,
    paged_decode_shared_prefix,
    find_prefix_groups,
    find_prefix_groups_anywhere,
    PrefixGroups,
    shared_prefix_descriptors,
    prepare_prefix_groups,
    paged_prefill,
    choose_partition,
    choose_launch,
    reserve_decode_workspace,
    sizing_graph_workspace,
    decode_workspace_bytes,
    release_decode_workspaces,
    check_block_tables,
    HAS_FLASH_ATTN,
    HAS_TRITON,
)
from .model_runner import ModelRunner, ModelRunnerConfig, DecodeState
from .qwen3_paged import Qwen3PagedConfig, Qwen3PagedModel
from . import _native

__all__ = [
    "InferenceContext", "set_context", "get_context", "reset_context",
    "Block", "BlockPool", "BlockTable", "KVCacheManager", "PrefixCache", "CachedBlock", "RadixAttentionCache", "RadixNode", "CUDAGraphRunner", "DecodeState", "slot_mapping", "prefill_metadata", "gather_kv_cache", "add_rms_norm", "silu_mul", "HAS_FP8",
    "PagedAttention", "PartitionedPagedAttention", "store_kv_cache", "qk_norm_rope_store", "sample_tokens",
    "paged_decode", "paged_decode_shared_prefix", "find_prefix_groups", "find_prefix_groups_anywhere", "PrefixGroups", "shared_prefix_descriptors", "prepare_prefix_groups", "paged_prefill", "choose_partition", "choose_launch", "reserve_decode_workspace", "sizing_graph_workspace",
    "decode_workspace_bytes", "release_decode_workspaces", "check_block_tables",
    "HAS_FLASH_ATTN", "HAS_TRITON",
    "ModelRunner", "ModelRunnerConfig", "Qwen3PagedConfig", "Qwen3PagedModel",
]
