"""Per-forward metadata handed from the model runner to the attention layers.

Same surface as the reference's src/inference/context.py:22-75: a module-global
InferenceContext that set_context() replaces (never mutates), get_context() returns and
reset_context() clears.  The forward pass is single-threaded by design, so a module global
is enough; the tensors are int32 and live on the device the attention runs on.
"""
from dataclasses import dataclass
from typing import Optional

import torch


@dataclass
class InferenceContext:
    """What an attention layer needs to know about the current step."""
    is_prefill: bool = False
    # prefill: cumulative new-token counts [S+1] and cumulative key counts (cached + new) [S+1]
    cu_seqlens_q: Optional[torch.Tensor] = None
    cu_seqlens_k: Optional[torch.Tensor] = None
    max_seqlen_q: int = 0
    max_seqlen_k: int = 0
    # token -> physical slot (block_id * block_size + offset); negative = do not write
    slot_mapping: Optional[torch.Tensor] = None
    # decode: tokens visible to each sequence, the one just written included
    context_lens: Optional[torch.Tensor] = None
    # [num_seqs, max_blocks] physical block ids; entries past the context are never read
    block_tables: Optional[torch.Tensor] = None
    # decode, optional (no counterpart in the reference): rows that share prefixes as the same
    # physical blocks, as attention.prepare_prefix_groups() returns them (a PrefixGroups); None = read
    # every row alone
    prefix_groups: Optional[object] = None
    # decode, optional (no counterpart in the reference): what the host knows about context_lens - an
    # upper bound on the longest row and the mean - so that the attention launch is sized for the rows
    # instead of for the width of the block table (attention.choose_partition); 0 = unknown
    longest_context_len: int = 0
    mean_context_len: float = 0.0


_CONTEXT = InferenceContext()


def set_context(
    is_prefill: bool,
    cu_seqlens_q: Optional[torch.Tensor] = None,
    cu_seqlens_k: Optional[torch.Tensor] = None,
    max_seqlen_q: int = 0,
    max_seqlen_k: int = 0,
    slot_mapping: Optional[torch.Tensor] = None,
    context_lens: Optional[torch.Tensor] = None,
    block_tables: Optional[torch.Tensor] = None,
    prefix_groups: Optional[object] = None,
    longest_context_len: int = 0,
    mean_context_len: float = 0.0,
):
    """Install the context for the next model forward."""
    global _CONTEXT
    _CONTEXT = InferenceContext(
        is_prefill=is_prefill,
        cu_seqlens_q=cu_seqlens_q,
        cu_seqlens_k=cu_seqlens_k,
        max_seqlen_q=max_seqlen_q,
        max_seqlen_k=max_seqlen_k,
        slot_mapping=slot_mapping,
        context_lens=context_lens,
        block_tables=block_tables,
        prefix_groups=prefix_groups,
        longest_context_len=longest_context_len,
        mean_context_len=mean_context_len,
    )


def get_context() -> InferenceContext:
    return _CONTEXT


def reset_context():
    """Drop the tensor references once the forward is done."""
    global _CONTEXT
    _CONTEXT = InferenceContext()
