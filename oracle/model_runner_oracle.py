"""Literal restatement of how the reference's ModelRunner derives the per-step attention
metadata (TEST INFRASTRUCTURE ONLY; plain Python loops, lists out):

  prefill_metadata   src/inference/model_runner.py:464-540
  decode_metadata    src/inference/model_runner.py:542-588
  block_tables       src/inference/model_runner.py:814-828
  batch_decode_slots src/inference/model_runner.py:670-682
  load_kv_from_paged_cache  src/inference/model_runner.py:340-420 (one layer, tensors in / out)

Pinned by the closed form "slot of position p = block_table[p // BS] * BS + p % BS" in
tests/test_model_runner_host.py.
"""


def block_tables(sequences):
    lists = [seq.get("block_table", []) for seq in sequences]
    if not lists or all(len(bt) == 0 for bt in lists):
        return None
    width = max(len(bt) for bt in lists)
    tables = [[-1] * width for _ in lists]
    for i, bt in enumerate(lists):
        for j, block_id in enumerate(bt):
            tables[i][j] = block_id
    return tables


def prefill_metadata(sequences, block_size):
    input_ids, positions, slot_mapping = [], [], []
    cu_q, cu_k = [0], [0]
    max_q = max_k = 0
    has_prefix = False
    for seq in sequences:
        start = seq["num_cached_tokens"]
        num_tokens = seq["num_scheduled_tokens"]
        end = start + num_tokens
        input_ids.extend(seq["token_ids"][start:end])
        positions.extend(range(start, end))
        bt = seq.get("block_table", [])
        if bt:
            start_block = start // block_size
            end_block = (end + block_size - 1) // block_size
            for i in range(start_block, end_block):
                slot_start = bt[i] * block_size
                if i == start_block:
                    slot_start += start % block_size
                if i != end_block - 1:
                    slot_end = bt[i] * block_size + block_size
                else:
                    slot_end = bt[i] * block_size + end - i * block_size
                slot_mapping.extend(range(slot_start, slot_end))
        cu_q.append(cu_q[-1] + num_tokens)
        cu_k.append(cu_k[-1] + end)
        max_q = max(max_q, num_tokens)
        max_k = max(max_k, end)
        if start > 0:
            has_prefix = True
    return dict(input_ids=input_ids, positions=positions, slot_mapping=slot_mapping or None,
                cu_seqlens_q=cu_q, cu_seqlens_k=cu_k, max_seqlen_q=max_q, max_seqlen_k=max_k,
                block_tables=block_tables(sequences) if has_prefix else None)


def decode_metadata(sequences, block_size):
    input_ids, positions, slot_mapping, context_lens = [], [], [], []
    for seq in sequences:
        position = len(seq["token_ids"]) - 1
        last = seq.get("last_block_num_tokens", None)
        if last is None:
            last = (position % block_size) + 1
        input_ids.append(seq["token_ids"][-1])
        positions.append(position)
        slot_mapping.append(seq["block_table"][-1] * block_size + last - 1)
        context_lens.append(len(seq["token_ids"]))
    return dict(input_ids=input_ids, positions=positions, slot_mapping=slot_mapping,
                context_lens=context_lens, block_tables=block_tables(sequences))


def batch_decode_slots(positions, block_tables, block_size):
    """src/inference/model_runner.py:670-682: the slot of each sequence's new token, read from
    its own table row.  (The reference indexes without checks; rows whose position falls
    outside the table, or on a padding id, are reported as None here.)"""
    slots = []
    for i, token_pos in enumerate(positions):
        block_idx = token_pos // block_size
        offset = token_pos % block_size
        if token_pos < 0 or block_idx >= len(block_tables[i]) or block_tables[i][block_idx] < 0:
            slots.append(None)
            continue
        slots.append(block_tables[i][block_idx] * block_size + offset)
    return slots


def load_kv_from_paged_cache(k_cache, v_cache, block_tables, context_lens):
    """src/inference/model_runner.py:361-420 for one layer: slot of every (sequence, past
    position) by the double loop, gather, zero the rows past each sequence's past length,
    [batch, len, heads, dim] -> [batch, heads, len, dim].  Returns None when nothing is cached,
    as the reference does."""
    import torch
    num_blocks, block_size, num_kv_heads, head_dim = k_cache.shape
    batch = len(block_tables)
    past_lens = [int(n) - 1 for n in context_lens]
    max_past_len = max(past_lens) if past_lens else 0
    if max_past_len <= 0:
        return None
    k_flat = k_cache.reshape(num_blocks * block_size, num_kv_heads, head_dim)
    v_flat = v_cache.reshape(num_blocks * block_size, num_kv_heads, head_dim)
    slot_indices = torch.zeros(batch, max_past_len, dtype=torch.long)
    for b in range(batch):
        for pos in range(max(past_lens[b], 0)):
            slot_indices[b, pos] = int(block_tables[b][pos // block_size]) * block_size + pos % block_size
    k_gathered = k_flat[slot_indices.view(-1)].view(batch, max_past_len, num_kv_heads, head_dim).clone()
    v_gathered = v_flat[slot_indices.view(-1)].view(batch, max_past_len, num_kv_heads, head_dim).clone()
    for b in range(batch):
        if past_lens[b] < max_past_len:
            k_gathered[b, max(past_lens[b], 0):] = 0
            v_gathered[b, max(past_lens[b], 0):] = 0
    return k_gathered.transpose(1, 2).contiguous(), v_gathered.transpose(1, 2).contiguous()
