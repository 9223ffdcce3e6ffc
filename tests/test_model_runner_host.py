"""ModelRunner's per-step metadata (CPU): equal to the loop-by-loop restatement of the
reference, which in turn is pinned by the slot closed form."""
import random

import torch

from oracle import model_runner_oracle as ref


def random_sequences(rng, n, block_size, prefill):
    seqs, next_block = [], 0
    for _ in range(n):
        total = rng.randint(1, 200)
        nblocks = (total + block_size - 1) // block_size
        bt = list(range(next_block, next_block + nblocks))
        rng.shuffle(bt)
        next_block += nblocks
        seq = {"token_ids": [rng.randint(0, 999) for _ in range(total)], "block_table": bt}
        if prefill:
            cached = rng.choice([0, 0, rng.randint(0, total - 1)])
            seq["num_cached_tokens"] = cached
            seq["num_scheduled_tokens"] = rng.randint(1, total - cached)
            # the table covers cached + scheduled tokens only
            need = (cached + seq["num_scheduled_tokens"] + block_size - 1) // block_size
            seq["block_table"] = bt[:need]
        seqs.append(seq)
    return seqs


def as_list(t):
    return None if t is None else t.tolist()


def test_oracle_slot_closed_form():
    rng = random.Random(1)
    for bs in (8, 16):
        seqs = random_sequences(rng, 12, bs, prefill=True)
        m = ref.prefill_metadata(seqs, bs)
        want = []
        for s in seqs:
            for p in range(s["num_cached_tokens"], s["num_cached_tokens"] + s["num_scheduled_tokens"]):
                want.append(s["block_table"][p // bs] * bs + p % bs)
        assert m["slot_mapping"] == want
        d = ref.decode_metadata(random_sequences(rng, 9, bs, prefill=False), bs)
        assert all(c == p + 1 for c, p in zip(d["context_lens"], d["positions"]))


def test_prepare_prefill_matches_reference_loops(pa):
    rng = random.Random(2)
    for bs in (8, 16):
        runner = pa.ModelRunner(None, pa.ModelRunnerConfig(block_size=bs, device="cpu"))
        for trial in range(5):
            seqs = random_sequences(rng, rng.randint(1, 9), bs, prefill=True)
            ids, pos = runner.prepare_prefill(seqs)
            ctx = pa.get_context()
            want = ref.prefill_metadata(seqs, bs)
            assert ids.tolist() == want["input_ids"] and pos.tolist() == want["positions"]
            assert ctx.is_prefill and as_list(ctx.slot_mapping) == want["slot_mapping"]
            assert as_list(ctx.cu_seqlens_q) == want["cu_seqlens_q"]
            assert as_list(ctx.cu_seqlens_k) == want["cu_seqlens_k"]
            assert (ctx.max_seqlen_q, ctx.max_seqlen_k) == (want["max_seqlen_q"], want["max_seqlen_k"])
            assert as_list(ctx.block_tables) == want["block_tables"]
            for t in (ctx.slot_mapping, ctx.cu_seqlens_q, ctx.cu_seqlens_k, ctx.block_tables):
                assert t is None or t.dtype == torch.int32
    pa.reset_context()


def test_prepare_decode_matches_reference_loops(pa):
    rng = random.Random(3)
    runner = pa.ModelRunner(None, pa.ModelRunnerConfig(block_size=16, device="cpu"))
    for trial in range(5):
        seqs = random_sequences(rng, rng.randint(1, 12), 16, prefill=False)
        if trial == 0:
            seqs[0]["last_block_num_tokens"] = 3
        ids, pos = runner.prepare_decode(seqs)
        ctx = pa.get_context()
        want = ref.decode_metadata(seqs, 16)
        assert ids.tolist() == want["input_ids"] and pos.tolist() == want["positions"]
        assert not ctx.is_prefill
        assert as_list(ctx.slot_mapping) == want["slot_mapping"]
        assert as_list(ctx.context_lens) == want["context_lens"]
        assert as_list(ctx.block_tables) == want["block_tables"]
        assert ctx.block_tables.dtype == torch.int32 and ctx.context_lens.dtype == torch.int32
    pa.reset_context()


def test_no_tables_means_none(pa):
    runner = pa.ModelRunner(None, pa.ModelRunnerConfig(block_size=16, device="cpu"))
    runner.prepare_prefill([{"token_ids": [1, 2, 3], "num_cached_tokens": 0, "num_scheduled_tokens": 3}])
    ctx = pa.get_context()
    assert ctx.slot_mapping is None and ctx.block_tables is None
    pa.reset_context()


def test_mock_mode_returns_random_logits_and_resets_the_context(pa):
    """src/inference/model_runner.py:152-158: no model bound -> random fp32 logits."""
    import torch
    r = pa.ModelRunner(None, pa.ModelRunnerConfig(vocab_size=97, device="cpu"))
    ids, pos = r.prepare_decode([{"token_ids": [1, 2, 3], "block_table": [0]}, {"token_ids": [4], "block_table": [1]}])
    assert pa.get_context().context_lens is not None
    logits = r.run(ids, pos, is_prefill=False)
    assert logits.shape == (2, 97) and logits.dtype == torch.float32
    assert pa.get_context().context_lens is None
