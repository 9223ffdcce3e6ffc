"""Slot mapping on the device (pa_slot_mapping), bit-exact against the host loops of the
reference's ModelRunner as restated in oracle/model_runner_oracle.py, and the two callers built
on it: ModelRunner.run_batch_decode and CUDAGraphRunner."""
import copy
import ctypes

import pytest
import torch

from oracle import model_runner_oracle as mro

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("bs", [1, 16, 24])
def test_decode_slots_equal_the_host_loop(pa, gpu, bs):
    g = torch.Generator().manual_seed(40 + bs)
    B, W, NB = 97, 33, 500
    tables = torch.randint(0, NB, (B, W), generator=g, dtype=torch.int32)
    lens = torch.randint(1, W * bs + 1, (B,), generator=g)
    for i in range(B):                                   # padding beyond the sequence: -1, 0 or stale
        used = (int(lens[i]) + bs - 1) // bs
        tables[i, used:] = (-1, 0, 7)[i % 3]
    positions = lens - 1
    want = mro.batch_decode_slots(positions.tolist(), tables.tolist(), bs)
    assert None not in want
    got = pa.slot_mapping(positions.to(gpu), tables.to(gpu), bs, NB)
    assert got.dtype == torch.int32 and got.tolist() == want
    # a view of a wider table (row stride > width), int32 positions, preallocated output
    wide = torch.full((B, W + 9), -1, dtype=torch.int32)
    wide[:, :W] = tables
    out = torch.empty(B, dtype=torch.int32, device=gpu)
    assert pa.slot_mapping(positions.int().to(gpu), wide.to(gpu)[:, :W], bs, NB, out=out) is out
    assert out.tolist() == want


def test_positions_outside_the_table_or_pool_give_minus_one(pa, gpu):
    bs, NB = 4, 10
    tables = torch.tensor([[3, 9, -1], [10, 2, 5], [1, 1, 1], [0, 0, 0]], dtype=torch.int32)
    positions = torch.tensor([9, 0, 12, -1])            # padding id; id == NB; past the width; negative
    assert pa.slot_mapping(positions.to(gpu), tables.to(gpu), bs, NB).tolist() == [-1, -1, -1, -1]
    positions = torch.tensor([7, 5, 11, 0])
    assert pa.slot_mapping(positions.to(gpu), tables.to(gpu), bs, NB).tolist() == [9 * 4 + 3, 2 * 4 + 1, 1 * 4 + 3, 0]
    want = mro.batch_decode_slots(positions.tolist(), tables.tolist(), bs)
    assert want == [39, 9, 7, 0]


def test_prefill_slots_equal_the_host_loop(pa, gpu):
    bs, NB = 16, 300
    g = torch.Generator().manual_seed(41)
    seqs = []
    free = torch.randperm(NB, generator=g).tolist()
    for cached, new in [(0, 40), (32, 1), (50, 0), (7, 77), (0, 16), (100, 130)]:     # one chunk is empty
        total = cached + new
        table = [free.pop() for _ in range((total + bs - 1) // bs)]
        seqs.append({"token_ids": list(range(total)), "block_table": table,
                     "num_cached_tokens": cached, "num_scheduled_tokens": new})
    meta = mro.prefill_metadata(seqs, bs)
    width = max(len(s["block_table"]) for s in seqs)
    tables = torch.full((len(seqs), width), -1, dtype=torch.int32)
    for i, s in enumerate(seqs):
        tables[i, :len(s["block_table"])] = torch.tensor(s["block_table"], dtype=torch.int32)
    got = pa.slot_mapping(torch.tensor(meta["positions"]).to(gpu), tables.to(gpu), bs, NB,
                          cu_seqlens_q=torch.tensor(meta["cu_seqlens_q"], dtype=torch.int32).to(gpu))
    assert got.tolist() == meta["slot_mapping"]


def test_slot_mapping_c_abi_errors(lib, gpu):
    pos = torch.zeros(4, dtype=torch.int64, device=gpu)
    bt = torch.zeros(4, 8, dtype=torch.int32, device=gpu)
    out = torch.empty(4, dtype=torch.int32, device=gpu)
    call = lambda *a: lib.pa_slot_mapping(*a)
    P, T, O = pos.data_ptr(), bt.data_ptr(), out.data_ptr()
    assert call(P, None, T, 8, O, 4, 4, 8, 16, 100, None) == 0
    assert call(P, None, T, 8, O, 0, 4, 8, 16, 100, None) == 0            # nothing to do
    assert call(None, None, T, 8, O, 4, 4, 8, 16, 100, None) != 0
    assert call(P, None, T, 8, O, 4, 3, 8, 16, 100, None) != 0            # rows != tokens without cu_seqlens_q
    assert call(P, None, T, 4, O, 4, 4, 8, 16, 100, None) != 0            # stride < width
    assert call(P, None, T, 8, O, 4, 4, 8, 0, 100, None) != 0             # block size
    assert call(P, None, T, 8, O, 4, 4, 8, 16, 1 << 28, None) != 0        # slots would overflow int32
    assert b"pa_slot_mapping" in lib.pa_last_error()
    torch.cuda.synchronize()


def _small_session(pa, gpu, seed):
    from test_gpu_model import Session, small_model
    return Session(pa, small_model(pa, seed=seed), gpu)


def test_run_batch_decode_equals_prepare_decode_and_run(pa, gpu):
    """The same step two ways: host lists through prepare_decode, and device tensors through
    run_batch_decode (src/inference/model_runner.py:639-708)."""
    a = _small_session(pa, gpu, 11)
    b = _small_session(pa, gpu, 11)
    g = torch.Generator().manual_seed(12)
    for n in (9, 40, 17, 64):
        p = torch.randint(0, 512, (n,), generator=g).tolist()
        a.add(p)
        b.add(p)
    a.prefill()
    b.prefill()
    for step in range(3):
        nxt = torch.randint(0, 512, (4,), generator=g).tolist()
        want = a.decode(nxt)
        for s, t in zip(b.seqs, nxt):
            s["token_ids"].append(int(t))
            b._grow(s, len(s["token_ids"]))
            s["done"] = len(s["token_ids"])
        width = max(len(s["block_table"]) for s in b.seqs)
        tables = torch.tensor([s["block_table"] + [-1] * (width - len(s["block_table"])) for s in b.seqs],
                              dtype=torch.int32, device=gpu)
        lens = torch.tensor([len(s["token_ids"]) for s in b.seqs], dtype=torch.int32, device=gpu)
        ids = torch.tensor([[s["token_ids"][-1]] for s in b.seqs], device=gpu)         # [batch, 1] as the engine passes it
        got = b.runner.run_batch_decode(ids, (lens - 1).long(), tables, lens)
        assert pa.get_context().slot_mapping is None                                   # context reset afterwards
        torch.testing.assert_close(got.float().cpu(), want.float().cpu(), rtol=1e-3, atol=1e-3)
        assert torch.equal(a.pool.kv_cache_tensor.cpu(), b.pool.kv_cache_tensor.cpu())


def test_graph_runner_replays_equal_eager_and_padding_rows_are_inert(pa, gpu):
    """CUDAGraphRunner (src/inference/cuda_graph.py:30-233) around a paged decode step."""
    eager = _small_session(pa, gpu, 13)
    graph = _small_session(pa, gpu, 13)
    g = torch.Generator().manual_seed(14)
    for n in (9, 40, 17):
        p = torch.randint(0, 512, (n,), generator=g).tolist()
        eager.add(p)
        graph.add(p)
    eager.prefill()
    graph.prefill()
    # slot 0 is live (block 0 is the first sequence's first block): a padding row that wrote to it,
    # as zero-filled buffers would make it, shows up as a difference between the two pools
    assert graph.seqs[0]["block_table"][0] == 0
    W = 16

    def step(input_ids, positions, slot_mapping, context_lens, block_tables):
        pa.set_context(False, slot_mapping=slot_mapping, context_lens=context_lens, block_tables=block_tables)
        return graph.gpu_model(input_ids, positions=positions)

    runner = pa.CUDAGraphRunner(max_batch_size=4)
    assert runner.supported_batch_sizes == [1, 2, 4] and not runner.is_captured(3)
    assert runner.replay(3, torch.zeros(3, dtype=torch.long, device=gpu)) is None
    saved = graph.pool.kv_cache_tensor.clone()           # warm-up and capture run on the inert buffers
    for bs in (4, 2):
        runner.capture(step, bs, (bs,), hidden_size=512, device="cuda:0", slot_mapping=(bs,),
                       context_lens=(bs,), block_tables=(bs, W))
    assert torch.equal(graph.pool.kv_cache_tensor, saved)
    assert runner.is_captured(3) and runner.is_captured(2) and not runner.is_captured(1) and not runner.is_captured(5)
    for it in range(5):
        nxt = torch.randint(0, 512, (3,), generator=g).tolist()
        want = eager.decode(nxt)
        for s, t in zip(graph.seqs, nxt):
            s["token_ids"].append(int(t))
            graph._grow(s, len(s["token_ids"]))
        live = graph.seqs if it != 3 else graph.seqs[:2]            # once with a smaller batch: the 2-graph
        n = len(live)
        lens = torch.tensor([len(s["token_ids"]) for s in live], dtype=torch.int32, device=gpu)
        tables = torch.tensor([s["block_table"] + [-1] * (W - len(s["block_table"])) for s in live],
                              dtype=torch.int32, device=gpu)
        slots = pa.slot_mapping((lens - 1).long(), tables, 16, graph.pool.num_blocks)
        ids = torch.tensor([s["token_ids"][-1] for s in live], device=gpu)
        got = runner.replay(n, ids, (lens - 1).long(), slot_mapping=slots, context_lens=lens, block_tables=tables)
        if it == 3:                                                   # the third sequence's token is stored eagerly
            s = graph.seqs[2]
            one = torch.tensor([len(s["token_ids"])], dtype=torch.int32, device=gpu)
            t1 = torch.tensor([s["block_table"] + [-1] * (W - len(s["block_table"]))], dtype=torch.int32, device=gpu)
            step(torch.tensor([s["token_ids"][-1]], device=gpu), (one - 1).long(),
                 pa.slot_mapping((one - 1).long(), t1, 16, graph.pool.num_blocks), one, t1)
        torch.cuda.synchronize()
        torch.testing.assert_close(got.float().cpu(), want[:n].float().cpu(), rtol=2e-3, atol=2e-3)
        assert torch.equal(graph.pool.kv_cache_tensor, eager.pool.kv_cache_tensor), "a padding row wrote to the pool"
        _ = (want.float() @ want.float().t()).sum().item()             # eager work between replays
    st = runner.get_stats()
    assert sorted(st["captured_sizes"]) == [2, 4] and st["total_captures"] == 2 and st["total_replays"] == 5
    assert st["graph_pool_active"]
    runner.invalidate()
    assert not runner.is_captured(2) and runner.get_stats()["captured_sizes"] == []
    pa.reset_context()


def test_prepare_prefill_on_the_device_equals_the_reference_loops(pa, gpu):
    """ModelRunner.prepare_prefill on the GPU: one upload (ids, cumulative lengths, tables), positions and
    slots made by pa_prefill_metadata - every field equal to the reference's host loops."""
    import random
    from test_model_runner_host import random_sequences, as_list
    rng = random.Random(12)
    for bs in (8, 16):
        runner = pa.ModelRunner(None, pa.ModelRunnerConfig(block_size=bs, device="cuda:0"))
        for trial in range(6):
            seqs = random_sequences(rng, rng.randint(1, 9), bs, prefill=True)
            if trial == 5:
                for s in seqs:
                    s["num_cached_tokens"] = 0                         # no prefix anywhere: no tables in the context
                    s["num_scheduled_tokens"] = min(s["num_scheduled_tokens"], len(s["block_table"]) * bs)
            ids, pos = runner.prepare_prefill(seqs)
            ctx = pa.get_context()
            torch.cuda.synchronize()
            want = mro.prefill_metadata(seqs, bs)
            assert ids.is_cuda and ids.dtype == torch.long and pos.dtype == torch.long
            assert ids.tolist() == want["input_ids"] and pos.tolist() == want["positions"]
            assert ctx.is_prefill and as_list(ctx.slot_mapping) == want["slot_mapping"]
            assert as_list(ctx.cu_seqlens_q) == want["cu_seqlens_q"] and as_list(ctx.cu_seqlens_k) == want["cu_seqlens_k"]
            assert (ctx.max_seqlen_q, ctx.max_seqlen_k) == (want["max_seqlen_q"], want["max_seqlen_k"])
            assert as_list(ctx.block_tables) == want["block_tables"]
            for t in (ctx.slot_mapping, ctx.cu_seqlens_q, ctx.cu_seqlens_k, ctx.block_tables):
                assert t is None or (t.dtype == torch.int32 and t.is_cuda)
    # no tables at all: positions only
    runner.prepare_prefill([{"token_ids": [1, 2, 3], "num_cached_tokens": 0, "num_scheduled_tokens": 3}])
    ctx = pa.get_context()
    assert ctx.slot_mapping is None and ctx.block_tables is None
    pa.reset_context()


def test_prefill_chunks_take_their_tables_from_the_decode_state(pa, gpu):
    """Sequences reserve a DecodeState row before their first chunk: the block table goes to the device
    once, every chunk's slots come from that row, and the row joins the decode steps when the prompt is in."""
    bs, NB = 16, 400
    g = torch.Generator().manual_seed(43)
    free = torch.randperm(NB, generator=g).tolist()
    st = pa.DecodeState(6, 16, bs, NB, device=gpu)
    runner = pa.ModelRunner(None, pa.ModelRunnerConfig(block_size=bs, device="cuda:0"))
    st.admit([free.pop()], 5, 9)                                   # row 0 is taken by a decoding sequence
    seqs = []
    for total in (150, 40, 97):
        table = [free.pop() for _ in range((total + bs - 1) // bs)]
        row = st.reserve(table)
        seqs.append({"token_ids": [int(x) for x in torch.randint(0, 999, (total,), generator=g)], "block_table": table,
                     "state_row": row, "num_cached_tokens": 0, "num_scheduled_tokens": 0})
    assert [s["state_row"] for s in seqs] == [1, 2, 3] and st.rows_in_use == 1      # reserved rows do not decode yet
    chunk = 64
    while any(s["num_cached_tokens"] < len(s["token_ids"]) for s in seqs):
        batch = []
        for s in seqs:
            left = len(s["token_ids"]) - s["num_cached_tokens"]
            if left:
                s["num_scheduled_tokens"] = min(chunk, left)
                batch.append(s)
        ids, pos = runner.prepare_prefill(batch, state=st)
        ctx = pa.get_context()
        torch.cuda.synchronize()
        want = mro.prefill_metadata(batch, bs)
        assert ids.tolist() == want["input_ids"] and pos.tolist() == want["positions"]
        assert ctx.slot_mapping.tolist() == want["slot_mapping"]
        assert ctx.cu_seqlens_q.tolist() == want["cu_seqlens_q"] and ctx.cu_seqlens_k.tolist() == want["cu_seqlens_k"]
        if want["block_tables"] is None:
            assert ctx.block_tables is None
        else:                                                     # the state's rows: wider than the reference's, same entries
            got = ctx.block_tables.tolist()
            for g_row, w_row in zip(got, want["block_tables"]):
                real = [x for x in w_row if x >= 0]
                assert g_row[:len(real)] == real and all(x == -1 for x in g_row[len(real):])
        for s in batch:
            s["num_cached_tokens"] += s["num_scheduled_tokens"]
    for s in seqs:
        st.activate(s["state_row"], len(s["token_ids"]), 7)
    assert st.rows_in_use == 4
    st.step(None)
    torch.cuda.synchronize()
    assert st.context_lens.tolist()[:4] == [6, 151, 41, 98]
    want_slots = [s["block_table"][len(s["token_ids"]) // bs] * bs + len(s["token_ids"]) % bs if len(s["token_ids"]) % bs
                  else -1 for s in seqs]
    got_slots = st.slot_mapping.tolist()[1:4]
    for s, got_s, want_s in zip(seqs, got_slots, want_slots):
        if len(s["token_ids"]) % bs:
            assert got_s == want_s
    with pytest.raises(RuntimeError, match="not a reserved row"):
        st.activate(1, 10, 3)
    pa.reset_context()


def test_prepare_decode_on_the_device_equals_the_reference_loops(pa, gpu):
    """ModelRunner.prepare_decode on the GPU: the five fields go up side by side through a ring of pinned
    staging buffers as one copy - every field equal to the reference's host loops, over more steps
    than the ring has buffers, batches that grow past a buffer's size, and while earlier steps' tensors
    are still held (a later step must not overwrite what an earlier one handed out)."""
    import random
    from test_model_runner_host import random_sequences, as_list
    rng = random.Random(21)
    runner = pa.ModelRunner(None, pa.ModelRunnerConfig(block_size=16, device="cuda:0"))
    held = []
    for trial in range(11):
        n = rng.randint(1, 12) if trial < 8 else 300 * (trial - 7)        # then 300, 600, 900 rows
        seqs = random_sequences(rng, n, 16, prefill=False)
        if trial == 0:
            seqs[0]["last_block_num_tokens"] = 3
        ids, pos = runner.prepare_decode(seqs)
        ctx = pa.get_context()
        want = mro.decode_metadata(seqs, 16)
        held.append((ids, pos, ctx.slot_mapping, ctx.context_lens, ctx.block_tables, want))
        assert ids.is_cuda and ids.dtype == torch.long and pos.dtype == torch.long
        for t in (ctx.slot_mapping, ctx.context_lens, ctx.block_tables):
            assert t.dtype == torch.int32 and t.is_cuda and t.is_contiguous() and t.data_ptr() % 16 == 0
        assert ctx.longest_context_len == max(want["context_lens"])
    torch.cuda.synchronize()
    for ids, pos, slots, lens, tables, want in held:
        assert ids.tolist() == want["input_ids"] and pos.tolist() == want["positions"]
        assert as_list(slots) == want["slot_mapping"] and as_list(lens) == want["context_lens"]
        assert as_list(tables) == want["block_tables"]
    # The converted rows of a step are kept for the next one: whatever a caller does to a list between two
    # steps must show - a block appended, the last block replaced (copy-on-write), a block in the middle
    # replaced in place (same length, same first and last id), a list swapped for another, a tuple.
    seqs = [{"token_ids": [7] * (16 * 5 + 3), "block_table": [10 * i + j for j in range(6)]} for i in range(1, 7)]

    def check():
        runner.prepare_decode(seqs)
        ctx = pa.get_context()
        want = mro.decode_metadata(seqs, 16)
        assert as_list(ctx.block_tables) == want["block_tables"] and as_list(ctx.slot_mapping) == want["slot_mapping"]

    check()
    check()
    seqs[0]["block_table"].append(777)
    seqs[0]["token_ids"] += [7] * 16
    seqs[1]["block_table"][-1] = 888
    seqs[2]["block_table"][2] = 999
    seqs[3]["block_table"] = list(seqs[4]["block_table"])
    seqs[5]["block_table"] = tuple(seqs[5]["block_table"])
    check()
    seqs[2]["block_table"][2] = 22
    seqs.reverse()
    check()
    pa.reset_context()
