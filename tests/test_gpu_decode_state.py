"""Device-resident decode metadata (DecodeState, pa_decode_advance): the tensors it keeps on the
GPU equal, bit for bit, what the reference's prepare_decode builds on the host for the same
sequences (oracle/model_runner_oracle.py), and a decode loop driven by it - eagerly and through
graphs recorded over the state - produces the logits and the cache of the prepare_decode path."""
import random

import pytest
import torch

from oracle import model_runner_oracle as mro

pytestmark = pytest.mark.gpu


def test_state_equals_host_metadata_through_admits_steps_and_retires(pa, gpu):
    BS, NB, ROWS, WIDTH = 4, 400, 12, 24
    rng = random.Random(5)
    st = pa.DecodeState(ROWS, WIDTH, BS, NB, device=gpu)
    free = list(range(NB))
    rng.shuffle(free)
    seqs = {}                                   # row -> {"token_ids": [...], "block_table": [...]}
    next_tok = 1000

    def admit():
        nonlocal next_tok
        n = rng.randrange(1, 40)
        table = [free.pop() for _ in range((n + BS - 1) // BS)]
        row = st.admit(table, n, next_tok)
        assert row not in seqs and row == min(set(range(ROWS)) - set(seqs))      # lowest free row
        seqs[row] = {"token_ids": list(range(n)) + [next_tok], "block_table": list(table)}
        next_tok += 1

    for _ in range(5):
        admit()
    fresh = set(seqs)                            # rows that have not taken a step yet
    for step in range(60):
        toks = torch.zeros(ROWS, dtype=torch.long)      # what the previous step "sampled", by row
        for row, s in seqs.items():
            if row not in fresh:
                s["token_ids"].append(7000 + step * 16 + row)
                toks[row] = s["token_ids"][-1]
        need = st.rows_needing_block()
        want_need = [r for r, s in seqs.items() if (len(s["token_ids"]) - 1) % BS == 0
                     and (len(s["token_ids"]) - 1) // BS >= len(s["block_table"])]
        assert sorted(need) == sorted(want_need)
        grants = {}
        for r in need:
            grants[r] = free.pop()
            seqs[r]["block_table"].append(grants[r])
        st.step(grants or None, toks.to(gpu) if step % 3 else toks[:st.rows_in_use].to(gpu))
        fresh = set()
        rows = sorted(seqs)
        meta = mro.decode_metadata([seqs[r] for r in rows], BS)
        n = st.rows_in_use
        assert n == (max(rows) + 1 if rows else 0)
        lens, pos, slots, ids = (t.cpu().tolist() for t in (st.context_lens, st.positions, st.slot_mapping, st.input_ids))
        tables = st.block_tables.cpu()
        for i, r in enumerate(rows):
            assert (lens[r], pos[r], slots[r], ids[r]) == (meta["context_lens"][i], meta["positions"][i],
                                                           meta["slot_mapping"][i], meta["input_ids"][i])
            k = len(seqs[r]["block_table"])
            assert tables[r, :k].tolist() == seqs[r]["block_table"] and bool((tables[r, k:] == -1).all())
        for r in set(range(ROWS)) - set(rows):
            assert lens[r] == 0 and slots[r] == -1
        # churn: retire and admit between steps
        if rows and rng.random() < 0.25:
            r = rng.choice(rows)
            assert st.retire(r) == seqs[r]["block_table"]
            free.extend(seqs.pop(r)["block_table"])
        while len(seqs) < ROWS and rng.random() < 0.3:
            before = set(seqs)
            admit()                              # takes part from the next step on, feeding its own next_token
            fresh |= set(seqs) - before
    with pytest.raises(RuntimeError, match="need a new block"):
        for _ in range(BS + 1):
            st.step(None)


def test_state_errors(pa, gpu):
    st = pa.DecodeState(2, 4, 16, 100, device=gpu)
    with pytest.raises(RuntimeError, match="at least one cached token"):
        st.admit([1], 0, 5)
    with pytest.raises(RuntimeError, match="does not fit"):
        st.admit([1, 2, 3, 4, 5], 70, 5)
    with pytest.raises(RuntimeError, match="does not fit"):
        st.admit([1], 17, 5)
    st.admit([1], 3, 5)
    st.admit([2], 3, 5)
    with pytest.raises(RuntimeError, match="rows are in use"):
        st.admit([3], 3, 5)
    with pytest.raises(RuntimeError, match="next_tokens"):
        st.step(None, torch.zeros(2, dtype=torch.long))            # a CPU tensor


def test_c_abi_decode_advance_errors(lib, gpu):
    bt = torch.full((4, 8), -1, dtype=torch.int32, device=gpu)
    lens = torch.tensor([5, 0, 16, 127], dtype=torch.int32, device=gpu)
    bt[0, 0], bt[2, 1], bt[3, 7] = 3, 9, 2
    pos = torch.zeros(4, dtype=torch.long, device=gpu)
    slots = torch.zeros(4, dtype=torch.int32, device=gpu)
    f = lib.pa_decode_advance
    ids = torch.tensor([11, 12, 13, 14], device=gpu)
    nxt = torch.tensor([21, 22, 23, 24], device=gpu)
    fresh = torch.tensor([0, 0, 1, 0], dtype=torch.int32, device=gpu)
    assert f(bt.data_ptr(), 8, lens.data_ptr(), pos.data_ptr(), slots.data_ptr(), None, ids.data_ptr(), nxt.data_ptr(),
             fresh.data_ptr(), 4, 8, 16, 100, None) == 0
    torch.cuda.synchronize()
    assert ids.tolist() == [21, 12, 13, 24] and fresh.tolist() == [0, 0, 0, 0]     # inactive and fresh rows keep theirs
    assert lens.tolist() == [6, 0, 17, 128] and pos.tolist() == [5, 0, 16, 127]
    assert slots.tolist() == [3 * 16 + 5, -1, 9 * 16, 2 * 16 + 15]
    # the next token of row 3 lies past the table: no slot, the row still advances
    assert f(bt.data_ptr(), 8, lens.data_ptr(), pos.data_ptr(), slots.data_ptr(), None, None, None, None, 4, 8, 16, 100, None) == 0
    torch.cuda.synchronize()
    assert slots.tolist()[3] == -1 and lens.tolist()[3] == 129
    assert f(None, 8, lens.data_ptr(), pos.data_ptr(), slots.data_ptr(), None, None, None, None, 4, 8, 16, 100, None) != 0
    assert f(bt.data_ptr(), 4, lens.data_ptr(), pos.data_ptr(), slots.data_ptr(), None, None, None, None, 4, 8, 16, 100, None) != 0
    assert f(bt.data_ptr(), 8, lens.data_ptr(), pos.data_ptr(), slots.data_ptr(), None, None, None, None, 4, 8, 0, 100, None) != 0
    assert f(bt.data_ptr(), 8, lens.data_ptr(), pos.data_ptr(), slots.data_ptr(), None, None, None, None, 0, 8, 16, 100, None) == 0
    assert f(bt.data_ptr(), 8, lens.data_ptr(), pos.data_ptr(), slots.data_ptr(), None, None, nxt.data_ptr(), None,
             4, 8, 16, 100, None) != 0                                  # next_tokens without input_ids
    assert b"pa_decode_advance" in lib.pa_last_error()


@pytest.mark.parametrize("graphs", [False, True])
def test_decode_loop_over_the_state_equals_the_prepare_decode_path(pa, gpu, graphs):
    from test_gpu_model import Session, small_model
    model = small_model(pa, seed=17)
    ref = Session(pa, model, gpu)                     # host lists every step
    dev = Session(pa, model, gpu, graphs=None)        # device-resident state
    dev.runner.config.enable_cuda_graph = graphs
    g = torch.Generator().manual_seed(18)
    prompts = [torch.randint(0, 512, (n,), generator=g).tolist() for n in (9, 40, 17, 31)]
    for p in prompts:
        ref.add(p)
        dev.add(p)
    first_ref = ref.prefill()[0].argmax(-1).tolist()
    first_dev = dev.prefill()[0].argmax(-1)
    assert first_dev.tolist() == first_ref
    st = pa.DecodeState(8, 16, 16, dev.pool.num_blocks, device=gpu)
    rows = [st.admit(s["block_table"], len(s["token_ids"]), t) for s, t in zip(dev.seqs, first_ref)]
    assert rows == [0, 1, 2, 3]
    if graphs:
        dev.runner.capture_decode_state_graphs(st, [4, 8])
        assert torch.equal(dev.pool.kv_cache_tensor, ref.pool.kv_cache_tensor)     # capture wrote nothing
    toks = first_ref
    next_dev = None
    for step in range(20):
        want = ref.decode(toks)                                         # appends toks, runs the step
        grants = {}
        for r in st.rows_needing_block():
            dev.seqs[r]["block_table"].append(dev.free.pop())
            grants[r] = dev.seqs[r]["block_table"][-1]
        st.step(grants or None, next_dev)
        got = dev.runner.run_decode_state(st)
        torch.testing.assert_close(got.float().cpu(), want.float().cpu(), rtol=2e-3, atol=2e-3)
        next_dev = pa.sample_tokens(got, temperature=0.0)               # greedy, stays on the device
        toks = want.argmax(-1).tolist()
        assert next_dev.tolist() == toks
        if step == 9:                                                   # one sequence leaves mid-run
            torch.cuda.synchronize()
            assert torch.equal(dev.pool.kv_cache_tensor, ref.pool.kv_cache_tensor)
        _ = (want.float() @ want.float().t()).sum().item()              # eager work between replays
    torch.cuda.synchronize()
    assert torch.equal(dev.pool.kv_cache_tensor, ref.pool.kv_cache_tensor)
    assert [st.num_tokens(r) for r in rows] == [len(s["token_ids"]) for s in ref.seqs]
    pa.reset_context()


def test_graphs_per_context_bucket_follow_the_rows(pa, gpu):
    """Tables far wider than the rows: graphs are recorded per context bucket (and, where the launch
    policy splits ragged batches differently, per flavour), each step replays the smallest bucket that
    holds the longest row, and the logits are those of the prepare_decode path whichever graph ran."""
    from test_gpu_model import Session, small_model
    model = small_model(pa, seed=19)
    ref = Session(pa, model, gpu, num_blocks=160)
    dev = Session(pa, model, gpu, num_blocks=160, graphs=None)
    dev.runner.config.enable_cuda_graph = True
    g = torch.Generator().manual_seed(20)
    prompts = [torch.randint(0, 512, (n,), generator=g).tolist() for n in (9, 700, 17, 300)]
    for p in prompts:
        ref.add(p)
        dev.add(p)
    first = ref.prefill()[0].argmax(-1).tolist()
    assert dev.prefill()[0].argmax(-1).tolist() == first
    st = pa.DecodeState(8, 128, 16, dev.pool.num_blocks, device=gpu)            # tables of 2048 tokens
    rows = [st.admit(s["block_table"], len(s["token_ids"]), t) for s, t in zip(dev.seqs, first)]
    # at the benchmark shape a ragged batch of 64 rows is split where a full one is read in one pass (256
    # rows are read in one pass either way); the test asks for the second graph of one bucket itself
    big = pa.ModelRunner(None, pa.ModelRunnerConfig(num_heads=16, num_kv_heads=8, head_dim=128))
    assert big._ragged_launch_differs(64, 4096) and not big._ragged_launch_differs(256, 1024)
    dev.runner._ragged_launch_differs = lambda bs, bucket: bucket == 710
    dev.runner.capture_decode_state_graphs(st, [4, 8], context_buckets=[256, 710, 1024])
    assert dev.runner._state_buckets[id(st)] == [256, 710, 1024, 2048]
    recorded = {(bs, bk, rg) for (_, bs, ps, bk, rg) in dev.runner._state_graphs}
    assert {(4, 256, False), (4, 710, False), (4, 1024, False), (4, 2048, False), (8, 2048, False)} <= recorded
    assert {(4, 710, True), (8, 710, True)} == {x for x in recorded if x[2]}
    assert torch.equal(dev.pool.kv_cache_tensor, ref.pool.kv_cache_tensor)     # capture wrote nothing
    seen = []
    real_for = dev.runner._state_graph_for

    def spy(state, n, want, longest=0, mean=0.0):
        hit = real_for(state, n, want, longest, mean)
        bucket = next(b for b in dev.runner._state_buckets[id(state)] if b >= longest)
        seen.append((bucket, hit[2]))
        return hit
    dev.runner._state_graph_for = spy
    toks, next_dev, live = first, None, list(rows)
    for step in range(24):
        if step == 16:                      # the long row leaves: the batch fits a smaller bucket again
            st.retire(1)
            live.remove(1)
        want = ref.decode(toks)
        grants = {}
        for r in st.rows_needing_block():
            dev.seqs[r]["block_table"].append(dev.free.pop())
            grants[r] = dev.seqs[r]["block_table"][-1]
        st.step(grants or None, next_dev)
        assert st.known_lengths()[0] == max(len(ref.seqs[r]["token_ids"]) for r in live)
        got = dev.runner.run_decode_state(st)
        torch.testing.assert_close(got[live].float().cpu(), want[live].float().cpu(), rtol=2e-3, atol=2e-3)
        next_dev = pa.sample_tokens(got, temperature=0.0)
        toks = want.argmax(-1).tolist()
        assert [next_dev.tolist()[r] for r in live] == [toks[r] for r in live]
        _ = (want.float() @ want.float().t()).sum().item()              # eager work between replays
    buckets = [b for b, _ in seen]
    assert buckets[0] == 710 and 1024 in buckets and buckets[-1] == 710 and 2048 not in buckets and 256 not in buckets
    assert buckets.index(1024) == 710 - 701 + 1                          # the step whose longest row reaches 711 tokens
    stats = dev.runner.decode_state_stats
    assert stats["eager"] == 0 and stats["plain_graph"] + stats["ragged_graph"] == 24
    assert stats["ragged_graph"] == sum(1 for _, rg in seen if rg) > 0   # rows of 10 ... 700 tokens: ragged
    pa.reset_context()


def test_state_keeps_prefix_groups_through_admits_and_retires(pa, gpu):
    """Host side of the group bookkeeping: rebuilt when a row is admitted or retired, never by a step; the
    device descriptors hold what the host list says."""
    BS = 16
    st = pa.DecodeState(8, 32, BS, 1000, device=gpu, num_q_heads=16, num_kv_heads=8, prefix_partition_sizes=(256, 64))
    assert st.tracks_prefixes and st.prefix_partition_sizes == (256, 64) and st.max_group_rows == 8
    prompt_a = list(range(100, 117))                      # 17 blocks = 272 tokens
    prompt_b = list(range(300, 305))                      # 5 blocks = 80 tokens
    st.admit(prompt_a + [1], 280, 7)
    st.admit(prompt_b + [2], 82, 7)
    st.admit(prompt_a + [3], 275, 7)
    st.admit([900, 901], 20, 7)
    st.sync_prefix_groups()
    # prompt a shares one partition of 256 (or four of 64: no more tokens), prompt b has one row only
    assert st.prefix_groups_host == [([0, 2], 256)] and st.prefix_partition_size == 256
    st.admit(prompt_b + [4], 85, 7)                       # row 4: b's second sample shares 64 tokens
    st.sync_prefix_groups()
    # 64-token partitions now save 256 + 64 tokens of reads against 256 with the coarse size: the finer size wins
    assert st.prefix_partition_size == 64 and st.prefix_groups_host == [([0, 2], 256), ([1, 4], 64)]
    pg = st.prefix_groups(5)
    assert (pg.num_groups, pg.max_group_rows, pg.max_shared_partitions, pg.partition_size) == (2, 2, 4, 64)
    torch.cuda.synchronize()
    assert pg.group_desc[:2].tolist() == [[0, 2, 4, 0], [2, 2, 1, 0]] and int(pg.group_desc[2:].abs().sum()) == 0
    assert pg.group_rows[:4].tolist() == [0, 2, 1, 4] and pg.row_skip.tolist() == [4, 1, 4, 0, 1]
    for _ in range(3):                                    # steps change nothing
        st.step(None)
        assert not st._groups_dirty and st.prefix_groups_host == [([0, 2], 256), ([1, 4], 64)]
    st.retire(0)
    assert st.prefix_groups(5).groups == [([1, 4], 64)]
    torch.cuda.synchronize()
    assert st._row_skip.tolist()[:5] == [0, 1, 0, 0, 1]
    st.retire(4)
    assert st.prefix_groups(5) is None and st.prefix_partition_size is None
    torch.cuda.synchronize()
    assert int(st._groups_dev.abs().sum()) == 0          # nothing on the device names a row any more
    # the capacity view a graph is recorded over
    cap = st.prefix_groups(8, 256, for_graph=True)
    assert (cap.num_groups, cap.max_group_rows, cap.max_shared_partitions, cap.partition_size) == (4, 8, 2, 256)
    # a state that was not told the head layout keeps no groups
    assert pa.DecodeState(4, 8, BS, 100, device=gpu).prefix_groups(4) is None


@pytest.mark.parametrize("graphs", [False, True])
def test_forked_samples_decode_through_shared_prefix_groups(pa, gpu, graphs):
    """Samples forked from prefilled prompts (KVCacheManager.fork_sequence, copy-on-write of the shared last
    block), interleaved rows, a retirement and a late fork: the decode loop over DecodeState takes the
    shared-prefix launch (recorded in a graph or eager) whenever the state holds a group, and its logits
    equal those of the same sequences decoded from private, unshared blocks through prepare_decode."""
    from test_gpu_model import Session, small_model
    BS = 16
    model = small_model(pa, seed=23)                  # 4 query / 2 KV heads: up to 8 rows per group
    ref = Session(pa, model, gpu, num_blocks=128)     # every sequence owns all its blocks
    ref.runner.config.share_prefix_decode = False
    dev = Session(pa, model, gpu, num_blocks=128, graphs=None)
    dev.runner.config.enable_cuda_graph = graphs
    mgr = pa.KVCacheManager(dev.pool, BS)
    g = torch.Generator().manual_seed(24)
    prompts = {"a": torch.randint(0, 512, (70,), generator=g).tolist(),     # 4 full blocks + 6 tokens
               "b": torch.randint(0, 512, (40,), generator=g).tolist(),     # 2 full blocks + 8 tokens
               "c": torch.randint(0, 512, (50,), generator=g).tolist()}
    # prefill each prompt once on the device path, from the manager's blocks
    first = {}
    for name, toks in prompts.items():
        table = mgr.allocate_for_sequence((name, 0), len(toks)).get_physical_block_ids()
        ids, pos = dev.runner.prepare_prefill([{"token_ids": toks, "block_table": table, "num_cached_tokens": 0,
                                                "num_scheduled_tokens": len(toks)}])
        first[name] = int(dev.runner.run(ids, pos, is_prefill=True)[-1].argmax())
    order = [("a", 0), ("b", 0), ("a", 1), ("c", 0), ("a", 2), ("b", 1), ("a", 3)]     # samples interleaved
    for name, s in order:
        if s:
            mgr.fork_sequence((name, 0), (name, s))
    st = pa.DecodeState(8, 8, BS, dev.pool.num_blocks, device=gpu, num_q_heads=4, num_kv_heads=2,
                        prefix_partition_sizes=(64, 32))
    seq_of_row, ref_of_row, tokens = {}, {}, {}
    for name, s in order:
        tok = (first[name] + 17 * s) % 512                               # the samples diverge at once
        row = st.admit(mgr.get_block_table((name, s)), len(prompts[name]), tok)
        seq_of_row[row], tokens[row] = (name, s), tok
        ref.add(prompts[name])
        ref_of_row[row] = len(ref.seqs) - 1
    ref.prefill()
    st.sync_prefix_groups()
    assert st.prefix_groups_host == [([0, 2, 4, 6], 64), ([1, 5], 32)] and st.prefix_partition_size == 32
    if graphs:
        dev.runner.capture_decode_state_graphs(st, [8])
    next_dev = None
    for step in range(24):
        if step == 8:                      # a sample of prompt a leaves: its group shrinks
            mgr.free_sequence(seq_of_row[2])
            st.retire(2)
            del seq_of_row[2]
        if step == 12:                     # a late fork of b's first sample (generated tokens included) takes the free row
            parent_row = next(r for r, sq in seq_of_row.items() if sq == ("b", 0))
            mgr.fork_sequence(("b", 0), ("b", 9))
            history = ref.seqs[ref_of_row[parent_row]]["token_ids"]
            row = st.admit(mgr.get_block_table(("b", 9)), len(history), 5)
            assert row == 2
            seq_of_row[2], tokens[2] = ("b", 9), 5
            ref.add(list(history))
            ref.prefill()
            ref_of_row[2] = len(ref.seqs) - 1
            st.sync_prefix_groups()
            assert ([1, 2, 5], 32) in st.prefix_groups_host
        # the manager makes room for every row's new token: a new block, or a private copy of a shared last block
        grants = {}
        for row, sq in seq_of_row.items():
            before = mgr.get_block_table(sq)
            assert mgr.append_token(sq)
            after = mgr.get_block_table(sq)
            if len(after) > len(before) or after[-1] != before[-1]:
                grants[row] = after[-1]
        mgr.apply_copies()
        st.step(grants or None, next_dev)
        got = dev.runner.run_decode_state(st)
        # the same step on private blocks
        ref_tokens = [0] * len(ref.seqs)
        for row, tok in tokens.items():
            ref_tokens[ref_of_row[row]] = tok
        want = ref.decode(ref_tokens)
        for row in seq_of_row:
            torch.testing.assert_close(got[row].float().cpu(), want[ref_of_row[row]].float().cpu(), rtol=2e-3, atol=2e-3)
        next_dev = pa.sample_tokens(got, temperature=0.0)
        picked = next_dev.tolist()
        for row in seq_of_row:
            tokens[row] = picked[row]
    stats = dev.runner.decode_state_stats
    if graphs:
        assert stats["shared_prefix_graph"] == 24 and stats["plain_graph"] == 0 and stats["eager"] == 0
    else:
        assert stats["eager"] == 24
    # without the last group the plain graph takes over
    for row, sq in list(seq_of_row.items()):
        if sq[0] in ("a", "b") and row != 0:
            st.retire(row)
    st.sync_prefix_groups()
    assert st.prefix_partition_size is None
    st.step(None, next_dev)
    dev.runner.run_decode_state(st)
    assert stats["plain_graph" if graphs else "eager"] == (1 if graphs else 25)
    pa.reset_context()
