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
