"""The pieces together, the way the reference's engine drives them (src/inference/engine.py:582-616,
1100-1130, 1540-1560): requests arrive with a shared system prompt, the radix cache aliases its
blocks, only the tails are prefilled, K samples of one prompt fork and copy on write, the running
batch lives in a DecodeState and steps through graph replays, sequences finish and free their
rows and blocks while others are admitted.  Every request's greedy continuation must equal the one
the same model produces for that request alone, with private blocks and host-built metadata."""
import pytest
import torch

pytestmark = pytest.mark.gpu


def test_continuous_batch_with_prefix_reuse_forks_and_graph_steps(pa, gpu):
    from test_gpu_model import Session, small_model
    BS = 16
    model = small_model(pa, seed=23)
    g = torch.Generator().manual_seed(24)
    system = torch.randint(0, 512, (3 * BS,), generator=g).tolist()
    tails = [torch.randint(0, 512, (n,), generator=g).tolist() for n in (5, 21, 40, 9, 33)]
    requests = [{"prompt": system + t, "new": n} for t, n in zip(tails, (14, 6, 25, 11, 18))]
    requests.append({"prompt": requests[0]["prompt"], "new": 9, "fork_of": 0})       # second sample of request 0

    # ---- each request alone: private blocks, prepare_decode every step ----------------------------
    want = []
    for req in requests:
        solo = Session(pa, model, gpu)
        solo.add(req["prompt"])
        tok = int(solo.prefill()[0].argmax(-1)[0])
        out = [tok]
        for _ in range(req["new"] - 1):
            tok = int(solo.decode([tok]).argmax(-1)[0])
            out.append(tok)
        want.append(out)

    # ---- the shared engine --------------------------------------------------------------------------
    sess = Session(pa, model, gpu, num_blocks=96)          # model, pool and runner; its own lists are unused
    pool, runner = sess.pool, sess.runner
    runner.config.enable_cuda_graph = True
    mgr = pa.KVCacheManager(pool, BS)
    cache = pa.RadixAttentionCache(BS, 64, block_pool=pool)
    state = pa.DecodeState(4, 16, BS, pool.num_blocks, device=gpu)
    runner.capture_decode_state_graphs(state, [2, 4])
    running = {}                                           # row -> {"id", "out", "left"}
    waiting = [0, 5, 1, 2, 3, 4]                          # the second sample of request 0 forks right after its prefill
    got = {}
    next_tokens = None
    hits = []
    steps = 0
    while waiting or running:
        # admit while rows are free; a fork waits until its parent has been prefilled and is still running
        for rid in list(waiting):
            if len(running) == state.max_batch:
                break
            req = requests[rid]
            if "fork_of" in req:
                parent_row = next((r for r, s in running.items() if s["id"] == req["fork_of"]), None)
                assert parent_row is not None and len(running[parent_row]["out"]) == 1
                mgr.fork_sequence(req["fork_of"], rid)
                table = mgr.get_block_table(rid)
                first = running[parent_row]["out"][0]
                hits.append(("fork", len(table)))
            else:
                prompt = req["prompt"]
                matched, ids = cache.match_prefix(prompt)
                keep = min(matched, (len(prompt) - 1) // BS * BS) // BS          # at least one token to compute
                matched, ids = keep * BS, ids[:keep]
                table = mgr.allocate_for_sequence(rid, len(prompt), shared_block_ids=ids).get_physical_block_ids()
                tok_ids, pos = runner.prepare_prefill([{"token_ids": prompt, "block_table": table,
                                                        "num_cached_tokens": matched,
                                                        "num_scheduled_tokens": len(prompt) - matched}])
                first = int(runner.run(tok_ids, pos, is_prefill=True).argmax(-1)[0])
                cache.insert(prompt, table)
                cache.release_prefix(prompt)
                hits.append(("prefix", matched))
            row = state.admit(table, len(req["prompt"]), first)
            running[row] = {"id": rid, "out": [first], "left": req["new"] - 1}
            waiting.remove(rid)
        # retire what is done before stepping
        for row in [r for r, s in running.items() if s["left"] == 0]:
            s = running.pop(row)
            got[s["id"]] = s["out"]
            state.retire(row)
            mgr.free_sequence(s["id"])
        if not running:
            assert not waiting, "nothing runs and nothing can be admitted"
            continue
        grants = {}
        for row, s in running.items():
            before = mgr.get_block_table(s["id"])
            assert mgr.append_token(s["id"])
            after = mgr.get_block_table(s["id"])
            if after != before:                            # a new block, or a private copy of a shared one
                grants[row] = after[-1]
        mgr.apply_copies()
        state.step(grants or None, next_tokens)
        logits = runner.run_decode_state(state)
        next_tokens = pa.sample_tokens(logits, temperature=0.0)
        toks = next_tokens.tolist()
        for row, s in running.items():
            s["out"].append(toks[row])
            s["left"] -= 1
        steps += 1
        assert steps < 200
    assert hits[0] == ("prefix", 0) and all(h == ("prefix", 3 * BS) for h in hits[1:] if h[0] == "prefix")
    assert ("fork", (len(requests[0]["prompt"]) + BS - 1) // BS) in hits
    for rid, req in enumerate(requests):
        assert got[rid] == want[rid], "request %d" % rid
    assert pool.num_used_blocks == cache.size              # only the cache holds blocks now
    cache.invalidate_all()
    assert pool.num_free_blocks == pool.num_blocks
    pa.reset_context()
