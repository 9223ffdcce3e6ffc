"""Decode over batches whose rows share prefixes as the same physical blocks (the fourth benchmark
configuration: n samples per prompt): partitions inside a group's shared prefix are computed once
per group.  The result must be the partitioned decode's, i.e. the oracle's within the path's
tolerances (rtol 1e-3 / atol 2e-3 for 16-bit caches, 1e-2 / 1e-2 for fp8)."""
import pytest
import torch

import cases
from test_gpu_decode import TOL, check, oracle_decode

pytestmark = pytest.mark.gpu


def host_tables(c):
    """Per-row lists of block ids, as the cache manager holds them on the host."""
    bs = c["k_cache"].shape[1]
    rows = []
    for b, n in enumerate(c["context_lens"].tolist()):
        rows.append(c["block_tables"][b, :(n + bs - 1) // bs].tolist())
    return rows


def shared_decode(pa, c, gpu, groups, **kw):
    d = cases.to_device(c, gpu)
    out = pa.paged_decode_shared_prefix(d["q"], d["k_cache"], d["v_cache"], d["block_tables"], d["context_lens"],
                                        d["scale"], groups, d["k_scale"], d["v_scale"], **kw)
    torch.cuda.synchronize()
    return out.cpu()


@pytest.mark.parametrize("cache", ["fp16", "fp8", "bf16"])
@pytest.mark.parametrize("hq,hkv", [(16, 8), (8, 8), (32, 8), (6, 2)])
def test_samples_of_a_prompt_share_its_prefix(pa, gpu, cache, hq, hkv):
    group = 16 // (hq // hkv)                      # as many samples per prompt as one group can hold
    prompts = 3
    lens = [560 + 13 * i + (i % group) * 5 for i in range(prompts * group)]
    pool = sum((n + 15) // 16 - (32 if i % group else 0) for i, n in enumerate(lens)) + 16
    c = cases.make_case(400 + hq, lens, pool, num_heads=hq, num_kv_heads=hkv, cache=cache,
                        q_dtype=torch.bfloat16 if cache == "bf16" else torch.float16, shared_prefix=(group, 32))
    groups = pa.find_prefix_groups(host_tables(c), lens, 16, hq, hkv, 128)
    assert groups == [(i * group, group, 512) for i in range(prompts)]
    want = oracle_decode(c)
    got = shared_decode(pa, c, gpu, groups, partition_size=128)
    check(got, want, cache)
    # the same launch shape without sharing
    plain = shared_decode(pa, c, gpu, [], partition_size=128)
    check(plain, want, cache)
    torch.testing.assert_close(got.float(), plain.float(), rtol=1e-3, atol=1e-3)


def test_ragged_groups_loners_and_partial_partitions(pa, gpu):
    """Groups of 2, 3 and 8 rows with different shared lengths, rows of no group between them, a shared
    length that is not a whole number of partitions (the remainder is computed per row)."""
    lens = [900, 950, 300, 700, 710, 720, 50, 1300, 1290, 1280, 1270, 1260, 1250, 1240, 1230, 17]
    c = cases.make_case(77, lens, 1000, shared_prefix=None)
    # alias leading blocks by hand: rows 0-1 share 50 blocks, rows 3-5 share 21, rows 7-14 share 70
    tb = c["block_tables"]
    for first, rows, blocks in ((0, 2, 50), (3, 3, 21), (7, 8, 70)):
        for m in range(1, rows):
            tb[first + m, :blocks] = tb[first, :blocks]
    # the aliased rows now read the leader's blocks: the oracle follows the tables, so it stays the reference
    want = oracle_decode(c)
    groups = pa.find_prefix_groups(host_tables(c), lens, 16, 16, 8, 256)
    assert groups == [(0, 2, 768), (3, 3, 256), (7, 8, 1024)]
    check(shared_decode(pa, c, gpu, groups, partition_size=256), want, "fp16")
    # finer partitions, 8 waves
    groups64 = pa.find_prefix_groups(host_tables(c), lens, 16, 16, 8, 64)
    assert groups64 == [(0, 2, 768), (3, 3, 320), (7, 8, 1088)]
    check(shared_decode(pa, c, gpu, groups64, partition_size=64, waves=8), want, "fp16")


@pytest.mark.parametrize("cache", ["fp16", "fp8"])
def test_fourth_benchmark_configuration_at_full_size(pa, gpu, cache):
    """32 prompts x 8 samples = 256 rows, 1024 shared tokens per prompt, private suffixes U[64, 512]: the
    shared-prefix launch on the whole batch, groups and partition size from the finder, against the
    oracle - and the same rows shuffled, so that no group's rows are neighbours."""
    c = cases.config4(cache=cache)
    lens = c["context_lens"].tolist()
    tables = host_tables(c)
    pg = pa.prepare_prefix_groups(tables, lens, 16, 16, 8, gpu)
    assert pg.partition_size == 1024 and pg.groups == [(list(range(8 * i, 8 * i + 8)), 1024) for i in range(32)]
    assert pg.group_rows is None
    want = oracle_decode(c)
    d = cases.to_device(c, gpu)
    got = pa.paged_decode_shared_prefix(d["q"], d["k_cache"], d["v_cache"], d["block_tables"], d["context_lens"],
                                        d["scale"], None, d["k_scale"], d["v_scale"], descriptors=pg)
    torch.cuda.synchronize()
    check(got.cpu(), want, cache)
    # finer partitions (more of them shared: 4 x 256 per prompt)
    check(shared_decode(pa, c, gpu, pa.find_prefix_groups(tables, lens, 16, 16, 8, 256), partition_size=256), want, cache)
    # the rows in a random order: groups are lists of rows
    perm = torch.randperm(256, generator=torch.Generator().manual_seed(4)).tolist()
    far = pa.prepare_prefix_groups([tables[i] for i in perm], [lens[i] for i in perm], 16, 16, 8, gpu, anywhere=True)
    assert far.partition_size == 1024 and far.num_groups == 32 and far.group_rows is not None
    inv = {old: new for new, old in enumerate(perm)}
    assert sorted(far.groups) == sorted((sorted(inv[r] for r in range(8 * i, 8 * i + 8)), 1024) for i in range(32))
    idx = torch.tensor(perm, device=gpu)
    got = pa.paged_decode_shared_prefix(d["q"][idx].contiguous(), d["k_cache"], d["v_cache"],
                                        d["block_tables"][idx].contiguous(), d["context_lens"][idx].contiguous(),
                                        d["scale"], None, d["k_scale"], d["v_scale"], descriptors=far)
    torch.cuda.synchronize()
    check(got.cpu(), want[perm], cache)


@pytest.mark.parametrize("hq,hkv", [(16, 8), (32, 8)])
@pytest.mark.parametrize("cache", ["fp16", "fp8"])
def test_groups_of_rows_anywhere_in_the_batch(pa, gpu, cache, hq, hkv):
    """Samples of three prompts interleaved with each other and with rows of their own; padding groups of no
    partitions between the real ones (what a recorded launch at full capacity holds)."""
    group = 16 // (hq // hkv)
    lens = [300 + 7 * i for i in range(3 * group)] + [90, 500]
    pool = sum((n + 15) // 16 for n in lens) + 16
    c = cases.make_case(900 + hq, lens, pool, num_heads=hq, num_kv_heads=hkv, cache=cache, shared_prefix=None)
    tb = c["block_tables"]
    for p_ in range(3):
        for m in range(1, group):
            tb[p_ * group + m, :16] = tb[p_ * group, :16]            # 256 shared tokens per prompt
    order = torch.randperm(len(lens), generator=torch.Generator().manual_seed(hq)).tolist()
    for key in ("q", "block_tables", "context_lens"):
        c[key] = c[key][order].contiguous()
    lens = c["context_lens"].tolist()
    want = oracle_decode(c)
    groups = pa.find_prefix_groups_anywhere(host_tables(c), lens, 16, hq, hkv, 128)
    assert len(groups) == 3 and all(len(rows) == group and tokens == 256 for rows, tokens in groups)
    assert any(rows != list(range(rows[0], rows[0] + group)) for rows, _ in groups)
    check(shared_decode(pa, c, gpu, groups, partition_size=128), want, cache)
    # the descriptors a recorded graph uses: more groups than there are, the spare ones empty
    pg = pa.shared_prefix_descriptors(groups, len(lens), gpu, 128)
    desc = torch.zeros(8, 4, dtype=torch.int32, device=gpu)
    desc[1], desc[4], desc[6] = pg.group_desc[0], pg.group_desc[1], pg.group_desc[2]
    padded = pa.PrefixGroups(128, desc, pg.group_rows, pg.row_skip, 8, group, 5, 0)
    d = cases.to_device(c, gpu)
    got = pa.paged_decode_shared_prefix(d["q"], d["k_cache"], d["v_cache"], d["block_tables"], d["context_lens"],
                                        d["scale"], None, d["k_scale"], d["v_scale"], descriptors=padded)
    torch.cuda.synchronize()
    check(got.cpu(), want, cache)


def test_corrupt_descriptors_do_not_fault(pa, gpu, monkeypatch):
    """Everything the kernel reads from the descriptors is clamped before it indexes anything: rows outside
    the batch, more rows than the operand holds, a row list index past the list, negative skips.  The launch
    must come back (with wrong numbers for the rows involved), and the checker must name the damage."""
    lens = [600, 610, 620, 630, 300]
    c = cases.make_case(6, lens, 220, shared_prefix=(4, 32))
    d = cases.to_device(c, gpu)
    good = pa.shared_prefix_descriptors([([0, 1, 2, 3], 512)], 5, gpu, 128)
    want = oracle_decode(c)
    for damage in ("rows", "row_index", "first", "skip"):
        desc, rows, skip = good.group_desc.clone(), good.group_rows, good.row_skip.clone()
        rows = torch.tensor([0, 1, 2, 3, 0], dtype=torch.int32, device=gpu)
        desc[0, 0] = 0
        if damage == "rows":
            desc[0, 1] = 4000
        elif damage == "row_index":
            rows[2] = 70000
        elif damage == "first":
            desc[0, 0] = 123456
        else:
            skip[4] = -7
        bad = pa.PrefixGroups(128, desc, rows, skip, 1, 4, 4, 0)
        out = pa.paged_decode_shared_prefix(d["q"], d["k_cache"], d["v_cache"], d["block_tables"], d["context_lens"],
                                            d["scale"], None, descriptors=bad)
        torch.cuda.synchronize()
        assert out.shape == d["q"].shape
        if damage == "skip":
            check(out.cpu(), want, "fp16")           # a negative skip is read as no skip: still the right answer
        if damage in ("rows", "row_index", "first"):
            monkeypatch.setenv("PA_DEBUG_TABLES", "1")
            with pytest.raises(RuntimeError, match="shared table entries differ|rows too short|outside the groups"):
                pa.paged_decode_shared_prefix(d["q"], d["k_cache"], d["v_cache"], d["block_tables"], d["context_lens"],
                                              d["scale"], None, descriptors=bad)
            monkeypatch.delenv("PA_DEBUG_TABLES")


def test_descriptor_check_and_refusals(pa, gpu, monkeypatch):
    lens = [600, 610, 620, 630]
    c = cases.make_case(5, lens, 200, shared_prefix=(4, 32))
    d = cases.to_device(c, gpu)
    good = [(0, 4, 512)]
    monkeypatch.setenv("PA_DEBUG_TABLES", "1")
    shared_decode(pa, c, gpu, good, partition_size=128)                      # passes the check
    with pytest.raises(RuntimeError, match="shared table entries differ"):   # claims more than is shared
        shared_decode(pa, c, gpu, [(0, 4, 576)], partition_size=64)
    monkeypatch.delenv("PA_DEBUG_TABLES")
    # more rows per group than the operand has columns for
    with pytest.raises(RuntimeError, match="must not exceed 16"):
        pa.paged_decode_shared_prefix(d["q"].repeat(1, 4, 1).contiguous(), d["k_cache"], d["v_cache"], d["block_tables"],
                                      d["context_lens"], d["scale"], [(0, 4, 512)], partition_size=128)
    with pytest.raises(RuntimeError, match="reaches outside the batch"):
        shared_decode(pa, c, gpu, [(2, 4, 512)], partition_size=128)


@pytest.mark.parametrize("layer", ["PagedAttention", "PartitionedPagedAttention"])
def test_attention_layers_take_the_groups_from_the_context(pa, gpu, layer):
    """What the runner does in a decode step: groups found on the host in the block-id lists, handed
    to the layers through the context; the layer's output equals the one without the groups."""
    lens = [700 + 9 * i for i in range(8)] + [300, 900]
    c = cases.make_case(31, lens, sum((n + 15) // 16 for n in lens) + 16, shared_prefix=None)
    tb = c["block_tables"]
    for m in range(1, 8):
        tb[m, :36] = tb[0, :36]                   # 8 samples share 576 tokens; rows 8, 9 are on their own
    want = oracle_decode(c)
    d = cases.to_device(c, gpu)
    att = getattr(pa, layer)(16, 8, 128)
    att.k_cache, att.v_cache = d["k_cache"], d["v_cache"]
    pg = pa.prepare_prefix_groups(host_tables(c), lens, 16, 16, 8, gpu)
    assert pg.groups == [(list(range(8)), 512)] and pg.partition_size == 512
    new_k = torch.zeros(10, 8, 128, dtype=torch.float16, device=gpu)
    outs = {}
    for name, groups in (("shared", pg), ("plain", None)):
        pa.set_context(False, context_lens=d["context_lens"], block_tables=d["block_tables"], prefix_groups=groups)
        outs[name] = att(d["q"], new_k, new_k).cpu()          # no slot mapping: nothing is written
        pa.reset_context()
    check(outs["shared"], want, "fp16")
    check(outs["plain"], want, "fp16")
    assert not torch.equal(outs["shared"], outs["plain"])       # another launch, not the same numbers by accident
