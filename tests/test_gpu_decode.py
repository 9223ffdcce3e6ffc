"""Paged decode attention on the GPU against the oracle (the reference's PyTorch paged
attention restated on the CPU).  Tolerances are the ones stated for the path: rtol 1e-3 / atol 2e-3 for 16-bit
caches, rtol 1e-2 / atol 1e-2 for fp8 caches."""
import pytest
import torch

import cases
from oracle import paged_attention_oracle as oracle

pytestmark = pytest.mark.gpu

# bf16 (no tolerance is stated for it): the oracle is evaluated in fp32 on the bf16 inputs, and the
# GPU result may differ from it by the 16-bit tolerance plus the one rounding of the output to
# bf16 (2^-8 relative) - the scheme of the prefill tests.
TOL = {"fp16": dict(rtol=1e-3, atol=2e-3), "bf16": dict(rtol=1e-3 + 2.0 ** -8, atol=2e-3),
       "fp8": dict(rtol=1e-2, atol=1e-2)}


def oracle_decode(c):
    q, kc, vc = c["q"], c["k_cache"], c["v_cache"]
    if q.dtype == torch.bfloat16 or kc.dtype == torch.bfloat16:
        q = q.float()
        if kc.dtype != cases.FP8:
            kc, vc = kc.float(), vc.float()
    return oracle.decode(q, kc, vc, c["block_tables"], c["context_lens"],
                         c["scale"], c["k_scale"], c["v_scale"], c["cache_dtype"])


def gpu_decode(pa, c, gpu, partition_size=None, **shape):
    d = cases.to_device(c, gpu)
    out = pa.paged_decode(d["q"], d["k_cache"], d["v_cache"], d["block_tables"], d["context_lens"],
                          d["scale"], d["k_scale"], d["v_scale"], partition_size=partition_size, **shape)
    torch.cuda.synchronize()
    return out.cpu()


def check(got, want, kind):
    assert not torch.isnan(got).any(), "NaN in the output: a read outside the context"
    torch.testing.assert_close(got.float(), want.float(), **TOL[kind])


def test_config1_fp16(pa, gpu):
    c = cases.config1()
    check(gpu_decode(pa, c, gpu), oracle_decode(c), "fp16")


@pytest.mark.parametrize("waves", [1, 2, 4, 8])
@pytest.mark.parametrize("cache", ["fp16", "fp8", "bf16"])
def test_every_workgroup_width(pa, lib, gpu, waves, cache):
    c = cases.make_case(40 + waves, [1, 15, 16, 17, 100, 333, 512, 47], 128, cache=cache,
                        q_dtype=torch.bfloat16 if cache == "bf16" else torch.float16)
    want = oracle_decode(c)
    got_single = gpu_decode(pa, c, gpu, waves=waves)
    got_part = gpu_decode(pa, c, gpu, partition_size=64, waves=waves)
    check(got_single, want, cache)
    check(got_part, want, cache)


@pytest.mark.parametrize("hq,hkv,d", [(16, 8, 128), (8, 8, 128), (32, 8, 128), (16, 2, 64),
                                       (4, 4, 64), (12, 4, 128), (64, 8, 128), (32, 2, 128),
                                       (24, 4, 128), (40, 8, 64), (48, 4, 64)])
@pytest.mark.parametrize("cache", ["fp16", "fp8"])
def test_head_shapes(pa, gpu, hq, hkv, d, cache):
    """GQA ratios 1, 2, 3, 4, 5, 6, 8, 12 and 16: the map h -> h // G (attention.py:366-370)."""
    c = cases.make_case(hq * 3 + d, [5, 64, 129, 700], 96, num_heads=hq, num_kv_heads=hkv,
                        head_dim=d, cache=cache)
    want = oracle_decode(c)
    check(gpu_decode(pa, c, gpu), want, cache)
    check(gpu_decode(pa, c, gpu, partition_size=128), want, cache)


@pytest.mark.parametrize("hq,hkv", [(32, 8), (64, 8), (32, 2), (24, 4)])
@pytest.mark.parametrize("qpw", [1, 2, 4])
@pytest.mark.parametrize("cache", ["fp16", "fp8", "bf16"])
def test_query_group_layouts_keep_the_result(pa, gpu, hq, hkv, qpw, cache):
    """Wide GQA groups: however the query heads of a KV head are spread over a wave's registers,
    the wave groups of a workgroup and separate workgroups, the output is the same."""
    if (hq // hkv) % qpw:
        pytest.skip("q_heads_per_wave must divide the GQA ratio")
    c = cases.make_case(hq + qpw, [3, 200, 1025, 77], 96, num_heads=hq, num_kv_heads=hkv, cache=cache,
                        q_dtype=torch.bfloat16 if cache == "bf16" else torch.float16)
    want = oracle_decode(c)
    check(gpu_decode(pa, c, gpu, q_heads_per_wave=qpw), want, cache)
    check(gpu_decode(pa, c, gpu, partition_size=256, q_heads_per_wave=qpw), want, cache)
    # 4 waves: no split of the query group over wave groups when two heads sit in a wave
    check(gpu_decode(pa, c, gpu, q_heads_per_wave=qpw, waves=4), want, cache)


@pytest.mark.parametrize("bs", [8, 32, 128, 256])
@pytest.mark.parametrize("cache", ["fp16", "fp8"])
def test_block_sizes(pa, gpu, bs, cache):
    lens = [1, bs - 1, bs, bs + 1, 5 * bs + 3, 301]
    c = cases.make_case(bs, lens, 64, block_size=bs, cache=cache)
    want = oracle_decode(c)
    check(gpu_decode(pa, c, gpu), want, cache)
    check(gpu_decode(pa, c, gpu, partition_size=48), want, cache)


@pytest.mark.parametrize("qdt", [torch.float32, torch.bfloat16])
def test_query_dtypes_against_fp64(pa, gpu, qdt):
    c = cases.make_case(77, [33, 260, 17], 40, q_dtype=qdt)
    got = gpu_decode(pa, c, gpu)
    assert got.dtype == qdt
    want = oracle.decode_f64(c["q"], c["k_cache"], c["v_cache"], c["block_tables"],
                             c["context_lens"], c["scale"])
    torch.testing.assert_close(got.double(), want, **TOL["fp16" if qdt == torch.float32 else "bf16"])
    check(got, oracle_decode(c), "fp16" if qdt == torch.float32 else "bf16")


def test_fp32_query_is_accurate_to_fp32_level(pa, gpu):
    c = cases.make_case(78, [200, 31], 32, q_dtype=torch.float32)
    got = gpu_decode(pa, c, gpu).double()
    want = oracle.decode_f64(c["q"], c["k_cache"], c["v_cache"], c["block_tables"],
                             c["context_lens"], c["scale"])
    torch.testing.assert_close(got, want, rtol=1e-4, atol=2e-5)


@pytest.mark.parametrize("pad", [-1, 0, 123456])
def test_padding_rows_and_garbage_table_tails(pa, gpu, pad):
    c = cases.make_case(11, [0, 40, 0, 16, 250], 64, pad=pad, extra_cols=5)
    got = gpu_decode(pa, c, gpu)
    assert float(got[0].abs().max()) == 0.0 and float(got[2].abs().max()) == 0.0
    check(got, oracle_decode(c), "fp16")
    gotp = gpu_decode(pa, c, gpu, partition_size=32)
    assert float(gotp[0].abs().max()) == 0.0
    check(gotp, oracle_decode(c), "fp16")


def test_ctx1_returns_the_single_value_row(pa, gpu):
    c = cases.make_case(12, [1, 1, 1, 1], 8)
    got = gpu_decode(pa, c, gpu)
    for b in range(4):
        blk = int(c["block_tables"][b, 0])
        for h in range(16):
            assert torch.equal(got[b, h], c["v_cache"][blk, 0, h // 2])


def test_strided_query_and_preallocated_output(pa, gpu):
    c = cases.make_case(13, [90, 300], 40)
    d = cases.to_device(c, gpu)
    wide = torch.zeros(2, 16 * 128 + 256, dtype=torch.float16, device=gpu)
    wide[:, :16 * 128] = d["q"].view(2, -1)
    qv = wide[:, :16 * 128].view(2, 16, 128)
    out = torch.empty(2, 16, 128, dtype=torch.float16, device=gpu)
    res = pa.paged_decode(qv, d["k_cache"], d["v_cache"], d["block_tables"], d["context_lens"],
                          d["scale"], out=out)
    torch.cuda.synchronize()
    assert res is out
    check(out.cpu(), oracle_decode(c), "fp16")


def test_config2_fp8_headline_shape(pa, gpu):
    c = cases.config2()
    got = gpu_decode(pa, c, gpu)
    check(got, oracle_decode(c), "fp8")
    # the same launch through the explicit 512-token partitioning
    check(gpu_decode(pa, c, gpu, partition_size=512), oracle_decode(c), "fp8")


def test_config2_fp8_per_tensor_scale(pa, gpu):
    c = cases.config2(seed=2002, batch=8, ctx=4096, per_tensor_scale=True)
    check(gpu_decode(pa, c, gpu), oracle_decode(c), "fp8")


def test_config2_shape_fp16(pa, gpu):
    c = cases.config2(seed=1102, cache="fp16", batch=16)
    check(gpu_decode(pa, c, gpu), oracle_decode(c), "fp16")


def test_config3_partitioned_long_context(pa, gpu):
    c = cases.config3()
    want = oracle_decode(c)                      # single-pass reference, as the config asks
    check(gpu_decode(pa, c, gpu, partition_size=512), want, "fp16")
    check(gpu_decode(pa, c, gpu), want, "fp16")   # automatic split


def test_config4_shared_prefix(pa, gpu):
    c = cases.config4()
    t = c["block_tables"]
    assert torch.equal(t[1, :64], t[0, :64]) and torch.equal(t[15, :64], t[8, :64])
    check(gpu_decode(pa, c, gpu), oracle_decode(c), "fp16")


def test_partials_match_the_reference_partition_outputs(pa, lib, gpu):
    c = cases.make_case(31, [700, 64, 1030], 160, q_dtype=torch.float32)
    d = cases.to_device(c, gpu)
    B, H, D, P = 3, 16, 128, 256
    parts = (d["block_tables"].shape[1] * 16 + P - 1) // P
    nbytes = lib.pa_workspace_bytes(B, H, D, parts)
    ws = torch.zeros(nbytes, dtype=torch.uint8, device=gpu)
    rc = lib.pa_decode_partials(d["q"].data_ptr(), 2, H * D, d["k_cache"].data_ptr(),
                                d["v_cache"].data_ptr(), None, None, 0, d["block_tables"].data_ptr(),
                                d["block_tables"].stride(0), d["block_tables"].shape[1],
                                d["context_lens"].data_ptr(), B, H, 8, D,
                                16, c["num_blocks"], c["scale"], P, parts, ws.data_ptr(), nbytes, 0, 0, 0, None)
    assert rc == 0, lib.pa_last_error()
    out = torch.empty(B, H, D, dtype=torch.float32, device=gpu)
    rc = lib.pa_merge(ws.data_ptr(), nbytes, d["context_lens"].data_ptr(), out.data_ptr(), 2, H * D,
                      B, H, D, P, parts, None)
    assert rc == 0, lib.pa_last_error()
    torch.cuda.synchronize()
    rows = B * H * parts
    scal = ((rows * 4 + 255) // 256) * 256
    wsc = ws.cpu()
    mx = wsc[:rows * 4].view(torch.float32).view(B, H, parts)
    sm = wsc[scal:scal + rows * 4].view(torch.float32).view(B, H, parts)
    po = wsc[2 * scal:2 * scal + rows * D * 4].view(torch.float32).view(B, H, parts, D)
    for b in range(B):
        n = int(c["context_lens"][b])
        for p in range((n + P - 1) // P):
            o, lse = oracle.partition_attention(c["q"][b:b + 1], c["k_cache"], c["v_cache"],
                                                c["block_tables"][b], p * P, min((p + 1) * P, n), 16,
                                                c["scale"])
            torch.testing.assert_close(po[b, :, p], o[0], rtol=1e-4, atol=1e-5)
            torch.testing.assert_close(mx[b, :, p] + torch.log(sm[b, :, p]), lse[0], rtol=1e-5, atol=1e-5)
    check(out.cpu(), oracle_decode(c), "fp16")


def test_more_partitions_than_workspace_rows_still_exact(pa, lib, gpu):
    # max_partitions smaller than ceil(ctx/P): the last partition absorbs the rest
    c = cases.make_case(32, [900, 100], 80)
    d = cases.to_device(c, gpu)
    B, H, D, P, parts = 2, 16, 128, 128, 3
    nbytes = lib.pa_workspace_bytes(B, H, D, parts)
    ws = torch.empty(nbytes, dtype=torch.uint8, device=gpu)
    out = torch.empty(B, H, D, dtype=torch.float16, device=gpu)
    rc = lib.pa_decode(d["q"].data_ptr(), 0, H * D, d["k_cache"].data_ptr(), d["v_cache"].data_ptr(),
                       None, None, 0, d["block_tables"].data_ptr(), d["block_tables"].stride(0),
                       d["block_tables"].shape[1], d["context_lens"].data_ptr(), out.data_ptr(), H * D, B, H, 8, D, 16,
                       c["num_blocks"], c["scale"], P, parts, ws.data_ptr(), nbytes, 0, 0, 0, None)
    assert rc == 0, lib.pa_last_error()
    torch.cuda.synchronize()
    check(out.cpu(), oracle_decode(c), "fp16")


def test_c_abi_argument_errors(lib, gpu):
    t = torch.zeros(16, dtype=torch.float16, device=gpu)
    p = t.data_ptr()
    base = dict(q=p, kc=p, vc=p, bt=p, cl=p, out=p)
    def call(**kw):
        a = dict(hq=16, hkv=8, d=128, bs=16, psize=0, parts=1, ws=None, wsb=0, kvd=0, waves=0, hpw=0, qpw=0)
        a.update(kw)
        return lib.pa_decode(base["q"], 0, a["hq"] * a["d"], base["kc"], base["vc"], None, None,
                             a["kvd"], base["bt"], 1, 1, base["cl"], base["out"], a["hq"] * a["d"], 1,
                             a["hq"], a["hkv"], a["d"], a["bs"], 4, 1.0, a["psize"], a["parts"],
                             a["ws"], a["wsb"], a["waves"], a["hpw"], a["qpw"], None)
    assert call(d=96) == -2 and b"head_dim" in lib.pa_last_error()
    assert call(bs=12) == -2
    assert call(bs=4) == -2
    assert call(hq=15) == -1
    assert call(kvd=3) == -1                      # fp8 without scales
    assert call(parts=4, psize=500, ws=p, wsb=1 << 30) == -2      # not a multiple of 16
    assert call(parts=4, psize=512) == -4         # workspace missing
    assert call(waves=3) == -1 and call(hpw=3) == -1 and call(qpw=3) == -1
    assert call(hq=32, hpw=2, qpw=4) == -2        # the vector kernel: several KV heads per wave need a GQA ratio <= 2
    assert call(hq=32, hpw=4) == -2 and call(hq=32, qpw=16, waves=1) == -2     # the matrix kernel: 1 or 2 heads, 2+ waves
    assert call(hq=32, qpw=16, hpw=2, waves=8) == -2
    assert call(hq=32, qpw=8) == -1 and call(hq=24, hkv=8, qpw=2) == -2
    assert call(hpw=4, waves=2) == -2


@pytest.mark.parametrize("adaptive", [True, False])
def test_partitioned_module_adaptive_and_exact_splits_agree(pa, gpu, adaptive):
    # long contexts at a small batch (split finer than the layer's size is never used) and a large
    # batch (no split needed): the layer's answer does not depend on how the launch was cut
    for seed, lens in ((50, [3000, 5000, 4097, 700]), (51, [300] * 130)):
        c = cases.make_case(seed, lens, sum((l + 15) // 16 for l in lens) + 8)
        d = cases.to_device(c, gpu)
        attn = pa.PartitionedPagedAttention(16, 8, 128, partition_size=512)
        attn.adaptive = adaptive
        attn.k_cache, attn.v_cache = d["k_cache"], d["v_cache"]
        pa.set_context(False, context_lens=d["context_lens"], block_tables=d["block_tables"])
        got = attn._decode_attention(d["q"], pa.get_context()).cpu()
        pa.reset_context()
        check(got, oracle_decode(c), "fp16")


@pytest.mark.parametrize("cache", ["fp16", "fp8"])
@pytest.mark.parametrize("hpw", [None, 1, 2, 4, 8])
@pytest.mark.parametrize("lens", [[2999, 301, 1777], [4100] * 5, [257, 5003], [1200] * 12, [33, 2000, 640, 3100, 90, 1500, 2111]])
def test_launch_policy_splits_and_head_pairing_keep_the_result(pa, lib, gpu, cache, hpw, lens):
    """The launch's own choices - partition sizes that are multiples of 16 rather than powers of
    two, one to eight KV heads per wave - never show in the output."""
    c = cases.make_case(sum(lens) % 97, lens, sum((n + 15) // 16 for n in lens) + 7, cache=cache)
    want = oracle_decode(c)
    psize, parts = pa.choose_partition(len(lens), 16, 8, c["block_tables"].shape[1] * 16, 128, 1 if cache == "fp8" else 2)
    assert psize % 16 == 0 and (parts == 1 or parts * psize >= max(lens))
    got = gpu_decode(pa, c, gpu, kv_heads_per_wave=hpw)
    odd = gpu_decode(pa, c, gpu, partition_size=16 * 23, kv_heads_per_wave=hpw)   # 368 tokens: neither a power of two nor a block multiple of 8 tiles
    check(got, want, cache)
    check(odd, want, cache)
    if hpw in (4, 8):
        check(gpu_decode(pa, c, gpu, kv_heads_per_wave=hpw, waves=8), want, cache)


@pytest.mark.parametrize("cache", ["fp16", "fp8"])
@pytest.mark.parametrize("hq", [16, 32])
@pytest.mark.parametrize("batch", [3, 64, 65, 150, 300])
def test_ragged_batches_pack_their_partitions(pa, gpu, cache, hq, batch):
    """A partitioned launch numbers only the (row, partition) pairs that hold tokens and every
    workgroup finds its pair from the context lengths: rows of very different lengths, empty rows
    between them, more rows than a wave has lanes (each lane then counts several rows), extra table
    columns (workgroups beyond the work), on the vector and the matrix kernel."""
    gen = torch.Generator().manual_seed(batch * 7 + hq)
    lens = torch.randint(1, 700, (batch,), generator=gen)
    lens[torch.rand(batch, generator=gen) < 0.2] = 0               # empty rows anywhere
    lens[int(torch.randint(0, batch, (1,), generator=gen))] = 1500  # one long row
    lens = lens.tolist()
    c = cases.make_case(batch + hq, lens, sum((n + 15) // 16 for n in lens) + 5, num_heads=hq, cache=cache, extra_cols=9)
    want = oracle_decode(c)
    for psize in (128, 256, 368):
        got = gpu_decode(pa, c, gpu, partition_size=psize)
        live = torch.tensor(lens) > 0
        check(got[live], want[live], cache)
        assert not got[~live].any(), "an empty row is a zero row"


@pytest.mark.parametrize("cache", ["fp16", "fp8"])
def test_known_lengths_size_the_launch_and_never_change_the_result(pa, gpu, cache):
    """longest_context / mean_context only shape the launch: right, too small (rows longer than the
    bound end in the last partition) or absurd, the output is the oracle's."""
    lens = [900, 40, 2500, 1300, 7, 1999]
    c = cases.make_case(77, lens, sum((n + 15) // 16 for n in lens) + 5, cache=cache, extra_cols=300)   # tables 7300 tokens wide
    want = oracle_decode(c)
    for longest, mean in ((2500, 1124.0), (2500, None), (1000, 500.0), (256, 10.0), (10 ** 6, 10.0 ** 6), (None, 1124.0)):
        check(gpu_decode(pa, c, gpu, longest_context=longest, mean_context=mean), want, cache)
        check(gpu_decode(pa, c, gpu, partition_size=512, longest_context=longest), want, cache)
    width = c["block_tables"].shape[1] * 16
    elem = 1 if cache == "fp8" else 2
    blind = pa.choose_partition(len(lens), 16, 8, width, 128, elem)
    told = pa.choose_partition(len(lens), 16, 8, width, 128, elem, longest_context=2500, mean_context=1124.0)
    assert told[0] * told[1] < blind[0] * blind[1], "the launch is sized for the rows, not for the table"
    # the layers take the same hints from the context
    d = cases.to_device(c, gpu)
    for cls in (pa.PagedAttention, pa.PartitionedPagedAttention):
        attn = cls(16, 8, 128, cache_dtype=cache)
        attn.k_cache, attn.v_cache, attn.k_scale, attn.v_scale = d["k_cache"], d["v_cache"], d["k_scale"], d["v_scale"]
        pa.set_context(False, context_lens=d["context_lens"], block_tables=d["block_tables"],
                       longest_context_len=2500, mean_context_len=1124.0)
        got = attn._decode_attention(d["q"], pa.get_context()).cpu()
        pa.reset_context()
        check(got, want, cache)


def test_table_check_counts_what_the_kernels_would_clamp(pa, gpu, monkeypatch):
    c = cases.make_case(60, [100, 40, 0, 33], 32)
    d = cases.to_device(c, gpu)
    assert pa.check_block_tables(d["block_tables"], d["context_lens"], 16, c["num_blocks"]) == (0, 0)
    bad = d["block_tables"].clone()
    bad[0, 2] = c["num_blocks"]          # inside row 0's context (7 blocks): counted
    bad[1, 1] = -5                        # inside row 1's context (3 blocks): counted
    bad[1, 5] = -5                        # past row 1's context: never read, not counted
    bad[2, 0] = 99999                     # padded row: not counted
    lens = d["context_lens"].clone()
    lens[3] = 16 * bad.shape[1] + 1       # needs one more column than the table has ...
    pads = bad.shape[1] - 3               # ... and now covers the -1 padding behind its 3 blocks
    assert pa.check_block_tables(bad, lens, 16, c["num_blocks"]) == (2 + pads, 1)
    # the attention launch itself survives such a table (clamped reads) ...
    out = pa.paged_decode(d["q"], d["k_cache"], d["v_cache"], bad, lens, d["scale"])
    torch.cuda.synchronize()
    assert out.shape == d["q"].shape
    # ... and names it when asked to
    monkeypatch.setenv("PA_DEBUG_TABLES", "1")
    with pytest.raises(RuntimeError, match="outside the pool"):
        pa.paged_decode(d["q"], d["k_cache"], d["v_cache"], bad, lens, d["scale"])
    got = pa.paged_decode(d["q"], d["k_cache"], d["v_cache"], d["block_tables"], d["context_lens"], d["scale"])
    check(got.cpu(), oracle_decode(c), "fp16")


def test_graph_workspace_grows_outside_captures_and_outlives_graphs(pa, gpu):
    """A partitioned launch recorded in a graph keeps its workspace address: a later, larger
    recorded launch grows the graphs' workspace without freeing the one already recorded, and
    growth inside a capture is an error instead of an allocation from the graph's pool."""
    pa.release_decode_workspaces()
    small = cases.make_case(61, [3000, 2000], 2 * 188 + 8)
    d = cases.to_device(small, gpu)
    want = oracle_decode(small)
    out = torch.empty_like(d["q"])

    def run_small():
        pa.paged_decode(d["q"], d["k_cache"], d["v_cache"], d["block_tables"], d["context_lens"],
                        d["scale"], partition_size=256, out=out)

    # growth inside a capture is refused
    with pytest.raises(RuntimeError, match="cannot grow during a graph capture"):
        g0 = torch.cuda.CUDAGraph()
        with torch.cuda.graph(g0):
            run_small()
    torch.cuda.synchronize()
    with pa.sizing_graph_workspace():
        run_small()                               # the warm-up before a capture sizes the graphs' workspace (1 MiB minimum)
    torch.cuda.synchronize()
    ws_first = pa.reserve_decode_workspace(gpu, 1, for_graphs=True)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        run_small()
    torch.cuda.synchronize()
    # a larger launch for a later graph: more partials than the first workspace holds
    large = cases.make_case(62, [4000] * 24, 24 * 250 + 8)
    dl = cases.to_device(large, gpu)
    with pa.sizing_graph_workspace():
        big_out = pa.paged_decode(dl["q"], dl["k_cache"], dl["v_cache"], dl["block_tables"], dl["context_lens"],
                                  dl["scale"], partition_size=64)
    torch.cuda.synchronize()
    ws_second = pa.reserve_decode_workspace(gpu, 1, for_graphs=True)
    assert ws_second.numel() > ws_first.numel() and ws_second.data_ptr() != ws_first.data_ptr()
    check(big_out.cpu(), oracle_decode(large), "fp16")
    # fill fresh allocations with garbage: had the first workspace been freed, this would land in it
    junk = [torch.full((1 << 20,), float("nan"), device=gpu) for _ in range(4)]
    for _ in range(3):
        out.fill_(float("nan"))
        graph.replay()
        torch.cuda.synchronize()
        check(out.cpu(), want, "fp16")
        pa.paged_decode(dl["q"], dl["k_cache"], dl["v_cache"], dl["block_tables"], dl["context_lens"],
                        dl["scale"], partition_size=64)
        torch.cuda.synchronize()
    del junk


def test_partitioned_launches_on_two_streams_do_not_share_partials(pa, gpu):
    """Eager launches take their workspace per (device, stream): two partitioned launches in flight on
    different streams of one GPU each merge their own partials."""
    a = cases.make_case(63, [4000] * 16, 16 * 250 + 8)
    b = cases.make_case(64, [3500] * 16, 16 * 250 + 8)
    da, db = cases.to_device(a, gpu), cases.to_device(b, gpu)
    want_a, want_b = oracle_decode(a), oracle_decode(b)
    side = torch.cuda.Stream()
    torch.cuda.synchronize()
    outs_a, outs_b = [], []
    for _ in range(4):
        outs_a.append(pa.paged_decode(da["q"], da["k_cache"], da["v_cache"], da["block_tables"], da["context_lens"],
                                      da["scale"], partition_size=128))
        with torch.cuda.stream(side):
            outs_b.append(pa.paged_decode(db["q"], db["k_cache"], db["v_cache"], db["block_tables"], db["context_lens"],
                                          db["scale"], partition_size=128))
    torch.cuda.synchronize()
    main_ws = pa.reserve_decode_workspace(gpu, 1)
    with torch.cuda.stream(side):
        side_ws = pa.reserve_decode_workspace(gpu, 1)
    assert main_ws.data_ptr() != side_ws.data_ptr()
    for o in outs_a:
        check(o.cpu(), want_a, "fp16")
    for o in outs_b:
        check(o.cpu(), want_b, "fp16")


# ---- the matrix kernel (q_heads_per_wave = 16; the launch's own choice from a GQA ratio of 3) -------

@pytest.mark.parametrize("hq,hkv,d", [(32, 8, 128), (64, 8, 128), (16, 8, 128), (8, 8, 128), (12, 4, 128),
                                       (40, 8, 64), (48, 2, 64), (40, 2, 128), (34, 2, 128)])
@pytest.mark.parametrize("cache", ["fp16", "fp8", "bf16"])
def test_matrix_kernel_head_shapes(pa, gpu, hq, hkv, d, cache):
    """Ratios 1 ... 24 (more than 16 query heads per KV head run as slices of 16, the last one ragged),
    one and two KV heads per wave, every workgroup width, single pass and partitions."""
    lens = [3, 200, 1025, 77, 32, 33, 64, 1]
    c = cases.make_case(hq + d, lens, 128, num_heads=hq, num_kv_heads=hkv, head_dim=d, cache=cache,
                        q_dtype=torch.bfloat16 if cache == "bf16" else torch.float16)
    want = oracle_decode(c)
    for kw in (dict(), dict(partition_size=256), dict(waves=4), dict(waves=2, partition_size=48),
               dict(kv_heads_per_wave=2), dict(kv_heads_per_wave=2, waves=2, partition_size=80),
               dict(kv_heads_per_wave=1, waves=8, partition_size=32)):
        check(gpu_decode(pa, c, gpu, q_heads_per_wave=16, **kw), want, cache)


@pytest.mark.parametrize("bs", [8, 32, 128, 256])
@pytest.mark.parametrize("cache", ["fp16", "fp8"])
def test_matrix_kernel_block_sizes_and_empty_rows(pa, gpu, bs, cache):
    lens = [1, 0, bs - 1, bs, bs + 1, 5 * bs + 3, 0, 301]
    c = cases.make_case(300 + bs, lens, 64, block_size=bs, num_heads=32, num_kv_heads=4, cache=cache, pad=-1)
    want = oracle_decode(c)
    live = [i for i, n in enumerate(lens) if n > 0]
    for kw in (dict(), dict(partition_size=48), dict(kv_heads_per_wave=2, partition_size=64)):
        got = gpu_decode(pa, c, gpu, q_heads_per_wave=16, **kw)
        check(got[live], want[live], cache)
        assert float(got[[1, 6]].float().abs().max()) == 0.0       # rows without context come back as zeros


def ramp_keys_along_the_pool(c, lo=0.2, hi=3.0):
    """Keys grow along the pool (and so, block by block, along the contexts that map it): later tiles hold
    larger scores than the first one.  An fp8 cache is scaled through its per-token multiplier."""
    nb, bs = c["k_cache"].shape[0], c["k_cache"].shape[1]
    ramp = torch.linspace(lo, hi, nb * bs).view(nb, bs)
    if c["cache_dtype"] == "fp8":
        c["k_scale"] = c["k_scale"] / ramp
    else:
        c["k_cache"] = (c["k_cache"].float() * ramp.view(nb, bs, 1, 1)).to(c["k_cache"].dtype)


@pytest.mark.parametrize("qdt,cache", [(torch.float32, "fp16"), (torch.bfloat16, "fp16"), (torch.float16, "fp16"),
                                       (torch.float16, "fp8"), (torch.bfloat16, "bf16")])
def test_matrix_kernel_query_dtypes_and_large_scores(pa, gpu, qdt, cache):
    """Scores far from zero (queries and keys of norm ~40): the reference point of the exponentials is
    set by the first tile and moved when a later one outgrows it."""
    c = cases.make_case(77, [700, 45, 2048, 9], 256, num_heads=32, num_kv_heads=8, q_dtype=qdt, cache=cache)
    c["q"] = (c["q"].float() * 3.5).to(qdt)
    ramp_keys_along_the_pool(c)
    want = oracle_decode(c)
    kind = "fp8" if cache == "fp8" else "bf16" if qdt == torch.bfloat16 else "fp16"
    check(gpu_decode(pa, c, gpu, q_heads_per_wave=16), want, kind)
    check(gpu_decode(pa, c, gpu, q_heads_per_wave=16, partition_size=512, kv_heads_per_wave=2), want, kind)


@pytest.mark.parametrize("v_factor", [1e-2, 1e-3])
@pytest.mark.parametrize("path", ["matrix", "vector"])
def test_fp8_small_values_behind_an_attention_sink(pa, gpu, path, v_factor):
    """An fp8 cache whose V is small (per-token amax of 1e-2 .. 1e-3 of the usual) read by rows that put most
    of their weight on one key of their first tile and spread the rest, ~1e-4 each, over thousands of keys.
    A kernel that folds 1 / v_scale into the probability before rounding it to fp16 loses that tail
    (p / v_scale underflows fp16) while the row sum still counts it.  The problem is linear in V, so the
    fp8 tolerance scales with the factor V was shrunk by."""
    hq, hkv = (32, 8) if path == "matrix" else (16, 8)
    lens = [3000, 1500, 4096, 700]
    c = cases.make_case(311, lens, sum((n + 15) // 16 for n in lens) + 8, num_heads=hq, num_kv_heads=hkv, cache="fp8")
    g = torch.Generator().manual_seed(312)
    # the sink: position 0 of every sequence holds a key along the mean query of each KV head's group,
    # q.k * scale about 9 above the N(0, 1) scores of the other keys
    gq = hq // hkv
    qf = c["q"].float().view(len(lens), hkv, gq, 128)
    k_sink = (0.8 * qf.sum(2)).half()                                   # [batch, hkv, 128]
    v_sink = torch.randn(len(lens), hkv, 128, generator=g).half()
    slots = (c["block_tables"][:, 0].long() * 16).to(torch.int32)
    oracle.store_kv_cache(k_sink, v_sink, c["k_cache"], c["v_cache"], slots, c["k_scale"], c["v_scale"], "fp8")
    # shrink V through its per-token multiplier: dequantised value = byte / v_scale
    jitter = 0.5 + 1.5 * torch.rand(c["v_scale"].shape, generator=g)
    c["v_scale"] = c["v_scale"] / (v_factor * jitter)
    want = oracle_decode(c)
    assert want.abs().max() < 20 * v_factor
    for kw in (dict(), dict(partition_size=512)):
        got = gpu_decode(pa, c, gpu, q_heads_per_wave=16 if path == "matrix" else 0, **kw)
        assert not torch.isnan(got).any()
        torch.testing.assert_close(got.float() / v_factor, want.float() / v_factor, rtol=1e-2, atol=1e-2)


def test_matrix_kernel_is_the_choice_for_wide_groups(pa, gpu):
    """From a ratio of 3 on the launch takes the matrix kernel by itself: same result as when it is
    named, bit for bit, and the vector kernel agrees to rounding."""
    c = cases.make_case(91, [500, 131, 64, 1999], 192, num_heads=24, num_kv_heads=8)
    auto = gpu_decode(pa, c, gpu)
    named = gpu_decode(pa, c, gpu, q_heads_per_wave=16)
    vector = gpu_decode(pa, c, gpu, q_heads_per_wave=1)
    assert torch.equal(auto, named)
    torch.testing.assert_close(auto.float(), vector.float(), rtol=1e-3, atol=1e-3)
    check(auto, oracle_decode(c), "fp16")


def test_matrix_kernel_refuses_what_it_cannot_run(pa, gpu):
    c = cases.make_case(5, [100, 50], 32, num_heads=28, num_kv_heads=7)
    for kw in (dict(waves=1), dict(kv_heads_per_wave=2), dict(kv_heads_per_wave=4)):
        with pytest.raises(RuntimeError, match="matrix path"):
            gpu_decode(pa, c, gpu, q_heads_per_wave=16, **kw)


@pytest.mark.parametrize("cache", ["fp16", "fp8"])
def test_matrix_kernel_in_a_replayed_graph(pa, gpu, cache):
    """Single pass and partitioned launches of the matrix kernel recorded in one graph; every replay,
    with eager work and new context lengths between the replays, equals the eager result."""
    lens = [900, 31, 1500, 257]
    c = cases.make_case(123, lens, 192, num_heads=32, num_kv_heads=4, cache=cache)
    d = cases.to_device(c, gpu)
    out1, out2 = torch.empty_like(d["q"]), torch.empty_like(d["q"])

    def run():
        pa.paged_decode(d["q"], d["k_cache"], d["v_cache"], d["block_tables"], d["context_lens"], d["scale"],
                        d["k_scale"], d["v_scale"], out=out1)
        pa.paged_decode(d["q"], d["k_cache"], d["v_cache"], d["block_tables"], d["context_lens"], d["scale"],
                        d["k_scale"], d["v_scale"], partition_size=256, out=out2)

    with pa.sizing_graph_workspace():
        run()                                     # warm-up: the graphs' workspace and kernel attributes
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        run()
    torch.cuda.synchronize()
    for shrink in (0, 100, 7):
        new_lens = [n - min(shrink, n - 1) for n in lens]
        d["context_lens"].copy_(torch.tensor(new_lens, dtype=torch.int32))
        c["context_lens"] = torch.tensor(new_lens, dtype=torch.int32)
        want = oracle_decode(c)
        out1.fill_(float("nan"))
        out2.fill_(float("nan"))
        graph.replay()
        torch.cuda.synchronize()
        check(out1.cpu(), want, cache)
        check(out2.cpu(), want, cache)
        _ = torch.randn(1 << 16, device=gpu).sum().item()      # eager work between the replays


def test_small_launches_are_split_for_graphs_and_not_for_eager_calls(pa, gpu):
    """One row of 1000 tokens: replayed from a graph the launch policy cuts it into 64-token partitions (a
    round of short workgroups), called eagerly it reads it in one pass (a second launch would cost the host
    more than the split saves); a warm-up inside sizing_graph_workspace() is shaped like the capture that
    follows, so the graphs' workspace is there when the capture needs it.  Same result every way."""
    assert pa.choose_partition(1, 16, 8, 1008)[1] > 1 and pa.choose_partition(1, 16, 8, 1008, eager=True) == (0, 1)
    c = cases.make_case(91, [1000], 80)
    want = oracle_decode(c)
    d = cases.to_device(c, gpu)
    out = torch.empty_like(d["q"])
    call = lambda: pa.paged_decode(d["q"], d["k_cache"], d["v_cache"], d["block_tables"], d["context_lens"], d["scale"], out=out)
    call()
    torch.cuda.synchronize()
    check(out.cpu(), want, "fp16")
    pa.release_decode_workspaces()
    with pa.sizing_graph_workspace():
        call()
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    out.zero_()
    with torch.cuda.graph(graph):
        call()                                   # raises if the warm-up had not sized the graphs' workspace
    for _ in range(3):
        out.zero_()
        graph.replay()
        torch.cuda.synchronize()
        check(out.cpu(), want, "fp16")
