"""The measuring aids of bench.py (libpa_probes.so, a library of its own beside the product's) run and
report what they say they do: the decode launch with its arithmetic taken out (pa_decode_load_probe),
the matrix-pipe rate probe (pa_mfma_rate_probe) and the plain read probe (pa_hbm_read_probe).  Their
timings belong to bench.py; here only the contracts are checked."""
import pytest
import torch

import cases

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def lib():
    import bench
    return bench.load_probes()


def test_the_product_library_holds_no_measuring_aid(pa):
    product = pa._native.load()
    for name in ("pa_decode_load_probe", "pa_mfma_rate_probe", "pa_hbm_read_probe"):
        assert not hasattr(product, name), name


def test_mfma_rate_probe_counts_its_work_and_rejects_bad_arguments(pa, lib, gpu):
    ops = torch.ones(65536, dtype=torch.float16, device=gpu)
    sink = torch.full((1024,), float("nan"), dtype=torch.float32, device=gpu)
    stream = torch.cuda.current_stream(gpu).cuda_stream
    cus = torch.cuda.get_device_properties(gpu).multi_processor_count
    flops = lib.pa_mfma_rate_probe(ops.data_ptr(), ops.numel(), 4, sink.data_ptr(), sink.numel(), stream)
    torch.cuda.synchronize()
    assert flops == cus * 8 * 4 * 16 * 32768
    got = sink[:cus].cpu()
    # all-ones operands: every product adds 16 to each element of its accumulator; 4 steps x 16 products over 4
    # chains = 16 products per chain = 256 per element; the sink sums two elements of each of the 4 chains
    assert torch.all(got == 4 * 2 * 256.0), got[:4]
    assert torch.isnan(sink[cus:]).all()
    assert lib.pa_mfma_rate_probe(None, ops.numel(), 4, sink.data_ptr(), sink.numel(), stream) == -1
    assert lib.pa_mfma_rate_probe(ops.data_ptr(), ops.numel(), 0, sink.data_ptr(), sink.numel(), stream) == -1
    assert b"steps" in lib.pa_probes_last_error()
    # buffers shorter than the launch reads or writes are refused
    assert lib.pa_mfma_rate_probe(ops.data_ptr(), 65535, 4, sink.data_ptr(), sink.numel(), stream) == -1
    assert lib.pa_mfma_rate_probe(ops.data_ptr(), ops.numel(), 4, sink.data_ptr(), cus - 1, stream) == -1
    assert b"sink" in lib.pa_probes_last_error()


def test_hbm_read_probe_reads_every_word_once(pa, lib, gpu):
    g = torch.Generator().manual_seed(5)
    words = torch.randint(-2 ** 31, 2 ** 31 - 1, (1 << 18,), generator=g, dtype=torch.int64).to(torch.int32)
    buf = words.to(gpu)
    stream = torch.cuda.current_stream(gpu).cuda_stream
    for groups, streaming in ((1, 0), (7, 1), (64, 0), (64, 1), (1000, 1)):
        sink = torch.zeros(groups, dtype=torch.int32, device=gpu)
        got = lib.pa_hbm_read_probe(buf.data_ptr(), buf.numel() * 4, groups, streaming, sink.data_ptr(), sink.numel(), stream)
        torch.cuda.synchronize()
        per = (buf.numel() // 4 // groups) * 4              # int32 words per workgroup
        assert got == per * groups * 4
        want = words[:per * groups].view(groups, per)
        acc = want[:, 0].clone()
        for j in range(1, per):                              # XOR fold on the host
            acc ^= want[:, j]
        assert torch.equal(sink.cpu(), acc), groups
    assert lib.pa_hbm_read_probe(buf.data_ptr(), 8, 1, 1, sink.data_ptr(), sink.numel(), stream) == -1
    assert lib.pa_hbm_read_probe(None, 1024, 1, 0, sink.data_ptr(), sink.numel(), stream) == -1
    assert lib.pa_hbm_read_probe(buf.data_ptr(), buf.numel() * 4, 64, 1, sink.data_ptr(), 63, stream) == -1


def test_decode_load_probe_runs_the_decode_launch_shape(pa, lib, gpu):
    product = pa._native.load()
    lens = cases.uniform_lens(5, 8, 128, 512)
    c = cases.make_case(1001, lens, 512, cache="fp8")
    d = cases.to_device(c, gpu)
    ws = torch.zeros(product.pa_workspace_bytes(8, 16, 128, 4), dtype=torch.uint8, device=gpu)
    rc = lib.pa_decode_load_probe(
        d["q"].data_ptr(), 0, 16 * 128, d["k_cache"].data_ptr(), d["v_cache"].data_ptr(), d["k_scale"].data_ptr(),
        d["v_scale"].data_ptr(), pa._native.DTYPE_FP8_E4M3, d["block_tables"].data_ptr(), d["block_tables"].stride(0),
        d["block_tables"].shape[1], d["context_lens"].data_ptr(), 8, 16, 8, 128, 16, c["num_blocks"], 128, 4,
        ws.data_ptr(), ws.numel(), 0, 0, 0, torch.cuda.current_stream(gpu).cuda_stream)
    torch.cuda.synchronize()
    assert rc == 0, lib.pa_probes_last_error()
    # too small a workspace is refused like in the real launch
    rc = lib.pa_decode_load_probe(
        d["q"].data_ptr(), 0, 16 * 128, d["k_cache"].data_ptr(), d["v_cache"].data_ptr(), d["k_scale"].data_ptr(),
        d["v_scale"].data_ptr(), pa._native.DTYPE_FP8_E4M3, d["block_tables"].data_ptr(), d["block_tables"].stride(0),
        d["block_tables"].shape[1], d["context_lens"].data_ptr(), 8, 16, 8, 128, 16, c["num_blocks"], 128, 4,
        ws.data_ptr(), 256, 0, 0, 0, torch.cuda.current_stream(gpu).cuda_stream)
    assert rc == -4
