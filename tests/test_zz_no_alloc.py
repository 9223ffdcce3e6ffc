"""pa_decode_noalloc (partition partials in the library's own device array, nothing allocated)
against pa_decode with a caller-owned workspace: same kernels, so the outputs must be equal bit
for bit - on two calls in a row, the second over a smaller input, so that whatever the first call
left in the shared array is shown not to matter."""
import pytest
import torch

import cases

pytestmark = pytest.mark.gpu

H, HKV, D, BS = 16, 8, 128, 16


def _args(d, c, out, H=H):
    t = d["block_tables"]
    fp8 = c["cache_dtype"] == "fp8"
    return [d["q"].data_ptr(), 0, H * D, d["k_cache"].data_ptr(), d["v_cache"].data_ptr(),
            d["k_scale"].data_ptr() if fp8 else None, d["v_scale"].data_ptr() if fp8 else None,
            3 if fp8 else 0, t.data_ptr(), t.stride(0), t.shape[1], d["context_lens"].data_ptr(),
            out.data_ptr(), H * D, t.shape[0], H, HKV, D, BS, c["num_blocks"], c["scale"]]


def _both(lib, gpu, c, psize, H=H):
    d = cases.to_device(c, gpu)
    batch = d["q"].shape[0]
    parts = max(1, (d["block_tables"].shape[1] * BS + psize - 1) // psize)
    nbytes = lib.pa_workspace_bytes(batch, H, D, parts)
    ws = torch.empty(nbytes, dtype=torch.uint8, device=gpu)
    want = torch.full((batch, H, D), float("nan"), dtype=torch.float16, device=gpu)
    got = torch.full_like(want, float("nan"))
    stream = torch.cuda.current_stream(gpu).cuda_stream
    rc = lib.pa_decode(*_args(d, c, want, H), psize, parts, ws.data_ptr(), nbytes, 0, 0, 0, stream)
    assert rc == 0, lib.pa_last_error()
    rc = lib.pa_decode_noalloc(*_args(d, c, got, H), psize, parts, 0, 0, 0, stream)
    assert rc == 0, lib.pa_last_error()
    torch.cuda.synchronize()
    return got.cpu(), want.cpu()


@pytest.mark.parametrize("cache", ["fp16", "fp8"])
def test_two_calls_in_a_row_second_one_smaller(lib, gpu, cache):
    big = cases.make_case(901, [3000, 517, 4096, 1, 2222, 1025], 6 * 256 + 16, cache=cache)
    small = cases.make_case(902, [700, 90], 64, cache=cache)
    allocated_before = torch.cuda.memory_allocated(gpu)
    for c, psize in ((big, 256), (small, 512)):
        got, want = _both(lib, gpu, c, psize)
        assert not torch.isnan(got).any()
        assert torch.equal(got.view(torch.int16), want.view(torch.int16))
    assert torch.cuda.memory_allocated(gpu) == allocated_before


def test_the_entry_point_takes_no_device_memory(lib, gpu):
    """torch's own counters cannot see a hipMalloc made inside the library, so the device-wide free bytes
    are read around the calls (hipMemGetInfo): with every input, output and the comparison workspace
    allocated beforehand, and the library's array resident since it was loaded, calls of the entry point -
    partitioned, over several shapes - must leave the free bytes where they were."""
    cs = [cases.make_case(906, [3000, 517, 4096, 1, 2222, 1025], 6 * 256 + 16),
          cases.make_case(907, [700, 90], 64, cache="fp8")]
    ds = [cases.to_device(c, gpu) for c in cs]
    outs = [torch.empty(d["q"].shape, dtype=torch.float16, device=gpu) for d in ds]
    stream = torch.cuda.current_stream(gpu).cuda_stream
    def run_all():
        for c, d, o in zip(cs, ds, outs):
            for psize in (256, 128, 1024):
                parts = (d["block_tables"].shape[1] * BS + psize - 1) // psize
                assert lib.pa_decode_noalloc(*_args(d, c, o), psize, parts, 0, 0, 0, stream) == 0, lib.pa_last_error()
        torch.cuda.synchronize()

    # a first call per launch shape: what the runtime sets up once per kernel and process (code object,
    # kernel attributes, the symbol lookup) is not what this test is about
    run_all()
    free_before, _total = torch.cuda.mem_get_info(gpu)
    torch_before = torch.cuda.memory_reserved(gpu)
    for _ in range(3):
        run_all()
    free_after, _total = torch.cuda.mem_get_info(gpu)
    assert torch.cuda.memory_reserved(gpu) == torch_before       # torch itself took nothing in between ...
    assert free_after == free_before, (free_before, free_after)   # ... and neither did anyone else on the device


def test_wide_query_groups_take_the_matrix_kernel_through_the_same_entry_point(lib, gpu):
    """32 query heads over 8 KV heads: the launch picks the matrix kernel; its partials go to the same array."""
    for seed, lens, psize in ((904, [2000, 333, 1500], 256), (905, [600], 128)):
        c = cases.make_case(seed, lens, sum((n + 15) // 16 for n in lens) + 8, num_heads=32)
        got, want = _both(lib, gpu, c, psize, H=32)
        assert not torch.isnan(got).any()
        assert torch.equal(got.view(torch.int16), want.view(torch.int16))


def test_single_pass_needs_no_scratch_and_oversized_launches_are_refused(lib, gpu):
    c = cases.make_case(903, [300, 64], 40)
    got, want = _both(lib, gpu, c, 1 << 20)          # one partition: straight to the output
    assert torch.equal(got.view(torch.int16), want.view(torch.int16))
    d = cases.to_device(c, gpu)
    out = torch.empty(2, H, D, dtype=torch.float16, device=gpu)
    a = _args(d, c, out)
    a[14] = 4096                                      # batch: partials of 4096 x 16 x 64 partitions > 16 MiB
    assert lib.pa_decode_noalloc(*a, 512, 64, 0, 0, 0, None) == -4
    assert b"scratch" in lib.pa_last_error()
