"""Residual add + RMSNorm and silu(gate) * up on the GPU (pa_add_rms_norm, pa_silu_mul) against
oracle/qwen3_block_oracle.py.  The residual sum is a single correctly rounded add: bit-exact.
The normed rows and the activation are floating point: rtol 1e-3 / atol 2e-3 for 16-bit types
(one unit in the last place of fp16 at |y| <= 2 is 1e-3 relative), 1e-5 for fp32."""
import pytest
import torch

from oracle import qwen3_block_oracle as ob

pytestmark = pytest.mark.gpu

TOL = {torch.float16: dict(rtol=1e-3, atol=2e-3), torch.bfloat16: dict(rtol=8e-3, atol=8e-3),
       torch.float32: dict(rtol=1e-5, atol=1e-5)}


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16, torch.float32])
@pytest.mark.parametrize("rows,hidden", [(64, 1024), (1, 1024), (5, 264), (33, 2048), (3, 4096), (2, 8192), (4099, 1024)])
def test_add_rms_norm_matches_oracle(pa, gpu, dtype, rows, hidden):
    g = torch.Generator().manual_seed(rows * 7 + hidden)
    x = (torch.randn(rows, hidden, generator=g) * 2).to(dtype)
    d = torch.randn(rows, hidden, generator=g).to(dtype)
    w = (torch.rand(hidden, generator=g) + 0.5).to(dtype)
    # norm alone
    same, normed = pa.add_rms_norm(x.to(gpu), w.to(gpu), 1e-6)
    assert torch.equal(same.cpu(), x)
    torch.testing.assert_close(normed.cpu().float(), ob.rms_norm(x, w, 1e-6).float(), **TOL[dtype])
    # add + norm, sum written over x
    xg = x.to(gpu)
    total, normed = pa.add_rms_norm(xg, w.to(gpu), 1e-6, delta=d.to(gpu))
    want_total, want_normed = ob.add_rms_norm(x, d, w, 1e-6)
    assert total.data_ptr() == xg.data_ptr()
    assert torch.equal(total.cpu(), want_total)
    torch.testing.assert_close(normed.cpu().float(), want_normed.float(), **TOL[dtype])
    # out of place, fp32 weight, rows that are views of a wider buffer
    wide = torch.zeros(rows, hidden + 24, dtype=dtype, device=gpu)
    wide[:, :hidden] = x.to(gpu)
    total2, normed2 = pa.add_rms_norm(wide[:, :hidden], w.float().to(gpu), 1e-6, delta=d.to(gpu), inplace_sum=False)
    assert torch.equal(total2.cpu(), want_total) and torch.equal(wide[:, :hidden].cpu(), x)
    torch.testing.assert_close(normed2.cpu().float(), want_normed.float(), **TOL[dtype])


def test_add_rms_norm_special_rows(pa, gpu):
    hidden = 1024
    w = torch.ones(hidden, dtype=torch.float16, device=gpu)
    x = torch.zeros(3, hidden, dtype=torch.float16, device=gpu)
    x[1, 5] = -4.0                                              # one-hot row: sqrt(hidden) * sign
    x[2] = 60000.0                                              # squares overflow fp16, not fp32
    _, y = pa.add_rms_norm(x, w, 1e-6)
    assert torch.equal(y[0].cpu(), torch.zeros(hidden, dtype=torch.float16))
    assert float(y[1, 5]) == -32.0 and float(y[1].abs().sum()) == 32.0
    torch.testing.assert_close(y[2].float().cpu(), torch.ones(hidden), rtol=1e-3, atol=0)
    # three leading dimensions
    x3 = torch.randn(2, 3, hidden, device=gpu).half()
    t3, y3 = pa.add_rms_norm(x3, w, 1e-6, delta=torch.ones_like(x3))
    assert t3.shape == y3.shape == (2, 3, hidden)
    torch.testing.assert_close(y3.cpu().float(), ob.rms_norm(t3.cpu(), w.cpu(), 1e-6).float(), rtol=1e-3, atol=2e-3)


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16, torch.float32])
@pytest.mark.parametrize("rows,width", [(64, 3072), (1, 8), (7, 200), (4096, 3072)])
def test_silu_mul_matches_oracle(pa, gpu, dtype, rows, width):
    g = torch.Generator().manual_seed(rows + width)
    gu = (torch.randn(rows, 2 * width, generator=g) * 3).to(dtype)
    gu[0, :4] = torch.tensor([0.0, 30.0, -30.0, -100.0]).to(dtype)
    want = ob.swiglu(gu[:, :width], gu[:, width:])
    got = pa.silu_mul(gu.to(gpu))                                            # packed gate|up
    torch.testing.assert_close(got.cpu().float(), want.float(), **TOL[dtype])
    got2 = pa.silu_mul(gu[:, :width].contiguous().to(gpu), gu[:, width:].contiguous().to(gpu))
    assert torch.equal(got2, got)
    assert got.shape == (rows, width)


def test_block_elementwise_c_abi_errors(lib, gpu):
    x = torch.zeros(4, 1024, dtype=torch.float16, device=gpu)
    w = torch.ones(1024, dtype=torch.float16, device=gpu)
    y = torch.empty_like(x)
    X, W, Y = x.data_ptr(), w.data_ptr(), y.data_ptr()
    n = lib.pa_add_rms_norm
    assert n(X, 1024, None, 0, W, 0, 1e-6, None, 0, Y, 1024, 0, 4, 1024, None) == 0
    assert n(X, 1024, None, 0, W, 0, 1e-6, None, 0, Y, 1024, 0, 0, 1024, None) == 0       # no rows
    assert n(None, 1024, None, 0, W, 0, 1e-6, None, 0, Y, 1024, 0, 4, 1024, None) != 0
    assert n(X, 1024, None, 0, W, 0, 1e-6, Y, 1024, Y, 1024, 0, 4, 1024, None) != 0       # sum_out without delta
    assert n(X, 1024, None, 0, W, 0, 1e-6, None, 0, Y, 1024, 3, 4, 1024, None) != 0       # fp8 activations
    assert n(X, 1024, None, 0, W, 0, 1e-6, None, 0, Y, 1024, 0, 4, 1020, None) != 0       # hidden % 8
    assert n(X, 1024, None, 0, W, 0, 1e-6, None, 0, Y, 1024, 0, 1, 16384, None) != 0      # too wide
    assert n(X, 512, None, 0, W, 0, 1e-6, None, 0, Y, 1024, 0, 4, 1024, None) != 0        # stride < hidden
    assert n(X + 2, 1024, None, 0, W, 0, 1e-6, None, 0, Y, 1024, 0, 3, 1016, None) != 0   # misaligned rows
    assert b"pa_add_rms_norm" in lib.pa_last_error()
    s = lib.pa_silu_mul
    assert s(X, 1024, X + 1024, 1024, Y, 1024, 0, 4, 512, None) == 0
    assert s(X, 1024, None, 1024, Y, 1024, 0, 4, 512, None) != 0
    assert s(X, 1024, X + 1024, 1024, Y, 1024, 0, 4, 500, None) != 0                      # width % 8
    assert s(X, 256, X + 1024, 1024, Y, 1024, 0, 4, 512, None) != 0                       # stride < width
    assert b"pa_silu_mul" in lib.pa_last_error()
    torch.cuda.synchronize()


def test_model_with_and_without_fused_elementwise_agrees(pa, gpu):
    """The decoder built from the fused kernels equals the one built from torch ops: same
    roundings, so logits agree to the last few bits, and the caches they write are identical."""
    from test_gpu_model import Session, small_model
    import dataclasses
    base = small_model(pa, seed=31)
    plain_model = pa.Qwen3PagedModel(dataclasses.replace(base.cfg, fused_elementwise=False)).eval()
    plain_model.load_state_dict(base.state_dict())
    fused, plain = Session(pa, base, gpu), Session(pa, plain_model, gpu)
    assert fused.gpu_model.cfg.fused_elementwise and not plain.gpu_model.cfg.fused_elementwise
    g = torch.Generator().manual_seed(32)
    for n in (21, 64, 50):
        p = torch.randint(0, 512, (n,), generator=g).tolist()
        fused.add(p)
        plain.add(p)
    torch.testing.assert_close(fused.prefill(chunk=32)[0].float().cpu(), plain.prefill(chunk=32)[0].float().cpu(),
                               rtol=1e-2, atol=1e-2)
    torch.testing.assert_close(fused.prefill()[0].float().cpu(), plain.prefill()[0].float().cpu(), rtol=1e-2, atol=1e-2)
    for step in range(3):
        nxt = torch.randint(0, 512, (3,), generator=g).tolist()
        torch.testing.assert_close(fused.decode(nxt).float().cpu(), plain.decode(nxt).float().cpu(), rtol=1e-2, atol=1e-2)
    blk = fused.seqs[0]["block_table"][0]
    torch.testing.assert_close(fused.pool.kv_cache_tensor[:, :, blk].float().cpu(),
                               plain.pool.kv_cache_tensor[:, :, blk].float().cpu(), rtol=1e-2, atol=1e-2)
