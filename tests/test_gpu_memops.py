"""GPU parity of slice/cat (bit-exact), add-N, combo-sum and SwiGLU kernels
(through torch.ops.xpu_ops -> C ABI) against the eager oracle."""
import pytest
import torch

from oracle import eager, inputs

pytestmark = pytest.mark.gpu

F32 = dict(rtol=1e-5, atol=1e-5)
LOW = dict(rtol=1.6e-2, atol=1e-5)


def _ops():
    import xpu_graph_amd.ops  # noqa: F401

    return torch.ops.xpu_ops


def _slice_cat(src, slice_lists):
    from xpu_graph_amd.ops import build_slice_table

    table, chunk, out_cols = build_slice_table(slice_lists, src.shape[1], src.element_size(), src.stride(0))
    table = table.to(src.device)
    if len(slice_lists) == 1:
        return [_ops().slice_cat(src, table, chunk, out_cols[0])], chunk
    return _ops().slice_cat_multi(src, table, chunk, out_cols), chunk


def test_slice_cat_c3_bit_exact(device):
    src, slices = inputs.c3_slice_cat(device=device)
    (got,), chunk = _slice_cat(src, [slices])
    assert chunk == 16  # 32-float slices move as 128-bit chunks even though the starts are not 16-byte aligned
    assert got.shape == (4096, 2048)
    assert torch.equal(got, eager.slice_cat_eager(src, slices))


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.int64, torch.uint8, torch.float64])
def test_slice_cat_ragged(device, dtype):
    g = torch.Generator().manual_seed(1)
    src = torch.randint(0, 255, (37, 1000), generator=g).to(dtype).to(device)
    slices = [(3, 10), (0, 1), (999, 1000), (500, 757), (10, 10), (128, 256), (1, 2)]
    (got,), _ = _slice_cat(src, [slices])
    assert torch.equal(got, eager.slice_cat_eager(src, slices))
    # brute force on the host: every output element is the source element the index list names
    idx = [c for s, e in slices for c in range(s, e)]
    host = src.cpu()
    want = torch.stack([host[:, c] for c in idx], dim=1)
    assert torch.equal(got.cpu(), want)


def test_slice_cat_multi_output(device):
    src = torch.randn(513, 4310, device=device)
    lists = [[(0, 32), (100, 164)], [(4000, 4310)], [(7, 8), (9, 10), (11, 13)], [(64, 128), (64, 128)]]
    outs, _ = _slice_cat(src, lists)
    assert len(outs) == 4
    for o, sl in zip(outs, lists):
        assert torch.equal(o, eager.slice_cat_eager(src, sl))


def test_slice_cat_strided_source_and_empty(device):
    big = torch.randn(64, 4096, device=device)
    src = big[:, 1024:3072]  # row stride 4096, storage offset 1024
    slices = [(5, 37), (1000, 2048)]
    (got,), _ = _slice_cat(src, [slices])
    assert torch.equal(got, eager.slice_cat_eager(src, slices))
    empty = torch.empty(0, 128, device=device)
    (got,), _ = _slice_cat(empty, [[(0, 64)]])
    assert got.shape == (0, 64)
    with pytest.raises(NotImplementedError):
        _slice_cat(torch.randn(2, 3, 4, device=device), [[(0, 1)]])


def test_addn_c3_fp32_bit_exact(device):
    ts = inputs.c3_addn(device=device)
    got = _ops().addn(ts)
    want = eager.addn_eager(ts)
    assert torch.equal(got, want)  # same left-to-right fp32 order as the eager chain
    torch.testing.assert_close(got, torch.stack(ts).sum(0), **F32)


@pytest.mark.parametrize("n", [1, 2, 4, 9, 64, 65, 130])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16])
def test_addn_counts_and_tails(device, n, dtype):
    ts = inputs.c3_addn(n, 13, 37, device=device, dtype=dtype)  # 481 elements: vector body + scalar tail
    got = _ops().addn(ts)
    ref32 = eager.addn_eager([t.float() for t in ts])
    if dtype == torch.float32:
        assert torch.equal(got, ref32)
    else:
        torch.testing.assert_close(got.float(), ref32, rtol=1.6e-2, atol=0.1)  # sums reach |16|: bf16 ulp 0.0625
    # an input view that is not 16-byte aligned goes through the scalar kernel
    base = torch.randn(13 * 37 + 1, device=device).to(dtype)
    ts2 = [base[1:].view(13, 37)] + ts[1:]
    got2 = _ops().addn(ts2)
    torch.testing.assert_close(got2.float(), eager.addn_eager([t.float() for t in ts2]), rtol=1.6e-2, atol=0.1)


@pytest.mark.parametrize("dim", [1, 2])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_combo_sum(device, dim, dtype):
    g = torch.Generator().manual_seed(3)
    shapes = [(86, 10, 32), (86, 4, 32), (5, 1, 7), (3, 50, 1), (128, 33, 129), (0, 4, 4), (2, 0, 3)]
    ins = [torch.randn(s, generator=g).to(dtype).to(device) for s in shapes]
    outs = _ops().combo_sum(ins, dim)
    assert len(outs) == len(ins)
    for o, t in zip(outs, ins):
        want = t.float().sum(dim=dim)
        assert o.shape == want.shape and o.dtype == dtype
        if dtype == torch.float32:
            torch.testing.assert_close(o, want, rtol=1e-5, atol=1e-5)
        else:
            torch.testing.assert_close(o.float(), want, rtol=1.6e-2, atol=1e-2)
    many = [torch.randn(4, 6, 8, device=device) for _ in range(70)]  # more jobs than one launch holds
    for o, t in zip(_ops().combo_sum(many, dim), many):
        torch.testing.assert_close(o, t.sum(dim=dim), **F32)


@pytest.mark.parametrize("rows,d", [(8192, 11008), (3, 40), (5, 33)])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32, torch.float16])
def test_silu_mul(device, rows, d, dtype):
    if rows * d > 1e7 and dtype != torch.bfloat16:
        pytest.skip("full size only in bf16")
    g = torch.Generator().manual_seed(4)
    x = torch.randn(rows, 2 * d, generator=g).to(dtype).to(device)
    got = _ops().silu_mul(x)
    want = (torch.nn.functional.silu(x[:, :d].float()) * x[:, d:].float())
    tol = F32 if dtype == torch.float32 else dict(rtol=1.6e-2, atol=1e-3)
    torch.testing.assert_close(got.float(), want, **tol)
    if dtype != torch.float32:
        torch.testing.assert_close(got, eager.silu_mul_eager(x), rtol=1.6e-2, atol=1e-2)
    got2 = _ops().silu_mul2(x[:, :d], x[:, d:])
    assert torch.equal(got2, got)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("n_slices,width", [(12, 64), (56, 32), (12, 4), (3, 1)])
def test_fused_slice_module_bit_exact(device, dtype, n_slices, width):
    """The FusedSlice module ([n, rows, width] gather, one launch per 32 slices) against plain slicing; starts are
    arbitrary element offsets as in the reference's tests (tests/mlu/test_fuse_slice.py:13-147)."""
    from xpu_graph_amd.passes.patterns.targets.mi355x.structure_replacements import FuseSliceModule

    g = torch.Generator().manual_seed(n_slices * 1000 + width)
    src = torch.randn(31, 43106, generator=g).to(dtype).to(device)
    starts = torch.randint(0, 43106 - width, (n_slices,), generator=g).tolist()
    got = FuseSliceModule(starts)(src, width)
    assert got.shape == (n_slices, 31, width)
    for k, s0 in enumerate(starts):
        assert torch.equal(got[k], src[:, s0 : s0 + width]), (k, s0)


def test_fused_slice_module_3d_and_strided(device):
    from xpu_graph_amd.passes.patterns.targets.mi355x.structure_replacements import FuseSliceModule

    src = torch.randn(5, 12, 4310, device=device)
    starts = [1257, 1198, 1156, 978, 972]
    got = FuseSliceModule(starts)(src, 4)
    assert got.shape == (5, 5, 12, 4)
    for k, s0 in enumerate(starts):
        assert torch.equal(got[k], src[:, :, s0 : s0 + 4])
    wide = torch.randn(64, 512, device=device)
    view = wide[:, 128:384]  # row stride 512, 256 columns
    got = FuseSliceModule([0, 100, 200])(view, 56)
    for k, s0 in enumerate([0, 100, 200]):
        assert torch.equal(got[k], view[:, s0 : s0 + 56])


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16, torch.float32])
@pytest.mark.parametrize("batch", [86, 512])
def test_slice_sum_cat_op(device, dtype, batch):
    """The shapes of the reference's test (tests/mlu/test_slice_sum_cat.py:67-84) plus slices that do not start at
    row 0, an empty one, a strided source and a column count that forces the scalar path."""
    x = torch.rand(batch, 32, 32, device=device).to(dtype)
    tol = F32 if dtype == torch.float32 else dict(rtol=1.6e-2, atol=1e-3)
    for params in ([(0, 2), (0, 4), (0, 8), (0, 16)], [(3, 9), (0, 32), (31, 32), (5, 5), (16, 20)]):
        got = _ops().slice_sum_cat(x, [a for a, _ in params], [b for _, b in params])
        torch.testing.assert_close(got, eager.slice_sum_cat_eager(x, params), **tol)
    wide = torch.rand(batch, 40, 48, device=device).to(dtype)
    view = wide[:, 4:36, 8:40]  # batch stride 1920, row stride 48, 32 columns
    got = _ops().slice_sum_cat(view, [0, 0, 7], [2, 32, 9])
    torch.testing.assert_close(got, eager.slice_sum_cat_eager(view, [(0, 2), (0, 32), (7, 9)]), **tol)
    odd = torch.rand(batch, 12, 13, device=device).to(dtype)
    got = _ops().slice_sum_cat(odd, [0, 2, 4], [12, 3, 11])
    torch.testing.assert_close(got, eager.slice_sum_cat_eager(odd, [(0, 12), (2, 3), (4, 11)]), **tol)


def test_slice_sum_cat_rejects(device):
    x = torch.rand(4, 8, 16, device=device)
    with pytest.raises(RuntimeError, match="xg_slice_sum_cat"):
        _ops().slice_sum_cat(x, [0, 0, 0], [2, 4, 9])  # end past the rows
    with pytest.raises(ValueError):
        _ops().slice_sum_cat(x, list(range(65)), list(range(65)))
    with pytest.raises(NotImplementedError):
        _ops().slice_sum_cat(x[0], [0], [1])


def test_clock_probe_reads_a_plausible_engine_clock(device):
    """xg_clock_probe on a side stream: every window reports wall-clock ticks at least the window length and a
    shader clock between 50 MHz and 3 GHz; a plain copy beside it does not disturb the launch."""
    import ctypes

    from xpu_graph_amd import _lib

    lib = _lib.lib()
    khz = int(lib.xg_wall_clock_khz())
    assert khz > 0
    n_win, win_us = 25, 20
    buf = torch.zeros(2 * n_win, dtype=torch.int64, device=device)
    a = torch.randn(1 << 22, device=device)
    b = torch.empty_like(a)
    side = torch.cuda.Stream()
    torch.cuda.synchronize()
    assert lib.xg_clock_probe(ctypes.c_void_p(buf.data_ptr()), n_win, win_us * khz // 1000, ctypes.c_void_p(side.cuda_stream)) == 0
    for _ in range(20):
        b.copy_(a)
    torch.cuda.synchronize()
    d = buf.view(n_win, 2).double().cpu()
    assert (d[:, 1] >= win_us * khz // 1000).all()
    ghz = d[:, 0] / d[:, 1] * khz / 1e6
    assert ((ghz > 0.05) & (ghz < 3.0)).all(), ghz
    assert torch.equal(a, b)
