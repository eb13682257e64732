"""Training on the mi355x target: the pregrad stage puts the HIP-backed norm and gate ops into the graph, AOT
differentiates through their backward formulas; values and gradients are compared with eager autograd
(reference tests/common/test_fuse_rmsnorm.py:66-85, here with the custom kernels in the forward pass)."""
import pytest
import torch
import torch.nn.functional as F

from xpu_graph_amd import OptLevel, Target, XpuGraph, XpuGraphConfig

pytestmark = pytest.mark.gpu


def backend():
    return XpuGraph(XpuGraphConfig(is_training=True, target=Target.mi355x, opt_level=OptLevel.level2, enable_cache=False))


def block(x, w, g, b, up):
    h = x * torch.rsqrt(x.pow(2).mean(-1, keepdim=True) + 1e-6) * w
    h = F.layer_norm(h, (h.shape[-1],), g, b, 1e-5)
    return F.silu(h) * up


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_norm_gate_block_values_and_gradients(device, dtype):
    torch.manual_seed(0)
    rows, cols = 512, 1024
    mk = lambda *s: torch.randn(*s, device=device).to(dtype).requires_grad_(True)  # noqa: E731
    args = [mk(rows, cols), mk(cols), mk(cols), mk(cols), mk(rows, cols)]
    dy = torch.randn(rows, cols, device=device).to(dtype)
    be = backend()
    y0 = torch.compile(block, backend=be, dynamic=False)(*args)
    g0 = torch.autograd.grad((y0,), args, (dy,))
    pregrad, forward = be.compiled_graphs[0], be.compiled_graphs[1]
    assert [n.target for n in pregrad.graph.nodes if n.op == "call_module"] == ["custom_rms_norm", "custom_layer_norm", "mi355x_silu_mul2"]
    assert [str(n.target) for n in forward.graph.nodes if n.op == "call_function"][:3] == [
        "xpu_ops.rms_norm.default", "xpu_ops.layer_norm.default", "xpu_ops.silu_mul2.default"]
    # reference: the same block in fp32 eager autograd
    ref_args = [a.detach().float().requires_grad_(True) for a in args]
    y1 = block(*ref_args)
    g1 = torch.autograd.grad((y1,), ref_args, (dy.float(),))
    if dtype == torch.float32:
        tol = dict(rtol=1e-4, atol=1e-4)
        torch.testing.assert_close(y0, y1, **tol)
        for a, c in zip(g0, g1):
            torch.testing.assert_close(a, c, rtol=1e-3, atol=1e-3)
    else:
        # bf16: the compiled path must be as close to the fp32 result as eager bf16 autograd is (x2 slack)
        eag_args = [a.detach().clone().requires_grad_(True) for a in args]
        y2 = block(*eag_args)
        g2 = torch.autograd.grad((y2,), eag_args, (dy,))
        err = lambda a, c: (a.float() - c).abs().mean().item()  # noqa: E731
        assert err(y0, y1) <= 2 * err(y2, y1) + 1e-3
        for a, c, e in zip(g0, g1, g2):
            assert err(a, c) <= 2 * err(e, c) + 1e-2 * c.abs().mean().item(), (err(a, c), err(e, c))


def test_swiglu_halves_gradient(device):
    def fn(x):
        d = x.shape[-1] // 2
        return F.silu(x[..., :d]) * x[..., d:]

    x = torch.randn(256, 512, device=device, requires_grad=True)
    dy = torch.randn(256, 256, device=device)
    be = backend()
    y0 = torch.compile(fn, backend=be, dynamic=False)(x)
    (g0,) = torch.autograd.grad((y0,), (x,), (dy,))
    assert "mi355x_silu_mul" in [n.target for n in be.compiled_graphs[0].graph.nodes if n.op == "call_module"]
    (g1,) = torch.autograd.grad((fn(x),), (x,), (dy,))
    torch.testing.assert_close(y0, fn(x), rtol=1e-5, atol=1e-5)
    torch.testing.assert_close(g0, g1, rtol=1e-4, atol=1e-4)


@pytest.mark.parametrize("dtype,wdtype", [(torch.float32, torch.float32), (torch.bfloat16, torch.bfloat16), (torch.bfloat16, torch.float32), (torch.float16, torch.float16)])
@pytest.mark.parametrize("rows,cols", [(1, 8), (37, 64), (300, 4096), (2050, 1024), (5, 16384), (1500, 2056)])
@pytest.mark.parametrize("with_res,with_gh,with_w", [(False, False, True), (True, True, True), (True, False, False)])
def test_rms_norm_backward_kernel(device, dtype, wdtype, rows, cols, with_res, with_gh, with_w):
    """xg_rms_norm_bwd against float64 autograd of the same forward (the residual sum rounded to the storage type,
    as the forward kernel rounds it): fp32 row statistics, one rounding of gx; the weight gradient summed over rows
    from per-block fp32 partials.  Row counts that do not divide among the blocks, one to eight chunks per lane."""
    import xpu_graph_amd.ops  # noqa: F401

    if dtype == torch.float32 and cols > 8192:
        pytest.skip("fp32 rows hold at most 8192 columns in the kernel")
    gen = torch.Generator().manual_seed(rows + cols)
    x = torch.randn(rows, cols, generator=gen).to(dtype).to(device)
    res = torch.randn(rows, cols, generator=gen).to(dtype).to(device) if with_res else None
    w = (1 + 0.2 * torch.randn(cols, generator=gen)).to(wdtype).to(device) if with_w else None
    gy = torch.randn(rows, cols, generator=gen).to(dtype).to(device)
    gh = torch.randn(rows, cols, generator=gen).to(dtype).to(device) if with_gh else None
    gx, gw = torch.ops.xpu_ops.rms_norm_bwd(x, res, w, gy, gh, 1e-6, True)
    h = (x + res) if with_res else x  # rounded to the storage type
    h64 = h.double().requires_grad_(True)
    w64 = w.double().requires_grad_(True) if with_w else None
    y = h64 * torch.rsqrt(h64.pow(2).mean(-1, keepdim=True) + 1e-6)
    y = y * w64 if with_w else y
    grads = torch.autograd.grad(y, (h64, w64) if with_w else (h64,), gy.double())
    want_gx = grads[0] + (gh.double() if with_gh else 0)
    ulp = {torch.float32: 2.0**-23, torch.bfloat16: 2.0**-8, torch.float16: 2.0**-11}[dtype]
    assert gx.shape == x.shape and gx.dtype == dtype
    torch.testing.assert_close(gx.double(), want_gx, rtol=1.01 * ulp, atol=want_gx.abs().max().item() * max(ulp * 2.0**-6, 2e-6))
    if with_w:
        wulp = {torch.float32: 2.0**-23, torch.bfloat16: 2.0**-8, torch.float16: 2.0**-11}[wdtype]
        assert gw.shape == w.shape and gw.dtype == wdtype
        torch.testing.assert_close(gw.double(), grads[1], rtol=1.01 * wulp, atol=grads[1].abs().max().item() * max(wulp * 2.0**-6, 1e-5))
    else:
        assert gw.numel() == 0


@pytest.mark.parametrize("dtype,wdtype", [(torch.float32, torch.float32), (torch.bfloat16, torch.bfloat16), (torch.bfloat16, torch.float32), (torch.float16, torch.float16)])
@pytest.mark.parametrize("rows,cols", [(1, 8), (37, 64), (300, 4096), (2050, 1024), (5, 16384), (1500, 2056)])
@pytest.mark.parametrize("with_res,with_gh,with_w", [(False, False, True), (True, True, True), (True, False, False)])
def test_layer_norm_backward_kernel(device, dtype, wdtype, rows, cols, with_res, with_gh, with_w):
    """xg_layer_norm_bwd against float64 autograd of the same forward, rows with a mean far from zero (the centred
    sums must not cancel): gx, the weight gradient and the bias gradient (the column sums of gy)."""
    import xpu_graph_amd.ops  # noqa: F401

    if dtype == torch.float32 and cols > 8192:
        pytest.skip("fp32 rows hold at most 8192 columns in the kernel")
    gen = torch.Generator().manual_seed(rows + 3 * cols)
    x = (3.0 + torch.randn(rows, cols, generator=gen)).to(dtype).to(device)
    res = torch.randn(rows, cols, generator=gen).to(dtype).to(device) if with_res else None
    w = (1 + 0.2 * torch.randn(cols, generator=gen)).to(wdtype).to(device) if with_w else None
    gy = torch.randn(rows, cols, generator=gen).to(dtype).to(device)
    gh = torch.randn(rows, cols, generator=gen).to(dtype).to(device) if with_gh else None
    gx, gw, gb = torch.ops.xpu_ops.layer_norm_bwd(x, res, w, gy, gh, 1e-5, True, True)
    h = (x + res) if with_res else x  # rounded to the storage type
    h64 = h.double().requires_grad_(True)
    w64 = w.double().requires_grad_(True) if with_w else None
    hc = h64 - h64.mean(-1, keepdim=True)
    y = hc * torch.rsqrt(hc.pow(2).mean(-1, keepdim=True) + 1e-5)
    y = y * w64 if with_w else y
    grads = torch.autograd.grad(y, (h64, w64) if with_w else (h64,), gy.double())
    want_gx = grads[0] + (gh.double() if with_gh else 0)
    ulp = {torch.float32: 2.0**-23, torch.bfloat16: 2.0**-8, torch.float16: 2.0**-11}[dtype]
    assert gx.shape == x.shape and gx.dtype == dtype
    # the row mean is an fp32 sum of up to 16384 values near 3: its rounding enters every centred value
    torch.testing.assert_close(gx.double(), want_gx, rtol=1.01 * ulp, atol=want_gx.abs().max().item() * max(ulp * 2.0**-6, 1e-5))
    out_dt = wdtype if with_w else dtype
    wulp = {torch.float32: 2.0**-23, torch.bfloat16: 2.0**-8, torch.float16: 2.0**-11}[out_dt]
    want_gb = gy.double().sum(0)
    assert gb.shape == (cols,) and gb.dtype == out_dt
    torch.testing.assert_close(gb.double(), want_gb, rtol=1.01 * wulp, atol=want_gb.abs().max().item() * max(wulp * 2.0**-6, 1e-5))
    if with_w:
        assert gw.shape == w.shape and gw.dtype == wdtype
        torch.testing.assert_close(gw.double(), grads[1], rtol=1.01 * wulp, atol=grads[1].abs().max().item() * max(wulp * 2.0**-6, 1e-5))
    else:
        assert gw.numel() == 0
    only_gx = torch.ops.xpu_ops.layer_norm_bwd(x, res, w, gy, gh, 1e-5, False, False)
    assert torch.equal(only_gx[0], gx) and only_gx[1].numel() == 0 and only_gx[2].numel() == 0


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16])
@pytest.mark.parametrize("shape", [(256, 512), (3, 5, 7), (1, 1), (8192, 1376)])
def test_gate_backward_kernel(device, dtype, shape):
    """xg_silu_mul2_bwd against autograd of silu(g) * u evaluated in float64 on the same inputs: fp32 math and one
    rounding per output (rtol 1e-5 for fp32, half an ulp of the output type otherwise); vector and scalar paths."""
    import xpu_graph_amd.ops  # noqa: F401

    gen = torch.Generator().manual_seed(sum(shape))
    g, u, gy = (torch.randn(*shape, generator=gen).to(dtype).to(device) for _ in range(3))
    dg, du = torch.ops.xpu_ops.silu_mul2_bwd(g, u, gy)
    g64, u64 = g.double().requires_grad_(True), u.double().requires_grad_(True)
    wg, wu = torch.autograd.grad(F.silu(g64) * u64, (g64, u64), gy.double())
    rtol = {torch.float32: 1e-5, torch.bfloat16: 2.0**-8, torch.float16: 2.0**-11}[dtype]
    for got, want in ((dg, wg), (du, wu)):
        assert got.dtype == dtype and got.shape == g.shape
        torch.testing.assert_close(got.double(), want, rtol=rtol * 1.01, atol=1e-6 if dtype == torch.float32 else rtol * 2.0**-10)


@pytest.mark.parametrize("act", ["none", "relu", "sigmoid", "silu", "gelu"])
@pytest.mark.parametrize("weight_trans", [True, False])
def test_dense_backward_formula(device, act, weight_trans):
    """Gradients of xpu_ops.dense (input gradient on the HIP kernel, weight gradient an Aten matmul) against
    autograd of the same layer evaluated in fp32."""
    import xpu_graph_amd.ops as xops

    xops.enable_autograd()
    torch.manual_seed(1)
    M, K, N = 384, 256, 192
    bf = torch.bfloat16
    x = torch.randn(M, K, device=device).to(bf).requires_grad_(True)
    w = (torch.randn(N, K, device=device) / 16 if weight_trans else torch.randn(K, N, device=device) / 16).to(bf).requires_grad_(True)
    b = torch.randn(N, device=device).to(bf).requires_grad_(True)
    r = torch.randn(M, N, device=device).to(bf).requires_grad_(True)
    dy = torch.randn(M, N, device=device).to(bf)
    y = torch.ops.xpu_ops.dense(x, w, weight_trans, b, r, act)
    g = torch.autograd.grad((y,), (x, w, b, r), (dy,))
    fx, fw, fb, fr = (t.detach().float().requires_grad_(True) for t in (x, w, b, r))
    z = fx @ (fw.t() if weight_trans else fw) + fb + fr
    ref = {"none": lambda t: t, "relu": torch.relu, "sigmoid": torch.sigmoid, "silu": F.silu, "gelu": F.gelu}[act](z)
    gref = torch.autograd.grad((ref,), (fx, fw, fb, fr), (dy.float(),))
    torch.testing.assert_close(y.float(), ref, rtol=1.6e-2, atol=3e-2)
    for name, a, c in zip("x w b r".split(), g, gref):
        scale = c.abs().mean().item()
        assert (a.float() - c).abs().mean().item() <= 2e-2 * scale + 1e-3, (name, (a.float() - c).abs().mean().item(), scale)


@pytest.mark.parametrize("in_features", [76, 100, 64])
def test_fp32_linear_trains_when_in_features_is_4_mod_8(device, in_features):
    """An fp32 Linear whose in_features is a multiple of 4 and not of 8 fuses (the forward loads four floats at a time)
    and its input gradient - a product whose OUTPUT width is in_features - does not fit the kernel: the backward
    formula takes the Aten product there.  Loss and gradients against eager autograd."""

    def layer(x, w, b):
        return F.silu(F.linear(x, w, b))

    torch.manual_seed(in_features)
    x = torch.randn(40, in_features, device=device, requires_grad=True)
    w = (torch.randn(64, in_features, device=device) / in_features**0.5).requires_grad_(True)
    b = torch.randn(64, device=device, requires_grad=True)
    be = backend()
    y = torch.compile(layer, backend=be, dynamic=False)(x, w, b)
    fwd_ops = [str(n.target) for n in be.compiled_graphs[1].graph.nodes if n.op == "call_function"]
    assert "xpu_ops.dense.default" in fwd_ops, fwd_ops
    g = torch.autograd.grad(y.pow(2).mean(), (x, w, b))
    args = [t.detach().double().requires_grad_(True) for t in (x, w, b)]
    want_y = layer(*args)
    want = torch.autograd.grad(want_y.pow(2).mean(), args)
    torch.testing.assert_close(y.double(), want_y, rtol=1e-5, atol=1e-5)
    for a, c in zip(g, want):
        torch.testing.assert_close(a.double(), c, rtol=1e-4, atol=1e-6)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16])
@pytest.mark.parametrize("act", ["relu", "gelu", "silu", "sigmoid"])
@pytest.mark.parametrize("shape", [(256, 512), (3, 5, 7), (1,), (4096, 1376)])
def test_activation_kernel_and_its_backward(device, dtype, act, shape):
    """xg_activation / xg_activation_bwd against float64 autograd of the same activation: fp32 math on the stored
    values, one rounding."""
    import xpu_graph_amd.ops  # noqa: F401

    gen = torch.Generator().manual_seed(len(shape) + shape[0])
    z = (2 * torch.randn(*shape, generator=gen)).to(dtype).to(device)
    gy = torch.randn(*shape, generator=gen).to(dtype).to(device)
    fn = {"relu": torch.relu, "gelu": F.gelu, "silu": F.silu, "sigmoid": torch.sigmoid}[act]
    z64 = z.double().requires_grad_(True)
    want_y = fn(z64)
    (want_g,) = torch.autograd.grad(want_y, z64, gy.double())
    y = torch.ops.xpu_ops.act(z, act)
    gz = torch.ops.xpu_ops.act_bwd(z, gy, act)
    ulp = {torch.float32: 2.0**-23, torch.bfloat16: 2.0**-8, torch.float16: 2.0**-11}[dtype]
    assert y.shape == z.shape and y.dtype == dtype and gz.shape == z.shape and gz.dtype == dtype
    # the hardware exp2 / reciprocal are good to about an ulp of fp32 each; near a zero of the result their error
    # shows against the size of the terms that cancel
    torch.testing.assert_close(y.double(), want_y.detach(), rtol=1.01 * ulp + 4e-7, atol=1e-6)
    torch.testing.assert_close(gz.double(), want_g, rtol=1.01 * ulp + 4e-7, atol=2e-6 * max(1.0, gy.abs().max().item()))


def test_mlp_training_step(device):
    """RMSNorm -> linear + bias -> SiLU -> linear, compiled for training on the mi355x target: the forward graph
    calls the HIP norm and dense kernels, loss and gradients follow eager."""

    def mlp(x, w1, b1, w2, nw):
        h = x * torch.rsqrt(x.pow(2).mean(-1, keepdim=True) + 1e-6) * nw
        return F.linear(F.silu(F.linear(h, w1, b1)), w2)

    torch.manual_seed(2)
    bf = torch.bfloat16
    mk = lambda *s, k=1.0: (torch.randn(*s, device=device) * k).to(bf).requires_grad_(True)  # noqa: E731
    args = [mk(4, 128, 512), mk(1024, 512, k=0.05), mk(1024, k=0.1), mk(512, 1024, k=0.05), mk(512)]
    be = backend()
    y0 = torch.compile(mlp, backend=be, dynamic=False)(*args)
    loss0 = y0.float().pow(2).mean()
    g0 = torch.autograd.grad(loss0, args)
    fwd_ops = [str(n.target) for n in be.compiled_graphs[1].graph.nodes if n.op == "call_function"]
    assert fwd_ops.count("xpu_ops.dense.default") == 2 and "xpu_ops.rms_norm.default" in fwd_ops
    assert not any("aten.mm" in t or "aten.addmm" in t for t in fwd_ops)
    # the activated layer of a differentiated graph keeps its pre-activation: activation and its backward are one
    # pass each, and the backward runs no product beyond the input- and weight-gradient ones
    bwd_ops = [str(n.target) for n in be.compiled_graphs[2].graph.nodes if n.op == "call_function"]
    assert fwd_ops.count("xpu_ops.act.default") == 1 and bwd_ops.count("xpu_ops.act_bwd.default") == 1, (fwd_ops, bwd_ops)
    assert bwd_ops.count("xpu_ops.dense.default") == 2 and not any("aten.sigmoid" in t or "aten.silu" in t for t in bwd_ops), bwd_ops
    ref_args = [a.detach().float().requires_grad_(True) for a in args]
    loss1 = mlp(*ref_args).pow(2).mean()
    g1 = torch.autograd.grad(loss1, ref_args)
    assert abs(loss0.item() - loss1.item()) <= 2e-2 * abs(loss1.item())
    eag_args = [a.detach().clone().requires_grad_(True) for a in args]
    g2 = torch.autograd.grad(mlp(*eag_args).float().pow(2).mean(), eag_args)
    err = lambda a, c: (a.float() - c).abs().mean().item()  # noqa: E731
    for a, c, e in zip(g0, g1, g2):
        assert err(a, c) <= 2 * err(e, c) + 1e-2 * c.abs().mean().item(), (err(a, c), err(e, c), c.abs().mean().item())


def test_gated_dense_backward_formula(device):
    """Gradients of xpu_ops.dense_glu (projections recomputed and input gradient on the HIP dense kernel, weight
    gradients Aten matmuls) against autograd of silu(x Wg^T) * (x Wu^T) evaluated in fp32."""
    import xpu_graph_amd.ops as xops

    xops.enable_autograd()
    torch.manual_seed(3)
    M, K, N = 384, 256, 192
    bf = torch.bfloat16
    x = torch.randn(M, K, device=device).to(bf).requires_grad_(True)
    wg = (torch.randn(N, K, device=device) / 16).to(bf).requires_grad_(True)
    wu = (torch.randn(N, K, device=device) / 16).to(bf).requires_grad_(True)
    dy = torch.randn(M, N, device=device).to(bf)
    y = torch.ops.xpu_ops.dense_glu(x, wg, wu)
    g = torch.autograd.grad((y,), (x, wg, wu), (dy,))
    fx, fg, fu = (t.detach().float().requires_grad_(True) for t in (x, wg, wu))
    ref = F.silu(fx @ fg.t()) * (fx @ fu.t())
    gref = torch.autograd.grad((ref,), (fx, fg, fu), (dy.float(),))
    torch.testing.assert_close(y.float(), ref, rtol=1.6e-2, atol=3e-2)
    for name, a, c in zip("x wg wu".split(), g, gref):
        scale = c.abs().mean().item()
        assert (a.float() - c).abs().mean().item() <= 2e-2 * scale + 1e-3, (name, (a.float() - c).abs().mean().item(), scale)


def test_gated_dense_that_saves_its_projections(device):
    """dense_glu_save returns the gated output bit-identical to dense_glu plus the two projections bit-identical to
    two dense layers (large tiles and the small-grid kernel), and its backward -- no recomputation -- gives the
    gradients of the recomputing formula bit for bit."""
    import xpu_graph_amd.ops as xops

    xops.enable_autograd()
    ops = torch.ops.xpu_ops
    for M, K, N in ((4096, 512, 2816), (96, 256, 264)):
        gen = torch.Generator().manual_seed(M + N)
        x = torch.randn(M, K, generator=gen).bfloat16().to(device)
        wg = (torch.randn(N, K, generator=gen) / K**0.5).bfloat16().to(device)
        wu = (torch.randn(N, K, generator=gen) / K**0.5).bfloat16().to(device)
        y, gate, up = ops.dense_glu_save(x, wg, wu)
        assert torch.equal(y, ops.dense_glu(x, wg, wu))
        assert torch.equal(gate, ops.dense(x, wg, True, None, None, "none")) and torch.equal(up, ops.dense(x, wu, True, None, None, "none"))
        dy = torch.randn(M, N, generator=gen).bfloat16().to(device)
        grads = []
        for op in ("dense_glu", "dense_glu_save"):
            leaves = [t.clone().requires_grad_(True) for t in (x, wg, wu)]
            out = getattr(ops, op)(*leaves)
            out = out[0] if op == "dense_glu_save" else out
            grads.append(torch.autograd.grad(out, leaves, dy))
        assert all(torch.equal(a, b) for a, b in zip(*grads))


def test_gated_mlp_training_step(device):
    """RMSNorm -> SwiGLU MLP (gate, up, down projections), compiled for training on the mi355x target: the forward
    graph calls the gated dense kernel once and the dense kernel once, loss and gradients follow eager."""

    def mlp(x, nw, wg, wu, wd):
        h = x * torch.rsqrt(x.pow(2).mean(-1, keepdim=True) + 1e-6) * nw
        return x + F.linear(F.silu(F.linear(h, wg)) * F.linear(h, wu), wd)

    torch.manual_seed(4)
    bf = torch.bfloat16
    mk = lambda *s, k=1.0: (torch.randn(*s, device=device) * k).to(bf).requires_grad_(True)  # noqa: E731
    args = [mk(4, 128, 512), mk(512), mk(1024, 512, k=0.05), mk(1024, 512, k=0.05), mk(512, 1024, k=0.05)]
    be = backend()
    y0 = torch.compile(mlp, backend=be, dynamic=False)(*args)
    loss0 = y0.float().pow(2).mean()
    g0 = torch.autograd.grad(loss0, args)
    fwd_ops = [str(n.target) for n in be.compiled_graphs[1].graph.nodes if n.op == "call_function"]
    # a graph that is differentiated runs the gated layer that also saves its two projections for the backward
    assert fwd_ops.count("xpu_ops.dense_glu_save.default") == 1 and fwd_ops.count("xpu_ops.dense.default") == 1, fwd_ops
    assert not any("aten.mm" in t or "aten.addmm" in t for t in fwd_ops)
    ref_args = [a.detach().float().requires_grad_(True) for a in args]
    loss1 = mlp(*ref_args).pow(2).mean()
    g1 = torch.autograd.grad(loss1, ref_args)
    assert abs(loss0.item() - loss1.item()) <= 2e-2 * abs(loss1.item())
    eag_args = [a.detach().clone().requires_grad_(True) for a in args]
    g2 = torch.autograd.grad(mlp(*eag_args).float().pow(2).mean(), eag_args)
    err = lambda a, c: (a.float() - c).abs().mean().item()  # noqa: E731
    for a, c, e in zip(g0, g1, g2):
        assert err(a, c) <= 2 * err(e, c) + 1e-2 * c.abs().mean().item(), (err(a, c), err(e, c), c.abs().mean().item())


@pytest.mark.parametrize("one_row", [False, True])
@pytest.mark.parametrize("table_grads", [False, True])
def test_rotary_backward_formula(device, table_grads, one_row):
    """The input gradient of xpu_ops.rope is the rotary kernel on a rewritten sine table (halves swapped, negated);
    the table gradients are Aten sums.  Against autograd of the written-out formula in fp32; the sine table has
    different halves so that the swap matters."""
    import xpu_graph_amd.ops as xops

    xops.enable_autograd()
    torch.manual_seed(5)
    B, H, S, D = 2, 4, 96, 64
    bf = torch.bfloat16
    x = torch.randn(B, S, H, D, device=device).to(bf).transpose(1, 2).requires_grad_(True)  # [B, H, S, D] view
    tshape = (D,) if one_row else (S, D)  # one row: shared by every position, so its gradient sums over them too
    cos = torch.randn(*tshape, device=device).to(bf).requires_grad_(table_grads)
    sin = torch.randn(*tshape, device=device).to(bf).requires_grad_(table_grads)
    dy = torch.randn(B, H, S, D, device=device).to(bf)
    wrt = (x, cos, sin) if table_grads else (x,)
    g = torch.autograd.grad((torch.ops.xpu_ops.rope(x, cos, sin),), wrt, (dy,))
    fx, fc, fs = (t.detach().float().requires_grad_(True) for t in (x, cos, sin))
    ref = fx * fc + torch.cat([-fx[..., D // 2:], fx[..., : D // 2]], dim=-1) * fs
    gref = torch.autograd.grad((ref,), (fx, fc, fs) if table_grads else (fx,), (dy.float(),))
    for name, a, c in zip("x cos sin".split(), g, gref):
        scale = c.abs().mean().item()
        assert a.shape == c.shape
        assert (a.float() - c).abs().mean().item() <= 1e-2 * scale + 1e-3, (name, (a.float() - c).abs().mean().item(), scale)


@pytest.mark.parametrize("causal", [True, False])
@pytest.mark.parametrize("kv_heads", [4, 2])
def test_attention_backward_formula(device, causal, kv_heads):
    """Gradients of xpu_ops.sdpa (the backward kernels, row statistics recomputed) against autograd of the written-out attention in
    fp32, with as many or fewer key/value heads than query heads."""
    import xpu_graph_amd.ops as xops

    xops.enable_autograd()
    torch.manual_seed(6)
    B, H, Sq, Skv, D = 2, 4, 96, 96 if causal else 160, 64
    bf = torch.bfloat16
    q = torch.randn(B, H, Sq, D, device=device).to(bf).requires_grad_(True)
    k = torch.randn(B, kv_heads, Skv, D, device=device).to(bf).requires_grad_(True)
    v = torch.randn(B, kv_heads, Skv, D, device=device).to(bf).requires_grad_(True)
    dy = torch.randn(B, H, Sq, D, device=device).to(bf)
    scale = D**-0.5
    y = torch.ops.xpu_ops.sdpa(q, k, v, causal, scale)
    g = torch.autograd.grad((y,), (q, k, v), (dy,))
    fq, fk, fv = (t.detach().float().requires_grad_(True) for t in (q, k, v))
    rep = H // kv_heads
    s = (fq @ fk.repeat_interleave(rep, 1).transpose(-1, -2)) * scale
    if causal:
        s = s.masked_fill(~torch.ones(Sq, Skv, dtype=torch.bool, device=device).tril(), float("-inf"))
    ref = torch.softmax(s, -1) @ fv.repeat_interleave(rep, 1)
    gref = torch.autograd.grad((ref,), (fq, fk, fv), (dy.float(),))
    torch.testing.assert_close(y.float(), ref, rtol=1.6e-2, atol=2e-2)
    for name, a, c in zip("q k v".split(), g, gref):
        scale_ = c.abs().mean().item()
        assert a.shape == c.shape
        assert (a.float() - c).abs().mean().item() <= 1e-2 * scale_ + 1e-3, (name, (a.float() - c).abs().mean().item(), scale_)


def test_attention_training_step(device):
    """A causal self-attention layer (projections, rotary-free, F.scaled_dot_product_attention) compiled for training
    on the mi355x target: the forward graph calls the attention and dense kernels, gradients follow eager."""

    def layer(x, wqkv, wo):
        B, S, E = x.shape
        q, k, v = (t.view(B, S, 4, 64).transpose(1, 2) for t in F.linear(x, wqkv).split(E, dim=-1))
        a = F.scaled_dot_product_attention(q, k, v, is_causal=True)
        return F.linear(a.transpose(1, 2).reshape(B, S, E), wo)

    torch.manual_seed(7)
    bf = torch.bfloat16
    mk = lambda *s, k=1.0: (torch.randn(*s, device=device) * k).to(bf).requires_grad_(True)  # noqa: E731
    args = [mk(2, 128, 256), mk(768, 256, k=0.06), mk(256, 256, k=0.06)]
    be = backend()
    y0 = torch.compile(layer, backend=be, dynamic=False)(*args)
    g0 = torch.autograd.grad(y0.float().pow(2).mean(), args)
    fwd_ops = [str(n.target) for n in be.compiled_graphs[1].graph.nodes if n.op == "call_function"]
    # a graph that is differentiated runs the attention that also saves the row statistics for the backward kernels
    assert fwd_ops.count("xpu_ops.sdpa_lse.default") == 1 and fwd_ops.count("xpu_ops.dense.default") == 2, fwd_ops
    bwd_ops = [str(n.target) for gm in be.compiled_graphs[2:] for n in gm.graph.nodes if n.op == "call_function"]
    assert bwd_ops.count("xpu_ops.sdpa_bwd.default") == 1 and bwd_ops.count("xpu_ops.dense_at.default") == 2, bwd_ops
    ref_args = [a.detach().float().requires_grad_(True) for a in args]
    g1 = torch.autograd.grad(layer(*ref_args).pow(2).mean(), ref_args)
    eag_args = [a.detach().clone().requires_grad_(True) for a in args]
    g2 = torch.autograd.grad(layer(*eag_args).float().pow(2).mean(), eag_args)
    err = lambda a, c: (a.float() - c).abs().mean().item()  # noqa: E731
    for a, c, e in zip(g0, g1, g2):
        assert err(a, c) <= 2 * err(e, c) + 1e-2 * c.abs().mean().item(), (err(a, c), err(e, c), c.abs().mean().item())


def test_attention_with_a_padding_mask_trains_on_the_kernels(device):
    """The attn_mask form in a training graph (reference passes/patterns/common/fuse_scaled_dot_product_attention.py:
    184-234): a mask that needs no gradient (padded keys, given as a graph input) goes to the attention kernels, forward
    and backward; a learned additive bias does need one, so that attention stays on Aten and the bias is trained."""

    def layer(x, wqkv, wo, mask):
        B, S, E = x.shape
        q, k, v = (t.view(B, S, 4, 64).transpose(1, 2) for t in F.linear(x, wqkv).split(E, dim=-1))
        a = F.scaled_dot_product_attention(q, k, v, attn_mask=mask)
        return F.linear(a.transpose(1, 2).reshape(B, S, E), wo)

    torch.manual_seed(11)
    bf = torch.bfloat16
    mk = lambda *s, k=1.0: (torch.randn(*s, device=device) * k).to(bf).requires_grad_(True)  # noqa: E731
    args = [mk(2, 128, 256), mk(768, 256, k=0.06), mk(256, 256, k=0.06)]
    pad = torch.zeros(2, 1, 128, 128, device=device, dtype=bf)
    pad[0, :, :, 100:] = float("-inf")
    pad[1, :, :, 77:] = float("-inf")
    be = backend()
    y0 = torch.compile(layer, backend=be, dynamic=False)(*args, pad)
    g0 = torch.autograd.grad(y0.float().pow(2).mean(), args)
    fwd_ops = [str(n.target) for n in be.compiled_graphs[1].graph.nodes if n.op == "call_function"]
    assert fwd_ops.count("xpu_ops.sdpa_masked_lse.default") == 1, fwd_ops
    bwd_ops = [str(n.target) for gm in be.compiled_graphs[2:] for n in gm.graph.nodes if n.op == "call_function"]
    assert bwd_ops.count("xpu_ops.sdpa_masked_bwd.default") == 1, bwd_ops
    ref_args = [a.detach().float().requires_grad_(True) for a in args]
    g1 = torch.autograd.grad(layer(*ref_args, pad.float()).pow(2).mean(), ref_args)
    eag_args = [a.detach().clone().requires_grad_(True) for a in args]
    g2 = torch.autograd.grad(layer(*eag_args, pad).float().pow(2).mean(), eag_args)
    err = lambda a, c: (a.float() - c).abs().mean().item()  # noqa: E731
    for a, c, e in zip(g0, g1, g2):
        assert err(a, c) <= 2 * err(e, c) + 1e-2 * c.abs().mean().item(), (err(a, c), err(e, c), c.abs().mean().item())

    bias = (torch.randn(1, 4, 128, 128, device=device) * 0.5).to(bf).requires_grad_(True)
    be2 = backend()
    y = torch.compile(layer, backend=be2, dynamic=False)(*args, bias)
    gb = torch.autograd.grad(y.float().pow(2).mean(), [bias])[0]
    ops2 = [str(n.target) for gm in be2.compiled_graphs[1:] for n in gm.graph.nodes if n.op == "call_function"]
    assert not any("sdpa_masked" in o for o in ops2), ops2

    def written_out(x, wqkv, wo, mask):  # (eager's fused attention backward refuses a bias that alone needs a gradient)
        B, S, E = x.shape
        q, k, v = (t.view(B, S, 4, 64).transpose(1, 2) for t in F.linear(x, wqkv).split(E, dim=-1))
        a = torch.softmax(q @ k.transpose(-1, -2) / 8.0 + mask, dim=-1) @ v
        return F.linear(a.transpose(1, 2).reshape(B, S, E), wo)

    ref_bias = bias.detach().float().requires_grad_(True)
    want = torch.autograd.grad(written_out(*[a.detach().float() for a in args], ref_bias).pow(2).mean(), [ref_bias])[0]
    assert (gb.float() - want).abs().mean().item() <= 0.1 * want.abs().mean().item() + 1e-6


def test_grouped_query_attention_trains_unrepeated(device):
    """`repeat_kv` + causal attention compiled for training: the pregrad stage hands the kernels the unrepeated keys and
    values, the backward kernels sum the gradients of a group's query heads, and dq, dk, dv follow fp32 autograd of the
    written-out form."""

    def repeat_kv(h, n):
        b, hk, s, d = h.shape
        return h[:, :, None, :, :].expand(b, hk, n, s, d).reshape(b, hk * n, s, d)

    def att(q, k, v):
        return F.scaled_dot_product_attention(q, repeat_kv(k, 4), repeat_kv(v, 4), is_causal=True)

    torch.manual_seed(5)
    bf = torch.bfloat16
    q = torch.randn(2, 8, 192, 64, device=device).to(bf).requires_grad_(True)
    k, v = (torch.randn(2, 2, 192, 64, device=device).to(bf).requires_grad_(True) for _ in range(2))
    be = backend()
    y = torch.compile(att, backend=be, dynamic=False)(q, k, v)
    g0 = torch.autograd.grad(y.float().pow(2).mean(), (q, k, v))
    fwd_ops = [str(n.target) for n in be.compiled_graphs[1].graph.nodes if n.op == "call_function"]
    assert fwd_ops.count("xpu_ops.sdpa_lse.default") == 1 and not any("expand" in o or "clone" in o for o in fwd_ops), fwd_ops
    ref = [t.detach().float().requires_grad_(True) for t in (q, k, v)]
    g1 = torch.autograd.grad(att(*ref).pow(2).mean(), ref)
    eag = [t.detach().clone().requires_grad_(True) for t in (q, k, v)]
    g2 = torch.autograd.grad(att(*eag).float().pow(2).mean(), eag)
    err = lambda a, c: (a.float() - c).abs().mean().item()  # noqa: E731
    for a, c, e in zip(g0, g1, g2):
        assert a.shape == c.shape
        assert err(a, c) <= 2 * err(e, c) + 1e-2 * c.abs().mean().item(), (err(a, c), err(e, c), c.abs().mean().item())


def test_llama_block_training_step(device):
    """The whole decoder block of benchmark config 5 (small batch and sequence), compiled for training on the mi355x
    target: the forward graph runs on the HIP kernels, and the gradients of every weight follow fp32 autograd as
    closely as eager bf16 does."""
    from collections import Counter

    from oracle import eager, inputs

    torch.manual_seed(8)
    x, p = inputs.c5_llama_block(B=2, S=128, device=device)
    names = sorted(p)

    def block(x, *w):
        return eager.llama_block_eager(x, dict(zip(names, w)), n_heads=32)

    args = [x.detach().requires_grad_(True)] + [p[n].detach().requires_grad_(True) for n in names]
    be = backend()
    y0 = torch.compile(block, backend=be, dynamic=False)(*args)
    g0 = torch.autograd.grad(y0.float().pow(2).mean(), args)
    ops = Counter(str(n.target) for n in be.compiled_graphs[1].graph.nodes if n.op == "call_function")
    assert ops["xpu_ops.dense_glu_save.default"] == 1 and ops["xpu_ops.dense.default"] >= 5 and ops["xpu_ops.rope.default"] == 2, ops
    assert ops["xpu_ops.add_rms_norm.default"] == 1, ops  # the attention residual add rides in the second norm
    ref_args = [a.detach().float().requires_grad_(True) for a in args]
    g1 = torch.autograd.grad(block(*ref_args).pow(2).mean(), ref_args)
    eag_args = [a.detach().clone().requires_grad_(True) for a in args]
    g2 = torch.autograd.grad(block(*eag_args).float().pow(2).mean(), eag_args)
    err = lambda a, c: (a.float() - c).abs().mean().item()  # noqa: E731
    for name, a, c, e in zip(["x"] + names, g0, g1, g2):
        assert err(a, c) <= 2 * err(e, c) + 2e-2 * c.abs().mean().item(), (name, err(a, c), err(e, c), c.abs().mean().item())


def test_llama_block_training_step_full_size_holds_no_score_matrix(device):
    """The block at its benchmark size (B4 S2048, 32 heads of 128): no tensor of the forward or backward graph is as
    large as one [B, H, S, S] score matrix, the step's peak memory is below eager's (which holds several), the
    backward runs the attention-backward and transposed-operand dense kernels, and the gradients follow fp32
    autograd as closely as eager bf16 does."""
    from collections import Counter

    from oracle import eager, inputs

    torch.manual_seed(9)
    B, S, H = 4, 2048, 32
    x, p = inputs.c5_llama_block(B=B, S=S, device=device)
    names = sorted(p)

    def block(x, *w):
        return eager.llama_block_eager(x, dict(zip(names, w)), n_heads=H)

    def step(fn, args):
        torch.cuda.synchronize()
        torch.cuda.reset_peak_memory_stats()
        base = torch.cuda.memory_allocated()
        g = torch.autograd.grad(fn(*args).float().pow(2).mean(), args)
        torch.cuda.synchronize()
        return g, torch.cuda.max_memory_allocated() - base

    args = [x.detach().requires_grad_(True)] + [p[n].detach().requires_grad_(True) for n in names]
    be = backend()
    compiled = torch.compile(block, backend=be, dynamic=False)
    step(compiled, args)  # compiles; the second step is the one measured
    g0, peak_compiled = step(compiled, args)
    eag_args = [a.detach().clone().requires_grad_(True) for a in args]
    g2, peak_eager = step(block, eag_args)
    score_elems = B * H * S * S
    for gm in be.compiled_graphs[1:]:
        for n in gm.graph.nodes:
            val = n.meta.get("val")
            vals = val if isinstance(val, (list, tuple)) else [val]
            assert all(not isinstance(t, torch.Tensor) or t.numel() < score_elems for t in vals), (n, [tuple(t.shape) for t in vals if isinstance(t, torch.Tensor)])
    assert peak_compiled < peak_eager, (peak_compiled, peak_eager)
    ops = Counter(str(n.target) for gm in be.compiled_graphs[2:] for n in gm.graph.nodes if n.op == "call_function")
    assert ops["xpu_ops.sdpa_bwd.default"] == 1 and ops["xpu_ops.dense_at.default"] >= 5, ops
    # gradient sums and layout copies ride on the kernels next to them: none is left as a launch of its own
    both = Counter(str(n.target) for gm in be.compiled_graphs[1:] for n in gm.graph.nodes if n.op == "call_function")
    assert both["aten.add.Tensor"] == 0 and both["aten.clone.default"] == 0, both
    ref_args = [a.detach().float().requires_grad_(True) for a in args]
    g1 = torch.autograd.grad(block(*ref_args).pow(2).mean(), ref_args)
    err = lambda a, c: (a.float() - c).abs().mean().item()  # noqa: E731
    for name, a, c, e in zip(["x"] + names, g0, g1, g2):
        assert err(a, c) <= 2 * err(e, c) + 2e-2 * c.abs().mean().item(), (name, err(a, c), err(e, c), c.abs().mean().item())
    print(f"peak memory of one training step: compiled {peak_compiled / 2**30:.2f} GiB, eager {peak_eager / 2**30:.2f} GiB")


@pytest.mark.parametrize("kind", ["rms", "layer"])
@pytest.mark.parametrize("with_sum", [True, False])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_add_norm_backward_formulas(device, kind, with_sum, dtype):
    """Gradients of the residual-add + norm ops (both addends, weight, bias; with the sum returned and used, or
    not returned) against autograd of the written-out formula in fp32."""
    import xpu_graph_amd.ops as xops

    xops.enable_autograd()
    torch.manual_seed(9)
    rows, cols = 96, 512
    mk = lambda *s: torch.randn(*s, device=device).to(dtype).requires_grad_(True)  # noqa: E731
    x, r, w, b = mk(rows, cols), mk(rows, cols), mk(cols), mk(cols)
    dy, dh = torch.randn(rows, cols, device=device).to(dtype), torch.randn(rows, cols, device=device).to(dtype)
    ops = torch.ops.xpu_ops
    if kind == "rms":
        out = ops.add_rms_norm(x, r, w, 1e-6) if with_sum else (ops.add_rms_norm_only(x, r, w, 1e-6),)
        wrt = (x, r, w)
    else:
        out = ops.add_layer_norm(x, r, w, b, 1e-5) if with_sum else (ops.add_layer_norm_only(x, r, w, b, 1e-5),)
        wrt = (x, r, w, b)
    g = torch.autograd.grad(tuple(out), wrt, (dy, dh)[: len(out)])
    fx, fr, fw, fb = (t.detach().float().requires_grad_(True) for t in (x, r, w, b))
    h = fx + fr
    if kind == "rms":
        y = h * torch.rsqrt(h.pow(2).mean(-1, keepdim=True) + 1e-6) * fw
        fwrt = (fx, fr, fw)
    else:
        y = F.layer_norm(h, (cols,), fw, fb, 1e-5)
        fwrt = (fx, fr, fw, fb)
    gref = torch.autograd.grad((y, h) if with_sum else (y,), fwrt, (dy.float(), dh.float())[: len(out)])
    tol = 1e-4 if dtype == torch.float32 else 1.5e-2
    for name, a, c in zip("x r w b".split(), g, gref):
        scale = c.abs().mean().item()
        assert (a.float() - c).abs().mean().item() <= tol * scale + 1e-6, (name, (a.float() - c).abs().mean().item(), scale)
