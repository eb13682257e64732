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
