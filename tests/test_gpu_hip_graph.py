"""HIP-graph replay of compiled mi355x graphs (reference GraphRunner: src/xpu_graph/device_graph_runner.py:11-141,
tests/npu/test_npu_graph_runner.py, tests/mlu/test_mlu_graph.py).  The recorded graph is replayed several times
with new input values and eager work and synchronisations in between; every replay is compared with eager."""
import pytest
import torch
import torch.nn.functional as F

from oracle import eager
from xpu_graph_amd import HIPGraphRunner, mi355x_compiler

pytestmark = pytest.mark.gpu


def mlp_block(x, res, g, w1, b1, w2):
    n, h = eager.add_rmsnorm_eager(x, res, g, 1e-6)
    y = F.silu(torch.addmm(b1, n, w1))
    return F.linear(y, w2) + h, h


def test_replays_match_eager(device):
    g = torch.Generator().manual_seed(0)
    bf = torch.bfloat16
    x = torch.randn(256, 512, generator=g).to(bf).to(device)
    res = torch.randn(256, 512, generator=g).to(bf).to(device)
    gam = (1 + 0.1 * torch.randn(512, generator=g)).to(bf).to(device)
    w1 = (0.05 * torch.randn(512, 1024, generator=g)).to(bf).to(device)
    b1 = (0.05 * torch.randn(1024, generator=g)).to(bf).to(device)
    w2 = (0.05 * torch.randn(512, 1024, generator=g)).to(bf).to(device)
    backend = mi355x_compiler()
    compiled = torch.compile(mlp_block, backend=backend, dynamic=False)
    with torch.no_grad():
        compiled(x, res, gam, w1, b1, w2)  # compile outside the capture
    mods = [n.target for n in backend.compiled_graphs[-1].graph.nodes if n.op == "call_module"]
    assert len(mods) >= 3, mods  # add+norm, dense+silu, dense

    runner = HIPGraphRunner(compiled)
    runner.capture(x, res, gam, w1, b1, w2, clone_args=True)
    for step in range(4):
        xs = torch.randn(256, 512, device=device).to(bf) * (step + 1)
        rs = torch.randn(256, 512, device=device).to(bf)
        scratch = torch.randn(1024, 1024, device=device)  # eager work between replays
        (scratch @ scratch).sum().item()  # ... and a synchronisation
        y, h = runner(xs, rs, gam, w1, b1, w2)
        y, h = y.clone(), h.clone()
        with torch.no_grad():
            y_ref, h_ref = mlp_block(xs, rs, gam, w1, b1, w2)
        assert torch.equal(h, h_ref)
        torch.testing.assert_close(y.float(), y_ref.float(), rtol=1.6e-2, atol=3e-2)


def test_runner_rejects_other_shapes_and_resets(device):
    f = torch.compile(lambda a: F.layer_norm(a + a, (64,)), backend=mi355x_compiler(), dynamic=False)
    a = torch.randn(8, 64, device=device).bfloat16()
    with torch.no_grad():
        f(a)
    runner = HIPGraphRunner(f)
    runner.capture(a, clone_args=True)
    torch.testing.assert_close(runner(a).float(), F.layer_norm(a + a, (64,)).float(), rtol=1.6e-2, atol=1e-2)
    with pytest.raises(RuntimeError, match="do not fit"):
        runner(torch.randn(4, 64, device=device).bfloat16())
    again = runner.clone()
    assert again.mempool is None
    again.capture(a, clone_args=True)
    torch.testing.assert_close(again(a).float(), F.layer_norm(a + a, (64,)).float(), rtol=1.6e-2, atol=1e-2)


def test_partitioned_mixed_graph_records_the_device_parts(device):
    """The reference's mixed-device case (tests/mlu/test_mlu_graph.py:62-120): device → host → device; the host
    part stays in the outer module, each device part is recorded and replayed with new inputs."""
    from torch.fx.experimental.proxy_tensor import make_fx

    from xpu_graph_amd.backends.device_graph import device_graph_compiler

    class Mixed(torch.nn.Module):
        def __init__(self):
            super().__init__()
            self.l1 = torch.nn.Linear(32, 32)
            self.l2 = torch.nn.Linear(32, 32)

        def forward(self, x):
            x = self.l1(x)
            x = x.cpu()
            x = x + 1.0
            x = x.to(device)
            return self.l2(x)

    model = Mixed().to(device)
    x1 = torch.randn(16, 32, device=device)
    with torch.no_grad():
        gm = make_fx(model)(x1)
        out = device_graph_compiler(gm, [x1], "cuda")
        regions = [m for _, m in out.named_children() if m.__class__.__name__ == "_LazyXPUGraph"]
        assert len(regions) == 2
        for step in range(3):
            x = torch.randn(16, 32, device=device) * (step + 1)
            torch.testing.assert_close(out(x).clone(), model(x), rtol=1e-3, atol=1e-3)
            (x @ x.t()).sum().item()
        assert all(r.recorded == 1 for r in regions)


def test_backend_with_device_graph_vendor_config(device):
    """XpuGraphConfig(vendor_compiler_config={"compiler": "device_graph"}) as in the reference
    (tests/mlu/test_mlu_graph.py:31-60): the compiled function records on its first call and replays afterwards;
    the recorded region holds the target's kernels."""
    from xpu_graph_amd import OptLevel, Target, XpuGraph, XpuGraphConfig

    bf = torch.bfloat16
    g = torch.Generator().manual_seed(1)
    gam = (1 + 0.1 * torch.randn(512, generator=g)).to(bf).to(device)
    w1 = (0.05 * torch.randn(512, 1024, generator=g)).to(bf).to(device)
    b1 = (0.05 * torch.randn(1024, generator=g)).to(bf).to(device)
    w2 = (0.05 * torch.randn(512, 1024, generator=g)).to(bf).to(device)
    backend = XpuGraph(
        XpuGraphConfig(False, target=Target.mi355x, opt_level=OptLevel.level2, enable_cache=False, vendor_compiler_config={"compiler": "device_graph"})
    )
    compiled = torch.compile(mlp_block, backend=backend, dynamic=False)
    for step in range(4):
        xs = torch.randn(256, 512, device=device).to(bf) * (step + 1)
        rs = torch.randn(256, 512, device=device).to(bf)
        with torch.no_grad():
            y, h = compiled(xs, rs, gam, w1, b1, w2)
            y, h = y.clone(), h.clone()
            y_ref, h_ref = mlp_block(xs, rs, gam, w1, b1, w2)
        (xs.float() @ xs.float().t()).sum().item()  # eager work and a synchronisation between replays
        assert torch.equal(h, h_ref)
        torch.testing.assert_close(y.float(), y_ref.float(), rtol=1.6e-2, atol=3e-2)
    outer = backend.compiled_graphs[-1]  # the partitioner rewrites the module in place: one region holds everything
    (region,) = [m for _, m in outer.named_children() if m.__class__.__name__ == "_LazyXPUGraph"]
    assert region.recorded == 1
    mods = [n.target for n in region.region.graph.nodes if n.op == "call_module"]
    assert len(mods) >= 3, mods  # add+norm, dense+silu, dense


def test_a_decode_step_replays_from_a_hip_graph(device):
    """One token against a cache of keys and values: the projections run on the row-streaming dense kernel, the
    attention on the key-split kernel (two launches and a workspace from the allocator, all inside the capture);
    every replay with new values matches eager."""

    def step(x, wq, wo, k_cache, v_cache, pad):
        B = x.shape[0]
        q = F.linear(x, wq).view(B, 1, 8, 128).transpose(1, 2)
        a = F.scaled_dot_product_attention(q, k_cache, v_cache, attn_mask=pad)
        return F.linear(a.transpose(1, 2).reshape(B, 1024), wo)

    g = torch.Generator().manual_seed(3)
    bf = torch.bfloat16
    B, S = 4, 1536
    mk = lambda *s, k=1.0: (torch.randn(*s, generator=g) * k).to(bf).to(device)  # noqa: E731
    x, wq, wo = mk(B, 1024), mk(1024, 1024, k=0.03), mk(1024, 1024, k=0.03)
    kc, vc = mk(B, 8, S, 128), mk(B, 8, S, 128)
    pad = torch.zeros(B, 1, 1, S, device=device, dtype=bf)
    pad[1, :, :, 1000:] = float("-inf")
    backend = mi355x_compiler()
    compiled = torch.compile(step, backend=backend, dynamic=False)
    with torch.no_grad():
        compiled(x, wq, wo, kc, vc, pad)
    mods = [n.target for n in backend.compiled_graphs[-1].graph.nodes if n.op == "call_module"]
    assert "mi355x_sdpa_masked" in mods, mods
    runner = HIPGraphRunner(compiled)
    runner.capture(x, wq, wo, kc, vc, pad, clone_args=True)
    for it in range(3):
        xs, ks, vs = mk(B, 1024), mk(B, 8, S, 128), mk(B, 8, S, 128)
        (torch.randn(512, 512, device=device) @ torch.randn(512, 512, device=device)).sum().item()
        y = runner(xs, wq, wo, ks, vs, pad).clone()
        with torch.no_grad():
            kr, vr = ks, vs
            q = F.linear(xs, wq).view(B, 1, 8, 128).transpose(1, 2)
            want = F.linear(F.scaled_dot_product_attention(q, kr, vr, attn_mask=pad).transpose(1, 2).reshape(B, 1024), wo)
        torch.testing.assert_close(y.float(), want.float(), rtol=1.6e-2, atol=2e-2)
