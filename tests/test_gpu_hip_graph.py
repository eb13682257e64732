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
    with pytest.raises(AssertionError):
        runner(torch.randn(4, 64, device=device).bfloat16())
    again = runner.clone()
    assert again.mempool is None
    again.capture(a, clone_args=True)
    torch.testing.assert_close(again(a).float(), F.layer_norm(a + a, (64,)).float(), rtol=1.6e-2, atol=1e-2)
