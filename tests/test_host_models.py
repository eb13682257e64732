"""Whole small modules through the backend, inference and training, default (target none) path on the CPU: the
behaviours the reference's model zoo pins (tests/common/test_models.py:7-86, test_inference.py:13-78,
test_training.py:13-49) -- a plain linear layer, a slice / negate / cat rewrite target, an in-place update of an
intermediate that is still read afterwards, data-dependent shapes (nonzero, scatter_) and dropout with the random
state forked around the golden run -- each with dynamic=True, with and without parameter freezing and with the
run-time parity guard switched on."""
import pytest
import torch
import torch.nn as nn

from xpu_graph_amd import OptLevel, XpuGraph, XpuGraphConfig
from xpu_graph_amd.test_utils import is_similar, need_xpu_graph_logs, skip_xpu_graph_cache

DIM = 16


class Linear1(nn.Module):
    def __init__(self):
        super().__init__()
        self.fc = nn.Linear(DIM, 1)

    def forward(self, x):
        return self.fc(x)


class RotateHalves(nn.Module):
    def __init__(self):
        super().__init__()
        self.fc = nn.Linear(DIM, 16)

    def forward(self, x):
        h = self.fc(x)
        return torch.cat([-h[..., 8:], h[..., :8]], 1).sum(dim=-1)


class InplaceAfterClone(nn.Module):
    def __init__(self):
        super().__init__()
        self.fc = nn.Linear(DIM, 16)

    def forward(self, x):
        h = torch.abs(self.fc(x)) + 1
        kept = h.clone()
        h.add_(1)
        return (h * kept).sum(dim=-1)


class DataDependentScatter(nn.Module):
    def __init__(self):
        super().__init__()
        self.fc = nn.Linear(DIM, 16)

    def forward(self, x):
        h = self.fc(x)
        idx = h.sum(dim=-1).nonzero().squeeze(-1)
        idx = idx[max(idx.shape[0] // 2, 1):]
        vals = h[idx].sum(-1)
        n = idx.max() + 1
        out = torch.zeros(n, dtype=vals.dtype, device=vals.device)
        out.scatter_(0, idx, vals)
        return torch.cat([out, torch.zeros(h.shape[0] - n, dtype=out.dtype, device=out.device)], dim=0)


class WithDropout(nn.Module):
    def __init__(self):
        super().__init__()
        self.fc = nn.Linear(DIM, 16)
        self.drop = nn.Dropout(0.5)

    def forward(self, x):
        return self.drop(self.fc(x))


ZOO = [Linear1, RotateHalves, InplaceAfterClone, DataDependentScatter, WithDropout]


def _pair(cls, train):
    golden, compiled = cls(), cls()
    compiled.load_state_dict(golden.state_dict())
    for m in (golden, compiled):
        m.train(train)
    return golden, compiled


def check_inference(cls, backend, bsz=80):
    golden, compiled = _pair(cls, train=False)
    compiled.forward = torch.compile(compiled.forward, backend=backend, dynamic=True)
    x = torch.randn(bsz, DIM)
    x_golden = x.clone()
    with torch.inference_mode():
        state = torch.random.get_rng_state()
        want = golden(x_golden)
        torch.random.set_rng_state(state)
        got = compiled(x)
    assert is_similar(x, x_golden)  # inputs untouched
    assert is_similar(got, want)


def check_training(cls, backend, steps=6, bsz=8):
    golden, compiled = _pair(cls, train=True)
    compiled.forward = torch.compile(compiled.forward, backend=backend, dynamic=True)
    x = torch.randn(bsz, DIM)
    target = torch.randn(bsz, 1)
    opt_g, opt_c = torch.optim.AdamW(golden.parameters()), torch.optim.AdamW(compiled.parameters())
    opt_c.load_state_dict(opt_g.state_dict())
    loss_fn = nn.MSELoss()
    for _ in range(steps):
        state = torch.random.get_rng_state()
        opt_g.zero_grad()
        loss_g = loss_fn(golden(x).reshape(bsz, -1).mean(-1, keepdim=True), target)
        loss_g.backward()
        opt_g.step()
        torch.random.set_rng_state(state)
        opt_c.zero_grad()
        loss_c = loss_fn(compiled(x).reshape(bsz, -1).mean(-1, keepdim=True), target)
        loss_c.backward()
        opt_c.step()
        assert is_similar(loss_g, loss_c), (loss_g.item(), loss_c.item())
    for pg, pc in zip(golden.parameters(), compiled.parameters()):
        assert is_similar(pg, pc)


@pytest.mark.parametrize("freeze", [False, True])
@pytest.mark.parametrize("cls", ZOO)
def test_inference_zoo(cls, freeze):
    backend = XpuGraph(XpuGraphConfig(is_training=False, opt_level=OptLevel.level2, freeze=freeze))
    with skip_xpu_graph_cache(backend):
        check_inference(cls, backend)
    torch._dynamo.reset()


@pytest.mark.parametrize("freeze", [False, True])
@pytest.mark.parametrize("cls", ZOO)
def test_inference_zoo_with_parity_guard(caplog, cls, freeze):
    backend = XpuGraph(XpuGraphConfig(is_training=False, opt_level=OptLevel.level2, freeze=freeze, enable_interceptor="rtol=1e-6,atol=1e-5"))
    with need_xpu_graph_logs(), skip_xpu_graph_cache(backend):
        check_inference(cls, backend)
    assert "Monitored inference" in caplog.text
    assert "diverges" not in caplog.text
    torch._dynamo.reset()


@pytest.mark.parametrize("cls", [Linear1, RotateHalves, InplaceAfterClone, WithDropout])
def test_training_zoo(cls):
    backend = XpuGraph(XpuGraphConfig(is_training=True, opt_level=OptLevel.level1, freeze=False))
    check_training(cls, backend)
    torch._dynamo.reset()


@pytest.mark.parametrize("partition_fn", ["MINCUT", "DEFAULT", "torch._functorch.partitioners.min_cut_rematerialization_partition", "dummy"])
def test_training_with_partitioner_and_parity_guard(caplog, monkeypatch, partition_fn):
    monkeypatch.setenv("XPUGRAPH_PARTITIONER", partition_fn)
    with need_xpu_graph_logs():
        backend = XpuGraph(XpuGraphConfig(is_training=True, opt_level=OptLevel.level1, freeze=False, enable_interceptor="rtol=1e-6,atol=1e-5"))
        check_training(Linear1, backend)
    assert "Monitored forward" in caplog.text and "Monitored backward" in caplog.text
    assert "diverges" not in caplog.text
    torch._dynamo.reset()
